"""Every new mechanism alone, through its kernel entry points, against the plain implementation (GPU):
norms, PolyNorm, convolution and recurrence with state carried over portions, rotation and attention with
key and value sizes of their own and a chunked mask (keys just inside and just outside a chunk, at page
borders, far back), products head by head."""
import math

import pytest
import torch

import plain_duvulix as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def dev(t, dtype=None):
    return t.to(DEV, dtype) if dtype is not None else t.to(DEV)


def close(got, want, dtype, scale=None):
    want = want.to(torch.float64)
    tol = (2e-5 if dtype == "float32" else 1.5e-2) * float(scale if scale is not None else want.abs().max())
    err = float((got.detach().cpu().to(torch.float64) - want).abs().max())
    assert err <= tol, f"error {err:.3g} > {tol:.3g}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_poly_norm(dtype):
    from cpmcu_amd import ops
    torch.manual_seed(1)
    for n, F in ((5, 100), (70, 777), (1, 4)):
        z = (torch.randn(n, F) * 1.7).to(DT[dtype])
        coef = torch.tensor([0.7, -1.3, 0.4, 0.25])
        out = torch.empty(n, F, dtype=DT[dtype], device=DEV)
        ops.poly_norm(dev(z), dev(coef), 1e-5, out)
        close(out, plain.poly_norm(z.double(), coef.double(), 1e-5), dtype)
    # float partial sums of a split product
    parts = torch.randn(3, 6, 50)
    out = torch.empty(6, 50, dtype=DT[dtype], device=DEV)
    ops.poly_norm(dev(parts), dev(coef), 1e-6, out)
    close(out, plain.poly_norm(parts.double().sum(0), coef.double(), 1e-6), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_grouped_norm_with_gate_on_column_slices(dtype):
    from cpmcu_amd import ops
    torch.manual_seed(2)
    n, W, groups = 9, 96, 3
    wide = torch.randn(n, 40 + 2 * W).to(DT[dtype])           # [gate | junk | x]: slices of a wider row
    y = torch.randn(n, W)
    w = torch.randn(W)
    out = torch.empty(n, W, dtype=DT[dtype], device=DEV)
    wd = dev(wide)
    ops.rms_norm_groups(dev(y), dev(w), 1e-5, out, groups=groups, gate=wd[:, :W])
    z = wide[:, :W].double()
    v = y.double() * (z * torch.sigmoid(z))
    want = plain.rms(v.view(n, groups, W // groups), 1e-5).reshape(n, W) * w.double()
    close(out, want, dtype)
    # no gate, one group, input a slice
    out2 = torch.empty(n, W, dtype=DT[dtype], device=DEV)
    ops.rms_norm_groups(wd[:, 40 + W:], dev(w), 1e-6, out2)
    close(out2, plain.rms(wide[:, 40 + W:].double(), 1e-6) * w.double(), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_branch_norm_add_norm(dtype):
    from cpmcu_amd import ops
    torch.manual_seed(3)
    n, H = 11, 200
    x, wb, w = torch.randn(n, H), torch.randn(H) * 0.1 + 1, torch.randn(H) * 0.1 + 1
    for b in (torch.randn(n, H).to(DT[dtype]), torch.randn(3, n, H)):
        bsum = b.double().sum(0) if b.dim() == 3 else b.double()
        xs = x.double() + plain.rms(bsum, 1e-5) * wb.double()
        want = plain.rms(xs, 1e-6) * w.double()
        xd = dev(x.clone())
        out = torch.empty(n, H, dtype=DT[dtype], device=DEV)
        ops.branch_norm_add_norm(xd, dev(b), dev(wb), 1e-5, dev(w), 1e-6, out)
        close(out, want, dtype)
        close(xd, xs, "float32")
        # wanted rows only: the residual stays as it was
        rows = torch.tensor([7, 0, 7], dtype=torch.int32)
        xd = dev(x.clone())
        out = torch.empty(3, H, dtype=DT[dtype], device=DEV)
        ops.branch_norm_add_norm(xd, dev(b), dev(wb), 1e-5, dev(w), 1e-6, out, rows=dev(rows))
        close(out, want[rows.long()], dtype)
        assert torch.equal(xd.cpu(), x)


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_convolution_in_portions_and_slots(taps):
    """Two sequences in slots 3 and 1, fed in portions of unequal sizes (down to one token): equal to the
    convolution over each whole sequence; a slot that is cleared starts from zeros again."""
    from cpmcu_amd import ops
    torch.manual_seed(4)
    C = 70
    w, b = torch.randn(C, taps), torch.randn(C)
    seqs = {3: torch.randn(23, C + 9), 1: torch.randn(17, C + 9)}
    want = {s: plain.causal_conv_silu(u[:, 4:4 + C].double(), w.double(), b.double()) for s, u in seqs.items()}
    state = torch.zeros(5, max(taps - 1, 0), C, device=DEV) if taps > 1 else None
    cuts = {3: [5, 1, 1, 2, 14], 1: [1, 2, 9, 5]}
    done = {3: 0, 1: 0}
    got = {3: [], 1: []}
    for step in range(5):
        live = [s for s in (3, 1) if step < len(cuts[s])]
        rows = torch.cat([seqs[s][done[s]:done[s] + cuts[s][step]] for s in live])
        cu = [0]
        for s in live:
            cu.append(cu[-1] + cuts[s][step])
        out = torch.empty(rows.shape[0], C, device=DEV)
        ops.conv_silu(dev(rows)[:, 4:4 + C], dev(w), dev(b), state, out, dev(torch.tensor(cu, dtype=torch.int32)),
                      dev(torch.tensor(live, dtype=torch.int32)), max(cuts[s][step] for s in live))
        for i, s in enumerate(live):
            got[s].append(out[cu[i]:cu[i + 1]].cpu())
            done[s] += cuts[s][step]
    for s in (3, 1):
        close(torch.cat(got[s]), want[s], "float32")
    if taps > 1:
        assert float(state[[0, 2, 4]].abs().max()) == 0.0            # other slots untouched


@pytest.mark.parametrize("shape", [(4, 16, 24, 1), (6, 8, 20, 3), (1, 48, 16, 1), (3, 40, 130, 3)])
def test_recurrence_in_portions(shape):
    from cpmcu_amd import ops
    H, P, N, G = shape
    torch.manual_seed(5)
    T = 41
    width = H * P + 2 * G * N
    xbc = torch.randn(T, width)
    dt_raw = torch.randn(T, H + 3)
    dt_bias, A_log, D = torch.randn(H) * 0.5, torch.log(0.05 + 3 * torch.rand(H)), torch.randn(H)
    x = xbc[:, :H * P].double().view(T, H, P)
    B = xbc[:, H * P:H * P + G * N].double().view(T, G, N).repeat_interleave(H // G, 1)
    C = xbc[:, H * P + G * N:].double().view(T, G, N).repeat_interleave(H // G, 1)
    want = plain.ssm_recurrence(x, B, C, plain.softplus(dt_raw[:, 1:1 + H].double() + dt_bias.double()), A_log.double(),
                                D.double()).reshape(T, H * P)
    state = torch.zeros(3, H, P, N, device=DEV)
    got = []
    done = 0
    for cut in (16, 1, 2, 1, 21):                                  # a tile's edge, single tokens, two tokens
        y = torch.empty(cut, H * P, device=DEV)
        ops.ssm_scan(dev(xbc[done:done + cut].contiguous()), dev(dt_raw[done:done + cut])[:, 1:1 + H], dev(dt_bias),
                     dev(A_log), dev(D), state, y, dev(torch.tensor([0, cut], dtype=torch.int32)),
                     dev(torch.tensor([2], dtype=torch.int32)), H, P, N, G)
        got.append(y.cpu())
        done += cut
    close(torch.cat(got), want, "float32")
    assert float(state[:2].abs().max()) == 0.0


def test_recurrence_remembers_far_back():
    """One head that hardly decays: an impulse at the first token is still in the output 900 tokens later,
    where every other input is zero, with the weight the decay gives it."""
    from cpmcu_amd import ops
    H, P, N, T = 2, 16, 8, 900
    xbc = torch.zeros(T, H * P + 2 * N)
    xbc[0, :H * P] = 1.0                                           # x at token 0
    xbc[0, H * P:H * P + N] = 1.0                                  # B at token 0
    xbc[:, H * P + N:] = 0.5                                       # C always
    dt_raw = torch.zeros(T, H)
    dt_bias = torch.tensor([0.0, 0.0])
    A_log = torch.tensor([math.log(1e-4), math.log(0.05)])
    D = torch.zeros(H)
    y = torch.empty(T, H * P, device=DEV)
    state = torch.zeros(1, H, P, N, device=DEV)
    ops.ssm_scan(dev(xbc), dev(dt_raw), dev(dt_bias), dev(A_log), dev(D), state, y,
                 dev(torch.tensor([0, T], dtype=torch.int32)), dev(torch.tensor([0], dtype=torch.int32)), H, P, N, 1)
    d = math.log(2.0)                                              # softplus(0)
    for h, A in enumerate((1e-4, 0.05)):
        want = N * 0.5 * d * math.exp(-A * d * (T - 1))
        assert float(y[T - 1, h * P]) == pytest.approx(want, rel=2e-4)
    assert float(y[T - 1, 0]) > 3.0 * float(y[T - 1, P])           # the slow head remembers, the fast one less


def _fill_cache(keys, values, page, dtype, slot_pages):
    """Pools and a page table that hold keys [T, G, dk] and values [T, G, dv] of one sequence in slot 1, in the
    given (scattered) pages, written by the rotation kernel without rotation."""
    from cpmcu_amd import ops
    T, G, dk = keys.shape
    dv = values.shape[2]
    pk, pv = -(-dk // 16) * 16, -(-dv // 16) * 16
    n_pages = max(slot_pages) + 1
    kp = torch.zeros(n_pages, page, G * pk, dtype=dtype, device=DEV)
    vp = torch.zeros(n_pages, page, G * pv, dtype=dtype, device=DEV)
    table = torch.zeros(2, len(slot_pages), dtype=torch.int32)
    table[1] = torch.tensor(slot_pages, dtype=torch.int32)
    table = dev(table)
    pos = dev(torch.arange(T, dtype=torch.int32))
    slot = dev(torch.ones(T, dtype=torch.int32))
    paged = dict(tok_slot=slot, page_table=table, page_size=page, pool_heads=G)
    ops.rotate_copy(dev(keys.reshape(T, G * dk), dtype), 0, dk, G, dk, 0, pos, None, 1.0, kp, ops.ROTATE_TO_KEYS,
                    pool_hd=pk, **paged)
    ops.rotate_copy(dev(values.reshape(T, G * dv), dtype), 0, dv, G, dv, 0, pos, None, 1.0, vp, ops.ROTATE_TO_VALUES,
                    pool_hd=pv, **paged)
    return kp, vp, table


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(4, 2, 48, 32, 40, 32), (6, 1, 24, 40, 33, 64), (2, 2, 80, 64, 0, 32), (3, 1, 136, 72, 64, 64)])
def test_attention_with_sizes_of_its_own_and_chunks(dtype, shape):
    from cpmcu_amd import ops
    H, G, dk, dv, chunk, page = shape
    torch.manual_seed(6)
    T = 150
    q = torch.randn(T, H, dk).to(DT[dtype])
    k = torch.randn(T, G, dk).to(DT[dtype])
    v = torch.randn(T, G, dv).to(DT[dtype])
    pages = [7, 2, 9, 0, 4][:-(-T // page)]
    kp, vp, table = _fill_cache(k, v, page, DT[dtype], pages)
    out = torch.empty(T, H * dv, dtype=DT[dtype], device=DEV)
    ops.attention_general(dev(q.reshape(T, H * dk)), out, H, G, dk, dv, 0.2, kp, vp, table, page,
                          dev(torch.arange(T, dtype=torch.int32)), dev(torch.ones(T, dtype=torch.int32)), chunk)
    s = torch.einsum("ihd,jhd->hij", q.double(), k.double().repeat_interleave(H // G, 1)) * 0.2
    want = plain.softmax_attend(s, plain.visible(T, chunk or None), v.double().repeat_interleave(H // G, 1))
    close(out, want.reshape(T, H * dv), dtype)


@pytest.mark.parametrize("splits", [1, 3, 16])
@pytest.mark.parametrize("shape", [(4, 2, 48, 32, 40, 32, 150), (6, 1, 24, 40, 33, 64, 150), (2, 2, 80, 64, 0, 32, 150),
                                   (20, 1, 136, 72, 64, 64, 150), (3, 1, 576, 512, 0, 64, 700), (35, 1, 320, 272, 100, 32, 90)])
def test_matrix_core_attention_against_the_plain_kernel_and_the_plain_implementation(shape, splits):
    """The bf16 kernel on the matrix cores: prompts (every token of a sequence at once, more than 64 tokens and
    fewer) and shares of the keys that are merged; head groups larger than a tile of 16, sizes that are padded
    in the cache, values wider than a wavefront's four can merge."""
    from cpmcu_amd import ops
    H, G, dk, dv, chunk, page, T = shape
    torch.manual_seed(16)
    q = torch.randn(T, H, dk).to(torch.bfloat16)
    k = torch.randn(T, G, dk).to(torch.bfloat16)
    v = torch.randn(T, G, dv).to(torch.bfloat16)
    pages = [7, 2, 9, 0, 4, 11, 1, 3, 12, 5, 6, 8][:-(-T // page)]
    kp, vp, table = _fill_cache(k, v, page, torch.bfloat16, pages)
    pos, slot = dev(torch.arange(T, dtype=torch.int32)), dev(torch.ones(T, dtype=torch.int32))
    s = torch.einsum("ihd,jhd->hij", q.double(), k.double().repeat_interleave(H // G, 1)) * dk ** -0.5
    want = plain.softmax_attend(s, plain.visible(T, chunk or None), v.double().repeat_interleave(H // G, 1)).reshape(T, H * dv)
    qd = dev(q.reshape(T, H * dk))
    for rows in ((0, T), (T - 5, T), (T // 2, T // 2 + 1)):           # a prompt, a few tokens, a single token
        a, b = rows
        out = torch.empty(b - a, H * dv, dtype=torch.bfloat16, device=DEV)
        po = torch.empty(b - a, H, splits, dv, device=DEV) if splits > 1 else None
        pm = torch.empty(b - a, H, splits, 2, device=DEV) if splits > 1 else None
        ops.attention_general_mfma(qd[a:b], out, H, G, dk, dv, dk ** -0.5, kp, vp, table, page, pos[a:b], slot[a:b], chunk,
                                   splits, po, pm)
        close(out, want[a:b], "bfloat16")


@pytest.mark.parametrize("shape", [(8, 2, 48, 32, 40), (6, 1, 64, 64, 33), (4, 4, 32, 96, 0), (5, 1, 40, 24, 100)])
def test_matrix_core_attention_with_several_tokens_a_tile(shape):
    """Prompts of more than 256 tokens whose kv heads serve few query heads: consecutive tokens of one sequence
    share a tile.  Two sequences of unequal length in one packed batch, the second continuing from cached
    tokens; runs never straddle the sequences."""
    from cpmcu_amd import ops
    H, G, dk, dv, chunk = shape
    torch.manual_seed(17)
    page, T1, T2, old2 = 64, 301, 140, 37                 # sequence 2 holds 37 tokens already
    L2 = old2 + T2
    k = [torch.randn(T1, G, dk).to(torch.bfloat16), torch.randn(L2, G, dk).to(torch.bfloat16)]
    v = [torch.randn(T1, G, dv).to(torch.bfloat16), torch.randn(L2, G, dv).to(torch.bfloat16)]
    q = [torch.randn(T1, H, dk).to(torch.bfloat16), torch.randn(L2, H, dk).to(torch.bfloat16)]
    pk, pv = -(-dk // 16) * 16, -(-dv // 16) * 16
    kp = torch.zeros(12, page, G * pk, dtype=torch.bfloat16, device=DEV)
    vp = torch.zeros(12, page, G * pv, dtype=torch.bfloat16, device=DEV)
    table = torch.zeros(3, 5, dtype=torch.int32)
    table[2, :5] = torch.tensor([3, 9, 0, 7, 5])
    table[0, :3] = torch.tensor([11, 1, 6])
    table = dev(table)
    for sl, kk, vv in ((2, k[0], v[0]), (0, k[1], v[1])):
        Tn = kk.shape[0]
        paged = dict(tok_slot=dev(torch.full((Tn,), sl, dtype=torch.int32)), page_table=table, page_size=page, pool_heads=G)
        pos = dev(torch.arange(Tn, dtype=torch.int32))
        ops.rotate_copy(dev(kk.reshape(Tn, G * dk)), 0, dk, G, dk, 0, pos, None, 1.0, kp, ops.ROTATE_TO_KEYS, pool_hd=pk, **paged)
        ops.rotate_copy(dev(vv.reshape(Tn, G * dv)), 0, dv, G, dv, 0, pos, None, 1.0, vp, ops.ROTATE_TO_VALUES, pool_hd=pv, **paged)
    want = []
    for i in range(2):
        s = torch.einsum("ihd,jhd->hij", q[i].double(), k[i].double().repeat_interleave(H // G, 1)) * 0.2
        want.append(plain.softmax_attend(s, plain.visible(q[i].shape[0], chunk or None),
                                         v[i].double().repeat_interleave(H // G, 1)).reshape(-1, H * dv))
    qd = dev(torch.cat([q[0], q[1][old2:]]).reshape(T1 + T2, H * dk))
    pos = dev(torch.cat([torch.arange(T1), torch.arange(old2, L2)]).to(torch.int32))
    slot = dev(torch.cat([torch.full((T1,), 2), torch.full((T2,), 0)]).to(torch.int32))
    tpt = ops.attention_general_tokens_per_tile(T1 + T2, H, G, pv)
    assert tpt == 16 // (H // G)
    tiles = ops.prefill_tiles([T1, T2], tpt, DEV)
    out = torch.empty(T1 + T2, H * dv, dtype=torch.bfloat16, device=DEV)
    ops.attention_general_mfma(qd, out, H, G, dk, dv, 0.2, kp, vp, table, page, pos, slot, chunk, tiles=tiles,
                               tokens_per_tile=tpt)
    close(out, torch.cat([want[0], want[1][old2:]]), "bfloat16")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_key_that_stands_out_at_the_edges_of_a_chunk(dtype):
    """The key at one position is made to dominate every query.  A query sees it exactly when it lies in the
    query's chunk and not after the query: the first and last position of a chunk, the positions around a page
    border, a key hundreds of tokens back in an unchunked mask."""
    from cpmcu_amd import ops
    H, G, dk, dv, page = 2, 1, 32, 48, 64
    T = 700
    torch.manual_seed(7)
    for chunk, star in ((96, 96), (96, 95), (96, 191), (64, 64), (50, 449), (0, 3), (0, 640)):
        k = torch.randn(T, G, dk) * 0.1
        q = torch.randn(T, H, dk) * 0.1
        q[:, :, 0] = 6.0
        k[star, 0, 0] = 6.0
        v = torch.randn(T, G, dv)
        kp, vp, table = _fill_cache(k, v, page, DT[dtype], list(range(10, -1, -1)))
        out = torch.empty(T, H * dv, dtype=DT[dtype], device=DEV)
        ops.attention_general(dev(q.reshape(T, H * dk), DT[dtype]), out, H, G, dk, dv, 1.0, kp, vp, table, page,
                              dev(torch.arange(T, dtype=torch.int32)), dev(torch.ones(T, dtype=torch.int32)), chunk)
        if dtype == "bfloat16":       # the matrix-core kernel must see and not see exactly the same keys
            out2 = torch.empty_like(out)
            ops.attention_general_mfma(dev(q.reshape(T, H * dk), DT[dtype]), out2, H, G, dk, dv, 1.0, kp, vp, table, page,
                                       dev(torch.arange(T, dtype=torch.int32)), dev(torch.ones(T, dtype=torch.int32)), chunk)
            assert float((out2.float() - out.float()).abs().max()) < 0.05, (chunk, star)
        out = out.float().cpu().view(T, H, dv)
        vs = v[star, 0].to(DT[dtype]).float()
        sees = [p for p in range(T) if p >= star and (chunk == 0 or p // chunk == star // chunk)]
        for p in {sees[0], sees[-1], sees[len(sees) // 2]}:
            assert float((out[p, 0] - vs).abs().max()) < 0.05, (chunk, star, p)
        blind = [p for p in (star - 1, sees[-1] + 1, min(sees[-1] + chunk, T - 1)) if 0 <= p < T and p not in sees]
        for p in blind:
            assert float((out[p, 1] - vs).abs().max()) > 0.3, (chunk, star, p)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rotation_of_part_of_a_head(dtype):
    from cpmcu_amd import ops
    torch.manual_seed(8)
    n, H, d, dims = 7, 3, 40, 24
    rot = {"base": 300.0, "dims": dims, "scaling": {"factor": 3.0, "original": 16, "fast": 4.0, "slow": 1.0}}
    f, mag = plain.frequencies(rot)
    x = torch.randn(n, 5 + H * d).to(DT[dtype])
    pos = torch.tensor([0, 1, 5, 77, 130, 200, 12], dtype=torch.int32)     # float angles: p * f carries 2^-24 of p
    out = torch.zeros(n, H * (d + 2), dtype=DT[dtype], device=DEV)
    ops.rotate_copy(dev(x), 5, d, H, d, dims, dev(pos), dev(f.float()), mag, out, ops.ROTATE_TO_ROWS, 2, d + 2)
    want = plain.rotate(x[:, 5:].double().view(n, H, d), pos, rot)
    got = torch.stack([out.cpu()[:, 2 + h * (d + 2):2 + h * (d + 2) + d] for h in range(H)], 1)
    close(got, want, dtype)
    assert float(out[:, :2].abs().max()) == 0.0                    # what lies before the destination stays


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_products_head_by_head_with_gate(dtype):
    from cpmcu_amd import ops
    torch.manual_seed(9)
    M, H, N, K = 70, 3, 40, 24
    x = torch.randn(M, 7 + H * (K + 8)).to(DT[dtype])
    w = (torch.randn(H, N, K) * 0.3).to(DT[dtype])
    gate = torch.randn(M, H + 2).to(DT[dtype])
    out = torch.zeros(M, H * (N + 16), dtype=DT[dtype], device=DEV)
    gd = dev(gate)
    ops.gemm_heads(dev(x), 7, K + 8, dev(w), out, 16, N + 16, gate=gd[:, 1:1 + H])
    for h in range(H):
        xs = x[:, 7 + h * (K + 8):7 + h * (K + 8) + K].double()
        want = xs @ w[h].double().T * torch.sigmoid(gate[:, 1 + h].double())[:, None]
        close(out[:, 16 + h * (N + 16):16 + h * (N + 16) + N], want, dtype)
    assert float(out[:, :16].abs().max()) == 0.0


@pytest.mark.parametrize("shape", [(70, 3, 40, 24), (8, 5, 200, 64), (1, 2, 16, 512), (300, 2, 130, 136)])
def test_products_head_by_head_on_the_matrix_cores(shape):
    from cpmcu_amd import ops
    torch.manual_seed(10)
    M, H, N, K = shape
    x = torch.randn(M, 8 + H * (K + 8)).to(torch.bfloat16)
    w = (torch.randn(H, N, K) * 0.3).to(torch.bfloat16)
    gate = torch.randn(M, H).to(torch.bfloat16)
    for gt in (None, dev(gate)):
        out = torch.zeros(M, H * (N + 3), dtype=torch.bfloat16, device=DEV)
        twin = torch.zeros_like(out)
        ops.gemm_heads(dev(x), 8, K + 8, dev(w), out, 0, N + 3, gate=gt)
        ops.gemm_heads(dev(x), 8, K + 8, dev(w), twin, 0, N + 3, gate=gt, plain=True)
        for h in range(H):
            want = x[:, 8 + h * (K + 8):8 + h * (K + 8) + K].double() @ w[h].double().T
            if gt is not None:
                want = want * torch.sigmoid(gate[:, h].double())[:, None]
            close(out[:, h * (N + 3):h * (N + 3) + N], want, "bfloat16")
            assert float(out[:, h * (N + 3) + N:(h + 1) * (N + 3)].abs().max()) == 0.0
        assert float((out.float() - twin.float()).abs().max()) <= 0.02 * float(twin.float().abs().max())
