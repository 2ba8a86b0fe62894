"""Gumodra's mechanisms alone, through their kernel entry points, against the plain implementation (GPU):
biased projections with per-head norms, rotation and keys that double as values; attention with a sliding window,
kept first tokens and a sink (plain and matrix-core kernels; keys just inside and just outside the window, kept
tokens at their edges, page borders, far back); the matrix-memory recurrence in portions, with a memory that
lasts; routing with groups and corrections; experts; gates of a parallel layer."""
import math

import pytest
import torch

import plain_gumodra as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F64 = torch.float64


def dev(t, dtype=None):
    return t.to(DEV, dtype) if dtype is not None else t.to(DEV)


def close(got, want, dtype, scale=None):
    want = want.to(F64)
    tol = (2e-5 if dtype == "float32" else 1.5e-2) * float(scale if scale is not None else want.abs().max())
    err = float((got.detach().cpu().to(F64) - want).abs().max())
    assert err <= tol, f"error {err:.3g} > {tol:.3g}"


def i32(x):
    return dev(torch.as_tensor(x, dtype=torch.int32))


def _pools(T, G, dk, dv, page, dtype, slot_pages):
    pk, pv = -(-dk // 16) * 16, -(-dv // 16) * 16
    n_pages = max(slot_pages) + 1
    kp = torch.zeros(n_pages, page, G * pk, dtype=dtype, device=DEV)
    vp = torch.zeros(n_pages, page, G * pv, dtype=dtype, device=DEV)
    table = torch.zeros(2, len(slot_pages), dtype=torch.int32)
    table[1] = torch.tensor(slot_pages, dtype=torch.int32)
    return kp, vp, dev(table)


def _fill(keys, values, page, dtype, slot_pages):
    """Pools and a page table holding keys [T, G, dk] and values [T, G, dv] of one sequence in slot 1."""
    from cpmcu_amd import ops
    T, G, dk = keys.shape
    dv = values.shape[2]
    kp, vp, table = _pools(T, G, dk, dv, page, dtype, slot_pages)
    paged = dict(tok_slot=i32([1] * T), page_table=table, page_size=page, pool_heads=G)
    pos = i32(range(T))
    ops.rotate_copy(dev(keys.reshape(T, G * dk), dtype), 0, dk, G, dk, 0, pos, None, 1.0, kp, ops.ROTATE_TO_KEYS,
                    pool_hd=kp.shape[2] // G, **paged)
    ops.rotate_copy(dev(values.reshape(T, G * dv), dtype), 0, dv, G, dv, 0, pos, None, 1.0, vp, ops.ROTATE_TO_VALUES,
                    pool_hd=vp.shape[2] // G, **paged)
    return kp, vp, table


def _attend(q, k, v, scale, window, keep_first, sink):
    H, G = q.shape[1], k.shape[1]
    s = torch.einsum("ihd,jhd->hij", q.double(), k.double().repeat_interleave(H // G, 1)) * scale
    w = plain.sink_softmax(s, plain.visible(q.shape[0], window or None, keep_first), sink.double() if sink is not None else None)
    return torch.einsum("hij,jhd->ihd", w, v.double().repeat_interleave(H // G, 1)).reshape(q.shape[0], -1)


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(4, 2, 32, 16), (5, 5, 20, 6), (3, 1, 24, 0), (2, 2, 48, 48)])
def test_projection_to_normed_rotated_heads_with_keys_as_values(dtype, shape):
    """From a row [q | k] and a bias: q heads and k heads normed per head with weights shared by the heads, the
    first features rotated; the value pages hold k as projected.  Read back through attention of one-hot queries."""
    from cpmcu_amd import ops
    H, G, d, rd = shape
    torch.manual_seed(21)
    T, page, eps = 75, 32, 1e-5
    row = torch.randn(T, (H + G) * d + 3).to(DT[dtype])           # a wider row: the kernel reads its first columns
    bias = torch.randn((H + G) * d) * 0.5
    qw, kw = torch.rand(d) + 0.5, torch.rand(d) + 0.5
    rot = {"base": 300.0, "dims": rd}
    pos = torch.arange(T)
    full = row[:, :(H + G) * d].double() + bias.double()
    q_raw, k_raw = full[:, :H * d].view(T, H, d), full[:, H * d:].view(T, G, d)
    q_want = plain.rotate(plain.rms(q_raw, eps) * qw.double(), pos, rot)
    k_want = plain.rotate(plain.rms(k_raw, eps) * kw.double(), pos, rot)
    kp, vp, table = _pools(T, G, d, d, page, DT[dtype], [4, 0, 2])
    q_out = torch.empty(T, H * d, dtype=DT[dtype], device=DEV)
    inv = dev((300.0 ** (-2.0 * torch.arange(rd // 2, dtype=F64) / rd)).float()) if rd else None
    ops.qkv_norm_rotate_store(dev(row), q_out, H, G, d, d, rd, i32(range(T)), i32([1] * T), inv, 1.0, kp, vp, table, page,
                              bias=dev(bias), q_norm=dev(qw), k_norm=dev(kw), eps=eps, values_from_keys=True)
    close(q_out, q_want.reshape(T, H * d), dtype)
    # what lies in the pages: attention with queries from the plain implementation must give the plain result
    qq = torch.randn(T, H, d).to(DT[dtype])
    out = torch.empty(T, H * d, dtype=DT[dtype], device=DEV)
    ops.attention_general(dev(qq.reshape(T, H * d)), out, H, G, d, d, 0.3, kp, vp, table, page, i32(range(T)), i32([1] * T))
    close(out, _attend(qq, k_want, k_raw, 0.3, 0, 0, None), dtype, scale=float(k_raw.abs().max()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(4, 2, 32, 24, 5, 32), (6, 1, 16, 70, 0, 64), (2, 2, 48, 33, 70, 64), (5, 5, 20, 17, 3, 32),
                                   (8, 4, 128, 48, 12, 64), (3, 1, 24, 0, 0, 32)])
def test_window_kept_tokens_and_sink(dtype, shape):
    from cpmcu_amd import ops
    H, G, d, window, keep, page = shape
    torch.manual_seed(22)
    T = 230
    q, k, v = (torch.randn(T, n, d).to(DT[dtype]) for n in (H, G, G))
    sink = torch.randn(H) * 2
    kp, vp, table = _fill(k, v, page, DT[dtype], [7, 2, 9, 0, 4, 11, 1, 3][:-(-T // page)])
    want = _attend(q, k, v, 0.25, window, keep, sink)
    pos, slot = i32(range(T)), i32([1] * T)
    out = torch.empty(T, H * d, dtype=DT[dtype], device=DEV)
    ops.attention_general(dev(q.reshape(T, H * d)), out, H, G, d, d, 0.25, kp, vp, table, page, pos, slot, 0, window, keep, dev(sink))
    close(out, want, dtype)
    if dtype == "bfloat16" and d % 8 == 0:
        qd = dev(q.reshape(T, H * d))
        for a, b, splits in ((0, T, 1), (T - 70, T, 1), (T - 3, T, 1), (T - 3, T, 3), (100, 101, 16), (T - 1, T, 2)):
            out = torch.empty(b - a, H * d, dtype=torch.bfloat16, device=DEV)
            po = torch.empty(b - a, H, splits, d, device=DEV) if splits > 1 else None
            pm = torch.empty(b - a, H, splits, 2, device=DEV) if splits > 1 else None
            ops.attention_general_mfma(qd[a:b], out, H, G, d, d, 0.25, kp, vp, table, page, pos[a:b], slot[a:b], 0, splits,
                                       po, pm, window=window, keep_first=keep, sink=dev(sink))
            close(out, want[a:b], "bfloat16")


def test_matrix_core_prompt_tiles_with_a_window():
    """Prompts of more than 256 tokens whose kv heads serve few query heads put consecutive tokens into one tile:
    the tile's tokens have windows of their own."""
    from cpmcu_amd import ops
    H, G, d, window, keep, page = 4, 2, 32, 50, 10, 64
    torch.manual_seed(23)
    T = 400
    q, k, v = (torch.randn(T, n, d).to(torch.bfloat16) for n in (H, G, G))
    sink = torch.randn(H)
    kp, vp, table = _fill(k, v, page, torch.bfloat16, [7, 2, 9, 0, 4, 11, 1])
    tpt = ops.attention_general_tokens_per_tile(T, H, G, d)
    assert tpt == 8
    tiles = ops.prefill_tiles([T], tpt, DEV)
    out = torch.empty(T, H * d, dtype=torch.bfloat16, device=DEV)
    ops.attention_general_mfma(dev(q.reshape(T, H * d)), out, H, G, d, d, 0.25, kp, vp, table, page, i32(range(T)), i32([1] * T),
                               tiles=tiles, tokens_per_tile=tpt, window=window, keep_first=keep, sink=dev(sink))
    close(out, _attend(q, k, v, 0.25, window, keep, sink), "bfloat16")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_key_that_stands_out_at_the_edges_of_the_window(dtype):
    """The key at one position is made to dominate every query that sees it: exactly the queries from its position
    to window - 1 later, or all later ones if it is a kept first token.  Positions around the window's edge, the
    kept tokens' edge and page borders, in the plain and the matrix-core kernel, for prompts and single tokens."""
    from cpmcu_amd import ops
    H, G, d, page = 2, 1, 32, 64
    T = 520
    torch.manual_seed(24)
    cases = [(44, 18, 100), (44, 18, 17), (44, 18, 18), (64, 0, 64), (64, 0, 63), (33, 70, 69), (33, 70, 70), (100, 3, 2),
             (100, 3, 300), (1, 0, 77), (500, 0, 10)]
    for window, keep, star in cases:
        k = torch.randn(T, G, d) * 0.1
        q = torch.randn(T, H, d) * 0.1
        q[:, :, 0] = 6.0
        k[star, 0, 0] = 6.0
        v = torch.randn(T, G, d)
        kp, vp, table = _fill(k, v, page, DT[dtype], list(range(9, -1, -1)))
        pos, slot = i32(range(T)), i32([1] * T)
        qd = dev(q.reshape(T, H * d), DT[dtype])
        out = torch.empty(T, H * d, dtype=DT[dtype], device=DEV)
        ops.attention_general(qd, out, H, G, d, d, 1.0, kp, vp, table, page, pos, slot, 0, window, keep, None)
        outs = [out]
        if dtype == "bfloat16":
            o2 = torch.empty_like(out)
            ops.attention_general_mfma(qd, o2, H, G, d, d, 1.0, kp, vp, table, page, pos, slot, window=window, keep_first=keep)
            o3 = torch.empty_like(out)
            for t in range(max(star - 2, 0), min(star + window + 3, T)):            # token by token, keys in shares
                po, pm = torch.empty(1, H, 4, d, device=DEV), torch.empty(1, H, 4, 2, device=DEV)
                ops.attention_general_mfma(qd[t:t + 1], o3[t:t + 1], H, G, d, d, 1.0, kp, vp, table, page, pos[t:t + 1],
                                           slot[t:t + 1], 0, 4, po, pm, window=window, keep_first=keep)
            outs += [o2, o3]
        vs = v[star, 0].to(DT[dtype]).float()
        sees = [p for p in range(T) if p >= star and (p - star < window or star < keep)]
        near = [p for p in (star - 1, star + window, star + window + 1) if 0 <= p < T and p not in sees]
        for n_out, o in enumerate(outs):
            o = o.float().cpu().view(T, H, d)
            inside = {sees[0], min(star + window - 1, T - 1)} if n_out == 2 else {sees[0], sees[-1], sees[len(sees) // 2],
                                                                                 min(star + window - 1, T - 1)}
            for p in inside:
                assert float((o[p, 0] - vs).abs().max()) < 0.05, (window, keep, star, p, n_out)
            for p in near:
                assert float((o[p, 1] - vs).abs().max()) > 0.3, (window, keep, star, p, n_out)


def test_a_sink_that_outweighs_every_key_silences_the_head():
    from cpmcu_amd import ops
    H, G, d, page, T = 2, 1, 16, 32, 40
    torch.manual_seed(25)
    q, k, v = (torch.randn(T, n, d) for n in (H, G, G))
    kp, vp, table = _fill(k, v, page, torch.float32, [1, 0])
    sink = torch.tensor([40.0, -40.0])
    out = torch.empty(T, H * d, device=DEV)
    ops.attention_general(dev(q.reshape(T, H * d)), out, H, G, d, d, 0.25, kp, vp, table, page, i32(range(T)), i32([1] * T),
                          0, 0, 0, dev(sink))
    out = out.cpu().view(T, H, d)
    assert float(out[:, 0].abs().max()) < 1e-6
    close(out[:, 1].reshape(T, d), _attend(q[:, 1:], k, v, 0.25, 0, 0, None), "float32")


# ---------------------------------------------------------------------------
def _mlstm_inputs(T, H, d, dv, seed, dtype, f_bias=0.0):
    g = torch.Generator().manual_seed(seed)
    width = 2 * H * d + 2 * H * dv + 2 * H + 5
    proj = torch.randn(T, width, generator=g).to(DT[dtype])
    i_bias, f_b = torch.randn(H, generator=g) * 0.5, torch.randn(H, generator=g) * 0.5 + f_bias
    offs = dict(q=3, k=3 + H * d, v=3 + 2 * H * d, i=3 + 2 * H * d + H * dv + 1, f=3 + 2 * H * d + H * dv + 1 + H)
    return proj, i_bias, f_b, offs


def _mlstm_want(proj, i_bias, f_b, offs, H, d, dv, cap):
    T = proj.shape[0]
    p = proj.double()
    q = p[:, offs["q"]:offs["q"] + H * d].view(T, H, d) * d ** -0.5
    k = p[:, offs["k"]:offs["k"] + H * d].view(T, H, d)
    v = p[:, offs["v"]:offs["v"] + H * dv].view(T, H, dv)
    a = cap * torch.tanh((p[:, offs["i"]:offs["i"] + H] + i_bias.double()) / cap)
    b = torch.nn.functional.logsigmoid(cap * torch.tanh((p[:, offs["f"]:offs["f"] + H] + f_b.double()) / cap))
    return plain.mlstm_recurrence(q, k, v, a, b).reshape(T, H * dv)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(3, 16, 24), (1, 40, 8), (2, 12, 7), (5, 32, 40), (2, 130, 70), (1, 256, 33), (2, 300, 9),
                                   (1, 1000, 5)])
def test_matrix_memory_in_portions(dtype, shape):
    """Two sequences in slots 2 and 0, fed in portions of unequal sizes (down to one token, across a tile of 32):
    equal to the recurrence over each whole sequence; other slots stay untouched."""
    from cpmcu_amd import ops
    H, d, dv = shape
    cap = 6.0
    seqs = {2: _mlstm_inputs(57, H, d, dv, 31, dtype), 0: _mlstm_inputs(38, H, d, dv, 32, dtype)}
    i_bias, f_b, offs = seqs[2][1], seqs[2][2], seqs[2][3]
    want = {s: _mlstm_want(x[0], i_bias, f_b, offs, H, d, dv, cap) for s, x in seqs.items()}
    S = torch.zeros(4, H, dv, d, device=DEV)
    n_st, m_st = torch.zeros(4, H, d, device=DEV), torch.zeros(4, H, device=DEV)
    cuts = {2: [33, 1, 1, 2, 20], 0: [1, 2, 31, 4]}
    done, got = {2: 0, 0: 0}, {2: [], 0: []}
    for step in range(5):
        live = [s for s in (2, 0) if step < len(cuts[s])]
        rows = torch.cat([seqs[s][0][done[s]:done[s] + cuts[s][step]] for s in live])
        cu = [0]
        for s in live:
            cu.append(cu[-1] + cuts[s][step])
        y = torch.empty(rows.shape[0], H * dv, device=DEV)
        den = torch.empty(rows.shape[0], H, device=DEV)
        ops.mlstm_scan(dev(rows), offs["q"], offs["k"], offs["v"], offs["i"], offs["f"], dev(i_bias), dev(f_b), cap, d ** -0.5,
                       S, n_st, m_st, y, den, i32(cu), i32(live), H, d, dv)
        y = (y.view(-1, H, dv) / den[:, :, None]).view(-1, H * dv)
        for i, s in enumerate(live):
            got[s].append(y[cu[i]:cu[i + 1]].cpu())
            done[s] += cuts[s][step]
    for s in (2, 0):
        close(torch.cat(got[s]), want[s], "float32", scale=max(float(want[s].abs().max()), 1.0))
    assert float(S[[1, 3]].abs().max()) == 0.0 and float(m_st[[1, 3]].abs().max()) == 0.0


def test_matrix_memory_remembers_far_back():
    """Forget gates held open: a value written at the first token with a key that nothing else uses is read back
    900 tokens later; with the forget gates shut it is gone."""
    from cpmcu_amd import ops
    H, d, dv, T, cap = 1, 16, 8, 900, 10.0
    for f_val, remembered in ((30.0, True), (-2.0, False)):
        proj = torch.zeros(T, 2 * d + dv + 2)
        g = torch.Generator().manual_seed(33)
        proj[:, d + 1:2 * d] = torch.randn(T, d - 1, generator=g)               # keys of later tokens avoid feature 0
        proj[:, 2 * d:2 * d + dv] = torch.randn(T, dv, generator=g)
        proj[0, d] = 4.0
        proj[0, d + 1:2 * d] = 0.0
        proj[T - 1, 0] = 4.0 * d ** 0.5                                          # the last query asks for feature 0
        proj[:, 2 * d + dv + 1] = f_val
        S, n_st, m_st = torch.zeros(1, H, dv, d, device=DEV), torch.zeros(1, H, d, device=DEV), torch.zeros(1, H, device=DEV)
        y, den = torch.empty(T, dv, device=DEV), torch.empty(T, 1, device=DEV)
        z = torch.zeros(1)
        done = 0
        for cut in (500, 399, 1):
            ops.mlstm_scan(dev(proj[done:done + cut]), 0, d, 2 * d, 2 * d + dv, 2 * d + dv + 1, dev(z), dev(z), cap, d ** -0.5,
                           S, n_st, m_st, y[done:done + cut], den[done:done + cut], i32([0, cut]), i32([0]), H, d, dv)
            done += cut
        y = y / den
        want = _mlstm_want(proj, z, z, dict(q=0, k=d, v=2 * d, i=2 * d + dv, f=2 * d + dv + 1), H, d, dv, cap)
        close(y, want, "float32", scale=max(float(want.abs().max()), 1.0))
        v0 = proj[0, 2 * d:2 * d + dv]
        cos = float(torch.nn.functional.cosine_similarity(y[T - 1].cpu(), v0, dim=0))
        assert (cos > 0.999) == remembered, (f_val, cos)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_head_norm_with_gate_after_it(dtype):
    from cpmcu_amd import ops
    torch.manual_seed(34)
    n, H, dv = 9, 3, 24
    wide = torch.randn(n, 10 + H * dv).to(DT[dtype])
    y, w = torch.randn(n, H * dv) * 3, torch.randn(H * dv)
    out = torch.empty(n, H * dv, dtype=DT[dtype], device=DEV)
    ops.rms_norm_groups(dev(y), dev(w), 1e-5, out, groups=H, gate=dev(wide)[:, 10:], gate_after=True)
    want = plain.rms(y.double().view(n, H, dv), 1e-5).reshape(n, -1) * w.double() * torch.sigmoid(wide[:, 10:].double())
    close(out, want, dtype)
    # a divisor a (row, head) first: what the recurrence leaves to its norm
    den = torch.rand(n, H) * 3 + 0.01
    ops.rms_norm_groups(dev(y), dev(w), 1e-5, out, groups=H, gate=dev(wide)[:, 10:], gate_after=True, divisor=dev(den))
    want = (plain.rms(y.double().view(n, H, dv) / den.double()[:, :, None], 1e-5).reshape(n, -1) * w.double()
            * torch.sigmoid(wide[:, 10:].double()))
    close(out, want, dtype)


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(96, 8, 3, (4, 2)), (100, 6, 2, (3, 3)), (64, 5, 1, None), (128, 64, 6, (8, 3)), (72, 4, 2, (2, 1)),
                                   (192, 12, 3, (4, 3))])
def test_routing(dtype, shape):
    from cpmcu_amd import ops
    Hd, E, top, groups = shape
    torch.manual_seed(41)
    n = 70
    h = torch.randn(n, Hd).to(DT[dtype])
    W = {"router": torch.randn(E, Hd) * 0.3, "correction": torch.randn(E) * 0.05}
    sgw = torch.randn(Hd) * 0.2
    r = {"experts": E, "top": top}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    idx_w, w_w = plain.route(h.double(), {k: v.double() for k, v in W.items()}, "", r)
    idx = torch.empty(n, top, dtype=torch.int32, device=DEV)
    wts = torch.empty(n, top, device=DEV)
    sg = torch.empty(n, device=DEV)
    ops.moe_route(dev(h), dev(W["router"]), dev(W["correction"]), dev(sgw), groups[0] if groups else 1,
                  groups[1] if groups else 1, top, idx, wts, sg)
    got = idx.cpu().long()
    assert torch.equal(got.sort(1).values, idx_w.sort(1).values)
    order = got.argsort(1), idx_w.argsort(1)
    close(wts.cpu().gather(1, order[0]), w_w.gather(1, order[1]), "float32", scale=1.0)
    close(sg, torch.sigmoid(h.double() @ sgw.double()), "float32", scale=1.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(96, 40, 8, 3), (100, 20, 6, 2), (64, 24, 5, 1), (128, 56, 12, 4)])
def test_experts(dtype, shape):
    from cpmcu_amd import ops
    Hd, F, E, top = shape
    torch.manual_seed(42)
    n = 37
    h = torch.randn(n, Hd).to(DT[dtype])
    gu = (torch.randn(E, 2 * F, Hd) * 0.2).to(DT[dtype])
    dn = (torch.randn(E, Hd, F) * 0.2).to(DT[dtype])
    idx = torch.stack([torch.randperm(E)[:top] for _ in range(n)]).to(torch.int32)
    w = torch.rand(n, top)
    shared = torch.randn(2, n, Hd)
    sgate = torch.rand(n)
    act = torch.empty(n, top, F, dtype=DT[dtype], device=DEV)
    ops.moe_gated(dev(h), dev(gu), dev(idx), act)
    hh = h.double()
    want_act = torch.stack([torch.stack([plain.silu(hh[t] @ gu[e, :F].double().T) * (hh[t] @ gu[e, F:].double().T)
                                         for e in idx[t].tolist()]) for t in range(n)])
    close(act, want_act, dtype)
    out = torch.empty(n, Hd, device=DEV)
    ops.moe_down(act, dev(dn), dev(idx), dev(w), out, dev(shared), dev(sgate))
    a = act.cpu().double()
    want = torch.stack([sum(w[t, j].double() * (a[t, j] @ dn[e].double().T) for j, e in enumerate(idx[t].tolist()))
                        for t in range(n)]) + sgate.double()[:, None] * shared.double().sum(0)
    close(out, want, "float32" if dtype == "float32" else "bfloat16")
    out2 = torch.empty(n, Hd, device=DEV)
    ops.moe_down(act, dev(dn), dev(idx), dev(w), out2)
    close(out2, want - sgate.double()[:, None] * shared.double().sum(0), "float32" if dtype == "float32" else "bfloat16")


@pytest.mark.parametrize("shape", [(96, 40, 8, 3, 300), (104, 24, 6, 2, 65), (64, 24, 5, 1, 700), (128, 72, 12, 4, 1000),
                                   (256, 136, 40, 6, 129)])
def test_experts_of_many_tokens_on_the_matrix_cores(shape):
    """Pairs grouped by expert in tiles of 64 rows: equal to the few-token kernels pair by pair, whatever row of a
    tile a pair lands in; experts that nobody chose, experts with more than a tile of tokens, a last tile partly
    empty."""
    from cpmcu_amd import ops
    Hd, F, E, top, n = shape
    torch.manual_seed(44)
    h = torch.randn(n, Hd).to(torch.bfloat16)
    gu = (torch.randn(E, 2 * F, Hd) * 0.2).to(torch.bfloat16)
    dn = (torch.randn(E, Hd, F) * 0.2).to(torch.bfloat16)
    busy = max(E - 2, top)                                        # the last experts stay without tokens
    idx = torch.stack([torch.randperm(busy)[:top] for _ in range(n)]).to(torch.int32)
    idx[:n // 2, 0] = 0                                           # and the first is crowded
    for t in range(n // 2):
        if (idx[t, 1:] == 0).any():
            idx[t, 1:][idx[t, 1:] == 0] = busy - 1 if busy - 1 not in idx[t].tolist() else idx[t, 0]
    idx = torch.stack([torch.tensor(sorted(set(r.tolist())) + [e for e in range(busy) if e not in r.tolist()])[:top]
                       for r in idx]).to(torch.int32)
    w = torch.rand(n, top)
    shared = torch.randn(n, Hd).to(torch.bfloat16)
    sgate = torch.rand(n)
    hd, gud, dnd, idxd, wd = dev(h), dev(gu), dev(dn), dev(idx), dev(w)
    act = torch.empty(n, top, F, dtype=torch.bfloat16, device=DEV)
    want = torch.empty(n, Hd, device=DEV)
    ops.moe_gated(hd, gud, idxd, act)
    ops.moe_down(act, gud.new_empty(0) if False else dnd, idxd, wd, want, dev(shared), dev(sgate))
    tiles = ops.moe_tiles(n, top, E)
    act2 = torch.empty_like(act)
    y = torch.empty(n, top, Hd, dtype=torch.bfloat16, device=DEV)
    rows = torch.empty(tiles * ops.MOE_TILE, dtype=torch.int32, device=DEV)
    te, nt = torch.empty(tiles, dtype=torch.int32, device=DEV), torch.empty(1, dtype=torch.int32, device=DEV)
    out = torch.empty(n, Hd, device=DEV)
    for _ in range(2):
        ops.moe_experts_mfma(hd, gud, dnd, idxd, wd, out, act2, y, rows, te, nt, dev(shared), dev(sgate))
        close(act2, act.float().cpu(), "bfloat16")
        close(out, want.cpu(), "bfloat16")
    counts = torch.bincount(idx.flatten().long(), minlength=E)
    assert int(nt) == int(((counts + 63) // 64).sum())
    placed = rows[:int(nt) * 64].cpu()
    assert sorted(placed[placed >= 0].tolist()) == list(range(n * top))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gates_of_a_parallel_layer(dtype):
    from cpmcu_amd import ops
    torch.manual_seed(43)
    n, Hd = 13, 100
    g = torch.randn(n, 2 * Hd + 4).to(DT[dtype])
    gb, ab = torch.randn(2 * Hd), torch.randn(Hd)
    a = torch.randn(3, n, Hd)
    f = torch.randn(n, Hd).to(DT[dtype])
    out = torch.empty(n, Hd, device=DEV)
    ops.gated_branches(dev(g)[:, :2 * Hd], dev(gb), dev(a), dev(ab), dev(f), None, out)
    gd = g.double()[:, :2 * Hd] + gb.double()
    want = torch.sigmoid(gd[:, :Hd]) * (a.double().sum(0) + ab.double()) + torch.sigmoid(gd[:, Hd:]) * f.double()
    close(out, want, "float32")
    ops.gated_branches(dev(g)[:, :Hd], dev(gb[:Hd]), dev(a), None, None, None, out)
    close(out, torch.sigmoid(gd[:, :Hd]) * a.double().sum(0), "float32")
    o2 = torch.empty(n, Hd, device=DEV)
    ops.bias_sum(dev(a), dev(ab), o2)
    close(o2, a.double().sum(0) + ab.double(), "float32")
