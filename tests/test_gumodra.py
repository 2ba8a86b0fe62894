"""Gumodra without a GPU: configuration, refusals, tensor names and cache needs; the plain implementation pinned by
closed forms and invariants; the cache's bookkeeping for groups that keep a window and a sequence's first tokens."""
import copy
import math
import random

import pytest
import torch

import plain_gumodra as plain
import tiny_gumodra as tg

F64 = torch.float64


# ---------------------------------------------------------------------------
# configuration and model
# ---------------------------------------------------------------------------
def _cfg(raw):
    import cpmcu_amd
    arch = cpmcu_amd.get_architecture(raw["architecture"])
    return arch, arch.config_class.from_dict(raw)


@pytest.mark.parametrize("raw", [tg.tiny_s(), tg.tiny_t()])
def test_configuration_reads_back(raw):
    arch, cfg = _cfg(raw)
    assert arch.config_class.from_dict(cfg.to_dict()) == cfg
    assert cfg.vocabulary_size == raw["vocab"] and len(cfg.layers) == len(raw["layers"])
    assert cfg.embedding_scale == raw["embedding"]["scale"]


def test_defaults_of_absent_keys():
    raw = tg.tiny_t()
    del raw["embedding"]
    del raw["layers"][0]["mixer"]["kv_heads"]
    del raw["layers"][0]["mixer"]["mask"]["keep_first"]
    _, cfg = _cfg(raw)
    assert cfg.embedding_scale == 1.0
    m = cfg.layers[0].mixer
    assert m.kv_heads == m.heads and m.keep_first == 0 and m.window == 17
    assert cfg.layers[2].mixer.window is None and cfg.layers[2].mixer.rot_dims == 0


@pytest.mark.parametrize("change, word", [
    (lambda r: r["layers"][0]["mixer"].update(vdim=24), "vdim"),
    (lambda r: r["layers"][0]["mixer"].update(kv_heads=2), "kv_heads"),
    (lambda r: r["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda r: r["layers"][0]["mixer"]["mask"].update(size=0), "mask.size"),
    (lambda r: r["layers"][0]["mlp"]["router"].update(top=7), "top"),
    (lambda r: r["layers"][0]["mlp"]["router"]["groups"].update(count=4), "groups"),
    (lambda r: r["layers"][2]["mlp"]["router"].update(top=3), "top"),
    (lambda r: r["layers"][1]["mixer"].update(gate_cap=0.0), "gate_cap"),
    (lambda r: r["layers"][1].update(type="mamba2"), "type"),
    (lambda r: r["layers"][1]["mlp"].update(kind="poly"), "kind"),
])
def test_refusals(change, word):
    from cpmcu_amd import ConfigError
    raw = tg.tiny_t()
    change(raw)
    with pytest.raises(ConfigError, match=word):
        _cfg(raw)


def test_tensor_names_and_cache_needs():
    arch, cfg = _cfg(tg.tiny_s())
    model = arch.build_model(cfg)
    specs = {s.name: tuple(s.shape) for s in model.all_weight_specs()}
    assert specs["l0.norm1"] == () and specs["final.norm"] == ()
    assert specs["l1.mix.q"] == (4 * 32, 96) and specs["l1.mix.k"] == (2 * 32, 96) and "l1.mix.v" not in specs
    assert specs["l1.mix.q.norm"] == (32,) and specs["l1.mix.sink"] == (4,) and specs["l1.mix.o.b"] == (96,)
    assert specs["l0.mix.i"] == (3, 96) and specs["l0.mix.f.b"] == (3,) and specs["l0.mix.norm"] == (72,)
    assert specs["l1.mlp.e7.down"] == (96, 40) and specs["l1.mlp.shared.sg"] == (1, 96) and specs["l1.mlp.correction"] == (8,)
    assert specs["l1.rg2.b"] == (96,) and "l3.rg2" not in specs and "l3.rg1" in specs
    assert "l4.mlp.shared.gate" not in specs and specs["l4.mlp.router"] == (5, 96)
    needs = model.cache_needs()
    assert needs[1].window == 24 and needs[1].keep_first == 5 and needs[4].keep_first == 70
    assert needs[0].streams == () and dict(needs[0].state)["memory"].shape == (3, 24, 16)
    assert arch.ignore_tensor(cfg, "l3.rg2") and not arch.ignore_tensor(cfg, "l2.rg2")


# ---------------------------------------------------------------------------
# the plain implementation
# ---------------------------------------------------------------------------
def test_visible_window_with_kept_first_tokens():
    m = plain.visible(7, size=2, keep_first=1)
    want = [[1, 0, 0, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0, 0], [1, 1, 1, 0, 0, 0, 0], [1, 0, 1, 1, 0, 0, 0],
            [1, 0, 0, 1, 1, 0, 0], [1, 0, 0, 0, 1, 1, 0], [1, 0, 0, 0, 0, 1, 1]]
    assert m.int().tolist() == want
    assert plain.visible(5).int().tolist() == torch.tril(torch.ones(5, 5)).int().tolist()
    assert plain.visible(6, size=100, keep_first=0).equal(plain.visible(6))


def test_sink_takes_its_share_of_the_softmax():
    s = torch.tensor([[[0.3, -1.0], [0.7, 0.2]]], dtype=F64)
    mask = plain.visible(2)
    w = plain.sink_softmax(s, mask, torch.tensor([0.5], dtype=F64))
    # first query: one key and the sink
    assert w[0, 0, 0].item() == pytest.approx(math.exp(0.3) / (math.exp(0.3) + math.exp(0.5)))
    assert w[0, 0, 1].item() == 0.0
    tot = math.exp(0.7) + math.exp(0.2) + math.exp(0.5)
    assert w[0, 1].tolist() == pytest.approx([math.exp(0.7) / tot, math.exp(0.2) / tot])
    far = plain.sink_softmax(s, mask, torch.tensor([-1e9], dtype=F64))
    assert torch.allclose(far, plain.sink_softmax(s, mask, None))


def test_rotation_composes_and_leaves_the_rest():
    rot = {"base": 100.0, "dims": 4}
    x = torch.randn(3, 2, 6, dtype=F64)
    pos = torch.tensor([0, 5, 9])
    y = plain.rotate(x, pos, rot)
    assert torch.equal(y[..., 4:], x[..., 4:]) and torch.allclose(y[0], x[0])
    assert torch.allclose(y[..., :4].norm(dim=-1), x[..., :4].norm(dim=-1))
    # scores depend on the distance only
    q, k = torch.randn(1, 1, 4, dtype=F64), torch.randn(1, 1, 4, dtype=F64)
    a = (plain.rotate(q, torch.tensor([7]), rot) * plain.rotate(k, torch.tensor([3]), rot)).sum()
    b = (plain.rotate(q, torch.tensor([14]), rot) * plain.rotate(k, torch.tensor([10]), rot)).sum()
    assert a.item() == pytest.approx(b.item())


def test_recurrence_equals_the_unstabilised_sums():
    """The running maximum only keeps the exponentials in range: the state times exp(m) is the plain weighted sum
    of the outer products, with weights exp(sum of the later log forget gates + the log input gate)."""
    g = torch.Generator().manual_seed(3)
    T, H, d, dv = 9, 2, 3, 4
    q, k = torch.randn(T, H, d, generator=g, dtype=F64), torch.randn(T, H, d, generator=g, dtype=F64)
    v = torch.randn(T, H, dv, generator=g, dtype=F64)
    a = torch.randn(T, H, generator=g, dtype=F64) * 2
    b = -torch.rand(T, H, generator=g, dtype=F64)
    got = plain.mlstm_recurrence(q, k, v, a, b)
    B = torch.cumsum(b, 0)
    m = torch.zeros(H, dtype=F64)
    for t in range(T):
        m = torch.maximum(b[t] + m, a[t])
        wts = torch.exp(B[t][None] - B[:t + 1] + a[:t + 1])                       # [t+1, H]
        C = torch.einsum("sh,shd,shv->hdv", wts, k[:t + 1], v[:t + 1])
        n = torch.einsum("sh,shd->hd", wts, k[:t + 1])
        num = torch.einsum("hdv,hd->hv", C, q[t]) * torch.exp(-m)[:, None]
        den = torch.maximum((n * q[t]).sum(-1).abs() * torch.exp(-m), torch.exp(-m)) + 1e-6
        assert torch.allclose(got[t], num / den[:, None], rtol=1e-10, atol=1e-12)


def test_recurrence_with_open_gates_counts_tokens():
    T = 5
    q = torch.ones(T, 1, 1, dtype=F64) * 2
    k = torch.ones(T, 1, 1, dtype=F64)
    v = torch.arange(1, T + 1, dtype=F64).view(T, 1, 1)
    z = torch.zeros(T, 1, dtype=F64)
    out = plain.mlstm_recurrence(q, k, v, z, z)           # m stays 0: S_t = sum of v, n_t = t
    for t in range(T):
        assert out[t, 0, 0].item() == pytest.approx(2 * sum(range(1, t + 2)) / (2 * (t + 1) + 1e-6))


def test_gates_are_capped():
    W = {"i": torch.tensor([[100.0]], dtype=F64), "i.b": torch.zeros(1, dtype=F64),
         "f": torch.tensor([[-100.0]], dtype=F64), "f.b": torch.zeros(1, dtype=F64)}
    a, b = plain.mlstm_gates(torch.ones(1, 1, dtype=F64), W, "", 4.0)
    assert a.item() == pytest.approx(4.0, abs=1e-9) and b.item() == pytest.approx(-4.0 - math.log1p(math.exp(-4.0)), abs=1e-9)


def test_router_groups_shut_experts_out():
    """6 experts in 3 groups of which 2 are kept: the best single expert of a shut-out group loses to lesser ones;
    a correction decides the choice and not the weights; negative choice scores still rank."""
    H = 6
    W = {"router": torch.eye(6, dtype=F64) * 1.0, "correction": torch.zeros(6, dtype=F64)}
    h = torch.tensor([[2.0, 0.1, 1.9, 1.8, 2.5, 0.0]], dtype=F64) - 5.0
    r = {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}}
    idx, w = plain.route(h, W, "", r)
    assert sorted(idx[0].tolist()) == [0, 4]              # groups {0,1}, {2,3}, {4,5}: 4 and 0 lead their groups
    assert w.sum().item() == pytest.approx(1.0)
    r1 = {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 1}}
    idx, _ = plain.route(h, W, "", r1)
    assert sorted(idx[0].tolist()) == [4, 5]              # only the best group: its second expert is the weakest of all
    W2 = dict(W, correction=torch.tensor([0, 0, 5.0, 5.0, 0, 0], dtype=F64) - 9.0)
    idx, w = plain.route(h, W2, "", {"experts": 6, "top": 2})
    assert sorted(idx[0].tolist()) == [2, 3]
    s = torch.softmax(h, -1)[0]
    assert w[0].tolist() == pytest.approx([float(s[i] / (s[2] + s[3])) for i in idx[0].tolist()])


def test_a_layer_without_feed_forward_has_one_gated_term():
    raw = tg.tiny_s()
    g = torch.Generator().manual_seed(5)
    names = {"l3.norm1": (), "l3.rg1": (96, 96), "l3.rg1.b": (96,), "l3.mix.q": (40, 96), "l3.mix.k": (40, 96),
             "l3.mix.v": (8, 96), "l3.mix.g": (8, 96), "l3.mix.o": (96, 8), "l3.mix.norm": (8,), "l3.mix.i": (1, 96),
             "l3.mix.i.b": (1,), "l3.mix.f": (1, 96), "l3.mix.f.b": (1,)}
    W = {k: torch.randn(s, generator=g, dtype=F64) * 0.1 for k, s in names.items()}
    x = torch.randn(4, 96, generator=g, dtype=F64)
    y = plain.layer(x, W, 3, raw["layers"][3], 1e-5)
    h = plain.scalar_norm(x, W["l3.norm1"], 1e-5)
    want = x + torch.sigmoid(h @ W["l3.rg1"].T + W["l3.rg1.b"]) * plain.mlstm(h, W, "l3.mix.", raw["layers"][3]["mixer"], 1e-5)
    assert torch.allclose(y, want)


# ---------------------------------------------------------------------------
# the cache: a trailing window and a sequence's first tokens
# ---------------------------------------------------------------------------
def _cache(window, keep_first, max_tokens=64 * 40, slots=3, page=32, step=50):
    from cpmcu_amd.cache.paged import CacheNeeds, SequenceCache, StreamSpec
    needs = [CacheNeeds(streams=(("k", StreamSpec(8)),), window=window, keep_first=keep_first),
             CacheNeeds(streams=(("k", StreamSpec(8)),))]
    return SequenceCache(needs, max_tokens, slots, 4096, page, "cpu", torch.float32, step)


@pytest.mark.parametrize("window, keep_first", [(44, 18), (33, 70), (100, 0), (5, 32), (64, 1)])
def test_window_group_keeps_what_its_queries_read(window, keep_first):
    c = _cache(window, keep_first)
    g = c.groups[0]
    rnd = random.Random(window * 100 + keep_first)
    s = c.acquire()
    length = 0
    while length < 1500:
        n = rnd.choice([1, 1, 1, 2, 7, 31, 50])
        assert c.room_for([[(s, n)]]) is None
        first = c.extend(s, n)
        assert first == length
        length += n
        c.check()
        # every key that a query of this step reads lies in a held page
        pages = g.pages[s]
        for p in range(first, length):
            for j in list(range(max(p - window + 1, 0), p + 1)) + list(range(min(keep_first, p + 1))):
                assert pages[j // 32] >= 0, f"query {p} reads key {j}, whose page was given back"
        held = g.held(s)
        assert held <= c.pages_to_hold(length, 50)[0]
        assert int(g.table_host[s, 0]) == pages[0] or keep_first == 0
    c.release(s)
    c.check()
    assert len(g.free_pages) == g.n_pages


def test_room_for_counts_as_extend_does():
    """room_for plays passes through on counts alone; it must say yes exactly when extend succeeds."""
    from cpmcu_amd.cache.paged import CacheError
    rnd = random.Random(11)
    for trial in range(30):
        window, keep_first = rnd.choice([(44, 18), (33, 70), (20, 0), (70, 33)])
        c = _cache(window, keep_first, max_tokens=32 * rnd.choice([6, 9, 14]), slots=3, step=2048)
        slots = [c.acquire() for _ in range(3)]
        for _ in range(40):
            passes = [[(rnd.choice(slots), rnd.choice([1, 3, 30, 64, 100]))] for _ in range(rnd.choice([1, 2, 3]))]
            verdict = c.room_for(passes)
            shadow = copy.deepcopy(c)
            ok = True
            try:
                for one in passes:
                    for slot, n in one:
                        shadow.extend(slot, n)
            except CacheError:
                ok = False
            assert (verdict is None) == ok, (window, keep_first, passes, verdict)
            if ok:
                c = shadow
                slots = list(c.live)
            c.check()


def test_pool_of_a_window_group_counts_the_kept_pages():
    from cpmcu_amd.cache.paged import CacheNeeds, SequenceCache, StreamSpec
    needs = [CacheNeeds(streams=(("k", StreamSpec(4)),), window=10, keep_first=100)]
    c = SequenceCache(needs, 64 * 100, 2, 6400, 64, "cpu", torch.float32, 1)
    # a sequence holds two pages of kept tokens and the window's pages, however long it grows
    s = c.acquire()
    for _ in range(700):
        c.extend(s, 1)
    assert c.groups[0].held(s) <= 2 + 2 and c.groups[0].pages[s][0] >= 0 and c.groups[0].pages[s][1] >= 0
    assert c.groups[0].pages[s][2] == -1
    assert c.capacity()[0] >= 2 * 4
    before = SequenceCache.plan_bytes(needs, 64 * 100, 2, 6400, 64, torch.float32, 1)
    assert before == c.bytes() + 2 * 100 * 4
