"""Duvulix without a GPU: configuration, registry and schedule, weight names, and what pins the plain
implementation (tests/plain_duvulix.py) by closed forms and invariants."""
import copy
import math

import pytest
import torch

import plain_duvulix as plain
import tiny_duvulix as td


def _arch():
    import cpmcu_amd
    return cpmcu_amd.get_architecture("Duvulix")


@pytest.mark.parametrize("raw", [td.tiny_p(), td.tiny_q()])
def test_config_round_trip(raw):
    cfg = _arch().config_class.from_dict(raw)
    assert cfg.to_dict() == raw
    assert cfg.vocabulary_size == raw["vocab"] and cfg.longest_sequence is None


def test_architecture_is_named_by_a_plain_string():
    from cpmcu_amd.config.base import architecture_name
    assert architecture_name({"architecture": "Duvulix"}) == "Duvulix"
    assert architecture_name({"architectures": ["X"], "architecture": "Duvulix"}) == "X"


def test_config_refuses_what_the_design_excludes():
    from cpmcu_amd.config.base import ConfigError
    C = _arch().config_class
    bad = td.tiny_p()
    bad["layers"][4]["mixer"]["kv_from"] = 1                 # not a latent layer
    with pytest.raises(ConfigError, match="no latent cache"):
        C.from_dict(bad)
    bad = td.tiny_p()
    bad["layers"][4]["mixer"]["kv_rank"] = 32                # differs from the layer whose cache is read
    with pytest.raises(ConfigError, match="must equal"):
        C.from_dict(bad)
    bad = td.tiny_p()
    bad["layers"][2]["mixer"]["kv_from"] = 4                 # a later layer
    with pytest.raises(ConfigError, match="earlier"):
        C.from_dict(bad)
    bad = td.tiny_p()
    bad["layers"][1]["mixer"]["kv_heads"] = 3
    with pytest.raises(ConfigError, match="multiple"):
        C.from_dict(bad)
    bad = td.tiny_p()
    bad["layers"][0]["type"] = "lstm"
    with pytest.raises(ConfigError, match="not supported"):
        C.from_dict(bad)
    bad = td.tiny_p()
    bad["layers"][0]["mlp"]["kind"] = "experts"
    with pytest.raises(ConfigError, match="not supported"):
        C.from_dict(bad)


def test_schedule_and_cache_entries():
    a = _arch()
    m = a.build_model(a.config_class.from_dict(td.tiny_p()))
    runs = [(r.layer, r.cache, r.writes_cache) for r in m.schedule]
    assert runs == [(0, 0, True), (1, 1, True), (2, 2, True), (3, 3, True), (4, 2, False)]
    needs = m.cache_needs()
    assert len(needs) == 4
    assert needs[0].streams == () and {n for n, _ in needs[0].state} == {"ssm", "conv"}
    assert needs[1].window == 40 and needs[3].window is None
    # the latent cache holds kv_rank + rot_dim key features and kv_rank value features for all heads together
    assert dict(needs[2].streams)["k"].width == 80 and dict(needs[2].streams)["v"].width == 64
    m = a.build_model(a.config_class.from_dict(td.tiny_q()))
    # head sizes that are no multiple of 16 are padded in the cache
    assert dict(m.cache_needs()[0].streams)["k"].width == 80 and dict(m.cache_needs()[2].streams)["k"].width == 32
    assert {n for n, _ in m.cache_needs()[1].state} == {"ssm"}          # a single tap keeps no inputs


def test_weight_names_and_shapes():
    a = _arch()
    raw = td.tiny_p()
    specs = {s.name: tuple(s.shape) for s in a.build_model(a.config_class.from_dict(raw)).all_weight_specs()}
    assert specs["embed"] == (200, 96) and specs["head"] == (200, 96) and specs["final.norm"] == (96,)
    assert specs["l0.mix.in"] == (2 * 64 + 2 * 24 + 4, 96) and specs["l0.mix.conv"] == (64 + 48, 3)
    assert specs["l0.mix.conv.b"] == (112,) and specs["l0.mix.norm"] == (64,) and specs["l0.mix.o"] == (96, 64)
    assert specs["l1.mix.q"] == (192, 96) and specs["l1.mix.k"] == (96, 96) and specs["l1.mix.v"] == (64, 96)
    assert "l1.norm2" not in specs and "l1.mlp.up" not in specs and "l1.norm1b" in specs
    assert specs["l2.mix.q"] == (3 * 48, 96) and specs["l2.mix.dkv"] == (80, 96) and specs["l2.mix.dkv.norm"] == (64,)
    assert specs["l2.mix.uk"] == (96, 64) and specs["l2.mix.uv"] == (144, 64) and specs["l2.mix.g"] == (3, 96)
    assert "l4.mix.dkv" not in specs and "l4.mix.dkv.norm" not in specs and specs["l4.mix.uk"] == (80, 64)
    assert specs["l2.mlp.act"] == (4,) and specs["l2.mlp.up"] == (224, 96) and specs["l2.mlp.down"] == (96, 224)


def test_yarn_frequencies_of_the_part_equal_the_plain_ones():
    from cpmcu_amd.parts import POSITION_ENCODINGS
    from cpmcu_amd.parts.base import Runtime, Workspace
    rt = Runtime(torch.device("cpu"), torch.float32, Workspace("cpu"), 256)
    for rot in ({"base": 10000.0, "dims": 32, "scaling": {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}},
                {"base": 250000.0, "dims": 128, "scaling": {"factor": 8.0, "original": 8192, "fast": 24.0, "slow": 0.5}},
                {"base": 500.0, "dims": 8, "scaling": {"factor": 8.0, "original": 32, "fast": 1.0, "slow": 1.0}}):
        sc = rot["scaling"]
        enc = POSITION_ENCODINGS.build("yarn", head_dim=rot["dims"], theta=rot["base"], factor=sc["factor"],
                                       original=sc["original"], fast=sc["fast"], slow=sc["slow"])
        enc.bind({}, rt)
        f, mag = plain.frequencies(rot)
        inv, m = enc.rotary_params()
        assert torch.equal(inv, f.to(torch.float32)) and m == pytest.approx(mag, rel=1e-12)


# ---- what pins the plain implementation ----
def test_plain_yarn_limits():
    # pairs that turn often keep their frequency, pairs that turn rarely are slowed by the factor, and the
    # magnitude is 0.1 ln(factor) + 1
    rot = {"base": 10000.0, "dims": 64, "scaling": {"factor": 4.0, "original": 512, "fast": 32.0, "slow": 1.0}}
    f, mag = plain.frequencies(rot)
    f0, _ = plain.frequencies({"base": 10000.0, "dims": 64})
    assert mag == pytest.approx(1 + 0.1 * math.log(4.0))
    assert f[0] == f0[0] and f[-1] == pytest.approx(float(f0[-1]) / 4.0)
    ratio = f0 / f
    assert bool(((ratio[1:] - ratio[:-1]) >= -1e-12).all()) and float(ratio.max()) <= 4.0 + 1e-9
    # without scaling a rotation keeps lengths and composes: position a then b is position a + b
    x = torch.randn(3, 2, 40, dtype=torch.float64)
    r = {"base": 100.0, "dims": 24}
    y = plain.rotate(x, torch.tensor([5, 9, 200]), r)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1)) and torch.equal(y[..., 24:], x[..., 24:])
    assert torch.allclose(plain.rotate(y, torch.tensor([7, 7, 7]), r), plain.rotate(x, torch.tensor([12, 16, 207]), r))


def test_plain_masks():
    assert torch.equal(plain.visible(7, 100), plain.visible(7))
    m = plain.visible(10, 4)
    assert m[7].tolist() == [False] * 4 + [True] * 4 + [False] * 2 and m[8].tolist() == [False] * 8 + [True, False]


def test_plain_recurrence_closed_form():
    # constant inputs: S_t = dt B x (1 + a + ... + a^t), a = exp(-A dt)
    T, H, P, N = 9, 2, 3, 4
    x, B, C = torch.full((T, H, P), 0.5, dtype=torch.float64), torch.full((T, H, N), 2.0, dtype=torch.float64), \
        torch.full((T, H, N), 0.25, dtype=torch.float64)
    dt = torch.full((T, H), 0.3, dtype=torch.float64)
    A_log, D = torch.tensor([0.0, math.log(2.0)], dtype=torch.float64), torch.tensor([1.0, -1.0], dtype=torch.float64)
    y = plain.ssm_recurrence(x, B, C, dt, A_log, D)
    for h, A in enumerate((1.0, 2.0)):
        a = math.exp(-A * 0.3)
        for t in (0, 4, 8):
            geo = sum(a ** k for k in range(t + 1))
            want = N * 0.25 * (0.3 * 2.0 * 0.5 * geo) + float(D[h]) * 0.5
            assert float(y[t, h, 0]) == pytest.approx(want, rel=1e-12)


def test_plain_convolution_and_poly_norm():
    x = torch.arange(10, dtype=torch.float64).view(5, 2)
    w = torch.tensor([[1.0, 0.0, 0.0], [0.0, 0.0, 1.0]], dtype=torch.float64)      # channel 0 reads two back, 1 itself
    y = plain.causal_conv_silu(x, w, torch.zeros(2, dtype=torch.float64))
    pre = torch.stack([torch.tensor([0.0, 0.0, 0.0, 2.0, 4.0], dtype=torch.float64), x[:, 1]], 1)
    assert torch.allclose(y, pre * torch.sigmoid(pre))
    z = torch.tensor([[1.0, -1.0, 1.0, -1.0]], dtype=torch.float64)
    out = plain.poly_norm(z, [2.0, 3.0, 5.0, 7.0], 0.0)          # N(z) = z, N(z^2) = 1, N(z^3) = z
    assert torch.allclose(out, 2 * z + 3 + 5 * z + 7)


def test_plain_latent_attention_equals_expanded_attention():
    """Latent attention is ordinary attention over keys [W_uk c | shared] and values W_uv c."""
    torch.manual_seed(3)
    T, W_, H, d, r, dv, R = 12, 20, 2, 6, 4, 5, 8
    m = {"heads": H, "dim": d, "rot_dim": r, "vdim": dv, "kv_rank": R, "scale": 0.3, "rot": {"base": 50.0, "dims": r}}
    Wt = {k: torch.randn(s, dtype=torch.float64) * 0.4 for k, s in
          {"q": (H * (d + r), W_), "dkv": (R + r, W_), "dkv.norm": (R,), "uk": (H * d, R), "uv": (H * dv, R),
           "g": (H, W_), "o": (W_, H * dv)}.items()}
    h = torch.randn(T, W_, dtype=torch.float64)
    cache = plain.latent_cache(h, Wt, "", m, 1e-6)
    got = plain.latent_attention(h, Wt, "", m, cache)
    c, kr = cache
    q = (h @ Wt["q"].T).view(T, H, d + r)
    want = torch.zeros(T, H, dv, dtype=torch.float64)
    for i in range(T):
        for hh in range(H):
            qi = torch.cat([q[i, hh, :d], plain.rotate(q[i:i + 1, hh:hh + 1, d:], torch.tensor([i]), m["rot"])[0, 0]])
            keys = torch.cat([c[:i + 1] @ Wt["uk"][hh * d:(hh + 1) * d].T, kr[:i + 1]], 1)
            p = torch.softmax(keys @ qi * 0.3, 0)
            want[i, hh] = (p[:, None] * (c[:i + 1] @ Wt["uv"][hh * dv:(hh + 1) * dv].T)).sum(0) \
                * torch.sigmoid(h[i] @ Wt["g"][hh])
    assert torch.allclose(got, want.reshape(T, H * dv) @ Wt["o"].T, atol=1e-12)
