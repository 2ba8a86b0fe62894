"""Gumodra: which parts, with which numbers.

A decoder whose layers each have one norm (an RMS norm with a single number as its weight), a mixer and an optional
feed-forward that both read the normed rows, and a sigmoid gate on each of the two results before they join the
residual: x += sigmoid(rg1 h + b) * mixer(h) + sigmoid(rg2 h + b) * ff(h), h = norm1(x).  The mixer is grouped-query
attention (biased q, k and output projections, the projected keys double as values, q and k normed per head before a
rotation of the first features, a sliding window that keeps the sequence's first tokens, a softmax sink a head) or
an mLSTM matrix memory; the feed-forward is a SiLU-gated layer or a mixture of such experts with a shared one.
The embedding is multiplied by a number from the configuration; head and embedding are separate tables; the model's
last norm is ``final.norm``.

Checkpoint tensors: ``embed``, ``head``, ``final.norm``, and per layer i ``l<i>.norm1``, ``l<i>.rg1|rg2`` (+ ``.b``),
``l<i>.mix.*`` (attention: q, k, o with ``.b``, q.norm, k.norm, sink; mlstm: q, k, v, g, o, norm, i, f with ``.b``)
and ``l<i>.mlp.gate|up|down`` or ``l<i>.mlp.router|correction|e<j>.gate|up|down|shared.gate|up|down|sg``.
"""
from __future__ import annotations

from ..config.gumodra import ARCHITECTURE, GumodraConfig
from ..parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, LMHead, TokenEmbedding
from ..registry import Architecture, register_architecture
from .decoder import DecoderModel

_FF_NAMES = {"gate": "gate", "up": "up", "down": "down"}


def _mixer(cfg: GumodraConfig, i: int):
    layer, p = cfg.layers[i], f"l{i}.mix."
    m = layer.mixer
    if layer.type == "attention":
        names = {"q": p + "q", "k": p + "k", "out": p + "o", "q_bias": p + "q.b", "k_bias": p + "k.b",
                 "out_bias": p + "o.b", "q_norm": p + "q.norm", "k_norm": p + "k.norm", "sink": p + "sink"}
        position = (POSITION_ENCODINGS.build("rope", head_dim=m.rot_dims, theta=m.rot_base) if m.rot_dims else None)
        return MIXERS.build("attention", names=names, hidden_size=cfg.width, num_heads=m.heads, num_kv_heads=m.kv_heads,
                            key_dim=m.dim, value_dim=m.vdim, position=position, scale=m.scale, mask_window=m.window,
                            mask_keep_first=m.keep_first if m.window is not None else 0, norm_eps=cfg.eps)
    names = {"q": p + "q", "k": p + "k", "v": p + "v", "gate": p + "g", "out": p + "o", "norm": p + "norm",
             "input_gate": p + "i", "input_gate_bias": p + "i.b", "forget_gate": p + "f", "forget_gate_bias": p + "f.b"}
    return MIXERS.build("mlstm", names=names, hidden_size=cfg.width, heads=m.heads, key_dim=m.dim, value_dim=m.vdim,
                        gate_cap=m.gate_cap, eps=cfg.eps)


def _feed_forward(cfg: GumodraConfig, i: int):
    ff, p = cfg.layers[i].mlp, f"l{i}.mlp."
    if ff is None:
        return None
    if ff.kind == "dense":
        return FEED_FORWARDS.build("gated_silu", prefix=p, hidden_size=cfg.width, intermediate_size=ff.ff, names=_FF_NAMES)
    names = {"router": p + "router", "correction": p + "correction", "expert": p + "e{e}.{part}",
             "shared_gate": p + "shared.gate", "shared_up": p + "shared.up", "shared_down": p + "shared.down",
             "shared_scale": p + "shared.sg"}
    return FEED_FORWARDS.build("routed_experts", names=names, hidden_size=cfg.width, expert_size=ff.ff,
                               experts=ff.experts, top=ff.top, groups=ff.groups, shared_size=ff.shared_ff)


def build(cfg: GumodraConfig) -> DecoderModel:
    norm = lambda name: NORMS.build("rms_norm", name=name, hidden_size=cfg.width, eps=cfg.eps, scalar=True)
    layers = []
    for i in range(len(cfg.layers)):
        p = f"l{i}."
        ff = _feed_forward(cfg, i)
        gates = [(p + "rg1", p + "rg1.b")] + ([(p + "rg2", p + "rg2.b")] if ff is not None else [])
        layers.append(BLOCKS.build("parallel_gated", norm=norm(p + "norm1"), mixer=_mixer(cfg, i), feed_forward=ff,
                                   hidden_size=cfg.width, gate_names=gates))
    embedding = TokenEmbedding("embed", cfg.vocab, cfg.width, cfg.embedding_scale)
    head = LMHead("head", cfg.vocab, cfg.width, 1.0)
    return DecoderModel(cfg, embedding, layers, norm("final.norm"), head)


def _ignore(cfg: GumodraConfig, name: str) -> bool:
    """A layer without a feed-forward has no second gate: a checkpoint that stores one all the same is read without it."""
    for i, layer in enumerate(cfg.layers):
        if layer.mlp is None and name in (f"l{i}.rg2", f"l{i}.rg2.b"):
            return True
    return False


register_architecture(Architecture(name=ARCHITECTURE, config_class=GumodraConfig, build=build, ignore_tensor=_ignore))
