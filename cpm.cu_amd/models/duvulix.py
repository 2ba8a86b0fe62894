"""Duvulix: which parts, with which numbers.

A decoder whose layers each choose one of three mixers (latent attention, grouped-query attention with a
chunked mask and YaRN-scaled rotation, a Mamba-2 state-space mixer) and an optional PolyNorm feed-forward, with
an RMS norm (weight stored around zero, multiplied as 1 + w) before and after every sub-layer:
x += norm1b(mixer(norm1 x)); x += norm2b(ff(norm2 x)).  Embedding and head are separate tables; the model's
last norm is ``final.norm``.  A latent-attention layer with ``kv_from`` reads the latent cache of an earlier
layer: in the schedule its run names that layer's cache entry and writes none.

Checkpoint tensors: ``embed``, ``head``, ``final.norm``, and per layer i ``l<i>.norm1|norm1b|norm2|norm2b``,
``l<i>.mix.*`` (latent attention: q, dkv, dkv.norm, uk, uv, g, o; attention: q, k, v, o; mamba2: in, conv,
conv.b, dt_bias, A_log, D, norm, o) and ``l<i>.mlp.up|down|act``.
"""
from __future__ import annotations

from typing import List, Optional

from ..config.duvulix import ARCHITECTURE, DuvulixConfig, Rotation
from ..parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, LMHead, TokenEmbedding
from ..registry import Architecture, register_architecture
from .decoder import DecoderModel, Run


def _position(rot: Rotation):
    if rot.dims == 0:
        return None
    if rot.scaling is not None:
        factor, original, fast, slow = rot.scaling
        return POSITION_ENCODINGS.build("yarn", head_dim=rot.dims, theta=rot.base, factor=factor, original=original,
                                        fast=fast, slow=slow)
    return POSITION_ENCODINGS.build("rope", head_dim=rot.dims, theta=rot.base)


def _mixer(cfg: DuvulixConfig, i: int):
    layer, p = cfg.layers[i], f"l{i}.mix."
    m = layer.mixer
    if layer.type == "latent_attention":
        names = {"q": p + "q", "down": p + "dkv", "down_norm": p + "dkv.norm", "up_k": p + "uk", "up_v": p + "uv",
                 "gate": p + "g", "out": p + "o"}
        return MIXERS.build("latent_attention", names=names, hidden_size=cfg.width, num_heads=m.heads, key_dim=m.dim,
                            rot_dim=m.rot_dim, value_dim=m.vdim, kv_rank=m.kv_rank, position=_position(m.rot),
                            scale=m.scale, eps=cfg.eps, shares_cache=m.kv_from is not None)
    if layer.type == "attention":
        names = {"q": p + "q", "k": p + "k", "v": p + "v", "out": p + "o"}
        return MIXERS.build("attention", names=names, hidden_size=cfg.width, num_heads=m.heads, num_kv_heads=m.kv_heads,
                            key_dim=m.dim, value_dim=m.vdim, position=_position(m.rot), scale=m.scale,
                            mask_chunk=m.mask_size)
    names = {"in": p + "in", "conv": p + "conv", "conv_bias": p + "conv.b", "dt_bias": p + "dt_bias",
             "A_log": p + "A_log", "D": p + "D", "norm": p + "norm", "out": p + "o"}
    return MIXERS.build("mamba2", names=names, hidden_size=cfg.width, heads=m.heads, head_dim=m.vdim,
                        state_size=m.state, groups=m.groups, conv_taps=m.conv, norm_groups=m.norm_groups, eps=cfg.eps)


def build(cfg: DuvulixConfig) -> DecoderModel:
    norm = lambda name: NORMS.build("rms_norm", name=name, hidden_size=cfg.width, eps=cfg.eps, unit_offset=True)
    layers, schedule = [], []
    entry_of: List[Optional[int]] = []
    n_entries = 0
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        ff = {}
        if layer.ff is not None:
            ff = dict(ff_norm=norm(p + "norm2"), ff_post_norm=norm(p + "norm2b"),
                      feed_forward=FEED_FORWARDS.build("poly_norm", up_name=p + "mlp.up", down_name=p + "mlp.down",
                                                       act_name=p + "mlp.act", hidden_size=cfg.width,
                                                       intermediate_size=layer.ff, eps=cfg.eps))
        layers.append(BLOCKS.build("sandwich_norm", mixer_norm=norm(p + "norm1"), mixer=_mixer(cfg, i),
                                   mixer_post_norm=norm(p + "norm1b"), **ff))
        src = getattr(layer.mixer, "kv_from", None)
        if src is None:
            entry_of.append(n_entries)
            schedule.append(Run(i, n_entries, True))
            n_entries += 1
        else:
            entry_of.append(None)
            schedule.append(Run(i, entry_of[src], False))
    embedding = TokenEmbedding("embed", cfg.vocab, cfg.width, 1.0)
    head = LMHead("head", cfg.vocab, cfg.width, 1.0)
    return DecoderModel(cfg, embedding, layers, norm("final.norm"), head, schedule)


register_architecture(Architecture(name=ARCHITECTURE, config_class=DuvulixConfig, build=build))
