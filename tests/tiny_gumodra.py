"""Tiny Gumodra configurations for the tests.  They differ from each other in every size, in the order of the
layers and in the options: grouped, single and ungrouped kv heads, a rotation that covers a whole head, part of it
or nothing, windows shorter and longer than a cache page, kept first tokens within and beyond a page, experts with
and without groups, with and without a shared expert, one expert a token, layers without a feed-forward."""
import json
import os


def tiny_s():
    """mlstm first; a window of 24 with 5 kept tokens and grouped experts; a single kv head with a window of 70
    (longer than a page) and nothing kept; an mlstm of one head without a feed-forward; 70 kept tokens (more than a
    page) with ungrouped experts and no shared one."""
    return {
        "architecture": "Gumodra", "vocab": 210, "width": 96, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0},
        "layers": [
            {"type": "mlstm", "mixer": {"heads": 3, "dim": 16, "vdim": 24, "gate_cap": 8.0},
             "mlp": {"kind": "dense", "ff": 136}},
            {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 32, "scale": 0.2,
                                            "rot": {"base": 10000.0, "dims": 16}, "mask": {"size": 24, "keep_first": 5}},
             "mlp": {"kind": "moe", "expert": {"ff": 40},
                     "router": {"experts": 8, "top": 3, "groups": {"count": 4, "keep": 2}}, "shared": {"ff": 56}}},
            {"type": "attention", "mixer": {"heads": 6, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 0.25,
                                            "rot": {"base": 500.0, "dims": 16}, "mask": {"size": 70, "keep_first": 0}},
             "mlp": {"kind": "dense", "ff": 120}},
            {"type": "mlstm", "mixer": {"heads": 1, "dim": 40, "vdim": 8, "gate_cap": 15.0}, "mlp": None},
            {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 48, "vdim": 48, "scale": 0.15,
                                            "rot": {"base": 30000.0, "dims": 32}, "mask": {"size": 33, "keep_first": 70}},
             "mlp": {"kind": "moe", "expert": {"ff": 24}, "router": {"experts": 5, "top": 1}}},
        ],
    }


def tiny_t():
    """Sizes that suit no vector access and no matrix-core tile: a width of 100, a vocabulary of 77, heads of 20
    features (padded in the cache) of which 6 rotate, an mlstm of 12 by 7, experts of 20; every group kept; a
    layer whose attention sees everything (no window) and rotates nothing; an embedding scale of 1."""
    return {
        "architecture": "Gumodra", "vocab": 77, "width": 100, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0},
        "layers": [
            {"type": "attention", "mixer": {"heads": 5, "kv_heads": 5, "dim": 20, "vdim": 20, "scale": 0.3,
                                            "rot": {"base": 1000.0, "dims": 6}, "mask": {"size": 17, "keep_first": 3}},
             "mlp": {"kind": "moe", "expert": {"ff": 20},
                     "router": {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 3}}, "shared": {"ff": 12}}},
            {"type": "mlstm", "mixer": {"heads": 2, "dim": 12, "vdim": 7, "gate_cap": 5.0},
             "mlp": {"kind": "dense", "ff": 52}},
            {"type": "attention", "mixer": {"heads": 3, "kv_heads": 1, "dim": 24, "vdim": 24, "scale": 0.2,
                                            "rot": {"base": 1000.0, "dims": 0}},
             "mlp": {"kind": "moe", "expert": {"ff": 28},
                     "router": {"experts": 4, "top": 2, "groups": {"count": 2, "keep": 1}}, "shared": {"ff": 20}}},
        ],
    }


def write_model(raw, out_dir, seed, std=0.08, norm_std=0.1):
    """A model folder with random weights through the package's own writer; config.json is the raw dictionary."""
    import cpmcu_amd
    from cpmcu_amd.weights import write_model_dir
    arch = cpmcu_amd.get_architecture(raw["architecture"])
    cfg = arch.config_class.from_dict(raw)
    write_model_dir(cfg, out_dir, seed, std=std, norm_std=norm_std)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(raw, f, indent=1)
    return out_dir
