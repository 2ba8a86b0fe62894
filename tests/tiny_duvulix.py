"""Tiny Duvulix configurations for the tests.  They differ from each other in every size, in the order of the
layers and in the options: grouped and ungrouped kv heads, a rotation that covers a whole head or part of it,
with and without YaRN scaling, chunked and plain masks, one or several norm groups, layers without a
feed-forward, a latent cache that two layers read."""
import json
import os


def tiny_p():
    """mamba2 first, a chunked attention with 2 kv heads for 4 heads and partial rotation, a latent pair, an
    unchunked attention whose key and value sizes are equal."""
    return {
        "architecture": "Duvulix", "vocab": 200, "width": 96, "norm": {"eps": 1e-5},
        "layers": [
            {"type": "mamba2", "mixer": {"heads": 4, "vdim": 16, "state": 24, "groups": 1, "conv": 3, "norm_groups": 4},
             "mlp": {"kind": "dense", "ff": 160}},
            {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 48, "vdim": 32, "scale": 0.15,
                                            "rot": {"base": 10000.0, "dims": 32,
                                                    "scaling": {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}},
                                            "mask": {"size": 40}},
             "mlp": None},
            {"type": "latent_attention", "mixer": {"heads": 3, "dim": 32, "rot_dim": 16, "vdim": 48, "kv_rank": 64,
                                                   "scale": 0.12, "rot": {"base": 100000.0, "dims": 16}},
             "mlp": {"kind": "dense", "ff": 224}},
            {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 32, "vdim": 32, "scale": 0.18,
                                            "rot": {"base": 5000.0, "dims": 32}},
             "mlp": {"kind": "dense", "ff": 128}},
            {"type": "latent_attention", "mixer": {"heads": 5, "dim": 16, "rot_dim": 16, "vdim": 16, "kv_rank": 64,
                                                   "scale": 0.2, "rot": {"base": 100000.0, "dims": 16}, "kv_from": 2},
             "mlp": {"kind": "dense", "ff": 160}},
        ],
    }


def tiny_q():
    """latent attention first, sizes that need padding in the cache (24, 40, 72), one group for all heads, a
    chunk of 33 tokens, a single-tap convolution, one norm group, one head."""
    return {
        "architecture": "Duvulix", "vocab": 131, "width": 72, "norm": {"eps": 1e-6},
        "layers": [
            {"type": "latent_attention", "mixer": {"heads": 2, "dim": 24, "rot_dim": 8, "vdim": 40, "kv_rank": 72,
                                                   "scale": 0.2, "rot": {"base": 30000.0, "dims": 8}},
             "mlp": None},
            {"type": "mamba2", "mixer": {"heads": 6, "vdim": 8, "state": 20, "groups": 3, "conv": 1, "norm_groups": 1},
             "mlp": {"kind": "dense", "ff": 100}},
            {"type": "attention", "mixer": {"heads": 6, "kv_heads": 1, "dim": 24, "vdim": 40, "scale": 0.25,
                                            "rot": {"base": 20000.0, "dims": 24}, "mask": {"size": 33}},
             "mlp": {"kind": "dense", "ff": 88}},
            {"type": "mamba2", "mixer": {"heads": 1, "vdim": 48, "state": 16, "groups": 1, "conv": 5, "norm_groups": 3},
             "mlp": {"kind": "dense", "ff": 100}},
        ],
    }


def tiny_r():
    """Sizes that suit no vector access and no matrix-core tile: a width of 100, a vocabulary of 77, heads of 20 and
    12 features, a latent of 36 with 4 rotated features, 5 kv heads of 3 query heads each, a state of 7."""
    return {
        "architecture": "Duvulix", "vocab": 77, "width": 100, "norm": {"eps": 1e-6},
        "layers": [
            {"type": "attention", "mixer": {"heads": 15, "kv_heads": 5, "dim": 20, "vdim": 12, "scale": 0.3,
                                            "rot": {"base": 1000.0, "dims": 6}, "mask": {"size": 17}},
             "mlp": {"kind": "dense", "ff": 52}},
            {"type": "latent_attention", "mixer": {"heads": 3, "dim": 20, "rot_dim": 4, "vdim": 12, "kv_rank": 36,
                                                   "scale": 0.25, "rot": {"base": 777.0, "dims": 4}},
             "mlp": {"kind": "dense", "ff": 30}},
            {"type": "mamba2", "mixer": {"heads": 3, "vdim": 5, "state": 7, "groups": 3, "conv": 2, "norm_groups": 5},
             "mlp": None},
            {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 40, "vdim": 40, "scale": 0.2,
                                            "rot": {"base": 1000.0, "dims": 40,
                                                    "scaling": {"factor": 16.0, "original": 24, "fast": 8.0, "slow": 1.0}}},
             "mlp": {"kind": "dense", "ff": 52}},
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
