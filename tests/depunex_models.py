"""Small Depunex configurations for the tests, and model folders with random weights for them.

The configurations differ from each other in every size and option: heads that share key/value heads or groups of B and C
and heads that do not, one head, values wider and narrower than keys, chunks shorter than a cache block, longer than one and
absent, rotations over a part of the head, the whole head or none, with and without stretched frequencies, convolutions of
one to five taps, states of fewer and more entries than a wavefront's share, experts with and without groups, layers with
a dense feed-forward, experts or none in every order, and a model without the hashed table, the side table and the cap.
"""
import os

import torch

MIXED = {
    "architecture": "Depunex", "vocab": 97, "width": 48, "norm": {"eps": 1e-5}, "logit_softcap": 9.0,
    "embedding": {"scale": 3.0, "bigram": {"buckets": 53, "mul_prev": 7, "mul_cur": 13}}, "token_side": {"dim": 6},
    "layers": [
        {"type": "parallel",
         "mixer": {"left": {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 16, "scale": 0.3, "mask": {"size": 20},
                            "rot": {"dims": 12, "base": 1000.0, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}}},
                   "right": {"inner": 40, "state": 10, "dt_rank": 3, "conv": 3}, "left_scale": 0.7, "right_scale": 1.3},
         "mlp": {"kind": "moe", "expert": {"ff": 24}, "router": {"experts": 8, "top": 2, "groups": {"count": 4, "keep": 2}}}},
        {"type": "mamba2", "mixer": {"heads": 4, "vdim": 12, "state": 20, "groups": 2, "norm_groups": 3, "conv": 4},
         "mlp": {"kind": "dense", "ff": 56, "limit": 0.8}},
        {"type": "mamba2", "mixer": {"heads": 2, "vdim": 40, "state": 72, "groups": 1, "norm_groups": 1, "conv": 2}, "mlp": None},
    ],
}
WIDE = {
    "architecture": "Depunex", "vocab": 130, "width": 64, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "mamba2", "mixer": {"heads": 1, "vdim": 136, "state": 16, "groups": 1, "norm_groups": 2, "conv": 5},
         "mlp": {"kind": "moe", "expert": {"ff": 16}, "router": {"experts": 6, "top": 3}}},
        {"type": "parallel",
         "mixer": {"left": {"heads": 2, "kv_heads": 2, "dim": 32, "vdim": 48, "scale": 0.2, "mask": {"size": 70},
                            "rot": {"dims": 32, "base": 10000.0}},
                   "right": {"inner": 100, "state": 16, "dt_rank": 5, "conv": 4}, "left_scale": 1.0, "right_scale": 0.5},
         "mlp": {"kind": "dense", "ff": 40, "limit": 2.0}},
        {"type": "parallel",
         "mixer": {"left": {"heads": 3, "kv_heads": 1, "dim": 16, "vdim": 8, "scale": 0.25},
                   "right": {"inner": 64, "state": 33, "dt_rank": 1, "conv": 1}, "left_scale": 1.5, "right_scale": 1.0},
         "mlp": {"kind": "moe", "expert": {"ff": 20}, "router": {"experts": 12, "top": 1, "groups": {"count": 3, "keep": 1}}}},
    ],
}
EDGES = {
    "architecture": "Depunex", "vocab": 64, "width": 32, "norm": {"eps": 1e-3}, "logit_softcap": 30.0,
    "embedding": {"scale": 1.5, "bigram": {"buckets": 7, "mul_prev": 1, "mul_cur": 1}}, "token_side": {"dim": 1},
    "layers": [
        {"type": "parallel",
         "mixer": {"left": {"heads": 1, "kv_heads": 1, "dim": 64, "vdim": 64, "scale": 0.125, "mask": {"size": 64},
                            "rot": {"dims": 2, "base": 10.0, "scaling": {"factor": 2.0, "low": 2.0, "high": 3.0, "original": 16}}},
                   "right": {"inner": 16, "state": 1, "dt_rank": 2, "conv": 2}, "left_scale": 1.0, "right_scale": 1.0},
         "mlp": None},
        {"type": "mamba2", "mixer": {"heads": 3, "vdim": 16, "state": 8, "groups": 3, "norm_groups": 6, "conv": 1},
         "mlp": {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 4, "top": 4, "groups": {"count": 2, "keep": 2}}}},
        {"type": "parallel",
         "mixer": {"left": {"heads": 4, "kv_heads": 4, "dim": 8, "vdim": 4, "scale": 0.5, "mask": {"size": 1}},
                   "right": {"inner": 72, "state": 24, "dt_rank": 4, "conv": 3}, "left_scale": 0.25, "right_scale": 2.0},
         "mlp": {"kind": "dense", "ff": 24, "limit": 0.25}},
        {"type": "parallel",
         "mixer": {"left": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 24, "scale": 0.3, "mask": {"size": 128},
                            "rot": {"dims": 8, "base": 100.0}},
                   "right": {"inner": 8, "state": 5, "dt_rank": 8, "conv": 5}, "left_scale": 1.0, "right_scale": 1.0},
         "mlp": {"kind": "moe", "expert": {"ff": 12}, "router": {"experts": 9, "top": 2, "groups": {"count": 3, "keep": 2}}}},
    ],
}
CONFIGS = {"mixed": MIXED, "wide": WIDE, "edges": EDGES}


def make_depunex_folder(raw_config, folder, seed, std=0.2, router_std=0.5):
    """A model folder for `raw_config` with the library's random weights, where the small tensors are then given values that
    make them matter: gains and layer scales away from one, biases and skips away from zero, step sizes and decay rates in
    the range where a state neither forgets at once nor keeps everything, a router whose scores differ."""
    from xeno_rt_amd.config import parse_config
    from xeno_rt_amd.weights import SafetensorsFile, write_random_model, write_safetensors

    folder = str(folder)
    write_random_model(parse_config(raw_config), folder, seed=seed, std=std)
    path = os.path.join(folder, "model.safetensors")
    with SafetensorsFile(path) as file:
        tensors = {name: file.read(name) for name in file.names()}
    generator = torch.Generator().manual_seed(seed + 1)

    def normal(shape, mean, deviation):
        return mean + deviation * torch.randn(shape, generator=generator)

    for name, tensor in tensors.items():
        last = name.split(".")[-1]
        if last in ("norm1", "ls1", "ls2") or name == "final.norm":
            new = normal(tensor.shape, 0.0 if last == "norm1" or name == "final.norm" else 1.0, 0.3)
        elif last == "norm":
            new = normal(tensor.shape, 1.0, 0.3)
        elif last in ("conv", "D"):
            new = normal(tensor.shape, 0.0, 0.5)
        elif name.endswith(("conv.b", "dt.b", "dt_bias")):
            new = normal(tensor.shape, 0.0 if name.endswith("conv.b") else -1.0, 0.5)
        elif last == "A_log":
            new = normal(tensor.shape, -1.0, 1.0)
        elif last == "router":
            new = normal(tensor.shape, 0.0, router_std)      # (wide models take a smaller one: a sigmoid of 17 is 1.0 in float32)
        elif name in ("bigram", "side.embed"):
            new = normal(tensor.shape, 0.0, 0.5)
        else:
            continue
        tensors[name] = new.to(tensor.dtype)
    write_safetensors(path, tensors)
    return folder
