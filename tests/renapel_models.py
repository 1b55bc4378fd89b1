"""Small Renapel configurations for the tests, and model folders with random weights for them.

The configurations differ from each other in every size and option: two, four, one and no copies of the residual stream;
heads that share key/value heads and heads that do not, one head, values wider and narrower than keys, key sizes that are no
multiples of eight; a query temperature that grows every few positions, every position, or is absent; tables of biases of
few and many rows whose number config.json names or leaves to the checkpoint; layers that read another layer's keys and
values right after it and several layers later; latents narrower and wider than a head, turned parts rotated whole and in
part; decays from one half to one; experts with and without groups, with one, some and all of them chosen, with and without
a scale; layers without a feed-forward; every order of the three mixers.
"""
import json
import os

import torch


def _moe(ff, limit, experts, top, groups=None, scale=None):
    router = {"experts": experts, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    if scale is not None:
        router["scale"] = scale
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": router}


MIXED = {
    "architecture": "Renapel", "vocab": 101, "width": 48, "norm": {"eps": 1e-5}, "streams": 2,
    "layers": [
        {"type": "lightning", "mixer": {"heads": 3, "dim": 20, "vdim": 12, "decay": [0.5, 0.9, 1.0]},
         "mlp": _moe(24, 1.5, 8, 2, groups=(4, 2), scale=1.7)},
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 16, "scale": 0.3, "bias_max": 40, "bias_rows": 12,
                                        "q_temp": {"coef": 0.4, "every": 16}}, "mlp": None},
        {"type": "latent_attention", "mixer": {"heads": 3, "dim": 16, "rot_dim": 8, "vdim": 12, "kv_rank": 24, "q_rank": 20, "scale": 0.2,
                                               "rot": {"dims": 8, "base": 1000.0}}, "mlp": _moe(16, 0.8, 6, 3)},
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 16, "scale": 0.25, "bias_max": 70, "bias_rows": 8,
                                        "kv_from": 1}, "mlp": _moe(20, 2.0, 4, 1, groups=(2, 1))},
    ],
}
WIDE = {
    "architecture": "Renapel", "vocab": 130, "width": 64, "norm": {"eps": 1e-6}, "streams": 4,
    "layers": [
        {"type": "latent_attention", "mixer": {"heads": 1, "dim": 40, "rot_dim": 16, "vdim": 72, "kv_rank": 80, "q_rank": 12, "scale": 0.15,
                                               "rot": {"dims": 8, "base": 10000.0}}, "mlp": _moe(32, 3.0, 12, 4, groups=(3, 3), scale=0.5)},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 32, "vdim": 48, "scale": 0.2, "bias_max": 200, "bias_rows": 32},
         "mlp": _moe(8, 1.0, 5, 5)},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 32, "vdim": 48, "scale": 0.1, "bias_max": 9, "bias_rows": 4,
                                        "q_temp": {"coef": 1.0, "every": 1}, "kv_from": 1}, "mlp": None},
        {"type": "lightning", "mixer": {"heads": 2, "dim": 64, "vdim": 40, "decay": [0.97, 0.75]}, "mlp": _moe(24, 0.5, 9, 2, groups=(3, 2))},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 32, "vdim": 48, "scale": 0.3, "bias_max": 64, "bias_rows": 16,
                                        "kv_from": 1}, "mlp": None},
    ],
}
EDGES = {
    "architecture": "Renapel", "vocab": 64, "width": 32, "norm": {"eps": 1e-3}, "streams": 1,
    "layers": [
        {"type": "attention", "mixer": {"heads": 6, "kv_heads": 1, "dim": 10, "vdim": 6, "scale": 0.5, "bias_max": 1000, "bias_rows": 6,
                                        "q_temp": {"coef": 0.1, "every": 70}}, "mlp": _moe(12, 0.25, 2, 1)},
        {"type": "lightning", "mixer": {"heads": 1, "dim": 72, "vdim": 136, "decay": [0.99]}, "mlp": None},
        {"type": "latent_attention", "mixer": {"heads": 5, "dim": 8, "rot_dim": 6, "vdim": 4, "kv_rank": 40, "q_rank": 48, "scale": 0.3,
                                               "rot": {"dims": 2, "base": 10.0}}, "mlp": _moe(8, 4.0, 16, 3, groups=(8, 2), scale=2.5)},
        {"type": "lightning", "mixer": {"heads": 4, "dim": 8, "vdim": 8, "decay": [0.6, 0.8, 0.9, 0.999]}, "mlp": _moe(16, 1.0, 3, 2)},
    ],
}
PLAIN = {          # no copies: one plain residual stream
    "architecture": "Renapel", "vocab": 80, "width": 40, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "latent_attention", "mixer": {"heads": 2, "dim": 12, "rot_dim": 4, "vdim": 20, "kv_rank": 16, "q_rank": 16, "scale": 0.25,
                                               "rot": {"dims": 4, "base": 100.0}}, "mlp": _moe(16, 1.0, 4, 2)},
        {"type": "lightning", "mixer": {"heads": 2, "dim": 16, "vdim": 20, "decay": [0.9, 0.95]}, "mlp": None},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 0.25, "bias_max": 30, "bias_rows": 10},
         "mlp": _moe(16, 2.0, 4, 2, groups=(2, 1))},
    ],
}
CONFIGS = {"mixed": MIXED, "wide": WIDE, "edges": EDGES, "plain": PLAIN}


def make_renapel_folder(raw_config, folder, seed, std=0.2, router_std=0.7, name_the_rows=True):
    """A model folder for `raw_config` with the library's random weights, where the small tensors are then given values that
    make them matter: gains away from one, biases, sinks and tables of biases away from zero, the copies' weights near a
    plain residual stream's but not on it, a router whose scores differ. name_the_rows False: config.json is written without
    the rows of the tables of biases, as a checkpoint's may be."""
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
        if last in ("norm1", "norm2", "norm") or name == "final.norm":
            new = normal(tensor.shape, 1.0, 0.3)
        elif last == "b" or last == "rel":
            new = normal(tensor.shape, 0.0, 0.5)
        elif last == "sink":
            new = normal(tensor.shape, 0.5, 1.0)
        elif last == "router":
            new = normal(tensor.shape, 0.0, router_std)
        elif ".hc" in name and last == "mix":
            new = torch.eye(tensor.shape[0]) + normal(tensor.shape, 0.0, 0.2)
        elif ".hc" in name and last == "in":
            new = normal(tensor.shape, 1.0 / tensor.shape[0], 0.2)
        elif ".hc" in name and last == "out":
            new = normal(tensor.shape, 1.0, 0.3)
        else:
            continue
        tensors[name] = new.to(tensor.dtype)
    write_safetensors(path, tensors)
    if not name_the_rows:
        with open(os.path.join(folder, "config.json")) as handle:
            written = json.load(handle)
        for layer in written["layers"]:
            layer["mixer"].pop("bias_rows", None)
        with open(os.path.join(folder, "config.json"), "w") as handle:
            json.dump(written, handle)
    return folder
