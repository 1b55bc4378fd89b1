"""Configuration of the Depunex decoder: layers that each have one norm, a mixer and a feed-forward side by side.

config.json names the design under `architecture` and lists the layers; each entry gives `type` (the mixer: `mamba2`, a
matrix state per head with one decay per head and token, or `parallel`, attention inside chunks of positions beside a
selective scan), the mixer's sizes under `mixer`, and `mlp`: a dense feed-forward (`kind` "dense": `ff`, `limit`), a
mixture of experts (`kind` "moe": `expert.ff`, `router.experts|top|groups.count|groups.keep`), or null. Beside the layers:
`vocab`, `width`, `norm.eps`, `embedding.scale` and, each optional, `embedding.bigram` (`buckets`, `mul_prev`, `mul_cur`),
`token_side.dim`, `logit_softcap`. What is absent does not exist in the model.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Optional, Tuple

from . import ConfigError, _positive_int, _require
from .sozopel import _number, _sizes

MIXER_TYPES = ("mamba2", "parallel")
MLP_KINDS = ("dense", "moe")


def _check_rotation(rot, where: str) -> None:
    if rot is None:
        return
    if not isinstance(rot, dict):
        raise ConfigError(f"config.json: {where}: 'rot' must be an object")
    _sizes(rot, ("dims",), where)
    if rot["dims"] % 2 != 0:
        raise ConfigError(f"config.json: {where}: a rotation turns pairs of dims, found {rot['dims']}")
    if _number(rot, "base", where) <= 0:
        raise ConfigError(f"config.json: {where}: 'base' must be positive")
    scaling = rot.get("scaling")
    if scaling is not None:
        if not isinstance(scaling, dict):
            raise ConfigError(f"config.json: {where}: 'scaling' must be an object")
        for key in ("factor", "low", "high", "original"):
            if _number(scaling, key, where + ".scaling") <= 0:
                raise ConfigError(f"config.json: {where}.scaling: '{key}' must be positive")
        if scaling["high"] == scaling["low"]:
            raise ConfigError(f"config.json: {where}.scaling: 'low' and 'high' must differ")


def _check_mixer(kind: str, mixer: dict, where: str) -> None:
    if kind == "mamba2":
        _sizes(mixer, ("heads", "vdim", "state", "groups", "norm_groups", "conv"), where)
        if mixer["heads"] % mixer["groups"] != 0:
            raise ConfigError(f"config.json: {where}: {mixer['heads']} heads cannot share {mixer['groups']} groups")
        if (mixer["heads"] * mixer["vdim"]) % mixer["norm_groups"] != 0:
            raise ConfigError(f"config.json: {where}: {mixer['norm_groups']} norm groups do not divide {mixer['heads'] * mixer['vdim']}")
        return
    left, right = mixer.get("left"), mixer.get("right")
    if not isinstance(left, dict) or not isinstance(right, dict):
        raise ConfigError(f"config.json: {where}: a parallel mixer has 'left' and 'right'")
    _sizes(left, ("heads", "kv_heads", "dim", "vdim"), where + ".left")
    if left["heads"] % left["kv_heads"] != 0:
        raise ConfigError(f"config.json: {where}.left: {left['heads']} heads cannot share {left['kv_heads']} key/value heads")
    _number(left, "scale", where + ".left")
    mask = left.get("mask")
    if mask is not None:
        if not isinstance(mask, dict):
            raise ConfigError(f"config.json: {where}.left: 'mask' must give the chunks' size")
        _sizes(mask, ("size",), where + ".left.mask")
    _check_rotation(left.get("rot"), where + ".left.rot")
    if left.get("rot") is not None and left["rot"]["dims"] > left["dim"]:
        raise ConfigError(f"config.json: {where}.left.rot: {left['rot']['dims']} rotated dims in a head of {left['dim']}")
    _sizes(right, ("inner", "state", "dt_rank", "conv"), where + ".right")
    _number(mixer, "left_scale", where)
    _number(mixer, "right_scale", where)


def _check_mlp(mlp: dict, where: str) -> None:
    if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
        raise ConfigError(f"config.json: {where}: 'kind' must be one of {MLP_KINDS}")
    if mlp["kind"] == "dense":
        _sizes(mlp, ("ff",), where)
        if _number(mlp, "limit", where) <= 0:
            raise ConfigError(f"config.json: {where}: 'limit' must be positive")
        return
    expert, router = mlp.get("expert"), mlp.get("router")
    if not isinstance(expert, dict) or not isinstance(router, dict):
        raise ConfigError(f"config.json: {where}: a mixture of experts has 'expert' and 'router'")
    _sizes(expert, ("ff",), where + ".expert")
    _sizes(router, ("experts", "top"), where + ".router")
    groups = router.get("groups")
    if groups is not None:
        if not isinstance(groups, dict):
            raise ConfigError(f"config.json: {where}.router: 'groups' must be an object")
        _sizes(groups, ("count", "keep"), where + ".router.groups")
        if router["experts"] % groups["count"] != 0 or groups["keep"] > groups["count"]:
            raise ConfigError(f"config.json: {where}.router: {router['experts']} experts in {groups['count']} groups, "
                              f"{groups['keep']} kept")
    open_experts = router["experts"] if groups is None else groups["keep"] * (router["experts"] // groups["count"])
    if router["top"] > open_experts:
        raise ConfigError(f"config.json: {where}.router: {router['top']} experts chosen of {open_experts} that can be")


@dataclass(frozen=True)
class DepunexConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    bigram: Optional[Tuple[int, int, int]]      # (buckets, mul_prev, mul_cur), or None
    token_side_dim: Optional[int]
    logit_softcap: Optional[float]
    layers: Tuple[dict, ...]                    # as config.json lists them: {"type", "mixer", "mlp"}
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None

    # what the rest of the library asks of any configuration
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def max_position_embeddings(self):
        return None                             # nothing in the design ends at a position

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, raw: dict) -> "DepunexConfig":
        layers = _require(raw, "layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        kept = []
        for index, layer in enumerate(layers):
            where = f"layers[{index}]"
            if not isinstance(layer, dict) or layer.get("type") not in MIXER_TYPES:
                raise ConfigError(f"config.json: {where}: 'type' must be one of {MIXER_TYPES}")
            if not isinstance(layer.get("mixer"), dict):
                raise ConfigError(f"config.json: {where}: 'mixer' must give the mixer's sizes")
            _check_mixer(layer["type"], layer["mixer"], where + ".mixer")
            mlp = layer.get("mlp")
            if mlp is not None:
                _check_mlp(mlp, where + ".mlp")
            kept.append(copy.deepcopy({"type": layer["type"], "mixer": layer["mixer"], "mlp": mlp}))
        norm = _require(raw, "norm")
        if not isinstance(norm, dict):
            raise ConfigError("config.json: 'norm' must be an object")
        embedding = raw.get("embedding") or {}
        if not isinstance(embedding, dict):
            raise ConfigError("config.json: 'embedding' must be an object")
        bigram = embedding.get("bigram")
        if bigram is not None:
            if not isinstance(bigram, dict):
                raise ConfigError("config.json: 'embedding.bigram' must be an object")
            _sizes(bigram, ("buckets",), "embedding.bigram")
            for key in ("mul_prev", "mul_cur"):
                if isinstance(bigram.get(key), bool) or not isinstance(bigram.get(key), int) or not 0 <= bigram[key] < 2 ** 31:
                    raise ConfigError(f"config.json: embedding.bigram: '{key}' must be an integer from 0 up, found {bigram.get(key)!r}")
            bigram = (int(bigram["buckets"]), int(bigram["mul_prev"]), int(bigram["mul_cur"]))
        side = raw.get("token_side")
        if side is not None:
            if not isinstance(side, dict):
                raise ConfigError("config.json: 'token_side' must be an object")
            _sizes(side, ("dim",), "token_side")
        cap = raw.get("logit_softcap")
        if cap is not None and (isinstance(cap, bool) or not isinstance(cap, (int, float)) or cap <= 0):
            raise ConfigError(f"config.json: 'logit_softcap' must be a positive number, found {cap!r}")
        eos = raw.get("eos_token_id")
        eos = () if eos is None else tuple(eos) if isinstance(eos, list) else (eos,)
        return cls(architecture=str(raw.get("architecture") or raw["architectures"][0]), vocab=_positive_int(raw, "vocab"),
                   width=_positive_int(raw, "width"), norm_eps=_number(norm, "eps", "norm"),
                   embedding_scale=_number(embedding, "scale", "embedding") if "scale" in embedding else 1.0, bigram=bigram,
                   token_side_dim=None if side is None else int(side["dim"]), logit_softcap=None if cap is None else float(cap),
                   layers=tuple(kept), eos_token_ids=tuple(int(e) for e in eos), bos_token_id=raw.get("bos_token_id"))

    def to_dict(self) -> dict:
        embedding = {"scale": self.embedding_scale}
        if self.bigram is not None:
            embedding["bigram"] = {"buckets": self.bigram[0], "mul_prev": self.bigram[1], "mul_cur": self.bigram[2]}
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "embedding": embedding, "layers": copy.deepcopy(list(self.layers))}
        if self.token_side_dim is not None:
            out["token_side"] = {"dim": self.token_side_dim}
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        return out

    def __hash__(self):
        return hash((self.architecture, self.vocab, self.width, len(self.layers)))
