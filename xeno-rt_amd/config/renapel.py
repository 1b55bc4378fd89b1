"""Configuration of the Renapel decoder: a residual stream in several copies, and layers of three kinds of mixer before
a mixture of experts.

config.json names the design under `architecture` and lists the layers; each entry gives `type` (the mixer: `lightning`,
a matrix state per head with a fixed decay; `attention`, grouped softmax attention with a bias by distance and a learnt
sink, whose keys and values may be another layer's (`kv_from`); `latent_attention`, attention whose keys and values are
made from a cached latent), the mixer's sizes under `mixer`, and `mlp`: a mixture of experts (`kind` "moe": `expert.ff`,
`expert.limit`, `router.experts|top|scale|groups.count|groups.keep`) or null. Beside the layers: `vocab`, `width`,
`norm.eps`, `streams` (the copies of the residual stream; absent: one plain residual stream without the copies' weights).
The rows of an attention layer's table of biases are the table's first dimension; config.json may name them (`bias_rows`)
or leave them to the checkpoint.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Dict, Optional, Tuple

from . import ConfigError, _positive_int, _require
from .sozopel import _number, _sizes

MIXER_TYPES = ("lightning", "attention", "latent_attention")


def _check_mixer(kind: str, mixer: dict, where: str, index: int, layers: list) -> None:
    if kind == "lightning":
        _sizes(mixer, ("heads", "dim", "vdim"), where)
        decay = mixer.get("decay")
        if (not isinstance(decay, list) or len(decay) != mixer["heads"]
                or not all(isinstance(d, (int, float)) and not isinstance(d, bool) for d in decay)):
            raise ConfigError(f"config.json: {where}: 'decay' must list one number per head")
        return
    if kind == "attention":
        _sizes(mixer, ("heads", "kv_heads", "dim", "vdim"), where)
        if mixer["heads"] % mixer["kv_heads"] != 0:
            raise ConfigError(f"config.json: {where}: {mixer['heads']} heads cannot share {mixer['kv_heads']} key/value heads")
        _number(mixer, "scale", where)
        if "bias_rows" in mixer:
            _sizes(mixer, ("bias_rows",), where)
        if _number(mixer, "bias_max", where) <= 0:
            raise ConfigError(f"config.json: {where}: 'bias_max' must be positive")
        temp = mixer.get("q_temp")
        if temp is not None:
            if not isinstance(temp, dict):
                raise ConfigError(f"config.json: {where}: 'q_temp' must be an object")
            _number(temp, "coef", where + ".q_temp")
            _sizes(temp, ("every",), where + ".q_temp")
        source = mixer.get("kv_from")
        if source is not None:
            if isinstance(source, bool) or not isinstance(source, int) or not 0 <= source < index:
                raise ConfigError(f"config.json: {where}: 'kv_from' must name an earlier layer, found {source!r}")
            other = layers[source]
            theirs = other.get("mixer") if isinstance(other, dict) else None
            if other.get("type") != "attention" or not isinstance(theirs, dict) or "kv_from" in theirs:
                raise ConfigError(f"config.json: {where}: layer {source} has no keys and values of its own to share")
            if any(theirs.get(key) != mixer[key] for key in ("kv_heads", "dim", "vdim")):
                raise ConfigError(f"config.json: {where}: layer {source} keeps keys and values of other sizes")
        return
    _sizes(mixer, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"), where)
    _number(mixer, "scale", where)
    rot = mixer.get("rot")
    if not isinstance(rot, dict):
        raise ConfigError(f"config.json: {where}: 'rot' must be an object")
    _sizes(rot, ("dims",), where + ".rot")
    if rot["dims"] % 2 != 0 or rot["dims"] > mixer["rot_dim"]:
        raise ConfigError(f"config.json: {where}.rot: {rot['dims']} dims turn in pairs inside a part of {mixer['rot_dim']}")
    if _number(rot, "base", where + ".rot") <= 0:
        raise ConfigError(f"config.json: {where}.rot: 'base' must be positive")


def _check_mlp(mlp: dict, where: str) -> None:
    if not isinstance(mlp, dict) or mlp.get("kind") != "moe":
        raise ConfigError(f"config.json: {where}: 'kind' must be 'moe'")
    expert, router = mlp.get("expert"), mlp.get("router")
    if not isinstance(expert, dict) or not isinstance(router, dict):
        raise ConfigError(f"config.json: {where}: a mixture of experts has 'expert' and 'router'")
    _sizes(expert, ("ff",), where + ".expert")
    if _number(expert, "limit", where + ".expert") <= 0:
        raise ConfigError(f"config.json: {where}.expert: 'limit' must be positive")
    _sizes(router, ("experts", "top"), where + ".router")
    if "scale" in router:
        _number(router, "scale", where + ".router")
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
class RenapelConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    streams: Optional[int]                      # None: a plain residual stream
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
    def from_dict(cls, raw: dict) -> "RenapelConfig":
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
            _check_mixer(layer["type"], layer["mixer"], where + ".mixer", index, layers)
            mlp = layer.get("mlp")
            if mlp is not None:
                _check_mlp(mlp, where + ".mlp")
            kept.append(copy.deepcopy({"type": layer["type"], "mixer": layer["mixer"], "mlp": mlp}))
        norm = _require(raw, "norm")
        if not isinstance(norm, dict):
            raise ConfigError("config.json: 'norm' must be an object")
        eos = raw.get("eos_token_id")
        eos = () if eos is None else tuple(eos) if isinstance(eos, list) else (eos,)
        return cls(architecture=str(raw.get("architecture") or raw["architectures"][0]), vocab=_positive_int(raw, "vocab"),
                   width=_positive_int(raw, "width"), norm_eps=_number(norm, "eps", "norm"),
                   streams=_positive_int(raw, "streams") if raw.get("streams") is not None else None, layers=tuple(kept),
                   eos_token_ids=tuple(int(e) for e in eos), bos_token_id=raw.get("bos_token_id"))

    def to_dict(self) -> dict:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "layers": copy.deepcopy(list(self.layers))}
        if self.streams is not None:
            out["streams"] = self.streams
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        return out

    @staticmethod
    def bias_table(index: int) -> str:
        """The tensor whose first dimension is the number of distance buckets of layer `index`."""
        return f"l{index}.mix.rel"

    def completed_from(self, shapes: Dict[str, tuple]) -> "RenapelConfig":
        """The same configuration with every 'bias_rows' that config.json left out read from the tensors' shapes."""
        layers = copy.deepcopy(list(self.layers))
        for index, layer in enumerate(layers):
            if layer["type"] != "attention" or "bias_rows" in layer["mixer"]:
                continue
            name = self.bias_table(index)
            if name not in shapes or len(shapes[name]) != 2:
                raise ConfigError(f"the checkpoint has no table '{name}' to read the number of distance buckets from")
            layer["mixer"]["bias_rows"] = int(shapes[name][0])
        return RenapelConfig(self.architecture, self.vocab, self.width, self.norm_eps, self.streams, tuple(layers),
                             self.eos_token_ids, self.bos_token_id)

    def __hash__(self):
        return hash((self.architecture, self.vocab, self.width, self.streams, len(self.layers)))
