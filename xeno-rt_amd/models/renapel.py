"""Renapel: a decoder on a residual stream in several copies, described in parts.

(A configuration without `streams` has one plain residual stream, x += mixer(norm1(x)), x += feed_forward(norm2(x)), and
no tensors `hc1.*`, `hc2.*`.) The embedding's rows start every copy of the stream; then the layers that config.json lists, each a block that reads a
weighted sum of the copies before each of its sublayers and writes all copies at once after it
(parts/block.py: HyperConnectionBlock); in the end the copies are added up, normed, and multiplied by the head. The mixers:
  lightning         a matrix state per head with a fixed decay, q, k and v through silu, the heads' outputs normed together
                    and gated by a sigmoid (parts/recurrent.py: LightningAttention)
  attention         grouped softmax attention without rotation: biases on q, k and v, every head of q and k divided by its
                    root mean square, a query temperature that grows with the position, a learnt bias by bucket of
                    distance, a learnt sink per head; a layer with `kv_from` has no keys and values of its own and reads
                    the cache entry of the layer it names (parts/attention.py: Attention)
  latent_attention  attention whose keys and values are made from a cached latent, part of every query and one shared key
                    part turned by rotary positions in pairs of neighbours, a learnt sink per head (parts/latent.py)
The feed-forward is a mixture of clamped experts chosen by softmax scores within the best groups, or absent.
Tensor names: `embed`, `l<i>.norm1|norm2`, `l<i>.hc1.in|out|mix`, `l<i>.hc2.*`, `l<i>.mix.*`, `l<i>.mlp.*`, `final.norm`, `head`.
"""
from __future__ import annotations

from ..config import register_architecture
from ..config.renapel import RenapelConfig
from ..parts import (Attention, DistanceBuckets, Embedding, ExpertsMLP, HyperConnectionBlock, LatentAttention, LightningAttention,
                     OutputHead, PreNormBlock, ResidualStreams, RMSNorm)
from .decoder import LayerCall, ModelSpec

SWISH_ALPHA = 1.702     # an expert's gate is g * sigmoid(SWISH_ALPHA * g)
GROUP_TOP = 1           # a group of experts scores as its best expert


def _mixer(kind: str, m: dict, p: str, c: RenapelConfig):
    if kind == "lightning":
        return LightningAttention(p, c.width, m["heads"], m["dim"], m["vdim"], m["decay"], c.norm_eps, state_name="mix.state")
    if kind == "latent_attention":
        return LatentAttention(p, c.width, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"], m["scale"], c.norm_eps,
                               m["rot"]["dims"], m["rot"]["base"])
    if "bias_rows" not in m:
        raise ValueError("the rows of an attention layer's table of biases are read from the checkpoint, or named as 'bias_rows'")
    temp = m.get("q_temp")
    return Attention(p, c.width, m["heads"], m["kv_heads"], m["dim"], position=DistanceBuckets(p + "rel", m["heads"], m["bias_rows"], m["bias_max"]),
                     qk_norm="plain", qk_norm_eps=c.norm_eps, scale=m["scale"], value_dim=m["vdim"], sink="sink", biases="qkv",
                     query_temperature=None if temp is None else (temp["coef"], temp["every"]),
                     keys_from_another="kv_from" in m,
                     names={"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b"})


def _feed_forward(mlp, p: str, c: RenapelConfig):
    if mlp is None:
        return None
    router = mlp["router"]
    groups = router.get("groups")
    return ExpertsMLP(p, c.width, mlp["expert"]["ff"], router["experts"], router["top"],
                      groups=None if groups is None else groups["count"], keep=None if groups is None else groups["keep"],
                      scores="softmax", group_top=GROUP_TOP, scale=router.get("scale", 1.0), clamp=(mlp["expert"]["limit"], SWISH_ALPHA))


def build_renapel(config: RenapelConfig) -> ModelSpec:
    c = config
    layers, schedule = [], []
    for index, layer in enumerate(c.layers):
        p = f"l{index}."
        feed_forward = _feed_forward(layer["mlp"], p + "mlp.", c)
        norm1, mixer = RMSNorm(p, c.width, c.norm_eps, name=p + "norm1"), _mixer(layer["type"], layer["mixer"], p + "mix.", c)
        norm2 = None if feed_forward is None else RMSNorm(p, c.width, c.norm_eps, name=p + "norm2")
        if c.streams is None:
            layers.append(PreNormBlock(norm1, mixer, norm2, feed_forward, unread=[] if feed_forward is not None else [p + "norm2"]))
        else:
            layers.append(HyperConnectionBlock(c.streams, c.width, norm1, mixer, p + "hc1.", norm2, feed_forward, p + "hc2.",
                                               unread=[p + "norm2"]))
        schedule.append(LayerCall(index, reads_cache_of=layer["mixer"].get("kv_from") if layer["type"] == "attention" else None))
    return ModelSpec(config=c, embedding=Embedding("", c.vocab, c.width, name="embed"), layers=layers, schedule=schedule,
                     final_norm=RMSNorm("", c.width, c.norm_eps, name="final.norm"), head=OutputHead("", c.vocab, c.width, name="head"),
                     streams=None if c.streams is None else ResidualStreams(c.streams, c.width))


register_architecture("Renapel", RenapelConfig, build_renapel)
