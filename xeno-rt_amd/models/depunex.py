"""Depunex: a decoder whose layers have one norm that a mixer and a feed-forward both read, described in parts.

Embedding times a constant, plus a row of a second table hashed from the token and the one before it; then the layers that
config.json lists. A layer is x += ls1 * mixer(norm1(x)) + ls2 * feed_forward(norm1(x)) with an RMS norm whose tensor holds
the gain minus one, and two vectors ls1, ls2; after it the token adds a gated projection of its stretch of a side table's
row, RMS-normed. The mixers:
  mamba2    a matrix state per head that decays by one number per head and token (parts/recurrent.py: StateSpaceDuality)
  parallel  left_scale * attention + right_scale * selective scan: grouped softmax attention with rotary positions on the
            first dims of every head (pairs of halves, frequencies stretched by wavelength) inside chunks of positions,
            beside a state vector per channel with step sizes from a low-rank projection (SelectiveStateSpace)
The feed-forward is a gated one with clamps (`dense`), a mixture of experts chosen by sigmoid scores within the best
groups (`moe`), or absent. Final norm, then the embedding table as the output head, and a tanh cap on the logits.
Tensor names: `embed`, `bigram`, `side.embed`, `l<i>.norm1|ls1|ls2`, `l<i>.mix.*`, `l<i>.mlp.*`, `l<i>.side.gate|proj|norm`,
`final.norm`.
"""
from __future__ import annotations

from ..config import register_architecture
from ..config.depunex import DepunexConfig
from ..parts import (Attention, ClampedGLU, ExpertsMLP, HashedPairEmbedding, OffsetRMSNorm, OutputHead, PairRotation, ParallelBlock,
                     SelectiveStateSpace, StateSpaceDuality, TokenSideInput, TokenSideTable, WeightedPair)
from .decoder import ModelSpec

GLU_ALPHA = 1.702       # the dense feed-forward's gate is g * sigmoid(GLU_ALPHA * g)


def _mixer(kind: str, m: dict, p: str, c: DepunexConfig):
    if kind == "mamba2":
        return StateSpaceDuality(p, c.width, m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"], m["conv"], c.norm_eps,
                                 state_name="mix.state")
    left, right = m["left"], m["right"]
    rot = left.get("rot")
    position = None if rot is None else PairRotation(rot["dims"], rot["base"], neighbours=False, scaling=rot.get("scaling"))
    mask = left.get("mask")
    attention = Attention(p + "left.", c.width, left["heads"], left["kv_heads"], left["dim"], position=position, scale=left["scale"],
                          value_dim=left["vdim"], chunk=None if mask is None else mask["size"], completed=True,
                          names={"q": "q", "k": "k", "v": "v", "o": "o"})
    scan = SelectiveStateSpace(p + "right.", c.width, right["inner"], right["state"], right["dt_rank"], right["conv"],
                               state_name="mix.right.state")
    return WeightedPair(attention, scan, m["left_scale"], m["right_scale"])


def _feed_forward(mlp, p: str, c: DepunexConfig):
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return ClampedGLU(p, c.width, mlp["ff"], mlp["limit"], GLU_ALPHA)
    router = mlp["router"]
    groups = router.get("groups")
    return ExpertsMLP(p, c.width, mlp["expert"]["ff"], router["experts"], router["top"],
                      groups=None if groups is None else groups["count"], keep=None if groups is None else groups["keep"])


def build_depunex(config: DepunexConfig) -> ModelSpec:
    c = config
    bigram = c.bigram
    embedding = HashedPairEmbedding("", c.vocab, c.width, scale=c.embedding_scale, name="embed",
                                    pair_name=None if bigram is None else "bigram",
                                    **({} if bigram is None else dict(buckets=bigram[0], mul_prev=bigram[1], mul_cur=bigram[2])))
    side = None if c.token_side_dim is None else TokenSideTable("side.embed", c.vocab, len(c.layers), c.token_side_dim)
    layers = []
    for index, layer in enumerate(c.layers):
        p = f"l{index}."
        feed_forward = _feed_forward(layer["mlp"], p + "mlp.", c)
        layers.append(ParallelBlock(
            OffsetRMSNorm(p + "norm1", c.width, c.norm_eps), _mixer(layer["type"], layer["mixer"], p + "mix.", c), feed_forward,
            hidden=c.width, mixer_scale=p + "ls1", feed_forward_scale=p + "ls2",
            after=None if side is None else TokenSideInput(p + "side.", c.width, side, index, c.norm_eps)))
    return ModelSpec(config=c, embedding=embedding, layers=layers, final_norm=OffsetRMSNorm("final.norm", c.width, c.norm_eps),
                     head=OutputHead("", c.vocab, c.width, tied_to=embedding, softcap=c.logit_softcap))


register_architecture("Depunex", DepunexConfig, build_depunex)
