"""Causal attention whose keys and values are made from a latent that is all the cache keeps.

With h the mixer's input, H heads, per head d plain and r turned query/key dims and e value dims, a latent of `kv_rank`:
  queries   c_q = RMSnorm(W_dq h) (gain `dq.norm`), q = W_uq c_q, head by head [d plain | r to turn]
  latent    W_dkv h = [kv_rank | r]: c = RMSnorm of the first kv_rank (gain `dkv.norm`); the last r are one key part for all
            heads, turned like the queries' parts and not normed
  per head  plain key W_uk,h c, value W_uv,h c; score = (q_plain . k_plain + q_turned . k_turned) * scale
  rotation  the first `rot_dims` of a part of r turn in pairs of neighbours (2i, 2i + 1) by position * base^(-2i / rot_dims)
  softmax   over the keys at or before the query, with one more term exp(sink_h) in the denominator (a learnt number per head)
  output    W_o on the heads' outputs side by side

What is cached per token is one row [c | turned key part] as the key of a single key/value head, and c as its value. The
per-head keys never exist: q_plain . (W_uk,h c) = (W_uk,h^T q_plain) . c, so the plain part of a query is multiplied by its
head's key matrix, transposed, and the score is an ordinary one against the cached row; the softmax's weights sum the
latents, and the head's value matrix turns that sum into the head's output. Both are products with a matrix per head
(`ops.linear_heads`); the attention itself is `ops.attention` with H query heads on one key/value head, which in bfloat16
takes the matrix-core kernel for such a cache (sixteen heads of a token as the columns of a score tile) where the key and
value sizes are whole tiles of 32, and the general kernel otherwise.
Norms, angles, scores and the softmax are float32; the products run in the compute dtype with float32 sums.

A bfloat16 step whose sequences all start (prompts of some length) does not go through the attention kernel: the step has the
prompts' cached rows at hand, so the scores of a stretch of queries, all heads at once, are one matrix product with those
rows (float32 sums), a kernel turns them into the softmax's weights (as two bfloat16 numbers each, the rounded weight and what
the rounding left), and two products with the latents, tokens along the rows, sum them up: the library's matrix-core products
instead of a kernel that takes a key a lane. A query's weights behind its own position are zeros that the products still
multiply: twice the arithmetic of a causal kernel, and still a twentieth of the time.
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import CacheNeeds, KVSpec, Mixer, Runtime, WeightSpec, register_part
from .position import PairRotation


class LatentAttention(Mixer):
    capturable = True

    def __init__(self, prefix: str, hidden: int, n_heads: int, dim: int, rot_dim: int, value_dim: int, kv_rank: int, q_rank: int,
                 scale: float, eps: float, rot_dims: int, rot_base: float, sink: str = "sink"):
        if min(n_heads, dim, value_dim, kv_rank, q_rank) <= 0 or rot_dim < 0:
            raise ValueError("latent attention: sizes must be positive")
        if rot_dims < 0 or rot_dims % 2 != 0 or rot_dims > rot_dim:
            raise ValueError(f"latent attention: {rot_dims} dims turn in pairs inside a part of {rot_dim}")
        self.prefix, self.hidden, self.n_heads, self.dim, self.rot_dim = prefix, hidden, int(n_heads), int(dim), int(rot_dim)
        self.value_dim, self.kv_rank, self.q_rank = int(value_dim), int(kv_rank), int(q_rank)
        self.scale, self.eps, self.sink_name = float(scale), float(eps), sink
        self.position = PairRotation(rot_dims, rot_base, neighbours=True) if rot_dims > 0 else None
        self.rot_dims = int(rot_dims)

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, w, heads = self.prefix, self.hidden, self.n_heads
        return {p + "dq": WeightSpec((self.q_rank, w)), p + "dq.norm": WeightSpec((self.q_rank,), init="ones", kind="vector"),
                p + "uq": WeightSpec((heads * (self.dim + self.rot_dim), self.q_rank)),
                p + "dkv": WeightSpec((self.kv_rank + self.rot_dim, w)), p + "dkv.norm": WeightSpec((self.kv_rank,), init="ones", kind="vector"),
                p + "uk": WeightSpec((heads * self.dim, self.kv_rank)), p + "uv": WeightSpec((heads * self.value_dim, self.kv_rank)),
                p + self.sink_name: WeightSpec((heads,), init="zeros", kind="vector"), p + "o": WeightSpec((w, heads * self.value_dim))}

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds(kv=KVSpec(1, self.kv_rank + self.rot_dim, None, self.kv_rank))

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        p, heads = self.prefix, self.n_heads
        if self.position is not None:
            self.position.bind(tensors, runtime)
        self.w_dq, self.w_dkv = runtime.weight(tensors[p + "dq"]), runtime.weight(tensors[p + "dkv"])
        self.w_uq, self.w_o = runtime.weight(tensors[p + "uq"]), runtime.weight(tensors[p + "o"])
        self.q_gain, self.kv_gain = runtime.vector(tensors[p + "dq.norm"]), runtime.vector(tensors[p + "dkv.norm"])
        # a matrix per head: the key matrices transposed (a transposition moves numbers and rounds none), the value matrices as they are
        self.w_uk_t = runtime.matrix(tensors[p + "uk"]).view(heads, self.dim, self.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = runtime.matrix(tensors[p + "uv"]).view(heads, self.value_dim, self.kv_rank)
        self.sink = tensors[p + self.sink_name].to(device=runtime.device, dtype=torch.float32).contiguous()

    DENSE_FROM = 64                     # prompts from this many tokens on have their scores as a matrix product
    DENSE_SCORES = 32 * 1024 * 1024     # most scores of a stretch of queries (float32: 128 MiB, and as much again for the weights)

    def _prompts_alone(self, h, batch, cache) -> bool:
        """Whether the step is one of prompts that start their sequences, long enough for the products of `_attend_prompts`."""
        counts, starts = getattr(batch, "host_counts", None), getattr(batch, "host_starts", None)
        if h.dtype != torch.bfloat16 or not cache.writable or not counts or starts is None or not hasattr(self.runtime.ops, "causal_softmax"):
            return False
        if sum(counts) != h.shape[0] or any(slot < 0 for slot in batch.host_slots):
            return False
        return all(start == 0 for start in starts) and min(counts) >= self.DENSE_FROM

    def _attend_prompts(self, full, rows, batch, summed) -> None:
        """summed[t, h] = the latents under the softmax's weights of query (t, h), for prompts that start their sequences:
        full [tokens, heads * (rank + rot)] the queries, rows [tokens, rank + rot] the cached rows of the same tokens."""
        rt = self.runtime
        ops = rt.ops
        heads, rank, width = self.n_heads, self.kv_rank, self.kv_rank + self.rot_dim
        stretch_of = lambda count: max(1, min(count, self.DENSE_SCORES // (heads * count)))
        # one set of buffers for all stretches of all prompts of the step, as large as the largest stretch needs
        most = max(stretch_of(count) * heads * count for count in batch.host_counts)
        most_sums = max(stretch_of(count) for count in batch.host_counts) * heads * rank
        scores_all, sums_all = rt.empty((most,), torch.float32), rt.empty((most_sums,), torch.float32)
        rounded_all, rest_all = rt.empty((most,)), rt.empty((most,))
        latents_all = rt.empty((rank * max(batch.host_counts),))
        at = 0
        for count in batch.host_counts:
            keys = rows[at:at + count]
            latents = latents_all[:rank * count].view(rank, count)
            ops.transpose(keys[:, :rank], latents)
            stretch = stretch_of(count)
            for first in range(0, count, stretch):
                n = min(stretch, count - first)
                shape = (n * heads, count)
                queries = full[at + first:at + first + n].view(n * heads, width)
                scores, rounded, rest = (flat[:n * heads * count].view(shape) for flat in (scores_all, rounded_all, rest_all))
                ops.linear(queries, keys, scores)
                ops.causal_softmax(scores, heads, first, self.scale, self.sink, rounded, rest)
                sums = sums_all[:n * heads * rank].view(n * heads, rank)
                ops.linear(rounded, latents, sums)
                ops.linear(rest, latents, sums, accumulate=True)
                ops.cast(sums, summed[at + first:at + first + n].view(n * heads, rank))
            at += count

    def _heads_out(self, h, batch, cache):
        """The heads' outputs [tokens, n_heads * value_dim]."""
        rt = self.runtime
        ops = rt.ops
        tokens, heads, rank, rot = h.shape[0], self.n_heads, self.kv_rank, self.rot_dim
        frequencies = None if self.position is None else self.position.pair_rotation()[0]
        prompts = self._prompts_alone(h, batch, cache)
        rows = rt.empty((tokens, rank + rot)) if prompts else None
        if cache.writable:
            down = rt.empty((tokens, rank + rot), torch.float32)
            ops.linear(h, self.w_dkv, down)
            ops.latent_complete(down, rank, rot, self.kv_gain, self.eps, frequencies, self.rot_dims, cache.kv, batch, like=h, rows_out=rows)
        low = rt.empty((tokens, self.q_rank), torch.float32)
        ops.linear(h, self.w_dq, low)
        c_q = rt.empty((tokens, self.q_rank))
        ops.rmsnorm(low, self.q_gain, self.eps, c_q)
        q = rt.empty((tokens, heads * (self.dim + rot)), torch.float32)
        ops.linear(c_q, self.w_uq, q)
        plain = rt.empty((tokens, heads * self.dim))
        full = rt.empty((tokens, heads * (rank + rot)))
        ops.latent_queries(q, heads, self.dim, rot, frequencies, self.rot_dims, batch, plain, full, rank)
        ops.linear_heads(plain, self.w_uk_t, full, out_head=rank + rot)
        summed = rt.empty((tokens, heads * rank))
        if prompts:
            self._attend_prompts(full, rows, batch, summed)
        else:
            ops.attention(full, heads, 1, rank + rot, cache.kv, batch, summed, scale=self.scale, value_dim=rank, sink=self.sink,
                          queries_alone=True)
        out = rt.empty((tokens, heads * self.value_dim))
        ops.linear_heads(summed, self.w_uv, out)
        return out

    def forward_into(self, h, batch, cache, out: torch.Tensor) -> None:
        """The mixer's output into `out` (float32 [tokens, hidden]) instead of onto the residual stream."""
        self.runtime.ops.linear(self._heads_out(h, batch, cache), self.w_o, out)

    def forward(self, h, batch, cache, residual: torch.Tensor) -> None:
        self.runtime.ops.linear(self._heads_out(h, batch, cache), self.w_o, residual, accumulate=True)


register_part("mixer", "latent_attention", LatentAttention)
