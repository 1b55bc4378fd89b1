"""Causal attention with grouped key/value heads over the cache.

The reference's attention (crates/xrt-models/src/llama.rs:447-577 decode,
:695-784 prefill): q, k, v projections without bias; optional RMSNorm of every
head of q and k with one weight [head_dim] each (:1025-1040), after the
projection and before the position encoding; keys (encoded) and values (raw)
appended to the cache; query head h reads key/value head h // group; a token at
position P sees keys 0..P; softmax of q.k * scale in float32; output projection
added to the residual stream.

Q, K and V are bound as one matrix [(n_heads + 2 n_kv_heads) head_dim][hidden], so
one product reads the normed activations once (the reference fuses the three
dispatches, llama.rs:447-464).

Beyond the reference's model, as options: values of a width of their own (`value_dim`), a short causal convolution
over time on every channel of q, k and v right after the projection (`convolution`, whose last inputs are kept per
sequence), a softmax with one more in its denominator (`sink`: a key of score 0 that has no value), a window, a
position encoding that biases the scores by distance, and tensor names of the caller's choice (`names`). With any of
the first three the step takes the general attention kernel, and the keys and values reach the cache through a
kernel of their own.

Further options make the step take the completed path (`_attend_completed`): one projection for q, k, v (and the
output gate) with float32 sums, one kernel that completes them (biases, head norms, a rotation of pairs by a table of
frequencies, the blend of the values with another layer's, the cache write), then the attention kernel that the
weights ask for. These options are: biases on the four projections (`biases`); weights that are sigmoid(score) of
every visible key instead of a softmax over them (`weights="sigmoid"`), with the heads' scores of a pair mixed by a
matrix (`head_mix`) and a number per head added (`score_bias`) before the sigmoid; a gate per token and head on the
heads' outputs, sigmoid of a projection of the mixer's input (`output_gate`); values blended with those that another
attention layer made of the same token, v <- (1 - lambda) v + lambda v_other (`values=SharedValues.source()` in the
layer whose values are kept for the step, `.reader(name)` in those that blend them in, lambda the tensor `name`); a
position encoding that says `pair_rotation()`, or one that says `score_bias_table()`; positions cut into stretches of
`chunk` from a sequence's first token on, a query seeing the keys of its own stretch only; or `completed=True`, which
asks for this path outright (float32 sums of the projection, whatever else the layer has). On this path too: biases on q, k
and v but not on the output (`biases="qkv"`); head norms without weights (`qk_norm="plain"`: every head of q and k divided by
its root mean square); a query temperature (`query_temperature=(coef, every)`: the queries at position p times
1 + coef * ln(floor((p + 1) / every) + 1)); a sink with a learnt score per head (`sink="name"` of the tensor [n_heads]: the
softmax's denominator also holds exp of it, neither scaled nor biased); and a layer without keys and values of its own
(`keys_from_another=True`: no k and v tensors; its schedule entry reads the cache entry of the layer whose keys and values it uses).
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from .base import CacheNeeds, KVSpec, Mixer, PositionEncoding, Runtime, WeightSpec, register_part


class SharedValues:
    """The values that one attention layer made of a step's tokens (float32 [tokens, kv_heads * value_dim], as projected,
    with their bias), kept while the step runs so that later layers can blend them into their own. A model makes one and
    hands `source()` to the layer that fills it and `reader(name)` to those that read it."""

    def __init__(self):
        self.tensor = None

    def source(self, unused_name: Optional[str] = None):
        return (self, "source", unused_name)

    def reader(self, blend_name: str):
        return (self, "reader", blend_name)


class Attention(Mixer):
    passes_norms = True

    @property
    def capturable(self) -> bool:
        return ((self.position is None or self.position.capturable)
                and (getattr(self, "convolution", None) is None or self.convolution.capturable))

    def __init__(self, prefix: str, hidden: int, n_heads: int, n_kv_heads: int, head_dim: int,
                 position: Optional[PositionEncoding] = None, qk_norm: bool = False,
                 qk_norm_eps: float = 0.0, scale: Optional[float] = None,
                 window: Optional[int] = None, value_dim: Optional[int] = None, sink: bool = False,
                 convolution=None, names: Optional[Dict[str, str]] = None, biases: bool = False, weights: str = "softmax",
                 head_mix: Optional[str] = None, score_bias: Optional[str] = None, output_gate: Optional[str] = None,
                 values=None, unread=(), chunk: Optional[int] = None, completed: bool = False, query_temperature=None,
                 keys_from_another: bool = False):
        if n_heads <= 0 or n_kv_heads <= 0 or n_heads % n_kv_heads != 0:
            raise ValueError(f"head counts {n_heads}/{n_kv_heads}: the first must be a multiple of the second")
        if weights not in ("softmax", "sigmoid"):
            raise ValueError(f"the weights of the keys are 'softmax' or 'sigmoid', found {weights!r}")
        if weights == "softmax" and (head_mix is not None or score_bias is not None):
            raise ValueError("a mix of the heads' scores and a number per head belong to sigmoid weights")
        if biases not in (True, False, "qkv") or qk_norm not in (True, False, "plain"):
            raise ValueError(f"biases are True, False or 'qkv', head norms True, False or 'plain'; found {biases!r} and {qk_norm!r}")
        self.value_dim = head_dim if value_dim is None else int(value_dim)
        self.sink_name = sink if isinstance(sink, str) else None     # a learnt score per head; sink=True is a score of 0
        self.sink = bool(sink)
        self.convolution = convolution
        self.biases, self.weights = bool(biases), weights
        self.output_bias = biases is True
        self.plain_norm = qk_norm == "plain"
        qk_norm = qk_norm is True
        self.query_temperature = None if query_temperature is None else (float(query_temperature[0]), int(query_temperature[1]))
        if self.query_temperature is not None and self.query_temperature[1] <= 0:
            raise ValueError(f"a query temperature grows every so many positions, found {query_temperature!r}")
        self.keys_from_another = bool(keys_from_another)
        self.head_mix_name, self.score_bias_name, self.gate_name = head_mix, score_bias, output_gate
        self.values = values
        self.unread = tuple(unread)         # tensors under the prefix that a checkpoint may carry and this layer does not read
        self.chunk = None if chunk is None else int(chunk)      # positions in stretches of this many; a query sees its own stretch only
        if self.chunk is not None and (self.chunk <= 0 or weights != "softmax"):
            raise ValueError("stretches of positions have a positive size and are served for softmax weights")
        self.completed = (bool(completed) or self.biases or weights == "sigmoid" or output_gate is not None or values is not None or self.chunk is not None
                          or hasattr(position, "pair_rotation") or hasattr(position, "score_bias_table") or self.sink_name is not None
                          or self.plain_norm or self.query_temperature is not None or self.keys_from_another)
        if self.completed and convolution is not None:
            raise ValueError("the completed path of attention has no convolution")
        if self.sink and weights != "softmax":
            raise ValueError("a sink joins a softmax's denominator")
        if self.keys_from_another and values is not None:
            raise ValueError("a layer without values of its own blends none")
        if weights == "sigmoid" and hasattr(position, "score_bias_table"):
            raise ValueError("a bias by distance is served for softmax weights")
        self.general = self.completed or self.sink or self.value_dim != head_dim or convolution is not None
        if head_dim <= 0 or (head_dim % 2 != 0 and not self.general):   # llama.rs:125-128 takes any size; the rotation pairs dims, so an even one
            raise ValueError(f"head_dim {head_dim} must be positive and even")
        if self.general and qk_norm and not self.completed:
            raise ValueError("attention with a sink, a convolution or values of another width takes no head norms")
        self.names = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
                      "q_norm": "q_norm.weight", "k_norm": "k_norm.weight", **(names or {})}
        for name in "qkvo":                                             # a projection's bias, unless the caller names it
            self.names.setdefault(name + "_bias", self.names[name].replace(".weight", "") + ".bias")
        self.prefix = prefix
        self.hidden = hidden
        self.n_heads = n_heads
        self.n_kv_heads = n_kv_heads
        self.head_dim = head_dim
        self.position = position
        self.qk_norm = qk_norm
        self.qk_norm_eps = float(qk_norm_eps)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)  # llama.rs:506
        self.window = window
        self.q_width = n_heads * head_dim
        self.kv_width = n_kv_heads * head_dim
        self.v_width = n_kv_heads * self.value_dim
        self.w_qkv = None
        self.w_o = None
        self.q_norm = None
        self.k_norm = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        p, n = self.prefix, self.names
        specs = {p + n["q"]: WeightSpec((self.q_width, self.hidden)),
                 p + n["o"]: WeightSpec((self.hidden, self.n_heads * self.value_dim))}
        if not self.keys_from_another:
            specs[p + n["k"]] = WeightSpec((self.kv_width, self.hidden))
            specs[p + n["v"]] = WeightSpec((self.v_width, self.hidden))
        if self.sink_name is not None:
            specs[p + self.sink_name] = WeightSpec((self.n_heads,), init="zeros", kind="vector")
        if self.qk_norm:
            specs[p + n["q_norm"]] = WeightSpec((self.head_dim,), init="ones", kind="vector")
            specs[p + n["k_norm"]] = WeightSpec((self.head_dim,), init="ones", kind="vector")
        if self.convolution is not None:
            specs.update(self.convolution.weight_specs())
        if self.biases:
            for name, width in (("q", self.q_width), ("k", self.kv_width), ("v", self.v_width), ("o", self.hidden)):
                if (name == "o" and not self.output_bias) or (name in "kv" and self.keys_from_another):
                    continue
                specs[p + n[name + "_bias"]] = WeightSpec((width,), init="zeros", kind="vector")
        if self.head_mix_name is not None:
            specs[p + self.head_mix_name] = WeightSpec((self.n_heads, self.n_heads), kind="vector")
        if self.score_bias_name is not None:
            specs[p + self.score_bias_name] = WeightSpec((self.n_heads,), init="zeros", kind="vector")
        if self.gate_name is not None:
            specs[p + self.gate_name] = WeightSpec((self.n_heads, self.hidden))
        if self.values is not None and self.values[2] is not None:
            specs[p + self.values[2]] = WeightSpec((), init="zeros", kind="vector")
        if self.completed and self.position is not None:
            specs.update(self.position.weight_specs())
        return specs

    @property
    def has_output_bias(self) -> bool:
        return self.output_bias

    def ignored_names(self):
        """Tensors that a checkpoint may carry for this layer and that it does not read (the share of a blend in a layer
        that blends nothing in, for one)."""
        return [self.prefix + name for name in self.unread]

    def cache_needs(self) -> CacheNeeds:
        needs = CacheNeeds(kv=KVSpec(self.n_kv_heads, self.head_dim, self.window,
                                     None if self.value_dim == self.head_dim else self.value_dim))
        return needs if self.convolution is None else needs.merged(self.convolution.cache_needs())

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        p, n = self.prefix, self.names
        if self.position is not None:
            self.position.bind(tensors, runtime)
        if self.completed:
            projected = "q" if self.keys_from_another else "qkv"
            self.w_proj = runtime.weight([tensors[p + n[name]] for name in projected]
                                         + ([tensors[p + self.gate_name]] if self.gate_name is not None else []))
            self.w_o = runtime.weight(tensors[p + n["o"]])
            self.bias_qkv = self.bias_o = self.head_norms = self.head_mix = self.score_bias = self.blend = self.sink_scores = None
            if self.biases:
                self.bias_qkv = tuple(runtime.vector(tensors[p + n[name + "_bias"]]) if name in projected else None for name in "qkv")
                if self.output_bias:
                    self.bias_o = runtime.vector(tensors[p + n["o_bias"]])
            if self.sink_name is not None:
                self.sink_scores = tensors[p + self.sink_name].to(device=runtime.device, dtype=torch.float32).contiguous()
            if self.qk_norm:
                self.head_norms = (runtime.vector(tensors[p + n["q_norm"]]), runtime.vector(tensors[p + n["k_norm"]]))
            if self.head_mix_name is not None:
                self.head_mix = tensors[p + self.head_mix_name].to(device=runtime.device, dtype=torch.float32).contiguous()
            if self.score_bias_name is not None:
                self.score_bias = tensors[p + self.score_bias_name].to(device=runtime.device, dtype=torch.float32).contiguous()
            if self.values is not None and self.values[1] == "reader":
                self.blend = runtime.vector(tensors[p + self.values[2]]).reshape(1)
            return
        if self.general:
            if self.position is not None and self.position.rotation() is not None:
                raise ValueError("attention with a sink, a convolution or values of another width takes no rotation")
            if self.convolution is not None:
                self.convolution.bind(tensors, runtime)
            self.w_qkv = runtime.weight([tensors[p + n[name]] for name in "qkv"])
            self.w_o = runtime.weight(tensors[p + n["o"]])
            return
        # q and k heads that a rotation over the whole head turns: their pairs are kept side by side
        rotation = None if self.position is None else self.position.rotation()
        whole = rotation is not None and rotation.rope_dim == self.head_dim
        self.w_qkv = runtime.weight([tensors[p + n[name]] for name in "qkv"],
                                    "rotary", head_dim=self.head_dim,
                                    rotated_heads=self.n_heads + self.n_kv_heads if whole else 0)
        self.w_o = runtime.weight(tensors[p + n["o"]])
        if self.qk_norm:
            self.q_norm = runtime.vector(tensors[p + n["q_norm"]])
            self.k_norm = runtime.vector(tensors[p + n["k_norm"]])

    def _attend_general(self, h, batch, cache):
        """The heads' outputs [tokens, n_heads * value_dim] on the general path: projection, convolution over time, the keys and
        values into the cache, attention."""
        rt = self.runtime
        ops = rt.ops
        tokens = h.shape[0]
        qkv = rt.empty((tokens, self.q_width + self.kv_width + self.v_width))
        ops.linear(h, self.w_qkv, qkv)
        if self.convolution is not None:
            qkv = self.convolution.forward(qkv, batch, cache)
        if cache.writable:
            ops.kv_store(qkv[:, self.q_width:self.q_width + self.kv_width], qkv[:, self.q_width + self.kv_width:],
                         self.n_kv_heads, self.head_dim, self.value_dim, cache.kv, batch)
        slopes = None if self.position is None else self.position.score_slopes()
        out = rt.empty((tokens, self.n_heads * self.value_dim))
        ops.attention(qkv, self.n_heads, self.n_kv_heads, self.head_dim, cache.kv, batch, out, scale=self.scale, window=self.window,
                      distance_slopes=slopes, value_dim=self.value_dim, sink=self.sink)
        return out

    def _attend_completed(self, h, batch, cache):
        """The heads' outputs [tokens, n_heads * value_dim] on the completed path."""
        rt = self.runtime
        ops = rt.ops
        tokens = h.shape[0]
        qkv_width = self.q_width if self.keys_from_another else self.q_width + self.kv_width + self.v_width
        proj = rt.empty((tokens, qkv_width + (self.n_heads if self.gate_name is not None else 0)), torch.float32)
        ops.linear(h, self.w_proj, proj)
        rotation = self.position.pair_rotation() if hasattr(self.position, "pair_rotation") else (None, 0, True, 1.0)
        values_in = values_out = None
        if self.values is not None:
            link, role, _ = self.values
            if role == "source":
                values_out = link.tensor = rt.empty((tokens, self.v_width), torch.float32)
            else:
                values_in = link.tensor
                if values_in is None or tuple(values_in.shape) != (tokens, self.v_width):
                    raise ValueError("the values to blend in are those of an earlier layer of this step, of the same width")
        q = rt.empty((tokens, self.q_width))
        ops.qkv_complete(proj, self.n_heads, self.n_kv_heads, self.head_dim, self.value_dim, batch, q,
                         kv=cache.kv if cache.writable and not self.keys_from_another else None, biases=self.bias_qkv,
                         norms=self.head_norms, norm_eps=self.qk_norm_eps, frequencies=rotation[0], rot_dims=rotation[1],
                         neighbours=rotation[2], magnitude=rotation[3], values_in=values_in, values_out=values_out, blend=self.blend,
                         plain_norm=self.plain_norm, query_temperature=self.query_temperature, queries_only=self.keys_from_another)
        out = rt.empty((tokens, self.n_heads * self.value_dim))
        if self.weights == "sigmoid":
            ops.attention_sigmoid(q, self.n_heads, self.n_kv_heads, self.head_dim, self.value_dim, cache.kv, batch, out, self.scale,
                                  window=self.window, head_mix=self.head_mix, head_bias=self.score_bias,
                                  gate=proj[:, qkv_width:] if self.gate_name is not None else None)
            return out
        if self.gate_name is not None:
            raise NotImplementedError("an output gate is served with sigmoid weights")
        table = self.position.score_bias_table() if hasattr(self.position, "score_bias_table") else None
        slopes = None if self.position is None else self.position.score_slopes()
        ops.attention(q, self.n_heads, self.n_kv_heads, self.head_dim, cache.kv, batch, out, scale=self.scale, window=self.window,
                      distance_slopes=slopes, value_dim=self.value_dim, distance_bias=table, queries_alone=True, chunk=self.chunk,
                      sink=self.sink_scores if self.sink_scores is not None else self.sink)
        return out

    def forward_into(self, h, batch, cache, out: torch.Tensor, bias_later: bool = False):
        """The mixer's output into `out` (float32 [tokens, hidden]) instead of onto the residual stream: for an attention
        that is one of several mixers side by side, or whose block puts a norm behind it. bias_later: the output
        projection's bias is not added but returned, for a caller that adds it on its own way."""
        if not self.general:
            raise NotImplementedError("only the general path writes its output aside")
        rt = self.runtime
        if not self.completed:
            rt.ops.linear(self._attend_general(h, batch, cache), self.w_o, out)
            return None
        rt.ops.linear(self._attend_completed(h, batch, cache), self.w_o, out)
        if self.bias_o is None or bias_later:
            return self.bias_o
        row = rt.empty((out.shape[0],), torch.int32)
        row.zero_()
        rt.ops.rows_add(self.bias_o.reshape(1, -1), row, out)
        return None

    def forward(self, h, batch, cache, residual: torch.Tensor, then=None):
        if self.completed:
            out = self.runtime.empty(residual.shape, torch.float32)
            self.forward_into(h, batch, cache, out)
            self.runtime.ops.add(residual, out)
            return None
        if self.general:
            self.runtime.ops.linear(self._attend_general(h, batch, cache), self.w_o, residual, accumulate=True)
            return None
        rt = self.runtime
        ops = rt.ops
        tokens = h.shape[0]
        kv = cache.kv
        qkv = rt.empty((tokens, self.q_width + 2 * self.kv_width))

        dims = (self.n_heads, self.n_kv_heads, self.head_dim)
        write_to = kv if cache.writable else None
        longest_run = int(getattr(batch, "max_count", 0) or 0)      # picks how the values are written; 0: unknown
        rotation = None if self.position is None else self.position.rotation()
        slopes = None if self.position is None else self.position.score_slopes()
        out = rt.empty((tokens, self.q_width))
        # A decode step of a model with head norms: the projection only, and the attention kernel finishes q, k and v
        # itself (norms, rotation, cache write) where it can; without head norms the projection's own kernel does that.
        finishes = getattr(ops, "attention_finishes_qkv", None)
        if (self.qk_norm and write_to is not None and slopes is None and (rotation is not None or self.position is None)
                and finishes is not None and finishes(qkv.dtype, *dims, batch, self.window, 0 if rotation is None else rotation.rope_dim,
                                                       None if rotation is None else rotation.table)):
            ops.linear(h, self.w_qkv, qkv)
            ops.attention(qkv, *dims, kv, batch, out, scale=self.scale,
                          finish=ops.QkvFinish(self.q_norm, self.k_norm, self.qk_norm_eps, None if rotation is None else rotation.table))
            return ops.linear(out, self.w_o, residual, accumulate=True,
                              then_norm=None if then is None else then.row_scale())
        if rotation is not None or self.position is None:
            # the projection, then in one pass (in the same kernel, where a step is short): head norms, rotation, cache write
            ops.linear_qkv(h, self.w_qkv, qkv, *dims, batch.positions, batch.slots,
                            q_norm=self.q_norm, k_norm=self.k_norm, norm_eps=self.qk_norm_eps,
                            rope_theta=None if rotation is None else rotation.theta,
                            rope_dim=0 if rotation is None else rotation.rope_dim,
                            rope_scale=1.0 if rotation is None else rotation.scale,
                            kv=write_to, longest_run=longest_run)
        else:
            # any other position encoding: norms, then the encoding, then the cache write
            ops.linear(h, self.w_qkv, qkv)
            if self.qk_norm:
                ops.qkv_prepare(qkv, *dims, batch.positions, batch.slots,
                                q_norm=self.q_norm, k_norm=self.k_norm, norm_eps=self.qk_norm_eps)
            self.position.apply(qkv, *dims, batch)
            if write_to is not None:
                ops.qkv_prepare(qkv, *dims, batch.positions, batch.slots, kv=write_to, longest_run=longest_run)

        ops.attention(qkv, *dims, kv, batch, out, scale=self.scale, window=self.window,
                      **({} if slopes is None else {"distance_slopes": slopes}))
        return ops.linear(out, self.w_o, residual, accumulate=True,
                          then_norm=None if then is None else then.row_scale())


register_part("mixer", "attention", Attention)
