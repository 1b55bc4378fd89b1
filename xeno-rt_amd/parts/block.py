"""Pre-norm block: x += mixer(norm1(x)); x += feed_forward(norm2(x)).

The order of the reference's layer loop (crates/xrt-models/src/llama.rs:433-602):
norm, attention, add, norm, feed-forward, add. The residual stream x is float32
and is updated in place; each part adds its own output to it.

Options beyond the reference's layer: a block without a feed-forward (only the first sublayer), and an input
transform per sublayer, a part that is applied to the normed rows before the mixer or the feed-forward reads them
(`forward(h, batch, cache)`; a short convolution over time, for one) and may keep state in the block's cache entry.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Block, CacheNeeds, Part, Runtime, WeightSpec, register_part


class PreNormBlock(Block):
    def __init__(self, mixer_norm, mixer, feed_forward_norm=None, feed_forward=None, mixer_input=None, feed_forward_input=None, unread=()):
        if (feed_forward is None) != (feed_forward_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        self.unread = list(unread)          # tensors that a checkpoint may carry for this block and that it does not read
        self.mixer_norm = mixer_norm
        self.mixer = mixer
        self.feed_forward_norm = feed_forward_norm
        self.feed_forward = feed_forward
        self.mixer_input = mixer_input
        self.feed_forward_input = feed_forward_input if feed_forward is not None else None

    def parts(self):
        return tuple(part for part in (self.mixer_norm, self.mixer_input, self.mixer, self.feed_forward_norm,
                                       self.feed_forward_input, self.feed_forward) if part is not None)

    @property
    def capturable(self) -> bool:
        return all(part.capturable for part in self.parts())

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs: Dict[str, WeightSpec] = {}
        for part in self.parts():
            specs.update(part.weight_specs())
        return specs

    def ignored_names(self):
        return self.unread + [name for part in self.parts() for name in getattr(part, "ignored_names", lambda: [])()]

    def cache_needs(self) -> CacheNeeds:
        return self.mixer.cache_needs().merged(*[part.cache_needs() for part in (self.mixer_input, self.feed_forward_input)
                                                 if part is not None])

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        for part in self.parts():
            part.bind(tensors, runtime)

    @property
    def passes_norms(self) -> bool:
        plain = self.mixer_input is None and self.feed_forward_input is None and self.feed_forward is not None
        return plain and bool(getattr(self.mixer, "passes_norms", False))

    def first_norm(self):
        return self.mixer_norm

    @staticmethod
    def _read(x, norm, transform, batch, cache):
        """What a sublayer reads: the normed rows, through the sublayer's input transform if it has one (which may do the
        norm's work as well: `forward_normed`)."""
        if transform is None:
            return norm.forward(x)
        if hasattr(transform, "forward_normed"):
            return transform.forward_normed(x, norm, batch, cache)
        return transform.forward(norm.forward(x), batch, cache)

    def forward(self, x, batch, cache, h=None, then=None):
        if not self.passes_norms:
            self.mixer.forward(self._read(x, self.mixer_norm, self.mixer_input, batch, cache), batch, cache, x)
            if self.feed_forward is not None:
                self.feed_forward.forward(self._read(x, self.feed_forward_norm, self.feed_forward_input, batch, cache), batch, x)
            return None
        if h is None:
            h = self.mixer_norm.forward(x)
        # a norm is left to the products around it only if the part after it reads nothing but products of it
        if self.passes_norms and getattr(self.feed_forward, "passes_norms", False):
            h = self.mixer.forward(h, batch, cache, x, then=self.feed_forward_norm)
        else:
            h = self.mixer.forward(h, batch, cache, x)
        if h is None:
            h = self.feed_forward_norm.forward(x)
        if then is not None and getattr(self.feed_forward, "passes_norms", False):
            return self.feed_forward.forward(h, batch, x, then=then)
        self.feed_forward.forward(h, batch, x)
        return None


class SandwichBlock(Block):
    """A norm before and a norm after each sublayer, and a number m that multiplies what a sublayer adds:
    x += m * post1(mixer(read1(pre1(x)))), then, if the block has a feed-forward, x += m * post2(feed_forward(pre2(x))).
    `mixer_input` is an input transform as in PreNormBlock. Mixer and feed-forward write their float32 output aside
    (`forward_into`), the post norm takes it from there onto the stream (`Norm.add_to`); a mixer that has an output bias
    and can leave it to the caller (`forward_into(..., bias_later=True)` returns it) has it added on the norm's way in,
    and where both are layer norms the first post norm goes on to the feed-forward's norm in the same pass."""

    def __init__(self, mixer_norm, mixer, mixer_post_norm, feed_forward_norm=None, feed_forward=None, feed_forward_post_norm=None,
                 residual_scale: float = 1.0, mixer_input=None):
        if len({feed_forward is None, feed_forward_norm is None, feed_forward_post_norm is None}) != 1:
            raise ValueError("a feed-forward and its two norms come together")
        self.mixer_norm, self.mixer, self.mixer_post_norm = mixer_norm, mixer, mixer_post_norm
        self.feed_forward_norm, self.feed_forward, self.feed_forward_post_norm = feed_forward_norm, feed_forward, feed_forward_post_norm
        self.residual_scale = float(residual_scale)
        self.mixer_input = mixer_input

    def parts(self):
        return tuple(part for part in (self.mixer_norm, self.mixer_input, self.mixer, self.mixer_post_norm, self.feed_forward_norm,
                                       self.feed_forward, self.feed_forward_post_norm) if part is not None)

    @property
    def capturable(self) -> bool:
        return all(part.capturable for part in self.parts())

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs: Dict[str, WeightSpec] = {}
        for part in self.parts():
            specs.update(part.weight_specs())
        return specs

    def ignored_names(self):
        return [name for part in self.parts() for name in getattr(part, "ignored_names", lambda: [])()]

    def cache_needs(self) -> CacheNeeds:
        return self.mixer.cache_needs().merged(*([self.mixer_input.cache_needs()] if self.mixer_input is not None else []))

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        for part in self.parts():
            part.bind(tensors, runtime)

    def first_norm(self):
        return self.mixer_norm

    def forward(self, x, batch, cache) -> None:
        rt = self.runtime
        h = PreNormBlock._read(x, self.mixer_norm, self.mixer_input, batch, cache)
        y = rt.empty(x.shape, torch.float32)
        post = self.mixer_post_norm
        takes_bias = hasattr(post, "centred")
        bias = self.mixer.forward_into(h, batch, cache, y, **({"bias_later": True} if takes_bias and getattr(self.mixer, "has_output_bias", False) else {}))
        extra = {} if bias is None else {"pre_bias": bias}
        if self.feed_forward is None:
            post.add_to(x, y, self.residual_scale, **extra)
            return
        if takes_bias and hasattr(self.feed_forward_norm, "centred"):
            h = post.add_to(x, y, self.residual_scale, then=self.feed_forward_norm, **extra)
        else:
            post.add_to(x, y, self.residual_scale, **extra)
            h = self.feed_forward_norm.forward(x)
        self.feed_forward.forward_into(h, batch, y)
        self.feed_forward_post_norm.add_to(x, y, self.residual_scale)


class ParallelBlock(Block):
    """One norm, and both sublayers read its output: with h = norm(x), x += a * mixer(h) + b * feed_forward(h), where a and b
    are vectors over the model width (`mixer_scale`, `feed_forward_scale`: tensor names, or None for ones). The sublayers
    write their float32 outputs aside and one pass adds them to the stream; a mixer that is itself a weighted sum of
    mixers (`forward_terms`) has its terms added in that same pass. `after`, if given, is a part that then adds what the
    step's tokens bring to the stream of their own (`forward(x, batch, reads=)`, reads being x in the compute dtype if the
    block has it at hand)."""

    def __init__(self, norm, mixer, feed_forward=None, hidden=None, mixer_scale=None, feed_forward_scale=None, after=None):
        self.norm, self.mixer, self.feed_forward, self.after = norm, mixer, feed_forward, after
        self.hidden = int(hidden if hidden is not None else norm.dim)
        self.scale_names = (mixer_scale, feed_forward_scale if feed_forward is not None else None)
        self.unread = [feed_forward_scale] if feed_forward is None and feed_forward_scale is not None else []
        self.scales = [None, None]

    def parts(self):
        return tuple(part for part in (self.norm, self.mixer, self.feed_forward, self.after) if part is not None)

    @property
    def capturable(self) -> bool:
        return all(part.capturable for part in self.parts())

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs: Dict[str, WeightSpec] = {name: WeightSpec((self.hidden,), init="ones", kind="vector")
                                        for name in self.scale_names if name is not None}
        for part in self.parts():
            specs.update(part.weight_specs())
        return specs

    def ignored_names(self):
        return self.unread + [name for part in self.parts() for name in getattr(part, "ignored_names", lambda: [])()]

    def cache_needs(self) -> CacheNeeds:
        return self.mixer.cache_needs()

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        for part in self.parts():
            part.bind(tensors, runtime)
        # (float32 whatever the file stores: the sum onto the stream is float32, and the gains of one pass share a type)
        self.scales = [None if name is None else runtime.vector(tensors[name]).to(torch.float32) for name in self.scale_names]

    def first_norm(self):
        return self.norm

    def forward(self, x, batch, cache) -> None:
        rt = self.runtime
        h = self.norm.forward(x)
        if hasattr(self.mixer, "forward_terms"):
            terms = [(y, self.scales[0], scale) for y, scale in self.mixer.forward_terms(h, batch, cache, x)]
        else:
            y = rt.empty(x.shape, torch.float32)
            self.mixer.forward_into(h, batch, cache, y)
            terms = [(y, self.scales[0], 1.0)]
        if self.feed_forward is not None:
            y = rt.empty(x.shape, torch.float32)
            self.feed_forward.forward_into(h, batch, y)
            terms.append((y, self.scales[1], 1.0))
        # what follows reads the updated stream in the compute dtype: written in the same pass
        reads = rt.empty(x.shape) if self.after is not None and rt.dtype != torch.float32 else None
        rt.ops.add_weighted(x, terms, copy=reads)
        if self.after is not None:
            self.after.forward(x, batch, reads=reads)


class ResidualStreams(Part):
    """The residual stream in `count` copies (hyper-connections): x [tokens, count, width], float32. All copies start as the
    embedding's rows (`open`); blocks read weighted sums of the copies and write all copies at once (`HyperConnectionBlock`);
    in the end the copies are added up and normed for the output head (`close`)."""
    capturable = True

    def __init__(self, count: int, width: int):
        if count <= 0:
            raise ValueError(f"a residual stream has one copy at least, found {count}")
        self.count, self.width = int(count), int(width)

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.ones = torch.ones(self.count, dtype=torch.float32, device=runtime.device)

    def open(self, x: torch.Tensor) -> torch.Tensor:
        streams = self.runtime.empty((x.shape[0], self.count, self.width), torch.float32)
        self.runtime.ops.streams_open(x, streams)
        return streams

    def close(self, streams: torch.Tensor, norm, rows=None) -> torch.Tensor:
        """norm(sum of the copies) of the tokens in `rows` (all, if None), in the compute dtype."""
        scale = norm.row_scale()
        if scale is None:
            raise ValueError("the norm behind a residual stream in copies is a plain RMS norm")
        out = self.runtime.empty((streams.shape[0] if rows is None else rows.shape[0], self.width))
        self.runtime.ops.streams_read(streams, self.ones, scale[0], scale[1], out, rows=rows)
        return out


class _StreamsRead:
    """What a block's first sublayer reads of the copies: the weights of the sum and the norm behind it."""

    def __init__(self, block):
        self.block = block

    def arguments(self, out):
        gain, eps = self.block.mixer_norm.row_scale()
        return self.block.weights[0]["in"], gain, eps, out


class HyperConnectionBlock(Block):
    """A pre-norm block on a residual stream in copies x_1 .. x_s. For each sublayer (the mixer, then the feed-forward if the
    block has one) with its three tensors `in` [s], `out` [s] and `mix` [s, s] (from, to): u = sum_s in[s] x_s,
    y = sublayer(norm(u)), then all copies at once from the old ones, x_t <- sum_s mix[s, t] x_s + out[t] y. The sublayers
    write their float32 output aside (`forward_into`); one kernel writes the copies and makes the next sublayer's read and
    norm in the same pass, across blocks too. Norms are plain RMS norms (`row_scale`)."""
    passes_norms = True

    def __init__(self, count: int, hidden: int, mixer_norm, mixer, mixer_connection: str, feed_forward_norm=None, feed_forward=None,
                 feed_forward_connection: Optional[str] = None, unread=()):
        if (feed_forward is None) != (feed_forward_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        if feed_forward is not None and feed_forward_connection is None:
            raise ValueError("a feed-forward on a stream in copies needs its connection's tensors")
        self.count, self.hidden = int(count), int(hidden)
        self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward = mixer_norm, mixer, feed_forward_norm, feed_forward
        self.connections = [mixer_connection] + ([feed_forward_connection] if feed_forward is not None else [])
        self.weights = []
        # what a checkpoint may carry for a block without a feed-forward and nobody reads: the second connection's tensors, and `unread`
        self.unread = [] if feed_forward is not None else (list(unread) + ([feed_forward_connection + name for name in ("in", "out", "mix")]
                                                                          if feed_forward_connection is not None else []))

    def parts(self):
        return tuple(part for part in (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward) if part is not None)

    @property
    def capturable(self) -> bool:
        return all(part.capturable for part in self.parts())

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs: Dict[str, WeightSpec] = {}
        for prefix in self.connections:
            specs[prefix + "in"] = WeightSpec((self.count,), init="ones", kind="vector")
            specs[prefix + "out"] = WeightSpec((self.count,), init="ones", kind="vector")
            specs[prefix + "mix"] = WeightSpec((self.count, self.count), init="normal", kind="vector")
        for part in self.parts():
            specs.update(part.weight_specs())
        return specs

    def ignored_names(self):
        return self.unread + [name for part in self.parts() for name in getattr(part, "ignored_names", lambda: [])()]

    def cache_needs(self) -> CacheNeeds:
        return self.mixer.cache_needs()

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        for part in self.parts():
            part.bind(tensors, runtime)
        for norm in (self.mixer_norm, self.feed_forward_norm):
            if norm is not None and norm.row_scale() is None:
                raise ValueError("the norms of a block on a stream in copies are plain RMS norms")
        # (float32 whatever the file stores: the sums over the copies are float32)
        self.weights = [{name: tensors[prefix + name].to(device=runtime.device, dtype=torch.float32).contiguous()
                         for name in ("in", "out", "mix")} for prefix in self.connections]

    def first_norm(self):
        return _StreamsRead(self)

    def forward(self, x, batch, cache, h=None, then=None):
        """x: the copies [tokens, count, hidden]. h: this block's first read, if the block before has made it; then: the next
        block's `first_norm()`, whose read this block's last write makes as well (returned; None without `then`)."""
        rt = self.runtime
        tokens = x.shape[0]
        if h is None:
            h = rt.empty((tokens, self.hidden))
            weights, gain, eps, _ = _StreamsRead(self).arguments(None)
            rt.ops.streams_read(x, weights, gain, eps, h)
        y = rt.empty((tokens, self.hidden), torch.float32)
        self.mixer.forward_into(h, batch, cache, y)
        after = None if then is None else then.arguments(rt.empty((tokens, self.hidden)))
        first = self.weights[0]
        if self.feed_forward is None:
            rt.ops.streams_write(x, first["mix"], first["out"], y, then=after)
            return None if after is None else after[3]
        second = self.weights[1]
        gain, eps = self.feed_forward_norm.row_scale()
        h = rt.empty((tokens, self.hidden))
        rt.ops.streams_write(x, first["mix"], first["out"], y, then=(second["in"], gain, eps, h))
        self.feed_forward.forward_into(h, batch, y)
        rt.ops.streams_write(x, second["mix"], second["out"], y, then=after)
        return None if after is None else after[3]


register_part("block", "hyper_connection", HyperConnectionBlock)
register_part("block", "parallel", ParallelBlock)
register_part("block", "pre_norm", PreNormBlock)
register_part("block", "sandwich", SandwichBlock)
