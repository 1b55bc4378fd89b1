"""Token embedding and output head.

Embedding: x = E[token_id, :], no scaling (crates/xrt-models/src/llama.rs:1042-1055).
Head: logits = W y in float32, W = lm_head.weight, or the embedding table when
the model ties them (llama.rs:299-305, 604-613).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import CacheNeeds, Part, Runtime, StateSpec, WeightSpec


class Embedding(Part):
    capturable = True

    def __init__(self, prefix: str, vocab: int, hidden: int, name: Optional[str] = None):
        self.prefix = prefix
        self.name = name if name is not None else prefix + "weight"       # the table's tensor
        self.vocab = vocab
        self.hidden = hidden
        self.table = None
        self.shared_with_head = False       # set by an OutputHead that is tied to this table

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.name: WeightSpec((self.vocab, self.hidden))}

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        # a table that is also the head's weight is kept as products like it; one that is only looked up stays plain
        tensor = tensors[self.name]
        self.table = runtime.weight(tensor) if self.shared_with_head else runtime.matrix(tensor)

    def forward(self, token_ids: torch.Tensor, positions: Optional[torch.Tensor] = None) -> torch.Tensor:
        """float32 residual stream [tokens, hidden] for int32 token ids (an embedding that knows nothing of positions
        does not look at them)."""
        x = self.runtime.empty((token_ids.shape[0], self.hidden), torch.float32)
        self.runtime.ops.embed(self.table, token_ids, x)
        return x


class PositionedEmbedding(Embedding):
    """x = E[token] + P[position]: a learnt vector for every position from 0 to max_positions - 1, added unscaled."""

    def __init__(self, prefix: str, vocab: int, hidden: int, max_positions: int, name: Optional[str] = None,
                 positions_name: Optional[str] = None):
        super().__init__(prefix, vocab, hidden, name)
        self.max_positions = int(max_positions)
        self.positions_name = positions_name if positions_name is not None else prefix + "positions"
        self.position_table = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs = super().weight_specs()
        specs[self.positions_name] = WeightSpec((self.max_positions, self.hidden))
        return specs

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.position_table = runtime.matrix(tensors[self.positions_name])

    def forward(self, token_ids: torch.Tensor, positions: Optional[torch.Tensor] = None) -> torch.Tensor:
        if positions is None:
            raise ValueError("an embedding with learnt positions needs the tokens' positions")
        x = super().forward(token_ids)
        self.runtime.ops.rows_add(self.position_table, positions, x)
        return x


class HashedPairEmbedding(Embedding):
    """x = E[token] * scale + B[row]: beside its own row a token reads a row of a second table that is hashed from the
    token before it and itself, row = (before * mul_prev + token * mul_cur) mod buckets; a sequence's first token reads
    row `buckets`, the table's last. The token before a step's first is kept per sequence (`keeps_state`: the model gives
    the embedding a cache entry of its own and calls `forward_step`). Without `pair_name` only the scale is applied."""
    keeps_state = True

    def __init__(self, prefix: str, vocab: int, hidden: int, scale: float = 1.0, name: Optional[str] = None,
                 pair_name: Optional[str] = None, buckets: int = 0, mul_prev: int = 0, mul_cur: int = 0):
        super().__init__(prefix, vocab, hidden, name)
        self.scale = float(scale)
        self.pair_name, self.buckets, self.mul_prev, self.mul_cur = pair_name, int(buckets), int(mul_prev), int(mul_cur)
        if pair_name is not None and self.buckets <= 0:
            raise ValueError("a hashed table needs its number of buckets")
        self.pair_table = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs = super().weight_specs()
        if self.pair_name is not None:
            specs[self.pair_name] = WeightSpec((self.buckets + 1, self.hidden))
        return specs

    def cache_needs(self) -> CacheNeeds:
        if self.pair_name is None:
            return CacheNeeds()
        return CacheNeeds(states=(("token_before", StateSpec((1,), torch.int32)),))

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        if self.pair_name is not None:
            self.pair_table = runtime.matrix(tensors[self.pair_name])

    def forward(self, token_ids, positions=None):
        raise NotImplementedError("an embedding that keeps the token before needs the step and its cache entry: forward_step")

    def forward_step(self, batch, cache) -> torch.Tensor:
        x = Embedding.forward(self, batch.token_ids)
        before = None if self.pair_table is None else cache.states["token_before"].view(-1)
        self.runtime.ops.bigram_add(x, self.scale, batch, self.pair_table, before, self.buckets, self.mul_prev, self.mul_cur)
        return x


class TokenSideTable(Part):
    """A second table with a row for every token id, [vocab, parts * dim]: each of `parts` readers (a layer, say) has its own
    stretch of `dim` columns of a token's row. One table serves all its readers and is bound once."""
    capturable = True

    def __init__(self, name: str, vocab: int, parts: int, dim: int):
        self.name, self.vocab, self.parts, self.dim = name, int(vocab), int(parts), int(dim)
        self.table = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.name: WeightSpec((self.vocab, self.parts * self.dim))}

    def bind(self, tensors, runtime: Runtime) -> None:
        if self.table is not None and getattr(self, "runtime", None) is runtime:
            return
        super().bind(tensors, runtime)
        self.table = runtime.matrix(tensors[self.name])


class TokenSideInput(Part):
    """What a token adds to the residual stream after a layer, from its stretch e of a side table's row:
    g = gelu_tanh(W_gate x) * e, y = W_proj g, x += y / sqrt(mean(y^2) + eps) * w (an RMS norm with a plain weight).
    W_gate reads the stream itself (rounded to the compute dtype), not a normed copy."""
    capturable = True

    def __init__(self, prefix: str, hidden: int, table: TokenSideTable, part: int, eps: float,
                 gate: str = "gate", proj: str = "proj", norm: str = "norm"):
        if not 0 <= part < table.parts:
            raise ValueError(f"stretch {part} of a table of {table.parts}")
        self.hidden, self.side, self.part, self.eps = hidden, table, int(part), float(eps)
        self.gate_name, self.proj_name, self.norm_name = prefix + gate, prefix + proj, prefix + norm

    def weight_specs(self) -> Dict[str, WeightSpec]:
        dim = self.side.dim
        specs = {self.gate_name: WeightSpec((dim, self.hidden)), self.proj_name: WeightSpec((self.hidden, dim)),
                 self.norm_name: WeightSpec((self.hidden,), init="ones", kind="vector")}
        specs.update(self.side.weight_specs())
        return specs

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.side.bind(tensors, runtime)
        self.w_gate = runtime.weight(tensors[self.gate_name])
        self.w_proj = runtime.weight(tensors[self.proj_name])
        self.norm_weight = runtime.vector(tensors[self.norm_name])

    def forward(self, x: torch.Tensor, batch, reads=None) -> None:
        """reads: x in the compute dtype, if the caller has it already."""
        rt = self.runtime
        tokens, dim = x.shape[0], self.side.dim
        if reads is None:
            reads = x
            if rt.dtype != torch.float32:
                reads = rt.empty(x.shape)
                rt.ops.cast(x, reads)
        sums = rt.empty((tokens, dim), torch.float32)
        rt.ops.linear(reads, self.w_gate, sums)
        g = rt.empty((tokens, dim))
        rt.ops.gated_rows(sums, self.side.table, batch.token_ids, self.part * dim, g)
        y = rt.empty(x.shape, torch.float32)
        rt.ops.linear(g, self.w_proj, y)
        rt.ops.add_normed(x, [(y, self.norm_weight)], self.eps, 1.0)


class OutputHead(Part):
    capturable = True

    def __init__(self, prefix: str, vocab: int, hidden: int, tied_to: Optional[Embedding] = None, name: Optional[str] = None,
                 softcap: Optional[float] = None):
        """softcap: logits <- softcap * tanh(logits / softcap)."""
        self.softcap = None if softcap is None else float(softcap)
        self.prefix = prefix
        self.name = name if name is not None else prefix + "weight"
        self.vocab = vocab
        self.hidden = hidden
        self.tied_to = tied_to
        if tied_to is not None:
            tied_to.shared_with_head = True
        self.weight = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        if self.tied_to is not None:
            return {}
        return {self.name: WeightSpec((self.vocab, self.hidden))}

    def ignored_names(self):
        """Tensors that a checkpoint may carry and that this part does not read."""
        return [self.name] if self.tied_to is not None else []

    def bind(self, tensors, runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        if self.tied_to is not None:
            self.weight = self.tied_to.table        # the same buffer, not a copy
        else:
            self.weight = runtime.weight(tensors[self.name])

    def forward(self, y: torch.Tensor) -> torch.Tensor:
        logits = self.runtime.empty((y.shape[0], self.vocab), torch.float32, outlives_the_step=True)
        self.runtime.ops.linear(y, self.weight, logits)
        if self.softcap is not None:
            self.runtime.ops.softcap(logits, self.softcap)
        return logits
