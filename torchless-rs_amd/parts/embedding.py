"""Token embedding (a row copy, no scaling: src/model/modules/embedding.rs:15-21
of the reference; `scale` multiplies the row for designs that have one) and the
output head (logits = W x, its own tensor unless the configuration ties it to the
embedding: src/model/mod.rs:364-369, 443-446; `scale` multiplies the logits)."""
from __future__ import annotations

from typing import Dict

import torch

from ..kernels import ops
from ..weights.binding import WeightSpec
from .base import Part, StreamPart, register_part
from .linear import Linear


class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, name: str = "embed_tokens.weight", scale: float = 1.0):
        self.V, self.H, self.name, self.scale = int(vocab_size), int(hidden_size), name, float(scale)
        self.table = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.name: WeightSpec((self.V, self.H))}

    def load(self, tensors, compute_dtype) -> None:
        self.table = tensors[self.name]

    def forward(self, ctx, ids: torch.Tensor, x: torch.Tensor) -> None:
        ops.embed(self.table, ids, x, self.scale)


class LMHead(Part):
    """`tied`: use the embedding table instead of a tensor of its own."""
    graph_safe = True

    def may_capture(self, n_rows: int) -> bool:
        return self.proj is not None and self.proj.own_kernels(n_rows)

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False, name: str = "weight", scale: float = 1.0):
        self.V, self.H, self.tied, self.name = int(vocab_size), int(hidden_size), bool(tied), name
        self.scale = float(scale)
        self.proj = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {} if self.tied else {self.name: WeightSpec((self.V, self.H))}

    def load(self, tensors, compute_dtype) -> None:
        self.proj = Linear(tensors["__embedding__"] if self.tied else tensors[self.name])

    def forward(self, ctx, y: torch.Tensor, logits: torch.Tensor) -> None:
        self.proj(y, logits)
        if self.scale != 1.0:
            ops.scale_(logits, self.scale)


register_part("embedding", "tokens", TokenEmbedding)
register_part("head", "linear", LMHead)


class PassEntry(StreamPart):
    """What the stream receives at the start of each pass over a run of layers that is gone
    through several times with the same weights: before every pass but the first the
    embedding's output is added again (`add_embedding`), and before every pass, the first
    too, row t of a learned table [passes, hidden] (tensor `name`), t the number of the pass."""
    graph_safe = True

    def __init__(self, hidden_size: int, passes: int, name: str = "step", add_embedding: bool = True):
        self.H, self.passes, self.name = int(hidden_size), int(passes), name
        self.needs_embedding = bool(add_embedding) and self.passes > 1
        self.table = None

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.name: WeightSpec((self.passes, self.H))}

    def load(self, tensors, compute_dtype) -> None:
        self.table = tensors[self.name].to(torch.float32).contiguous()
        self.rows = [self.table[t] for t in range(self.passes)]

    def forward(self, ctx, x: torch.Tensor, embedded, t: int) -> None:
        if not (0 <= t < self.passes):
            raise ValueError(f"pass {t} of {self.passes}")
        ops.stream_entry(x, embedded if (t > 0 and self.needs_embedding) else None, self.rows[t])


register_part("stream", "pass_entry", PassEntry)
