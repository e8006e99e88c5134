"""The two ends of the decoder: token embedding and output head.

The reference's LlamaForCausalLM holds ``model.embed_tokens`` (an nn.Embedding)
and ``lm_head`` (an nn.Linear without bias) and, where the head's tensor is
missing, copies the embedding into it
(python/lyapunov_engine/models/llama.py:172-177, 205, 224;
models/weight_loader.py:102-109).  Here the residual stream is float from the
first value on, logits are float, and a tied head uses the embedding's matrix
itself.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import EMBEDDINGS, HEADS, NORMS, STREAM_SHIFTS
from ..kernels import ops
from .base import Embedding, Head, Logits, StepContext, StreamShift, WeightSource, WeightSpec


@EMBEDDINGS.register("lookup")
class TokenEmbedding(Embedding):
    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0, tensor: str = "weight"):
        """``scale`` multiplies every row that is looked up; ``tensor`` is what the matrix is called
        after the part's prefix."""
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.scale, self.tensor = float(scale), tensor
        self.weight: Optional[torch.Tensor] = None

    def weight_specs(self):
        return [WeightSpec("weight", (WeightSource(self.tensor, (self.vocab_size, self.hidden_size)),))]

    def forward(self, ctx: StepContext, token_ids: torch.Tensor) -> torch.Tensor:
        h = torch.empty((token_ids.numel(), self.hidden_size), dtype=torch.float32, device=ctx.device)
        return ops.embedding(token_ids, self.weight, h, self.scale)


@EMBEDDINGS.register("lookup_sinusoid")
class SinusoidEmbedding(TokenEmbedding):
    """A looked-up row plus a position vector that is computed, not learned: entry 2i is
    sin(p * base^(-2i / hidden)), entry 2i + 1 the cosine of the same angle (angles in 64-bit);
    then, optionally, a norm of the sum (``norm``: a PartSpec of the NORMS registry, whose tensors
    stand under ``norm_name`` after the embedding's prefix).  The normed rows are the residual
    stream's first value, in 32-bit."""

    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0, tensor: str = "weight",
                 base: float = 10000.0, norm=None, norm_name: str = "norm."):
        super().__init__(vocab_size, hidden_size, scale, tensor)
        if not base > 0:
            raise ValueError(f"the sinusoid's base must be positive, not {base}")
        self.base, self.norm_name = float(base), norm_name
        self.norm = NORMS.build(norm) if norm is not None else None

    def children(self):
        return {self.norm_name: self.norm} if self.norm is not None else {}

    def forward(self, ctx: StepContext, token_ids: torch.Tensor) -> torch.Tensor:
        h = super().forward(ctx, token_ids)
        ops.add_sinusoid(h, ctx.positions, self.base)
        if self.norm is None:
            return h
        return self.norm.forward(ctx, h, out_dtype=torch.float32)


@HEADS.register("linear")
class LinearHead(Head):
    def __init__(self, vocab_size: int, hidden_size: int, tensor: str = "weight"):
        self.vocab_size, self.hidden_size, self.tensor = vocab_size, hidden_size, tensor
        self.weight: Optional[torch.Tensor] = None
        self._tied_to: Optional[Embedding] = None

    def tie(self, embedding: Embedding) -> None:
        self._tied_to = embedding

    def weight_specs(self):
        if self._tied_to is not None:
            return []
        return [WeightSpec("weight", (WeightSource(self.tensor, (self.vocab_size, self.hidden_size)),))]

    def materialize(self, device, dtype):
        if self._tied_to is not None:
            self.weight = self._tied_to.weight      # one matrix, two uses

    def forward(self, ctx: StepContext, x: torch.Tensor) -> Logits:
        return Logits(*ops.lm_head(x, self.weight))


@STREAM_SHIFTS.register("table")
class ShiftTable(StreamShift):
    """``count`` learned vectors of the stream's width in one tensor [count, hidden]; a call of the
    running order that names row i has it added to every row of the residual stream."""

    def __init__(self, count: int, hidden_size: int, tensor: str = "weight"):
        self.count, self.hidden_size, self.tensor = int(count), int(hidden_size), tensor
        self.weight: Optional[torch.Tensor] = None
        self.weight_f: Optional[torch.Tensor] = None

    def weight_specs(self):
        return [WeightSpec("weight", (WeightSource(self.tensor, (self.count, self.hidden_size)),))]

    def materialize(self, device, dtype):
        self.weight_f = self.weight.float().contiguous()

    def row(self, i: int) -> torch.Tensor:
        if not 0 <= i < self.count:
            raise IndexError(f"stream shift {i} of {self.count}")
        return self.weight_f[i]
