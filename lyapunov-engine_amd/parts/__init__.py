"""Parts of a decoder layer.  Importing the package registers the built-in ones."""
from . import (attention, block, embedding, filters, gated_attention, latent_attention, linear_recurrence, mingru, mlp, norm, rope,  # noqa: F401
               routed_experts, side_by_side, tempered_attention, window_attention)
from .base import (Block, Embedding, FeedForward, InputFilter, StreamShift, Head, FixedStep, GroupView, LayerCache, Logits, Mixer, Norm, PagedSpec, PageTensor,
                   Part, PositionEncoding, SLOT, StateSpec, StepBatch, StepContext, StepPlan, StepPlanner, WeightSource, WeightSpec)

__all__ = ["Block", "Embedding", "Head", "FeedForward", "InputFilter", "StreamShift", "FixedStep", "StepBatch", "StepPlan", "StepPlanner", "GroupView", "PagedSpec", "PageTensor", "SLOT", "LayerCache", "Logits", "Mixer", "Norm", "Part",
           "PositionEncoding", "StateSpec", "StepContext", "WeightSource", "WeightSpec"]
