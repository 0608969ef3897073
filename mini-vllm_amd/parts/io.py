"""The two ends of the model: token embedding and output head.

Reference: minivllm/models/models/qwen3.py:165,184 (``nn.Embedding``, no scaling) and
qwen3.py:201-204,219 (``lm_head``: a bias-free linear map over the rows whose logits are wanted,
sharing the embedding's table when ``tie_word_embeddings``). Logits are float32 here (the
reference keeps them in the model's dtype).

Both are parts like the others: a spec with the sizes and constants, a class registered under the
spec's kind. A head that scales or caps its logits, or an embedding with a learned offset, is
another registered class; the model code does not change.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict

import torch

from .base import Embedding, Head, PartSpec, Runtime, TensorDecl, register_embedding, register_head
from .plan import EmbeddingSpec, HeadSpec


@register_embedding(EmbeddingSpec.kind)
class TokenEmbedding(Embedding):
    spec_class = EmbeddingSpec
    carries_gather = True

    @classmethod
    def tensors(cls, spec: EmbeddingSpec) -> Dict[str, TensorDecl]:
        return {"weight": TensorDecl((spec.vocab_size, spec.hidden_size))}

    def __init__(self, spec: EmbeddingSpec, tensors: Dict[str, torch.Tensor], rt: Runtime):
        self.spec, self.rt = spec, rt
        self.table = tensors["weight"]

    def forward(self, ctx, resid: torch.Tensor, gather=None) -> None:
        self.rt.ops.embedding(ctx.token_ids, self.table, resid, self.spec.scale, gather=gather)


@register_head(HeadSpec.kind)
class LinearHead(Head):
    spec_class = HeadSpec

    @classmethod
    def tensors(cls, spec: HeadSpec) -> Dict[str, TensorDecl]:
        return {"weight": TensorDecl((spec.vocab_size, spec.hidden_size))}

    def __init__(self, spec: HeadSpec, tensors: Dict[str, torch.Tensor], rt: Runtime):
        self.spec, self.rt = spec, rt
        self.weight = tensors["weight"]

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        logits = self.rt.workspace.get("logits", (h.shape[0], self.spec.vocab_size), torch.float32)
        self.rt.ops.gemm(h, self.weight, logits)
        return logits


@dataclass(frozen=True)
class CappedHeadSpec(PartSpec):
    """A linear head whose logits are squashed into (-cap, cap): cap * tanh(logits / cap)."""
    kind = "capped_linear_head"
    vocab_size: int = 0
    hidden_size: int = 0
    cap: float = 30.0


@register_head(CappedHeadSpec.kind)
class CappedLinearHead(LinearHead):
    spec_class = CappedHeadSpec

    def __init__(self, spec: CappedHeadSpec, tensors: Dict[str, torch.Tensor], rt: Runtime):
        if not spec.cap > 0:
            raise ValueError(f"a logit cap must be positive, got {spec.cap}")
        super().__init__(spec, tensors, rt)

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        logits = super().forward(h, ctx)
        self.rt.ops.soft_cap(logits, self.spec.cap)
        return logits


@dataclass(frozen=True)
class ScaledHeadSpec(PartSpec):
    """A linear head whose logits are multiplied by a constant."""
    kind = "scaled_linear_head"
    vocab_size: int = 0
    hidden_size: int = 0
    scale: float = 1.0


@register_head(ScaledHeadSpec.kind)
class ScaledLinearHead(LinearHead):
    spec_class = ScaledHeadSpec

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        logits = super().forward(h, ctx)
        if self.spec.scale != 1.0:
            self.rt.ops.scale_f32(logits, self.spec.scale)
        return logits
