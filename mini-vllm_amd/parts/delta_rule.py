"""A recurrent mixer: the generalised delta rule with one matrix state per head.

Per token and head, with receptance r, key k, value v (``head_dim`` each), a decay w and a removal
rate a per key channel, and the unit key u = k / sqrt(sum(k^2) + key_eps):

    S <- diag(w) S - (a * u)(u^T S) + k v^T        (both subtracted terms read the old S)
    o  = S^T r

    w = exp(-decay_rate * sigmoid(W2 tanh(W1 h) + w0))      a = sigmoid(Wa h + a_bias)

Each head's o is divided by its root mean square, the heads are concatenated, multiplied by a
weight over all heads' channels and by sigmoid(Wg h), and projected back to the model's width.
S starts at zero and is float32 [heads, head_dim, head_dim] per request (``state``, each head's matrix
stored column by column), whatever the activation type; decays, rates, unit keys and the recurrence
itself are float32 too.

r, k, v, g, a and W1 read the same input and are one packed product; everything between that
product and the output projection is three kernels (prepare, scan, finish) for any mix of prompt
portions and single tokens, and one kernel for a step in which every request brings one token.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, Optional

import torch

from .base import Mixer, PartSpec, Runtime, TensorDecl, register_mixer


@dataclass(frozen=True)
class DeltaRuleSpec(PartSpec):
    kind = "delta_rule"
    hidden_size: int = 0
    num_heads: int = 0
    head_dim: int = 0
    decay_rank: int = 0                      # columns of W2 = rows of W1
    decay_rate: float = math.exp(-0.5)       # the decay of a channel lies in (exp(-decay_rate), 1)
    key_eps: float = 1e-6                    # inside the root of a key's length
    out_norm_eps: float = 1e-5               # of the per-head RMS of the output

    @property
    def inner(self) -> int:
        return self.num_heads * self.head_dim


@register_mixer(DeltaRuleSpec.kind)
class DeltaRule(Mixer):
    spec_class = DeltaRuleSpec
    PACKED = ("r", "k", "v", "g", "a", "w1")

    @classmethod
    def tensors(cls, spec: DeltaRuleSpec) -> Dict[str, TensorDecl]:
        inner, hid = spec.inner, spec.hidden_size
        t = {name: TensorDecl((inner, hid)) for name in ("r", "k", "v", "g", "a")}
        t["a_bias"] = TensorDecl((inner,), init="zeros_normal")
        t["w1"] = TensorDecl((spec.decay_rank, hid))
        t["w2"] = TensorDecl((inner, spec.decay_rank))
        t["w0"] = TensorDecl((inner,), init="zeros_normal")
        t["norm"] = TensorDecl((inner,), init="ones_normal")
        t["o"] = TensorDecl((hid, inner))
        return t

    @classmethod
    def state_shape(cls, spec: DeltaRuleSpec):
        return (spec.num_heads, spec.head_dim, spec.head_dim), torch.float32

    def __init__(self, spec: DeltaRuleSpec, tensors: Dict[str, torch.Tensor], rt: Runtime,
                 position: Optional[object] = None):
        if spec.num_heads < 1 or spec.head_dim < 1 or spec.decay_rank < 1:
            raise ValueError(f"delta rule: bad sizes {spec}")
        self.spec, self.rt = spec, rt
        dtypes = {tensors[p].dtype for p in self.PACKED}
        if len(dtypes) != 1:
            raise ValueError(f"delta rule: the projections are stored in different dtypes {dtypes}; cannot pack them")
        # every block of the packed rows starts at a multiple of 8 columns (the rank is padded with zero rows)
        pad = (-spec.decay_rank) % 8
        blocks = [tensors[p] for p in self.PACKED]
        if pad:
            blocks.append(torch.zeros((pad, spec.hidden_size), dtype=blocks[0].dtype, device=blocks[0].device))
        self.w_packed = torch.cat(blocks, dim=0).contiguous()
        self.width = self.w_packed.shape[0]
        # transposed, [rank, heads * head_dim]: neighbouring channels then read neighbouring words
        self.w2_t = tensors["w2"].t().contiguous()
        self.w0, self.a_bias = tensors["w0"], tensors["a_bias"]
        self.norm, self.w_o = tensors["norm"], tensors["o"]

    def forward(self, x: torch.Tensor, ctx, call: int) -> torch.Tensor:
        spec, rt, ops, ws = self.spec, self.rt, self.rt.ops, self.rt.workspace
        n, inner = x.shape[0], spec.inner
        packed = ws.get("delta.packed", (n, self.width), rt.dtype)
        ops.gemm(x, self.w_packed, packed)
        gated = ws.get("delta.gated", (n, inner), rt.dtype)
        plan = ctx.attention_plan
        if plan is not None and plan.decode_only:
            # every request brings one token: the three kernels below as one
            ops.delta_step(packed, spec.num_heads, spec.head_dim, spec.decay_rank, self.w2_t, self.w0, self.a_bias,
                           self.norm, spec.decay_rate, spec.key_eps, spec.out_norm_eps, ctx.state(call), ctx.token_seq,
                           ctx.state_slots, gated)
        else:
            # float32 [n, heads, 5, head_dim]: decay, rate * unit key, unit key, key, receptance
            coef = ws.get("delta.coef", (n, spec.num_heads, 5, spec.head_dim), torch.float32)
            ops.delta_prepare(packed, spec.num_heads, spec.head_dim, spec.decay_rank, self.w2_t, self.w0, self.a_bias,
                              spec.decay_rate, spec.key_eps, coef)
            raw = ws.get("delta.raw", (n, inner), torch.float32)
            ops.delta_scan(packed, coef, ctx.state(call), ctx.cu_seqlens, ctx.state_slots, ctx.n_seqs,
                           spec.num_heads, spec.head_dim, raw)
            ops.delta_finish(raw, packed, self.norm, spec.num_heads, spec.head_dim, spec.out_norm_eps, gated)
        y = ws.get("mixer.out", (n, spec.hidden_size), rt.dtype)
        return ops.gemm(gated, self.w_o, y, defer_sum=True) or y
