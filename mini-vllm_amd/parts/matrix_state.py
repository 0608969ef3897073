"""Recurrent mixers whose state is one decayed matrix per head, written with scalar gates.

Per token and head, with query q and key k (``key_dim`` each), value v (``value_dim``) and two
scalars a (how much of the old state stays) and b (how strongly the token is written):

    S <- a S;   u = b (v - [delta] S^T k);   S <- S + k u^T;   o = S^T q

so the read-out sees the token's own write.

* ``gated_delta`` (the gated delta rule): [delta] is on. q and k come from ``num_kv_heads`` groups
  (head h reads group h // (num_heads / num_kv_heads)); q, k and v pass a short causal convolution
  over time per channel (``conv_taps`` taps, the last one the current token's, zeros before the
  start) and SiLU; q and k are then made unit vectors, x / sqrt(sum(x^2) + unit_eps), q also times
  key_dim^-1/2. b = sigmoid(W_b h) and a = exp(-exp(A_log) * softplus(W_a h + dt_bias)) per head.
  o is divided by its root mean square per head, multiplied by a weight of ``value_dim`` numbers
  that the heads share and by silu(W_g h).
* ``mlstm`` (the matrix memory of the xLSTM): [delta] is off. q = W_q h * key_dim^-1/2. With the log
  input gate i = cap tanh((W_i h + b_i) / cap), the log forget gate
  f = logsigmoid(cap tanh((W_f h + b_f) / cap)) and a running maximum m (0 at the start),
  m' = max(f + m, i), the scalars are a = exp(f + m - m'), b = exp(i - m'). A normaliser n (the same
  recurrence on k alone) is kept as one more column of S, fed with the value 1, and
  o <- o / (max(|n . q|, exp(-m')) + denom_eps). o is then divided by its root mean square per head,
  multiplied by a weight over all heads' channels and by sigmoid(W_g h).

Both keep S as float32 [heads, columns, key_dim] per request (a head's matrix column by column),
zero at a request's start; the convolution's last ``conv_taps - 1`` inputs (activation type) and the
running maximum (float32 [heads]) are state too. Gates, unit vectors and the recurrence are float32
whatever the activation type. All projections of the mixer's input are one packed product; the
scan kernel is shared by the two mixers.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional

import torch

from .base import Mixer, PartSpec, Runtime, TensorDecl, register_mixer


def _pack(tensors: Dict[str, torch.Tensor], names, hidden: int, what: str):
    dtypes = {tensors[p].dtype for p in names}
    if len(dtypes) != 1:
        raise ValueError(f"{what}: the projections are stored in different dtypes {dtypes}; cannot pack them")
    blocks = [tensors[p] for p in names]
    rows = sum(b.shape[0] for b in blocks)
    pad = (-rows) % 8             # rows of the packed product keep a pitch of a multiple of 8 elements
    if pad:
        blocks.append(torch.zeros((pad, hidden), dtype=blocks[0].dtype, device=blocks[0].device))
    return torch.cat(blocks, dim=0).contiguous()


@dataclass(frozen=True)
class GatedDeltaSpec(PartSpec):
    kind = "gated_delta"
    hidden_size: int = 0
    num_heads: int = 0
    num_kv_heads: int = 0
    key_dim: int = 0
    value_dim: int = 0
    conv_taps: int = 1                  # 1: no convolution (a single tap still scales each channel)
    unit_eps: float = 1e-6              # inside the root of a query's or key's length
    out_norm_eps: float = 1e-6          # of the per-head RMS of the output

    @property
    def conv_channels(self) -> int:
        return 2 * self.num_kv_heads * self.key_dim + self.num_heads * self.value_dim


@register_mixer(GatedDeltaSpec.kind)
class GatedDelta(Mixer):
    spec_class = GatedDeltaSpec
    PACKED = ("q", "k", "v", "g", "b", "a")

    @classmethod
    def tensors(cls, spec: GatedDeltaSpec) -> Dict[str, TensorDecl]:
        hid, qk, vd = spec.hidden_size, spec.num_kv_heads * spec.key_dim, spec.num_heads * spec.value_dim
        t = {"q": TensorDecl((qk, hid)), "k": TensorDecl((qk, hid)), "v": TensorDecl((vd, hid)), "g": TensorDecl((vd, hid)),
             "b": TensorDecl((spec.num_heads, hid)), "a": TensorDecl((spec.num_heads, hid)),
             "q_conv": TensorDecl((qk, spec.conv_taps)), "k_conv": TensorDecl((qk, spec.conv_taps)),
             "v_conv": TensorDecl((vd, spec.conv_taps)),
             "A_log": TensorDecl((spec.num_heads,), init="zeros_normal"),
             "dt_bias": TensorDecl((spec.num_heads,), init="zeros_normal"),
             "norm": TensorDecl((spec.value_dim,), init="ones_normal"),
             "o": TensorDecl((hid, vd))}
        return t

    @classmethod
    def state_shapes(cls, spec: GatedDeltaSpec):
        shapes = {"state": ((spec.num_heads, spec.value_dim, spec.key_dim), torch.float32)}
        if spec.conv_taps > 1:
            shapes["conv"] = ((spec.conv_taps - 1, spec.conv_channels), None)      # the activation type
        return shapes

    def __init__(self, spec: GatedDeltaSpec, tensors: Dict[str, torch.Tensor], rt: Runtime, position: Optional[object] = None):
        if min(spec.num_heads, spec.num_kv_heads, spec.key_dim, spec.value_dim, spec.conv_taps) < 1 \
                or spec.num_heads % spec.num_kv_heads:
            raise ValueError(f"gated delta rule: bad sizes {spec}")
        self.spec, self.rt = spec, rt
        self.w_packed = _pack(tensors, self.PACKED, spec.hidden_size, "gated delta rule")
        self.width = self.w_packed.shape[0]
        self.gate_offset = spec.conv_channels
        self.conv_w = torch.cat([tensors["q_conv"], tensors["k_conv"], tensors["v_conv"]], dim=0).contiguous()
        self.a_log = tensors["A_log"].to(self.conv_w.dtype).contiguous()
        self.dt_bias = tensors["dt_bias"].to(self.conv_w.dtype).contiguous()
        self.norm, self.w_o = tensors["norm"].to(self.conv_w.dtype).contiguous(), tensors["o"]

    def forward(self, x: torch.Tensor, ctx, call: int) -> torch.Tensor:
        spec, rt, ops, ws = self.spec, self.rt, self.rt.ops, self.rt.workspace
        n, H, G, dk, dv = x.shape[0], spec.num_heads, spec.num_kv_heads, spec.key_dim, spec.value_dim
        packed = ws.get("mstate.packed", (n, self.width), rt.dtype)
        ops.gemm(x, self.w_packed, packed)
        gated = ws.get("mstate.gated", (n, H * dv), rt.dtype)
        y = ws.get("mixer.out", (n, spec.hidden_size), rt.dtype)
        plan = ctx.attention_plan
        # every request brings one token: everything between the two products as one kernel
        if plan is not None and plan.decode_only and ops.state_step(
                True, packed, H, G, dk, dv, self.norm, spec.out_norm_eps, ctx.state(call), ctx.token_seq, ctx.cu_seqlens,
                ctx.state_slots, ctx.n_seqs, gated, taps=spec.conv_taps, conv_w=self.conv_w, a_log=self.a_log,
                dt_bias=self.dt_bias, conv_state=ctx.state(call, "conv") if spec.conv_taps > 1 else None,
                unit_eps=spec.unit_eps):
            return ops.gemm(gated, self.w_o, y, defer_sum=True) or y
        qk = ws.get("mstate.qk", (n, G, 2, dk), torch.float32)
        vals = ws.get("mstate.vals", (n, H, dv), torch.float32)
        gates = ws.get("mstate.gates", (n, H, 4), torch.float32)
        ops.gated_delta_prepare(packed, H, G, dk, dv, spec.conv_taps, self.conv_w, self.a_log, self.dt_bias,
                                ctx.state(call, "conv") if spec.conv_taps > 1 else None, spec.unit_eps, ctx.token_seq,
                                ctx.cu_seqlens, ctx.state_slots, ctx.n_seqs, qk, vals, gates)
        raw = ws.get("mstate.raw", (n, H, dv), torch.float32)
        ops.state_scan(qk, vals, gates, ctx.state(call), ctx.cu_seqlens, ctx.state_slots, ctx.n_seqs, H, G, dk, dv, True, raw)
        ops.state_finish(raw, gates, packed, self.gate_offset, self.norm, H, dv, spec.out_norm_eps, ctx.token_seq, gated,
                         shared_weight=True, silu_gate=True)
        return ops.gemm(gated, self.w_o, y, defer_sum=True) or y


@dataclass(frozen=True)
class MLSTMSpec(PartSpec):
    kind = "mlstm"
    hidden_size: int = 0
    num_heads: int = 0
    key_dim: int = 0
    value_dim: int = 0
    gate_cap: float = 15.0              # both gates' pre-activations are squashed into (-cap, cap)
    denom_eps: float = 1e-6             # added to the denominator
    out_norm_eps: float = 1e-6          # of the per-head RMS of the output


@register_mixer(MLSTMSpec.kind)
class MLSTM(Mixer):
    spec_class = MLSTMSpec
    PACKED = ("q", "k", "v", "g", "i", "f")

    @classmethod
    def tensors(cls, spec: MLSTMSpec) -> Dict[str, TensorDecl]:
        hid, qk, vd = spec.hidden_size, spec.num_heads * spec.key_dim, spec.num_heads * spec.value_dim
        return {"q": TensorDecl((qk, hid)), "k": TensorDecl((qk, hid)), "v": TensorDecl((vd, hid)), "g": TensorDecl((vd, hid)),
                "i": TensorDecl((spec.num_heads, hid)), "f": TensorDecl((spec.num_heads, hid)),
                "i_bias": TensorDecl((spec.num_heads,), init="zeros_normal"),
                "f_bias": TensorDecl((spec.num_heads,), init="zeros_normal"),
                "norm": TensorDecl((vd,), init="ones_normal"), "o": TensorDecl((hid, vd))}

    @classmethod
    def state_shapes(cls, spec: MLSTMSpec):
        # the matrix with the normaliser as its last column; the running maximum
        return {"state": ((spec.num_heads, spec.value_dim + 1, spec.key_dim), torch.float32),
                "max": ((spec.num_heads,), torch.float32)}

    def __init__(self, spec: MLSTMSpec, tensors: Dict[str, torch.Tensor], rt: Runtime, position: Optional[object] = None):
        if min(spec.num_heads, spec.key_dim, spec.value_dim) < 1 or not spec.gate_cap > 0:
            raise ValueError(f"mlstm: bad sizes {spec}")
        self.spec, self.rt = spec, rt
        self.w_packed = _pack(tensors, self.PACKED, spec.hidden_size, "mlstm")
        self.width = self.w_packed.shape[0]
        self.gate_offset = spec.num_heads * (2 * spec.key_dim + spec.value_dim)
        self.i_bias = tensors["i_bias"].contiguous()
        self.f_bias = tensors["f_bias"].to(self.i_bias.dtype).contiguous()
        self.norm, self.w_o = tensors["norm"].to(self.i_bias.dtype).contiguous(), tensors["o"]

    def forward(self, x: torch.Tensor, ctx, call: int) -> torch.Tensor:
        spec, rt, ops, ws = self.spec, self.rt, self.rt.ops, self.rt.workspace
        n, H, dk, dv = x.shape[0], spec.num_heads, spec.key_dim, spec.value_dim
        packed = ws.get("mstate.packed", (n, self.width), rt.dtype)
        ops.gemm(x, self.w_packed, packed)
        gated = ws.get("mstate.gated", (n, H * dv), rt.dtype)
        y = ws.get("mixer.out", (n, spec.hidden_size), rt.dtype)
        plan = ctx.attention_plan
        if plan is not None and plan.decode_only and ops.state_step(
                False, packed, H, H, dk, dv, self.norm, spec.out_norm_eps, ctx.state(call), ctx.token_seq, ctx.cu_seqlens,
                ctx.state_slots, ctx.n_seqs, gated, i_bias=self.i_bias, f_bias=self.f_bias, cap=spec.gate_cap,
                max_state=ctx.state(call, "max"), denom_eps=spec.denom_eps):
            return ops.gemm(gated, self.w_o, y, defer_sum=True) or y
        qk = ws.get("mstate.qk", (n, H, 2, dk), torch.float32)
        vals = ws.get("mstate.vals", (n, H, dv + 1), torch.float32)
        gates = ws.get("mstate.gates", (n, H, 4), torch.float32)
        ops.mlstm_prepare(packed, H, dk, dv, self.i_bias, self.f_bias, spec.gate_cap, ctx.state(call, "max"), ctx.token_seq,
                          ctx.cu_seqlens, ctx.state_slots, ctx.n_seqs, qk, vals, gates)
        raw = ws.get("mstate.raw", (n, H, dv + 1), torch.float32)
        ops.state_scan(qk, vals, gates, ctx.state(call), ctx.cu_seqlens, ctx.state_slots, ctx.n_seqs, H, H, dk, dv + 1, False, raw)
        ops.state_finish(raw, gates, packed, self.gate_offset, self.norm, H, dv, spec.out_norm_eps, ctx.token_seq, gated,
                         shared_weight=False, silu_gate=False, normaliser=True, denom_eps=spec.denom_eps)
        return ops.gemm(gated, self.w_o, y, defer_sum=True) or y
