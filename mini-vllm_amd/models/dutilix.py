"""Dutilix as a plan of parts.

Every layer is a pre-norm block: x <- x + mixer(norm1(x)), then x <- x + ff(norm2(x)) when the layer has
a feed-forward. The mixer is the gated delta rule or the mLSTM matrix memory (``parts/matrix_state.py``)
or softmax attention over a cached latent with an output gate (``parts/latent_attention.py``); the
feed-forward is the gated SiLU pair or a routed mixture of such pairs with identity experts
(``parts/moe.py``). The logits are multiplied by a constant.

Tensor names on disk: ``embed``, ``head``, ``final.norm``; per layer i ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.mix.<name>`` and ``l<i>.mlp.{gate,up,down}`` or ``l<i>.mlp.{router,correction,e<j>.gate,e<j>.up,e<j>.down}``.
"""
from __future__ import annotations

import dataclasses
from typing import FrozenSet

from ..config.model_config import ConfigError, DutilixConfig
from ..parts.block import PreNormBlock, PreNormBlockSpec
from ..parts.io import ScaledHeadSpec
from ..parts.latent_attention import LatentAttentionSpec
from ..parts.matrix_state import GatedDeltaSpec, MLSTMSpec
from ..parts.mlp import SwiGLUSpec
from ..parts.moe import RoutedExpertsSpec
from ..parts.norm import RMSNormSpec
from ..parts.plan import Call, EmbeddingSpec, LayerPlan, ModelPlan, TensorLocation
from ..parts.rope import RotarySpec
from .registry import Architecture, register_architecture

_NORM_SLOTS = {"mixer": "norm1", "ffn": "norm2"}


def dutilix_plan(config: DutilixConfig) -> ModelPlan:
    hid, eps = config.hidden_size, config.norm_eps
    norm = RMSNormSpec(size=hid, eps=eps)
    layers, calls = [], []
    for i, l in enumerate(config.layers):
        m = l.mixer
        if (m.type == "delta" and m.conv < 1) or (m.type == "latent_attention" and (m.q_rank < 1 or m.kv_rank < 1)):
            raise ValueError(f"layer {i}: config.json states no taps (delta) or ranks (latent_attention); the stored "
                             f"tensors do (see dutilix_complete)")
        if m.type == "delta":
            mixer = GatedDeltaSpec(hidden_size=hid, num_heads=m.heads, num_kv_heads=m.kv_heads, key_dim=m.dim,
                                   value_dim=m.vdim, conv_taps=m.conv, unit_eps=1e-6, out_norm_eps=eps)
        elif m.type == "mlstm":
            mixer = MLSTMSpec(hidden_size=hid, num_heads=m.heads, key_dim=m.dim, value_dim=m.vdim, gate_cap=m.gate_cap,
                              denom_eps=1e-6, out_norm_eps=eps)
        else:
            rope = RotarySpec(rotary_dim=m.rot_dim, theta=m.rot_base, interleaved=False) if m.rot_dim else None
            mixer = LatentAttentionSpec(hidden_size=hid, num_heads=m.heads, plain_dim=m.dim, rot_dim=m.rot_dim,
                                        value_dim=m.vdim, q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale, norm_eps=eps,
                                        output_gate=True, position=rope)
        f = l.mlp
        if f is None:
            ffn = None
        elif f.kind == "dense":
            ffn = SwiGLUSpec(hidden_size=hid, intermediate_size=f.ff)
        else:
            ffn = RoutedExpertsSpec(hidden_size=hid, expert_size=f.ff, num_experts=f.experts, identity_experts=f.identity,
                                    top=f.top, groups=f.groups, keep_groups=f.groups_keep, correction=True,
                                    weight_sum_eps=1e-20)
        slots = PreNormBlock.slots_for(ffn is not None)
        layers.append(LayerPlan(block=PreNormBlockSpec(), mixer=mixer, ffn=ffn, norms=tuple((s, norm) for s in slots)))
        calls.append(Call(layer=i))
    plan = ModelPlan(hidden_size=hid, vocab_size=config.vocab_size, max_positions=config.max_position_embeddings,
                     embedding=EmbeddingSpec(vocab_size=config.vocab_size, hidden_size=hid, scale=1.0),
                     layers=tuple(layers), calls=tuple(calls), final_norm=norm,
                     head=ScaledHeadSpec(vocab_size=config.vocab_size, hidden_size=hid, scale=config.logit_scale))
    plan.validate()
    return plan


_MIXER_NAMES = {
    "delta": {"q": "q", "k": "k", "v": "v", "g": "g", "b": "b", "a": "a", "q_conv": "q.conv", "k_conv": "k.conv",
              "v_conv": "v.conv", "A_log": "A_log", "dt_bias": "dt_bias", "norm": "norm", "o": "o"},
    "mlstm": {"q": "q", "k": "k", "v": "v", "g": "g", "i": "i", "f": "f", "i_bias": "i.b", "f_bias": "f.b", "norm": "norm",
              "o": "o"},
    "latent_attention": {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk",
                         "uv": "uv", "g": "g", "o": "o"},
}


def dutilix_tensor_name(config: DutilixConfig, loc: TensorLocation) -> str:
    if loc.layer is None:
        if loc.role == "embedding":
            return "embed"
        if loc.role == "final_norm":
            return "final.norm"
        if loc.role == "head":
            return "head"
        raise KeyError(loc)
    prefix = f"l{loc.layer}."
    if loc.role == "mixer":
        return prefix + "mix." + _MIXER_NAMES[config.layers[loc.layer].mixer.type][loc.name]
    if loc.role == "ffn":
        if "." in loc.name:                          # an expert's tensor: "gate.3" is stored as e3.gate
            what, expert = loc.name.split(".")
            return f"{prefix}mlp.e{expert}.{what}"
        return prefix + "mlp." + loc.name
    if loc.role.startswith("norm."):
        return prefix + _NORM_SLOTS[loc.role[len("norm."):]]
    raise KeyError(loc)


def dutilix_ignorable(config: DutilixConfig) -> FrozenSet[str]:
    # a layer without a feed-forward may still store the norm in front of it
    return frozenset(f"l{i}.norm2" for i, l in enumerate(config.layers) if l.mlp is None)


def dutilix_complete(config: DutilixConfig, source) -> DutilixConfig:
    """The configuration with what only the stored tensors state, where config.json leaves it out: a delta layer's taps
    are the columns of ``l<i>.mix.q.conv``, an attention layer's ranks the lengths of ``l<i>.mix.dq.norm`` and
    ``l<i>.mix.dkv.norm``."""
    names = set(source.names())

    def length(name: str, axis: int) -> int:
        if name not in names or len(source.shape(name)) <= axis:
            raise ConfigError(f"the model has no tensor {name!r}, which states a size that config.json leaves out")
        return int(source.shape(name)[axis])

    layers = []
    for i, l in enumerate(config.layers):
        m = l.mixer
        if m.type == "delta" and m.conv < 1:
            m = dataclasses.replace(m, conv=length(f"l{i}.mix.q.conv", 1))
        if m.type == "latent_attention" and m.q_rank < 1:
            m = dataclasses.replace(m, q_rank=length(f"l{i}.mix.dq.norm", 0))
        if m.type == "latent_attention" and m.kv_rank < 1:
            m = dataclasses.replace(m, kv_rank=length(f"l{i}.mix.dkv.norm", 0))
        layers.append(dataclasses.replace(l, mixer=m))
    return dataclasses.replace(config, layers=tuple(layers))


DUTILIX = register_architecture(Architecture(
    name=DutilixConfig.architecture,
    config_class=DutilixConfig,
    plan=dutilix_plan,
    tensor_name=dutilix_tensor_name,
    ignorable=dutilix_ignorable,
    complete=dutilix_complete,
))
