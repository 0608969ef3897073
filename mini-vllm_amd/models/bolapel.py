"""Bolapel as a plan of parts.

Every layer is a sandwich block (a norm in front of and behind each sublayer) with a token shift
in front of its mixer. The mixer is the generalised delta rule (``parts/delta_rule.py``) or
attention with sigmoid weights inside chunks of the sequence, per-head score bias and per-head
output gate, query/key norm and a rotation over the first channels of each head
(``parts/attention.py``); an attention layer may read the keys and values of an earlier one
(``Call.cache_from``). The feed-forward is the gated SiLU pair; a layer may have none. The logits
are soft-capped.

Tensor names on disk: ``embed``, ``head``, ``final.norm``; per layer i ``l<i>.norm1``, ``.norm1b``,
``.norm2``, ``.norm2b``, ``.shift``, ``l<i>.mix.<name>`` and ``l<i>.mlp.{gate,up,down}``.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, FrozenSet, List

from ..config.model_config import BolapelConfig, ConfigError
from ..parts.attention import AttentionSpec
from ..parts.block import SandwichBlock, SandwichBlockSpec
from ..parts.delta_rule import DeltaRuleSpec
from ..parts.io import CappedHeadSpec
from ..parts.mlp import SwiGLUSpec
from ..parts.norm import RMSNormSpec
from ..parts.plan import Call, EmbeddingSpec, HeadSpec, LayerPlan, ModelPlan, TensorLocation
from ..parts.rope import RotarySpec
from .registry import Architecture, register_architecture

def bolapel_plan(config: BolapelConfig) -> ModelPlan:
    hid = config.hidden_size
    norm = RMSNormSpec(size=hid, eps=config.norm_eps)
    block = SandwichBlockSpec(hidden_size=hid, token_shift=True)
    # who reads whose keys: the owner's pages stay as long as any reader's chunk needs them
    readers: Dict[int, List[int]] = {}
    for i, l in enumerate(config.layers):
        if l.type == "attention":
            readers.setdefault(i if l.kv_from is None else l.kv_from, []).append(i)
    layers, calls = [], []
    for i, l in enumerate(config.layers):
        if l.type == "general_delta":
            if l.decay_rank is None:
                raise ValueError(f"layer {i}: the rank of the decay's matrices is unknown; config.json does not state "
                                 f"it, the stored tensors do (see bolapel_complete)")
            mixer = DeltaRuleSpec(hidden_size=hid, num_heads=l.heads, head_dim=l.dim, decay_rank=l.decay_rank,
                                  out_norm_eps=config.norm_eps)
            calls.append(Call(layer=i))
        else:
            rope = RotarySpec(rotary_dim=l.rot_dims, theta=l.rot_base, interleaved=False) if l.rot_dims else None
            mine = readers.get(i, [i])
            chunks = tuple(sorted({config.layers[j].chunk for j in mine if config.layers[j].chunk is not None}))
            mixer = AttentionSpec(
                hidden_size=hid, num_heads=l.heads, num_kv_heads=l.kv_heads, head_dim=l.dim, scale=l.scale,
                qk_norm=True, qk_norm_eps=config.norm_eps, bias=False, window=None, position=rope,
                shares_kv=l.kv_from is not None, value_dim=l.vdim, weighting="sigmoid", score_bias=True,
                chunk=l.chunk, head_gate=True,
                cache_chunks=() if l.kv_from is not None else chunks,
                cache_keeps_all=l.kv_from is None and any(config.layers[j].chunk is None for j in mine))
            calls.append(Call(layer=i, cache_from=l.kv_from))
        ffn = None if l.ff is None else SwiGLUSpec(hidden_size=hid, intermediate_size=l.ff)
        slots = SandwichBlock.slots_for(ffn is not None)
        layers.append(LayerPlan(block=block, mixer=mixer, ffn=ffn, norms=tuple((s, norm) for s in slots)))
    head = (HeadSpec(vocab_size=config.vocab_size, hidden_size=hid) if config.logit_softcap is None
            else CappedHeadSpec(vocab_size=config.vocab_size, hidden_size=hid, cap=config.logit_softcap))
    plan = ModelPlan(hidden_size=hid, vocab_size=config.vocab_size, max_positions=config.max_position_embeddings,
                     embedding=EmbeddingSpec(vocab_size=config.vocab_size, hidden_size=hid, scale=1.0),
                     layers=tuple(layers), calls=tuple(calls), final_norm=norm, head=head)
    plan.validate()
    return plan


_ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm",
                    "score_bias": "pb", "head_gate": "g"}
_DELTA_NAMES = {"r": "r", "k": "k", "v": "v", "g": "g", "a": "a", "a_bias": "a.b", "w1": "w1", "w2": "w2", "w0": "w0",
                "norm": "norm", "o": "o"}
_MLP_NAMES = {"gate": "gate", "up": "up", "down": "down"}


def bolapel_tensor_name(config: BolapelConfig, loc: TensorLocation) -> str:
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
        names = _DELTA_NAMES if config.layers[loc.layer].type == "general_delta" else _ATTENTION_NAMES
        return prefix + "mix." + names[loc.name]
    if loc.role == "ffn":
        return prefix + "mlp." + _MLP_NAMES[loc.name]
    if loc.role == "block":
        return prefix + loc.name
    if loc.role.startswith("norm."):
        return prefix + loc.role[len("norm."):]
    raise KeyError(loc)


def bolapel_ignorable(config: BolapelConfig) -> FrozenSet[str]:
    # a layer without a feed-forward may still store the two norms around it, and a layer that reads
    # another layer's keys and values may still store projections of its own: neither is used
    names = {f"l{i}.{n}" for i, l in enumerate(config.layers) if l.ff is None for n in ("norm2", "norm2b")}
    names |= {f"l{i}.mix.{n}" for i, l in enumerate(config.layers) if l.type == "attention" and l.kv_from is not None
              for n in ("k", "v", "k.norm")}
    return frozenset(names)


def bolapel_complete(config: BolapelConfig, source) -> BolapelConfig:
    """The configuration with what only the stored tensors state: the rank of every delta-rule
    layer's decay matrices is the number of rows of ``l<i>.mix.w1``."""
    names = set(source.names())
    layers = []
    for i, l in enumerate(config.layers):
        if l.type == "general_delta" and l.decay_rank is None:
            name = f"l{i}.mix.w1"
            if name not in names or len(source.shape(name)) != 2:
                raise ConfigError(f"the model has no matrix {name!r}, which states the rank of layer {i}'s decay")
            l = dataclasses.replace(l, decay_rank=int(source.shape(name)[0]))
        layers.append(l)
    return dataclasses.replace(config, layers=tuple(layers))


BOLAPEL = register_architecture(Architecture(
    name=BolapelConfig.architecture,
    config_class=BolapelConfig,
    plan=bolapel_plan,
    tensor_name=bolapel_tensor_name,
    ignorable=bolapel_ignorable,
    complete=bolapel_complete,
))
