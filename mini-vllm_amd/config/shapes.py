"""Named Qwen3 shapes for random-weights models: the sizes of the published Qwen3 dense models
(what their config.json files state) and a tiny one. Used by ``run.py --random-model`` and by the
benchmark; a shape is a dictionary of config.json keys that ``Qwen3Config.from_dict`` reads."""
from __future__ import annotations

from typing import Any, Dict

QWEN3_SHAPES: Dict[str, Dict[str, Any]] = {
    "tiny": dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                 intermediate_size=128, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6,
                 tie_word_embeddings=True),
    "0.6b": dict(num_hidden_layers=28, hidden_size=1024, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
                 intermediate_size=3072, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
                 tie_word_embeddings=True),
    "8b": dict(num_hidden_layers=36, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
               intermediate_size=12288, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
               tie_word_embeddings=False),
    "32b": dict(num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
                intermediate_size=25600, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
                tie_word_embeddings=False),
}


def named_shapes() -> Dict[str, Dict[str, Any]]:
    """Every named shape as a raw config.json dictionary, ``architectures`` included: the registry
    picks the architecture from it, as it does for a model folder. Another architecture's shapes are
    added here."""
    shapes = {name: qwen3_shape(name) for name in QWEN3_SHAPES}
    shapes["bolapel-tiny"] = bolapel_tiny_shape()
    for name in QWEN3_SHAPES:
        if name != "tiny":
            shapes[f"bolapel-{name}"] = bolapel_shape(name)
    return shapes


def named_shape(name: str, **overrides) -> Dict[str, Any]:
    shapes = named_shapes()
    if name not in shapes:
        raise KeyError(f"unknown shape {name!r} (known: {sorted(shapes)})")
    return dict(shapes[name], **overrides)


def qwen3_shape(name: str, **overrides) -> Dict[str, Any]:
    """The raw config dictionary of a named shape (``architectures`` and a position limit included)."""
    if name not in QWEN3_SHAPES:
        raise KeyError(f"unknown shape {name!r} (known: {sorted(QWEN3_SHAPES)})")
    raw = dict(QWEN3_SHAPES[name], architectures=["Qwen3ForCausalLM"], max_position_embeddings=40960)
    raw.update(overrides)
    return raw


def bolapel_shape(name: str, layers: int = None, chunk: int = 1024, delta_head_dim: int = 64, decay_rank: int = 64,
                  pattern: int = 4) -> Dict[str, Any]:
    """A Bolapel configuration with the width, feed-forward, vocabulary, head counts and head size of
    the named Qwen3 shape and as many layers: every ``pattern``-th layer is attention in chunks of
    ``chunk`` tokens (rotation over half of each head; every second of them reads the keys and values
    of the one before), the others are delta-rule layers with heads of ``delta_head_dim``. For
    random-weights models at sizes that resemble a real model's layers."""
    q = QWEN3_SHAPES[name]
    n = layers or q["num_hidden_layers"]
    hid, hd = q["hidden_size"], q["head_dim"]
    ff = {"kind": "dense", "ff": q["intermediate_size"]}
    out, owner = [], None
    for i in range(n):
        if i % pattern == pattern - 1:
            m = {"heads": q["num_attention_heads"], "kv_heads": q["num_key_value_heads"], "dim": hd, "vdim": hd,
                 "scale": hd ** -0.5, "mask": {"size": chunk}, "rot": {"dims": hd // 2, "base": q["rope_theta"]}}
            if owner is not None:
                m["kv_from"], owner = owner, None
            else:
                owner = i
            out.append({"type": "attention", "mixer": m, "mlp": ff})
        else:
            out.append({"type": "general_delta", "mlp": ff,
                        "mixer": {"heads": hid // delta_head_dim, "dim": delta_head_dim, "rank": decay_rank}})
    return {"architecture": "Bolapel", "vocab": q["vocab_size"], "width": hid, "layers": out,
            "norm": {"eps": q["rms_norm_eps"]}, "logit_softcap": 30.0}


def bolapel_tiny_shape() -> Dict[str, Any]:
    """A Bolapel model of a few thousand weights with every kind of layer: delta rule, attention in chunks
    with keys of its own, a layer without feed-forward, attention on another layer's keys."""
    ff = {"kind": "dense", "ff": 96}
    attn = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.25, "mask": {"size": 24},
            "rot": {"dims": 8, "base": 10000.0}}
    return {"architecture": "Bolapel", "vocab": 256, "width": 64, "norm": {"eps": 1e-5}, "logit_softcap": 20.0,
            "layers": [{"type": "general_delta", "mixer": {"heads": 2, "dim": 16, "rank": 8}, "mlp": ff},
                       {"type": "attention", "mixer": dict(attn), "mlp": ff},
                       {"type": "general_delta", "mixer": {"heads": 4, "dim": 8, "rank": 8}, "mlp": None},
                       {"type": "attention", "mixer": dict(attn, kv_from=1), "mlp": ff}]}
