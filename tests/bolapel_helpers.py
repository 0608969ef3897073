"""Shared by the Bolapel tests: tiny configurations that differ in every size and option, random
weights by on-disk name (made here, not by the engine), and the plain model's logits."""
from __future__ import annotations

import copy
from typing import Dict, List, Optional

import numpy as np
import torch

from plain import bolapel_plain as plain


def _delta(heads, dim, ff):
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _attn(heads, kv_heads, dim, vdim, chunk, rot_dims, base, scale, ff, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if chunk is not None:
        m["mask"] = {"size": chunk}
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": base}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


# P: a reader of another layer's keys with the owner's chunk; a layer without a feed-forward
BOLA_P = {"architecture": "Bolapel", "vocab": 200, "width": 64, "norm": {"eps": 1e-5}, "logit_softcap": 12.0,
          "layers": [_delta(2, 16, 96), _attn(4, 2, 32, 24, 20, 16, 10000.0, 0.21, 96),
                     _delta(4, 8, None), _attn(4, 2, 32, 24, 20, 16, 10000.0, 0.3, 128, kv_from=1)]}
# Q: head sizes that are no powers of two, rotation over the whole head, one kv head, a reader whose
# chunk differs from its owner's, two owners with different chunks (two cache groups), no cap
BOLA_Q = {"architecture": "Bolapel", "vocab": 333, "width": 96, "norm": {"eps": 3e-6},
          "layers": [_attn(3, 3, 16, 16, 7, 16, 500.0, 0.25, 72), _delta(3, 24, 80),
                     _attn(6, 1, 64, 40, 33, 32, 70000.0, 0.125, None), _delta(1, 40, 112),
                     _attn(6, 1, 64, 40, 50, 32, 70000.0, 0.11, 72, kv_from=2)]}
# R: sizes the bfloat16 serving kernels take (head size 64 for the delta rule, 128 / 64 for attention)
BOLA_R = {"architecture": "Bolapel", "vocab": 512, "width": 256, "norm": {"eps": 1e-6}, "logit_softcap": 30.0,
          "layers": [_delta(4, 64, 512), _attn(8, 2, 128, 128, 48, 64, 1000000.0, 0.0884, 512),
                     _delta(2, 128, 256), _attn(8, 2, 128, 128, 112, 64, 1000000.0, 0.07, 512, kv_from=1),
                     _attn(4, 4, 64, 64, 200, 64, 10000.0, 0.125, None)]}
# S: no mask (all keys), no rotation, values as large as keys, every head its own keys
BOLA_S = {"architecture": "Bolapel", "vocab": 150, "width": 48, "norm": {"eps": 2e-5}, "logit_softcap": 5.0,
          "layers": [_attn(2, 2, 24, 24, None, 0, 0.0, 0.2, 64), _delta(2, 12, None)]}
# T: delta-rule layers only (no cache group at all), a head size that is no multiple of four, rank 1
BOLA_T = {"architecture": "Bolapel", "vocab": 97, "width": 40, "norm": {"eps": 1e-5},
          "layers": [_delta(2, 30, 56), _delta(3, 16, None)]}
# U: attention layers only, two readers of one owner, chunks of one token and of three
BOLA_U = {"architecture": "Bolapel", "vocab": 120, "width": 56, "norm": {"eps": 1e-6}, "logit_softcap": 8.0,
          "layers": [_attn(2, 1, 16, 8, 5, 8, 300.0, 0.3, 48), _attn(2, 1, 16, 8, 1, 8, 300.0, 0.5, None, kv_from=0),
                     _attn(2, 1, 16, 8, 3, 8, 300.0, 0.2, 48, kv_from=0)]}
# V: nothing is a multiple of eight (width 50, vocabulary 77, heads of 6 and 10, values of 6, feed-forward 70)
BOLA_V = {"architecture": "Bolapel", "vocab": 77, "width": 50, "norm": {"eps": 1e-5}, "logit_softcap": 9.0,
          "layers": [_delta(3, 6, 70), _attn(3, 1, 10, 6, 11, 4, 1000.0, 0.3, 70), _delta(1, 10, None),
                     _attn(3, 1, 10, 6, 4, 4, 1000.0, 0.4, 70, kv_from=1)]}
BOLA = {"P": BOLA_P, "Q": BOLA_Q, "R": BOLA_R, "S": BOLA_S, "T": BOLA_T, "U": BOLA_U, "V": BOLA_V}
RANKS = {"P": 6, "Q": 5, "R": 32, "S": 3, "T": 1, "U": 2, "V": 3}


def tensor_shapes(cfg: Dict, rank: int) -> Dict[str, tuple]:
    V, W = cfg["vocab"], cfg["width"]
    shapes = {"embed": (V, W), "head": (V, W), "final.norm": (W,)}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        shapes[p + "norm1"] = (W,)
        shapes[p + "norm1b"] = (W,)
        shapes[p + "shift"] = (W,)
        if layer["type"] == "general_delta":
            inner = m["heads"] * m["dim"]
            for name in ("r", "k", "v", "g", "a"):
                shapes[p + "mix." + name] = (inner, W)
            shapes[p + "mix.a.b"] = (inner,)
            shapes[p + "mix.w1"] = (rank, W)
            shapes[p + "mix.w2"] = (inner, rank)
            shapes[p + "mix.w0"] = (inner,)
            shapes[p + "mix.norm"] = (inner,)
            shapes[p + "mix.o"] = (W, inner)
        else:
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            shapes[p + "mix.q"] = (H * D, W)
            shapes[p + "mix.q.norm"] = (D,)
            if m.get("kv_from") is None:
                shapes[p + "mix.k"] = (G * D, W)
                shapes[p + "mix.v"] = (G * Dv, W)
                shapes[p + "mix.k.norm"] = (D,)
            shapes[p + "mix.pb"] = (H,)
            shapes[p + "mix.g"] = (H, W)
            shapes[p + "mix.o"] = (W, H * Dv)
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            shapes[p + "norm2"] = (W,)
            shapes[p + "norm2b"] = (W,)
            shapes[p + "mlp.gate"] = (ff, W)
            shapes[p + "mlp.up"] = (ff, W)
            shapes[p + "mlp.down"] = (W, ff)
    return shapes


def make_weights(cfg: Dict, rank: int, seed: int, stored: torch.dtype = torch.bfloat16, qk_gain: float = 1.0
                 ) -> Dict[str, torch.Tensor]:
    """Matrices N(0, 1/sqrt(columns)), norm weights 1 + N(0, 0.1), shift weights uniform in (0, 1), the
    small vectors (score bias, rate bias, decay offset) N(0, 1). ``qk_gain`` multiplies the query/key
    norm weights, which makes the sigmoid weights steep so that a wrong key shows. Values are rounded to
    ``stored``."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg, rank).items():
        if len(shape) == 2:
            t = torch.randn(shape, generator=g) / shape[1] ** 0.5
        elif name.endswith("shift"):
            t = torch.rand(shape, generator=g)
        elif name.endswith((".pb", ".a.b", ".w0")):
            t = torch.randn(shape, generator=g)
        else:
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        if name.endswith(("q.norm", "k.norm")):
            t = t * qk_gain
        out[name] = t.to(stored)
    return out


def plain_logits(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int], rnd=None) -> np.ndarray:
    return plain.forward(cfg, weights, tokens, dtype=torch.float64, rnd=rnd).numpy()


def plain_logits_bf16(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int]) -> np.ndarray:
    return plain_logits(cfg, weights, tokens, rnd=plain.round_to_bfloat16)


def random_tokens(cfg: Dict, n: int, seed: int) -> List[int]:
    rng = np.random.default_rng(seed)
    return [int(t) for t in rng.integers(0, cfg["vocab"], size=n)]


def with_layers(cfg: Dict, layers: List[Dict]) -> Dict:
    c = copy.deepcopy(cfg)
    c["layers"] = copy.deepcopy(layers)
    return c
