"""Shared by the Dutilix tests: small configurations that differ in every size and option, random
weights by on-disk name (made here, not by the engine), and the plain model's logits."""
from __future__ import annotations

import copy
from typing import Dict, List, Optional

import numpy as np
import torch

from plain import dutilix_plain as plain


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, identity, top, groups=None, keep=None):
    router = {"experts": experts, "identity": identity, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups, "keep": keep}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def delta(heads, kv_heads, dim, vdim, conv, mlp):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp}


def mlstm(heads, dim, vdim, cap, mlp):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": mlp}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, mlp):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale}
    if rot_dim:
        m["rot"] = {"dims": rot_dim, "base": base}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


# A: every mixer and every feed-forward kind, a layer without feed-forward, grouped query/key heads, values of
# another size than keys, identity experts, groups of two
DUT_A = {"architecture": "Dutilix", "vocab": 200, "width": 64, "norm": {"eps": 1e-5}, "logit_scale": 0.5,
         "layers": [delta(4, 2, 16, 24, 4, moe(40, 8, 2, 3, groups=5, keep=3)),
                    latent(4, 16, 8, 12, 24, 32, 0.21, 10000.0, dense(96)),
                    mlstm(2, 16, 20, 10.0, None),
                    latent(2, 24, 16, 24, 40, 48, 0.16, 500.0, moe(48, 4, 0, 2, groups=2, keep=1))]}
# B: nothing is a multiple of eight; no groups, no identity experts in one router, as many identity as real
# experts in the other; every head its own keys; two taps; no logit scale
DUT_B = {"architecture": "Dutilix", "vocab": 77, "width": 50, "norm": {"eps": 3e-6},
         "layers": [mlstm(3, 10, 6, 15.0, moe(30, 6, 0, 2)),
                    delta(3, 3, 6, 10, 2, dense(70)),
                    latent(3, 10, 4, 6, 12, 20, 0.3, 1000.0, moe(22, 3, 3, 2, groups=3, keep=2)),
                    delta(6, 1, 10, 5, 5, None)]}
# C: sizes that resemble a real model's heads (keys of 64 and 128, a latent of 128, rotated part of 32)
DUT_C = {"architecture": "Dutilix", "vocab": 512, "width": 256, "norm": {"eps": 1e-6}, "logit_scale": 2.0,
         "layers": [delta(4, 2, 64, 128, 3, dense(512)),
                    latent(8, 64, 32, 64, 96, 128, 0.1, 1000000.0, moe(128, 8, 0, 2, groups=4, keep=2)),
                    mlstm(2, 128, 64, 12.0, dense(256)),
                    delta(2, 2, 128, 64, 4, moe(64, 6, 2, 4, groups=2, keep=2))]}
# D: one head everywhere, one tap (no convolution state), no rotated part, every expert chosen, a single group
DUT_D = {"architecture": "Dutilix", "vocab": 90, "width": 32, "norm": {"eps": 1e-5}, "logit_scale": 1.5,
         "layers": [delta(1, 1, 12, 8, 1, moe(16, 3, 1, 4, groups=1, keep=1)),
                    latent(1, 12, 0, 8, 8, 16, 0.29, 10000.0, None),
                    mlstm(1, 8, 12, 8.0, dense(40))]}
# E: mLSTM layers only (no cache group at all) and F: attention layers only (no state at all)
DUT_E = {"architecture": "Dutilix", "vocab": 120, "width": 48, "norm": {"eps": 1e-6},
         "layers": [mlstm(4, 12, 12, 9.0, dense(64)), mlstm(2, 20, 28, 20.0, None)]}
DUT_F = {"architecture": "Dutilix", "vocab": 150, "width": 56, "norm": {"eps": 2e-5}, "logit_scale": 0.8,
         "layers": [latent(7, 8, 8, 16, 16, 24, 0.25, 300.0, dense(48)), latent(2, 40, 2, 20, 32, 8, 0.15, 70000.0, None)]}
DUT = {"A": DUT_A, "B": DUT_B, "C": DUT_C, "D": DUT_D, "E": DUT_E, "F": DUT_F}


def tensor_shapes(cfg: Dict) -> Dict[str, tuple]:
    V, W = cfg["vocab"], cfg["width"]
    shapes = {"embed": (V, W), "head": (V, W), "final.norm": (W,)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        shapes[p + "norm1"] = (W,)
        x = p + "mix."
        H, dk, dv = m["heads"], m["dim"], m["vdim"]
        if layer["type"] == "delta":
            G = m["kv_heads"]
            for name, rows in (("q", G * dk), ("k", G * dk), ("v", H * dv)):
                shapes[x + name] = (rows, W)
                shapes[x + name + ".conv"] = (rows, m["conv"])
            shapes.update({x + "g": (H * dv, W), x + "b": (H, W), x + "a": (H, W), x + "A_log": (H,), x + "dt_bias": (H,),
                           x + "norm": (dv,), x + "o": (W, H * dv)})
        elif layer["type"] == "mlstm":
            shapes.update({x + "q": (H * dk, W), x + "k": (H * dk, W), x + "v": (H * dv, W), x + "g": (H * dv, W),
                           x + "i": (H, W), x + "f": (H, W), x + "i.b": (H,), x + "f.b": (H,), x + "norm": (H * dv,),
                           x + "o": (W, H * dv)})
        else:
            dr, qr, kr = m.get("rot_dim", 0), m["q_rank"], m["kv_rank"]
            shapes.update({x + "dq": (qr, W), x + "dq.norm": (qr,), x + "uq": (H * (dk + dr), qr), x + "dkv": (kr + dr, W),
                           x + "dkv.norm": (kr,), x + "uk": (H * dk, kr), x + "uv": (H * dv, kr), x + "g": (H * dv, W),
                           x + "o": (W, H * dv)})
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        shapes[p + "norm2"] = (W,)
        y = p + "mlp."
        if mlp["kind"] == "dense":
            shapes.update({y + "gate": (mlp["ff"], W), y + "up": (mlp["ff"], W), y + "down": (W, mlp["ff"])})
        else:
            r, ff = mlp["router"], mlp["expert"]["ff"]
            total = r["experts"] + r.get("identity", 0)
            shapes.update({y + "router": (total, W), y + "correction": (total,)})
            for e in range(r["experts"]):
                shapes.update({f"{y}e{e}.gate": (ff, W), f"{y}e{e}.up": (ff, W), f"{y}e{e}.down": (W, ff)})
    return shapes


def make_weights(cfg: Dict, seed: int, stored: torch.dtype = torch.bfloat16, router_gain: float = 3.0,
                 key_gain: float = 1.0) -> Dict[str, torch.Tensor]:
    """Matrices N(0, 1/sqrt(columns)); norm weights 1 + N(0, 0.1); convolution taps N(0, 0.6); decay, step and
    gate offsets N(0, 1), the forget gate's 3 + N(0, 1) (a long memory); the router's correction N(0, 0.05).
    ``router_gain`` multiplies the router's matrix (spread scores, fewer near ties); ``key_gain`` the matrices
    behind attention queries and keys (steep softmax, so that a wrong key shows). Rounded to ``stored``."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith(".conv"):
            t = 0.6 * torch.randn(shape, generator=g)
        elif len(shape) == 2:
            t = torch.randn(shape, generator=g) / shape[1] ** 0.5
            if name.endswith(".router"):
                t = t * router_gain
            if name.endswith((".uq", ".uk", ".dkv")):
                t = t * key_gain
        elif name.endswith((".A_log", ".dt_bias", ".i.b")):
            t = torch.randn(shape, generator=g)
        elif name.endswith(".f.b"):
            t = 3.0 + torch.randn(shape, generator=g)
        elif name.endswith(".correction"):
            t = 0.05 * torch.randn(shape, generator=g)
        else:
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        out[name] = t.to(stored)
    return out


def as_f64(weights: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: v.to(torch.float64) for k, v in weights.items()}


def plain_logits(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int], rnd=None) -> np.ndarray:
    return plain.forward(cfg, as_f64(weights), tokens, rnd=rnd)[0].numpy()


def plain_logits_bf16(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int]) -> np.ndarray:
    return plain_logits(cfg, weights, tokens, rnd=plain.round_to_bfloat16)


def plain_logits_f32(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int]) -> np.ndarray:
    """The plain model evaluated in float32: how far 32-bit arithmetic alone moves the logits."""
    return plain.forward(cfg, {k: v.to(torch.float32) for k, v in weights.items()}, tokens)[0].numpy()


def random_tokens(cfg: Dict, n: int, seed: int) -> List[int]:
    rng = np.random.default_rng(seed)
    return [int(t) for t in rng.integers(0, cfg["vocab"], size=n)]


def with_layers(cfg: Dict, layers: List[Dict]) -> Dict:
    c = copy.deepcopy(cfg)
    c["layers"] = copy.deepcopy(layers)
    return c
