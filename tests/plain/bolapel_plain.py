"""A plain, slow Bolapel forward pass: whole sequences, no cache, one function per mechanism.

It imports nothing from the engine and runs on the CPU in the dtype of its inputs (tests use
float64 or float32). ``weights`` maps the names on disk (``l0.mix.k``, ``l1.norm2b`` ...) to
tensors; ``cfg`` is the raw dictionary of ``config.json``.

Notation: n tokens of one sequence, positions 0..n-1; matrices are stored [out, in] and
applied as ``x @ W.T``.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch

DELTA_KEY_EPS = 1e-6                     # inside the root of a key's length
DECAY_RATE = math.exp(-0.5)              # the steepest decay is exp(-DECAY_RATE)


def rms_norm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) (* weight) over the last dimension."""
    y = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def token_shift(h: torch.Tensor, mix: torch.Tensor, before: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Row t becomes h[t] + (h[t-1] - h[t]) * mix with the rows as they were before; the row in
    front of the first one is ``before`` (zeros at the start of a sequence)."""
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    if before is not None:
        prev[0] = before
    return h + (prev - h) * mix


def delta_rule_scan(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, rate: torch.Tensor,
                    state: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """One head of the generalised delta rule, token by token.

    r, k, decay, rate: [n, dk]; v: [n, dv]; state [dk, dv] (zeros if None).
    With u = k / sqrt(sum(k^2) + 1e-6):  S <- diag(decay) S - (rate * u)(u^T S) + k v^T, both of
    the first two terms reading the old S; o = S^T r. Returns (o [n, dv], final state)."""
    n, dk = k.shape
    dv = v.shape[1]
    S = torch.zeros(dk, dv, dtype=k.dtype) if state is None else state.clone()
    out = torch.empty(n, dv, dtype=k.dtype)
    for t in range(n):
        u = k[t] / torch.sqrt((k[t] * k[t]).sum() + DELTA_KEY_EPS)
        read = u @ S                                   # u^T S, [dv]
        S = decay[t][:, None] * S - (rate[t] * u)[:, None] * read[None, :] + k[t][:, None] * v[t][None, :]
        out[t] = r[t] @ S                              # S^T r
    return out, S


def general_delta_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, heads: int, dim: int,
                        eps: float, rnd=None) -> torch.Tensor:
    """h [n, width] -> [n, width]. ``rnd`` rounds what an engine with 16-bit activations would store."""
    rnd = rnd or (lambda t: t)
    n = h.shape[0]
    g = lambda name: w[prefix + name]
    r = rnd(h @ g("r").T).view(n, heads, dim)
    k = rnd(h @ g("k").T).view(n, heads, dim)
    v = rnd(h @ g("v").T).view(n, heads, dim)
    lora = torch.tanh(rnd(h @ g("w1").T)) @ g("w2").T + g("w0")
    decay = torch.exp(-DECAY_RATE * torch.sigmoid(lora)).view(n, heads, dim)
    rate = torch.sigmoid(rnd(h @ g("a").T) + g("a.b")).view(n, heads, dim)
    out = torch.empty(n, heads, dim, dtype=h.dtype)
    for j in range(heads):
        o, _ = delta_rule_scan(r[:, j], k[:, j], v[:, j], decay[:, j], rate[:, j])
        out[:, j] = rms_norm(o, None, eps)
    y = rnd(out.reshape(n, heads * dim) * g("norm") * torch.sigmoid(rnd(h @ g("g").T)))
    return rnd(y @ g("o").T)


def partial_rotary(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [n, heads, d]: the first ``dims`` channels of every head are rotated, channel i paired with
    i + dims/2, by the angle position * base^(-2i/dims); the rest pass."""
    half = dims // 2
    freq = base ** (-2.0 * torch.arange(half, dtype=torch.float64) / dims)
    angle = positions.to(torch.float64)[:, None] * freq[None, :]
    c, s = angle.cos().to(x.dtype)[:, None, :], angle.sin().to(x.dtype)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat((a * c - b * s, b * c + a * s, x[..., dims:]), dim=-1)


def attention_keys_values(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, m: Dict, eps: float, rnd=None):
    """The keys (normed and rotated, as a cache would hold them) and values of a layer that owns them."""
    rnd = rnd or (lambda t: t)
    n = h.shape[0]
    G, D, Dv = m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    k = rnd(h @ w[prefix + "k"].T).view(n, G, D)
    v = rnd(h @ w[prefix + "v"].T).view(n, G, Dv)
    k = rms_norm(k, w[prefix + "k.norm"], eps)
    if m.get("rot"):
        k = partial_rotary(k, torch.arange(n), m["rot"]["dims"], m["rot"]["base"])
    return rnd(k), v


def chunked_sigmoid_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                              bias: Optional[torch.Tensor], chunk: Optional[int]) -> torch.Tensor:
    """q [n, H, D], k [n, G, D], v [n, G, Dv], bias [H]. Query i sees key j <= i of its own chunk
    (i // chunk == j // chunk); the weight of a visible key is sigmoid(score + bias[h]), not
    normalised over the keys."""
    n, H, D = q.shape
    G = k.shape[1]
    idx = torch.arange(n)
    seen = idx[None, :] <= idx[:, None]
    if chunk is not None:
        seen &= (idx[None, :] // chunk) == (idx[:, None] // chunk)
    out = torch.empty(n, H, v.shape[2], dtype=q.dtype)
    for hd in range(H):
        kv = hd // (H // G)
        score = (q[:, hd] @ k[:, kv].T) * scale + (0.0 if bias is None else bias[hd])
        weight = torch.sigmoid(score) * seen
        out[:, hd] = weight @ v[:, kv]
    return out


def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, m: Dict, eps: float,
                    keys_values, rnd=None) -> torch.Tensor:
    rnd = rnd or (lambda t: t)
    n = h.shape[0]
    H, D = m["heads"], m["dim"]
    q = rnd(h @ w[prefix + "q"].T).view(n, H, D)
    q = rms_norm(q, w[prefix + "q.norm"], eps)
    if m.get("rot"):
        q = partial_rotary(q, torch.arange(n), m["rot"]["dims"], m["rot"]["base"])
    q = rnd(q)
    k, v = keys_values
    chunk = m["mask"]["size"] if m.get("mask") else None
    o = chunked_sigmoid_attention(q, k, v, m["scale"], w[prefix + "pb"], chunk)
    gate = torch.sigmoid(rnd(h @ w[prefix + "g"].T))              # [n, H]
    o = rnd(o * gate[:, :, None])
    return rnd(o.reshape(n, -1) @ w[prefix + "o"].T)


def dense_feed_forward(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, rnd=None) -> torch.Tensor:
    rnd = rnd or (lambda t: t)
    gate = h @ w[prefix + "gate"].T
    return rnd(rnd(gate * torch.sigmoid(gate) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T)


def round_to_bfloat16(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.bfloat16).to(t.dtype)


def soft_cap(logits: torch.Tensor, cap: Optional[float]) -> torch.Tensor:
    return logits if not cap else cap * torch.tanh(logits / cap)


# ---------------------------------------------------------------------------------------
# the model
# ---------------------------------------------------------------------------------------
def forward(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
            return_layers: bool = False, rnd=None):
    """Logits [n, vocab] of one sequence (and the residual stream after every layer). ``rnd`` rounds
    what an engine with 16-bit activations would store (the residual stream and the recurrence stay wide)."""
    rnd = rnd or (lambda t: t)
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)]
    layers = []
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rnd(rms_norm(x, w[p + "norm1"], eps))
        h = rnd(token_shift(h, w[p + "shift"]))
        m = layer["mixer"]
        if layer["type"] == "general_delta":
            y = general_delta_mixer(h, w, p + "mix.", m["heads"], m["dim"], eps, rnd)
        elif layer["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kept[i] = attention_keys_values(h, w, p + "mix.", m, eps, rnd)
                src = i
            y = attention_mixer(h, w, p + "mix.", m, eps, kept[src], rnd)
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(y, w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = rnd(rms_norm(x, w[p + "norm2"], eps))
            x = x + rms_norm(dense_feed_forward(h, w, p + "mlp.", rnd), w[p + "norm2b"], eps)
        layers.append(x)
    h = rnd(rms_norm(x, w["final.norm"], eps))
    logits = soft_cap(h @ w["head"].T, cfg.get("logit_softcap"))
    return (logits, torch.stack(layers)) if return_layers else logits
