"""A plain, slow Dutilix forward pass: whole sequences, no cache, one function per mechanism.

It imports nothing from the engine and runs on the CPU in the dtype of its inputs (tests use
float64). ``weights`` maps the names on disk (``l0.mix.q``, ``l1.mlp.e3.up`` ...) to tensors; ``cfg``
is the raw dictionary of ``config.json``.

Notation: n tokens of one sequence at positions 0..n-1; matrices are stored [out, in] and applied
as ``x @ W.T``. Every recurrent function also takes and returns its state, so that a sequence can be
fed in pieces.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch

UNIT_EPS = 1e-6          # inside the root of a query's or key's length (delta mixer)
DENOM_EPS = 1e-6         # added to the mLSTM's denominator
WEIGHT_SUM_EPS = 1e-20   # added to the sum of the chosen experts' scores


def rms_norm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# ---------------------------------------------------------------------------------------
# delta mixer
# ---------------------------------------------------------------------------------------
def short_conv(x: torch.Tensor, taps: torch.Tensor, before: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Causal convolution along time, channel by channel. x [n, c]; taps [c, T], the last column
    multiplies the current token; ``before`` [T-1, c] are the inputs in front of x (zeros at the start
    of a sequence). Returns (y [n, c], the last T-1 inputs)."""
    n, c = x.shape
    T = taps.shape[1]
    hist = torch.zeros(T - 1, c, dtype=x.dtype) if before is None else before
    ext = torch.cat([hist, x], dim=0)                    # row t + T - 1 is x[t]
    y = torch.zeros_like(x)
    for j in range(T):
        y = y + ext[j:j + n] * taps[:, j]
    return y, ext[n:]


def gated_delta_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, beta: torch.Tensor,
                     state: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """One head. q, k [n, dk]; v [n, dv]; decay, beta [n]; state [dk, dv].
    S <- decay S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    n, dk = k.shape
    dv = v.shape[1]
    S = torch.zeros(dk, dv, dtype=k.dtype) if state is None else state.clone()
    out = torch.empty(n, dv, dtype=k.dtype)
    for t in range(n):
        S = decay[t] * S
        u = beta[t] * (v[t] - k[t] @ S)
        S = S + k[t][:, None] * u[None, :]
        out[t] = q[t] @ S
    return out, S


def delta_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, m: dict, eps: float,
                state: Optional[dict] = None, rnd=None) -> Tuple[torch.Tensor, dict]:
    """``rnd`` rounds what an engine with 16-bit activations would store (projections, the gated output)."""
    rnd = rnd or (lambda t: t)
    H, G, dk, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    n = h.shape[0]
    state = state or {}
    new = {}
    proj = {}
    for name in ("q", "k", "v"):
        y, new["conv." + name] = short_conv(rnd(h @ w[prefix + name].T), w[prefix + name + ".conv"], state.get("conv." + name))
        proj[name] = silu(y)
    q = proj["q"].view(n, G, dk)
    k = proj["k"].view(n, G, dk)
    v = proj["v"].view(n, H, dv)
    q = q / torch.sqrt(q.pow(2).sum(-1, keepdim=True) + UNIT_EPS) * dk ** -0.5
    k = k / torch.sqrt(k.pow(2).sum(-1, keepdim=True) + UNIT_EPS)
    beta = torch.sigmoid(rnd(h @ w[prefix + "b"].T))                                  # [n, H]
    decay = torch.exp(-torch.exp(w[prefix + "A_log"]) * torch.nn.functional.softplus(rnd(h @ w[prefix + "a"].T) + w[prefix + "dt_bias"]))
    gate = silu(rnd(h @ w[prefix + "g"].T)).view(n, H, dv)
    out = torch.empty(n, H, dv, dtype=h.dtype)
    states = []
    for head in range(H):
        g = head // (H // G)
        o, S = gated_delta_scan(q[:, g], k[:, g], v[:, head], decay[:, head], beta[:, head],
                                None if "S" not in state else state["S"][head])
        out[:, head] = o
        states.append(S)
    new["S"] = torch.stack(states)
    out = rnd(rms_norm(out, w[prefix + "norm"], eps) * gate)
    return rnd(out.reshape(n, H * dv) @ w[prefix + "o"].T), new


# ---------------------------------------------------------------------------------------
# mLSTM mixer
# ---------------------------------------------------------------------------------------
def mlstm_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, log_in: torch.Tensor, log_forget: torch.Tensor,
               state: Optional[tuple] = None) -> Tuple[torch.Tensor, tuple]:
    """One head. q, k [n, dk]; v [n, dv]; log gates [n]; state (S [dk, dv], nrm [dk], m scalar), all zero at
    the start. m' = max(f + m, i); S' = e^(f+m-m') S + e^(i-m') k v^T; nrm' likewise with k;
    o = S'^T q / (max(|nrm' . q|, e^(-m')) + 1e-6)."""
    n, dk = k.shape
    dv = v.shape[1]
    if state is None:
        S, nrm, m = torch.zeros(dk, dv, dtype=k.dtype), torch.zeros(dk, dtype=k.dtype), torch.zeros((), dtype=k.dtype)
    else:
        S, nrm, m = state[0].clone(), state[1].clone(), state[2].clone()
    out = torch.empty(n, dv, dtype=k.dtype)
    for t in range(n):
        m_new = torch.maximum(log_forget[t] + m, log_in[t])
        keep, take = torch.exp(log_forget[t] + m - m_new), torch.exp(log_in[t] - m_new)
        S = keep * S + take * k[t][:, None] * v[t][None, :]
        nrm = keep * nrm + take * k[t]
        m = m_new
        out[t] = (q[t] @ S) / (torch.maximum((nrm @ q[t]).abs(), torch.exp(-m)) + DENOM_EPS)
    return out, (S, nrm, m)


def mlstm_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, m: dict, eps: float,
                state: Optional[dict] = None, rnd=None) -> Tuple[torch.Tensor, dict]:
    rnd = rnd or (lambda t: t)
    H, dk, dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    n = h.shape[0]
    q = (rnd(h @ w[prefix + "q"].T) * dk ** -0.5).view(n, H, dk)
    k = rnd(h @ w[prefix + "k"].T).view(n, H, dk)
    v = rnd(h @ w[prefix + "v"].T).view(n, H, dv)
    log_in = cap * torch.tanh((rnd(h @ w[prefix + "i"].T) + w[prefix + "i.b"]) / cap)
    log_forget = torch.nn.functional.logsigmoid(cap * torch.tanh((rnd(h @ w[prefix + "f"].T) + w[prefix + "f.b"]) / cap))
    out = torch.empty(n, H, dv, dtype=h.dtype)
    new = []
    for head in range(H):
        o, st = mlstm_scan(q[:, head], k[:, head], v[:, head], log_in[:, head], log_forget[:, head],
                           None if state is None else state["heads"][head])
        out[:, head] = o
        new.append(st)
    out = rnd(rms_norm(out, None, eps).reshape(n, H * dv) * w[prefix + "norm"] * torch.sigmoid(rnd(h @ w[prefix + "g"].T)))
    return rnd(out @ w[prefix + "o"].T), {"heads": new}


# ---------------------------------------------------------------------------------------
# latent attention
# ---------------------------------------------------------------------------------------
def rotate_half_layout(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [n, ..., d]: the first ``dims`` channels are rotated, channel i with channel i + dims/2, by the
    angle position * base^(-2i/dims); the rest pass."""
    half = dims // 2
    freq = base ** (-2.0 * torch.arange(half, dtype=x.dtype) / dims)
    ang = positions.to(x.dtype)[:, None] * freq[None, :]                 # [n, half]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


def latent_attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, m: dict, eps: float,
                           positions: Optional[torch.Tensor] = None,
                           cache: Optional[tuple] = None, rnd=None) -> Tuple[torch.Tensor, tuple]:
    """``cache`` = (latents [j, kv_rank], rotated key parts [j, rot_dim]) of the tokens in front."""
    rnd = rnd or (lambda t: t)
    H, dn, dr, dv, rank = m["heads"], m["dim"], m.get("rot_dim", 0), m["vdim"], m["kv_rank"]
    n = h.shape[0]
    start = 0 if cache is None else cache[0].shape[0]
    pos = torch.arange(start, start + n) if positions is None else positions
    rot = (lambda x: rotate_half_layout(x, pos, m["rot"]["dims"], m["rot"]["base"])) if dr else (lambda x: x)
    cq = rnd(rms_norm(rnd(h @ w[prefix + "dq"].T), w[prefix + "dq.norm"], eps))
    q = rnd(cq @ w[prefix + "uq"].T).view(n, H, dn + dr)
    q_plain, q_rot = q[..., :dn], rot(q[..., dn:])
    down = rnd(h @ w[prefix + "dkv"].T)
    lat = rnd(rms_norm(down[:, :rank], w[prefix + "dkv.norm"], eps))
    k_rot = rnd(rot(down[:, rank:]))
    if cache is not None:
        lat, k_rot = torch.cat([cache[0], lat]), torch.cat([cache[1], k_rot])
    total = lat.shape[0]
    k_plain = (lat @ w[prefix + "uk"].T).view(total, H, dn)
    val = (lat @ w[prefix + "uv"].T).view(total, H, dv)
    score = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    visible = torch.arange(total)[None, :] <= pos[:, None]
    score = score.masked_fill(~visible[None], float("-inf"))
    out = torch.einsum("hij,jhd->ihd", torch.softmax(score, dim=-1), val).reshape(n, H * dv)
    out = rnd(out * torch.sigmoid(rnd(h @ w[prefix + "g"].T)))
    return rnd(out @ w[prefix + "o"].T), (lat, k_rot)


# ---------------------------------------------------------------------------------------
# feed-forwards
# ---------------------------------------------------------------------------------------
def gated_pair(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, rnd=None) -> torch.Tensor:
    rnd = rnd or (lambda t: t)
    return (rnd(silu(rnd(h @ gate.T)) * rnd(h @ up.T))) @ down.T


def route(h: torch.Tensor, router: torch.Tensor, correction: torch.Tensor, top: int, groups: int, keep: int):
    """(chosen [n, top] expert indices, weights [n, top]). Scores are the softmax of the router's logits over
    all outputs; the choice is made on scores + correction, among the experts of the ``keep`` groups whose
    largest such number is largest; the weights are the chosen experts' scores divided by their sum."""
    score = torch.softmax(h @ router.T, dim=-1)
    choice = score + correction
    n, E = choice.shape
    per = E // groups
    best = choice.view(n, groups, per).max(-1).values
    kept = torch.zeros(n, groups, dtype=torch.bool)
    kept.scatter_(1, best.topk(keep, dim=-1).indices, True)
    choice = choice.masked_fill(~kept.repeat_interleave(per, dim=1), float("-inf"))
    chosen = choice.topk(top, dim=-1).indices
    picked = score.gather(1, chosen)
    return chosen, picked / (picked.sum(-1, keepdim=True) + WEIGHT_SUM_EPS)


def mixture(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, mlp: dict, rnd=None) -> torch.Tensor:
    r = mlp["router"]
    real = r["experts"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    chosen, weight = route(h, w[prefix + "router"], w[prefix + "correction"], r["top"], groups["count"], groups["keep"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t].tolist(), weight[t]):
            if e >= real:                                # an identity expert
                out[t] += a * h[t]
            else:
                p = f"{prefix}e{e}."
                out[t] += a * gated_pair(h[t:t + 1], w[p + "gate"], w[p + "up"], w[p + "down"], rnd)[0]
    return out


def feed_forward(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, mlp: dict, rnd=None) -> torch.Tensor:
    if mlp["kind"] == "dense":
        return gated_pair(h, w[prefix + "gate"], w[prefix + "up"], w[prefix + "down"], rnd)
    if mlp["kind"] == "moe":
        return mixture(h, w, prefix, mlp, rnd)
    raise ValueError(mlp["kind"])


# ---------------------------------------------------------------------------------------
# the model
# ---------------------------------------------------------------------------------------
MIXERS = {"delta": delta_mixer, "mlstm": mlstm_mixer}


def round_to_bfloat16(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.bfloat16).to(t.dtype)


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], states: Optional[list] = None,
            return_layers: bool = False, rnd=None):
    """Logits [n, vocab] of ``tokens`` continuing a sequence whose per-layer ``states`` are given (None at
    the start). Returns (logits, new states[, residual stream after every layer]). ``rnd`` rounds what an
    engine with 16-bit activations would store; the residual stream stays as it is."""
    rnd = rnd or (lambda t: t)
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)]
    states = states or [None] * len(cfg["layers"])
    new_states, streams = [], []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        hin = rnd(rms_norm(x, w[p + "norm1"], eps))
        if layer["type"] == "latent_attention":
            y, st = latent_attention_mixer(hin, w, p + "mix.", layer["mixer"], eps, cache=states[i], rnd=rnd)
        else:
            y, st = MIXERS[layer["type"]](hin, w, p + "mix.", layer["mixer"], eps, states[i], rnd=rnd)
        new_states.append(st)
        x = x + y
        if layer.get("mlp") is not None:
            x = x + rnd(feed_forward(rnd(rms_norm(x, w[p + "norm2"], eps)), w, p + "mlp.", layer["mlp"], rnd))
        streams.append(x)
    logits = rnd(rms_norm(x, w["final.norm"], eps)) @ w["head"].T * cfg.get("logit_scale", 1.0)
    if return_layers:
        return logits, new_states, torch.stack(streams)
    return logits, new_states
