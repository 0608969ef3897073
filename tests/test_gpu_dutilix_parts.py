"""Each mechanism of Dutilix alone, the engine's kernels against the plain functions: the short
convolution with its kept inputs, the gated delta rule and the mLSTM on the shared scan (any mix of
requests, state carried, slots used again, padding, token by token against a prompt bit for bit), attention
over cached latents (far keys, page borders, first tokens), the router and the experts' kernels, the scaled
head."""
import math

import numpy as np
import pytest
import torch

from plain import dutilix_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def ops_for(dtype):
    from minivllm_amd.kernels.ops import Ops
    return Ops(dtype)


def i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


def step_ints(q_lens, slots, pad_rows=0, pad_seqs=0):
    seq = [s for s, n in enumerate(q_lens) for _ in range(n)] + [-1] * pad_rows
    cu = np.concatenate([[0], np.cumsum(q_lens)]).tolist()
    cu += [cu[-1]] * pad_seqs
    return i32(seq), i32(cu), i32(list(slots) + [0] * pad_seqs)


def close(got, want, tol, what=""):
    got, want = got.double().cpu(), want.double().cpu()
    assert torch.isfinite(got).all(), what
    err = float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err <= tol, f"{what}: relative error {err:.3e} exceeds {tol:.1e}"


# ---------------------------------------------------------------------------------------
# gated delta rule: prepare (convolution, unit vectors, gates), scan, finish
# ---------------------------------------------------------------------------------------
def delta_setup(H, G, dk, dv, taps, n, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    C = 2 * G * dk + H * dv
    width = C + H * dv + 2 * H
    width += (-width) % 8
    packed = torch.randn(n, width, generator=g).to(dtype)
    t = dict(conv=0.6 * torch.randn(C, taps, generator=g), a_log=torch.randn(H, generator=g), dt_bias=torch.randn(H, generator=g),
             norm=1 + 0.1 * torch.randn(dv, generator=g))
    return packed, {k: v.to(torch.bfloat16) for k, v in t.items()}


def delta_plain(packed, t, H, G, dk, dv, taps, eps, hist, S):
    """One request: (raw [n, H, dv], gated [n, H*dv], new kept inputs, new S [H, dk, dv]) in float64."""
    p = packed.double()
    n, C = p.shape[0], 2 * G * dk + H * dv
    y, kept = plain.short_conv(p[:, :C], t["conv"].double(), before=hist)
    y = plain.silu(y)
    q, k, v = y[:, :G * dk].view(n, G, dk), y[:, G * dk:2 * G * dk].view(n, G, dk), y[:, 2 * G * dk:].view(n, H, dv)
    q = q / torch.sqrt(q.pow(2).sum(-1, keepdim=True) + plain.UNIT_EPS) * dk ** -0.5
    k = k / torch.sqrt(k.pow(2).sum(-1, keepdim=True) + plain.UNIT_EPS)
    gate = plain.silu(p[:, C:C + H * dv]).view(n, H, dv)
    beta = torch.sigmoid(p[:, C + H * dv:C + H * dv + H])
    decay = torch.exp(-torch.exp(t["a_log"].double()) * torch.nn.functional.softplus(p[:, C + H * dv + H:C + H * dv + 2 * H] + t["dt_bias"].double()))
    raw = torch.empty(n, H, dv, dtype=torch.float64)
    new = []
    for h in range(H):
        raw[:, h], s = plain.gated_delta_scan(q[:, h // (H // G)], k[:, h // (H // G)], v[:, h], decay[:, h], beta[:, h], S[h])
        new.append(s)
    gated = (plain.rms_norm(raw, t["norm"].double(), eps) * gate).reshape(n, H * dv)
    return raw, gated, kept, torch.stack(new)


def run_delta(ops, packed, t, H, G, dk, dv, taps, eps, conv_state, state, q_lens, slots, pad_rows=0, pad_seqs=0):
    n = packed.shape[0]
    tsq, cu, sl = step_ints(q_lens, slots, pad_rows, pad_seqs)
    dev = {k: v.to(DEV) for k, v in t.items()}
    qk = torch.empty(n, G, 2, dk, dtype=torch.float32, device=DEV)
    vals = torch.empty(n, H, dv, dtype=torch.float32, device=DEV)
    gates = torch.empty(n, H, 4, dtype=torch.float32, device=DEV)
    raw = torch.full((n, H, dv), float("nan"), dtype=torch.float32, device=DEV)
    out = torch.empty(n, H * dv, dtype=packed.dtype, device=DEV)
    p = packed.to(DEV)
    ops.gated_delta_prepare(p, H, G, dk, dv, taps, dev["conv"], dev["a_log"], dev["dt_bias"], conv_state, plain.UNIT_EPS, tsq, cu, sl,
                            len(q_lens) + pad_seqs, qk, vals, gates)
    ops.state_scan(qk, vals, gates, state, cu, sl, len(q_lens) + pad_seqs, H, G, dk, dv, True, raw)
    ops.state_finish(raw, gates, p, 2 * G * dk + H * dv, dev["norm"], H, dv, eps, tsq, out, shared_weight=True, silu_gate=True)
    torch.cuda.synchronize()
    return raw, out


DELTA_SIZES = [(4, 2, 16, 24, 4), (3, 3, 6, 10, 2), (2, 1, 64, 128, 3), (1, 1, 12, 8, 1), (6, 2, 40, 20, 5), (2, 2, 128, 64, 4),
               (1, 1, 200, 7, 2)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, dk, dv, taps", DELTA_SIZES)
def test_gated_delta_mixed_step(dtype, H, G, dk, dv, taps):
    """Four requests of 9, 1, 4 and 2 tokens on slots out of order, two padding rows and a padding sequence;
    every request starts from a state and kept inputs that are not zero."""
    ops = ops_for(dtype)
    eps, q_lens, slots = 1e-5, [9, 1, 4, 2], [2, 0, 3, 1]
    n = sum(q_lens)
    packed, t = delta_setup(H, G, dk, dv, taps, n + 2, seed=H * 100 + dk, dtype=dtype)
    g = torch.Generator().manual_seed(1)
    C = 2 * G * dk + H * dv
    S0 = 0.3 * torch.randn(5, H, dk, dv, generator=g)
    hist0 = torch.randn(5, max(taps - 1, 1), C, generator=g).to(dtype)
    state = S0.transpose(2, 3).contiguous().to(DEV)                           # column by column
    conv_state = hist0.to(DEV).clone() if taps > 1 else None
    raw, out = run_delta(ops, packed, t, H, G, dk, dv, taps, eps, conv_state, state, q_lens, slots, pad_rows=2, pad_seqs=1)
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    base = 0
    for qn, slot in zip(q_lens, slots):
        want_raw, want, kept, S = delta_plain(packed[base:base + qn], t, H, G, dk, dv, taps, eps,
                                              hist0[slot, :taps - 1].double() if taps > 1 else None, S0[slot].double())
        close(raw[base:base + qn], want_raw, 2e-5, "scan output")
        close(out[base:base + qn], want, tol, "gated output")
        close(state[slot].transpose(1, 2), S, 2e-5, "state")
        if taps > 1:
            assert torch.equal(conv_state[slot].cpu().double(), kept), "kept inputs"
        base += qn
    assert torch.equal(state[4].cpu(), S0[4].transpose(1, 2)), "a slot nobody holds is not touched"
    assert (out[base:] == 0).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_delta_token_by_token_is_the_prompt_bit_for_bit(dtype):
    """120 tokens in one step, in portions of 1, 2, 3 (shorter than the four taps reach back), 50 and 64, and one by
    one: the same bits each way, state and kept inputs included."""
    ops = ops_for(dtype)
    H, G, dk, dv, taps, eps, n = 4, 2, 16, 24, 4, 1e-6, 120
    packed, t = delta_setup(H, G, dk, dv, taps, n, seed=7, dtype=dtype)
    C = 2 * G * dk + H * dv
    results = []
    for cuts in ([n], [1, 2, 3, 50, 64], [1] * n):
        state = torch.zeros(2, H, dv, dk, dtype=torch.float32, device=DEV)
        conv_state = torch.zeros(2, taps - 1, C, dtype=dtype, device=DEV)
        rows, base = [], 0
        for c in cuts:
            _, out = run_delta(ops, packed[base:base + c], t, H, G, dk, dv, taps, eps, conv_state, state, [c], [1])
            rows.append(out.clone())
            base += c
        results.append((torch.cat(rows), state.clone(), conv_state.clone()))
    for other in results[1:]:
        for a, b in zip(results[0], other):
            assert torch.equal(a, b)
    want = delta_plain(packed, t, H, G, dk, dv, taps, eps, None, torch.zeros(H, dk, dv, dtype=torch.float64))
    close(results[0][0], want[1], 2e-5 if dtype == torch.float32 else 1.2e-2, "against the plain scan")


def test_a_written_value_is_read_back_and_decays():
    """One key written with strength one is read back exactly by a query along it, fades by the decay with every
    later token whose key is orthogonal, and is replaced (not added to) by a second write along the same key."""
    ops = ops_for(torch.float32)
    H, G, dk, dv, n = 1, 1, 8, 4, 6
    qk = torch.zeros(n, G, 2, dk, device=DEV)
    vals = torch.zeros(n, H, dv, device=DEV)
    gates = torch.zeros(n, H, 4, device=DEV)
    gates[:, :, 0] = 0.5                                   # decay
    gates[[0, 4], :, 1] = 1.0                              # tokens 0 and 4 write with strength one
    qk[:, 0, 0, 0] = 1.0                                   # every query along channel 0
    qk[[0, 4], 0, 1, 0] = 1.0                              # keys of tokens 0 and 4 along channel 0
    qk[[1, 2, 3, 5], 0, 1, 1] = 1.0                        # the others along channel 1 (strength 0: nothing written)
    vals[0, 0] = torch.tensor([1.0, 2.0, 3.0, 4.0])
    vals[4, 0] = torch.tensor([-8.0, 0.0, 8.0, 16.0])
    state = torch.zeros(1, H, dv, dk, device=DEV)
    raw = torch.empty(n, H, dv, device=DEV)
    ops.state_scan(qk, vals, gates, state, i32([0, n]), i32([0]), 1, H, G, dk, dv, True, raw)
    first = torch.tensor([1.0, 2.0, 3.0, 4.0])
    for t, f in enumerate([1.0, 0.5, 0.25, 0.125]):
        assert torch.allclose(raw[t, 0].cpu(), first * f)
    assert torch.allclose(raw[4, 0].cpu(), vals[4, 0].cpu())                 # the delta rule overwrote what was there
    assert torch.allclose(raw[5, 0].cpu(), vals[4, 0].cpu() * 0.5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, dk, dv, taps", DELTA_SIZES)
def test_gated_delta_single_token_kernel(dtype, H, G, dk, dv, taps):
    """Steps of single tokens take one kernel per (row, head) instead of three: three such steps of four requests on
    slots out of order, a padding row and a padding sequence, give the bits of the three kernels, states and kept
    inputs included."""
    ops = ops_for(dtype)
    eps, slots, steps = 1e-5, [2, 0, 3, 1], 3
    n = len(slots) + 1
    C = 2 * G * dk + H * dv
    g = torch.Generator().manual_seed(5)
    S0 = 0.3 * torch.randn(5, H, dv, dk, generator=g)
    hist0 = torch.randn(5, max(taps - 1, 1), C, generator=g).to(dtype)
    results = []
    for fused in (False, True):
        state = S0.to(DEV).clone()
        conv_state = hist0.to(DEV).clone() if taps > 1 else None
        outs = []
        for step in range(steps):
            packed, t = delta_setup(H, G, dk, dv, taps, n, seed=50 + step, dtype=dtype)
            if not fused:
                outs.append(run_delta(ops, packed, t, H, G, dk, dv, taps, eps, conv_state, state, [1] * 4, slots, pad_rows=1, pad_seqs=1)[1].clone())
                continue
            tsq, cu, sl = step_ints([1] * 4, slots, 1, 1)
            dev = {k: v.to(DEV) for k, v in t.items()}
            out = torch.full((n, H * dv), 5.0, dtype=dtype, device=DEV)
            assert ops.state_step(True, packed.to(DEV), H, G, dk, dv, dev["norm"], eps, state, tsq, cu, sl, 5, out, taps=taps,
                                  conv_w=dev["conv"], a_log=dev["a_log"], dt_bias=dev["dt_bias"], conv_state=conv_state,
                                  unit_eps=plain.UNIT_EPS)
            torch.cuda.synchronize()
            outs.append(out.clone())
        results.append((torch.cat(outs), state.clone(), None if conv_state is None else conv_state.clone()))
    assert torch.equal(results[0][0], results[1][0]) and torch.equal(results[0][1], results[1][1])
    assert taps == 1 or torch.equal(results[0][2], results[1][2])
    assert torch.equal(results[1][1][4].cpu(), S0[4])


# ---------------------------------------------------------------------------------------
# mLSTM
# ---------------------------------------------------------------------------------------
def mlstm_setup(H, dk, dv, n, seed, dtype, gate_scale=3.0):
    g = torch.Generator().manual_seed(seed)
    width = 2 * H * dk + 2 * H * dv + 2 * H
    width += (-width) % 8
    packed = torch.randn(n, width, generator=g)
    packed[:, 2 * H * (dk + dv):] *= gate_scale            # gate pre-activations of a few units, so that the maximum moves
    t = dict(i_bias=torch.randn(H, generator=g), f_bias=2 + torch.randn(H, generator=g), norm=1 + 0.1 * torch.randn(H * dv, generator=g))
    return packed.to(dtype), {k: v.to(torch.bfloat16) for k, v in t.items()}


def mlstm_plain(packed, t, H, dk, dv, cap, eps, states):
    p = packed.double()
    n = p.shape[0]
    q = (p[:, :H * dk] * dk ** -0.5).view(n, H, dk)
    k = p[:, H * dk:2 * H * dk].view(n, H, dk)
    v = p[:, 2 * H * dk:2 * H * dk + H * dv].view(n, H, dv)
    g0 = 2 * H * dk + H * dv
    gate = torch.sigmoid(p[:, g0:g0 + H * dv])
    li = cap * torch.tanh((p[:, g0 + H * dv:g0 + H * dv + H] + t["i_bias"].double()) / cap)
    lf = torch.nn.functional.logsigmoid(cap * torch.tanh((p[:, g0 + H * dv + H:g0 + H * dv + 2 * H] + t["f_bias"].double()) / cap))
    out = torch.empty(n, H, dv, dtype=torch.float64)
    new = []
    for h in range(H):
        out[:, h], st = plain.mlstm_scan(q[:, h], k[:, h], v[:, h], li[:, h], lf[:, h], states[h])
        new.append(st)
    gated = plain.rms_norm(out, None, eps).reshape(n, H * dv) * t["norm"].double() * gate
    return out, gated, new


def run_mlstm(ops, packed, t, H, dk, dv, cap, eps, state, maxima, q_lens, slots, pad_rows=0, pad_seqs=0):
    n = packed.shape[0]
    tsq, cu, sl = step_ints(q_lens, slots, pad_rows, pad_seqs)
    dev = {k: v.to(DEV) for k, v in t.items()}
    qk = torch.empty(n, H, 2, dk, dtype=torch.float32, device=DEV)
    vals = torch.empty(n, H, dv + 1, dtype=torch.float32, device=DEV)
    gates = torch.empty(n, H, 4, dtype=torch.float32, device=DEV)
    raw = torch.full((n, H, dv + 1), float("nan"), dtype=torch.float32, device=DEV)
    out = torch.empty(n, H * dv, dtype=packed.dtype, device=DEV)
    p = packed.to(DEV)
    ns = len(q_lens) + pad_seqs
    ops.mlstm_prepare(p, H, dk, dv, dev["i_bias"], dev["f_bias"], cap, maxima, tsq, cu, sl, ns, qk, vals, gates)
    ops.state_scan(qk, vals, gates, state, cu, sl, ns, H, H, dk, dv + 1, False, raw)
    ops.state_finish(raw, gates, p, 2 * H * dk + H * dv, dev["norm"], H, dv, eps, tsq, out, shared_weight=False, silu_gate=False,
                     normaliser=True, denom_eps=plain.DENOM_EPS)
    torch.cuda.synchronize()
    return out


def plain_states_of(state, maxima, slot, H, dk, dv):
    s = state[slot].double().cpu()                         # [H, dv + 1, dk]
    return [(s[h, :dv].T.contiguous(), s[h, dv].clone(), maxima[slot, h].double().cpu()) for h in range(H)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, dk, dv, cap", [(2, 16, 20, 10.0), (3, 10, 6, 15.0), (2, 128, 64, 12.0), (1, 8, 12, 4.0), (4, 64, 64, 20.0)])
def test_mlstm_steps_and_states(dtype, H, dk, dv, cap):
    """A first step of four requests (150 tokens in one of them: more than the gate scan takes at a time), a second step
    that continues two of them on their states, with padding."""
    ops = ops_for(dtype)
    eps = 1e-5
    lens1, slots1 = [150, 1, 4, 2], [2, 0, 3, 1]
    lens2, slots2 = [3, 70], [3, 2]
    n1, n2 = sum(lens1), sum(lens2)
    packed, t = mlstm_setup(H, dk, dv, n1 + n2 + 2, seed=H * 10 + dv, dtype=dtype)
    state = torch.zeros(5, H, dv + 1, dk, dtype=torch.float32, device=DEV)
    maxima = torch.zeros(5, H, dtype=torch.float32, device=DEV)
    tol = 1e-4 if dtype == torch.float32 else 1.2e-2
    out1 = run_mlstm(ops, packed[:n1 + 2], t, H, dk, dv, cap, eps, state, maxima, lens1, slots1, pad_rows=2, pad_seqs=1)
    kept, base = {}, 0
    for qn, slot in zip(lens1, slots1):
        _, want, st = mlstm_plain(packed[base:base + qn], t, H, dk, dv, cap, eps, [None] * H)
        close(out1[base:base + qn], want, tol, "first step")
        kept[slot] = st
        for h, (S, nrm, m) in enumerate(plain_states_of(state, maxima, slot, H, dk, dv)):
            close(S, st[h][0], 1e-4, "matrix"); close(nrm, st[h][1], 1e-4, "normaliser")
            assert abs(float(m) - float(st[h][2])) < 1e-5
        base += qn
    assert (out1[base:] == 0).all() and float(state[4].abs().max()) == 0.0
    out2 = run_mlstm(ops, packed[n1 + 2:], t, H, dk, dv, cap, eps, state, maxima, lens2, slots2)
    base = 0
    for qn, slot in zip(lens2, slots2):
        _, want, _ = mlstm_plain(packed[n1 + 2 + base:n1 + 2 + base + qn], t, H, dk, dv, cap, eps, kept[slot])
        close(out2[base:base + qn], want, tol, "second step")
        base += qn


@pytest.mark.parametrize("dtype", DTYPES)
def test_mlstm_one_by_one_against_the_prompt(dtype):
    """100 tokens in one step and one by one: the same bits (the running maximum is taken in the order of the tokens
    however they are cut), and the rows agree with the plain scan."""
    ops = ops_for(dtype)
    H, dk, dv, cap, eps, n = 2, 16, 12, 6.0, 1e-6, 100
    packed, t = mlstm_setup(H, dk, dv, n, seed=3, dtype=dtype)
    outs = []
    for cuts in ([n], [1] * n):
        state = torch.zeros(1, H, dv + 1, dk, dtype=torch.float32, device=DEV)
        maxima = torch.zeros(1, H, dtype=torch.float32, device=DEV)
        rows, base = [], 0
        for c in cuts:
            rows.append(run_mlstm(ops, packed[base:base + c], t, H, dk, dv, cap, eps, state, maxima, [c], [0]).clone())
            base += c
        outs.append(torch.cat(rows))
    assert torch.equal(outs[1], outs[0]), "one by one against whole"
    close(outs[1], mlstm_plain(packed, t, H, dk, dv, cap, eps, [None] * H)[1], 3e-5 if dtype == torch.float32 else 1.2e-2, "plain")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, dk, dv, cap", [(2, 16, 20, 10.0), (3, 10, 6, 15.0), (2, 128, 64, 12.0), (1, 8, 12, 4.0), (4, 64, 64, 20.0),
                                            (1, 200, 255, 9.0)])
def test_mlstm_single_token_kernel(dtype, H, dk, dv, cap):
    """The one kernel for steps of single tokens against the four: the same maxima, outputs and states to rounding (the
    compiler joins a product and a sum of the gates' arithmetic in one of them and not in the other)."""
    ops = ops_for(dtype)
    eps, slots, steps = 1e-5, [1, 3, 0], 4
    n = len(slots) + 2
    results = []
    for fused in (False, True):
        state = torch.zeros(4, H, dv + 1, dk, dtype=torch.float32, device=DEV)
        maxima = torch.zeros(4, H, dtype=torch.float32, device=DEV)
        outs = []
        for step in range(steps):
            packed, t = mlstm_setup(H, dk, dv, n, seed=70 + step, dtype=dtype)
            if not fused:
                outs.append(run_mlstm(ops, packed, t, H, dk, dv, cap, eps, state, maxima, [1] * 3, slots, pad_rows=2, pad_seqs=1).clone())
                continue
            tsq, cu, sl = step_ints([1] * 3, slots, 2, 1)
            dev = {k: v.to(DEV) for k, v in t.items()}
            out = torch.full((n, H * dv), 5.0, dtype=dtype, device=DEV)
            assert ops.state_step(False, packed.to(DEV), H, H, dk, dv, dev["norm"], eps, state, tsq, cu, sl, 4, out,
                                  i_bias=dev["i_bias"], f_bias=dev["f_bias"], cap=cap, max_state=maxima, denom_eps=plain.DENOM_EPS)
            torch.cuda.synchronize()
            outs.append(out.clone())
        results.append((torch.cat(outs), state.clone(), maxima.clone()))
    close(results[1][0], results[0][0].double(), 2e-6 if dtype == torch.float32 else 8e-3, "outputs")
    close(results[1][1], results[0][1].double(), 2e-6, "states")
    close(results[1][2], results[0][2].double(), 2e-6, "maxima")
    assert float(results[1][1][2].abs().max()) == 0.0 and float(results[1][2][2].abs().max()) == 0.0     # slot 2 belongs to nobody


def test_mlstm_first_tokens_use_the_floor_of_the_denominator():
    """With the maximum starting at 0 and a very negative input gate, the first token's normaliser is tiny and the
    denominator is exp(-m) = 1: the output is q.k e^i v, not v."""
    ops = ops_for(torch.float32)
    H, dk, dv, cap = 1, 4, 3, 30.0
    width = 2 * H * dk + 2 * H * dv + 2 * H
    width += (-width) % 8
    packed = torch.zeros(2, width)
    packed[:, :dk] = 1.0; packed[:, dk:2 * dk] = 1.0; packed[:, 2 * dk:2 * dk + dv] = torch.tensor([1.0, 2.0, 3.0])
    packed[:, 2 * dk + 2 * dv] = -6.0                       # input gate
    packed[:, 2 * dk + 2 * dv + 1] = 20.0                   # forget gate: log f ~ 0
    t = dict(i_bias=torch.zeros(H), f_bias=torch.zeros(H), norm=torch.ones(H * dv))
    qk = torch.empty(2, H, 2, dk, device=DEV); vals = torch.empty(2, H, dv + 1, device=DEV); gates = torch.empty(2, H, 4, device=DEV)
    raw = torch.empty(2, H, dv + 1, device=DEV)
    state = torch.zeros(1, H, dv + 1, dk, device=DEV); maxima = torch.zeros(1, H, device=DEV)
    tsq, cu, sl = step_ints([2], [0])
    ops.mlstm_prepare(packed.to(DEV), H, dk, dv, t["i_bias"].to(DEV), t["f_bias"].to(DEV), cap, maxima, tsq, cu, sl, 1, qk, vals, gates)
    ops.state_scan(qk, vals, gates, state, cu, sl, 1, H, H, dk, dv + 1, False, raw)
    torch.cuda.synchronize()
    want, _ = plain.mlstm_scan(torch.full((2, dk), 0.5, dtype=torch.float64), torch.ones(2, dk, dtype=torch.float64),
                               torch.tensor([[1.0, 2.0, 3.0]] * 2, dtype=torch.float64),
                               cap * torch.tanh(torch.tensor([-6.0, -6.0], dtype=torch.float64) / cap),
                               torch.nn.functional.logsigmoid(cap * torch.tanh(torch.tensor([20.0, 20.0], dtype=torch.float64) / cap)))
    g = gates.cpu()
    assert abs(float(maxima[0, 0])) < 1e-6 and abs(float(g[0, 0, 2]) - 1.0) < 1e-6      # m stays 0, the floor is 1
    got = raw[:, 0, :dv].cpu().double() / (torch.maximum(raw[:, 0, dv].cpu().double().abs(), g[:, 0, 2].double()) + plain.DENOM_EPS)[:, None]
    assert float((got - want).abs().max()) < 1e-6 and float(want[0, 0]) < 0.01


# ---------------------------------------------------------------------------------------
# attention over cached latents
# ---------------------------------------------------------------------------------------
def latent_case(H, dn, dr, dv, qr, R, seed, dtype, n, key_gain=1.0):
    g = torch.Generator().manual_seed(seed)
    hid = 48
    w = {"dq": torch.randn(qr, hid, generator=g) / hid ** 0.5, "dq.norm": 1 + 0.1 * torch.randn(qr, generator=g),
         "uq": key_gain * torch.randn(H * (dn + dr), qr, generator=g) / qr ** 0.5,
         "dkv": key_gain * torch.randn(R + dr, hid, generator=g) / hid ** 0.5, "dkv.norm": 1 + 0.1 * torch.randn(R, generator=g),
         "uk": torch.randn(H * dn, R, generator=g) / R ** 0.5, "uv": torch.randn(H * dv, R, generator=g) / R ** 0.5,
         "g": torch.randn(H * dv, hid, generator=g) / hid ** 0.5, "o": torch.eye(H * dv)}
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    h = torch.randn(n, hid, generator=g).to(dtype)
    return w, h


def run_latent(ops, dtype, w, h, m, eps, positions, token_seq, block_table, page_size, pages, base=10000.0):
    """The mixer's kernels between its packed product and its output product, on projections made with torch."""
    H, dn, dr, dv, qr, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
    n = h.shape[0]
    dev = {k: v.to(DEV) for k, v in w.items()}
    hd = h.to(DEV)
    packed_w = torch.cat([dev["dq"], dev["dkv"], dev["g"]]).to(dtype)
    width = packed_w.shape[0] + (-packed_w.shape[0]) % 8
    packed = torch.zeros(n, width, dtype=dtype, device=DEV)
    packed[:, :packed_w.shape[0]] = (hd.float() @ packed_w.float().T).to(dtype)
    table = None
    if dr:
        inv = 1.0 / (base ** (torch.arange(0, dr, 2, dtype=torch.float) / dr))
        table = ops.rope_table(inv.to(DEV), 4096)
    cq = torch.empty(n, qr, dtype=dtype, device=DEV)
    ops.latent_prepare(packed, qr, R, dr, dev["dq.norm"], dev["dkv.norm"], eps, table, positions, token_seq, block_table,
                       page_size, cq, pages)
    q = (cq.float() @ dev["uq"].float().T).to(dtype)
    qa = torch.empty(n, H, R + dr, dtype=torch.float32, device=DEV)
    ops.head_linear(q.view(n, H, dn + dr), dev["uk"].view(H, dn, R).contiguous(), qa, token_seq, tail=dr, table=table, positions=positions)
    mixed = torch.full((n, H, R), float("nan"), dtype=torch.float32, device=DEV)
    ops.attention_latent(qa, mixed, pages, block_table, page_size, positions, token_seq, H, R, dr, m["scale"])
    out = torch.empty(n, H * dv, dtype=dtype, device=DEV)
    gate = packed[:, qr + R + dr:qr + R + dr + H * dv]
    ops.head_linear(mixed, dev["uv"].view(H, dv, R).transpose(1, 2).contiguous(), out, token_seq, gate=gate)
    torch.cuda.synchronize()
    return packed, cq, q, out


LATENT_SIZES = [(4, 16, 8, 12, 24, 32), (3, 10, 4, 6, 12, 20), (8, 64, 32, 64, 96, 128), (1, 12, 0, 8, 8, 16), (5, 24, 16, 24, 40, 48),
                (7, 8, 8, 16, 16, 24)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, dn, dr, dv, qr, R", LATENT_SIZES)
@pytest.mark.parametrize("page_size", [16, 4])
def test_latent_attention_prompt_and_continuation(dtype, H, dn, dr, dv, qr, R, page_size):
    """A prompt of 150 tokens on scattered pages (every position against the plain mixer), then a portion of 9 tokens and
    single tokens behind it, beside another request in the same steps; padding rows; NaN in every page nobody owns."""
    ops = ops_for(dtype)
    eps = 1e-5
    m = {"heads": H, "dim": dn, "rot_dim": dr, "vdim": dv, "q_rank": qr, "kv_rank": R, "scale": (dn + dr) ** -0.5,
         "rot": {"dims": dr, "base": 10000.0}}
    n_a, n_b = 163, 40
    w, h = latent_case(H, dn, dr, dv, qr, R, seed=H + dn, dtype=dtype, n=n_a + n_b, key_gain=2.0)
    ha, hb = h[:n_a], h[n_a:]
    w64 = {"x." + k: v.double() for k, v in w.items()}
    want_a = plain.latent_attention_mixer(ha.double(), w64, "x.", m, eps, rnd=None)[0]
    want_b = plain.latent_attention_mixer(hb.double(), w64, "x.", m, eps, rnd=None)[0]
    tol = 3e-5 if dtype == torch.float32 else 5e-2          # (single rows of a steep softmax, relative to the row's own largest value)
    n_pages = 64 if page_size == 16 else 256
    pages = torch.full((n_pages, page_size, R + dr), float("nan"), dtype=dtype, device=DEV)
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(5)).tolist()
    width = -(-n_a // page_size)
    bt = torch.full((2, width), -1, dtype=torch.int32)
    bt[0, :width] = torch.tensor(perm[:width])
    wb = -(-n_b // page_size)
    bt[1, :wb] = torch.tensor(perm[width:width + wb])
    bt = bt.to(DEV)
    # step 1: request a's first 150 tokens and request b's first 30, two padding rows
    pos = i32(list(range(150)) + list(range(30)) + [0, 0])
    tsq = i32([0] * 150 + [1] * 30 + [-1, -1])
    x = torch.cat([ha[:150], hb[:30], torch.zeros(2, h.shape[1], dtype=dtype)])
    out = run_latent(ops, dtype, w, x, m, eps, pos, tsq, bt, page_size, pages)[3]
    close(out[:150], want_a[:150], tol, "prompt a"); close(out[150:180], want_b[:30], tol, "prompt b")
    assert (out[180:] == 0).all()
    # step 2: nine more tokens of a beside one of b
    pos = i32(list(range(150, 159)) + [30]); tsq = i32([0] * 9 + [1])
    out = run_latent(ops, dtype, w, torch.cat([ha[150:159], hb[30:31]]), m, eps, pos, tsq, bt, page_size, pages)[3]
    close(out[:9], want_a[150:159], tol, "portion of a"); close(out[9:], want_b[30:31], tol, "token of b")
    # steps of single tokens
    for t in range(4):
        pos = i32([159 + t, 31 + t]); tsq = i32([0, 1])
        out = run_latent(ops, dtype, w, torch.stack([ha[159 + t], hb[31 + t]]), m, eps, pos, tsq, bt, page_size, pages)[3]
        close(out[:1], want_a[159 + t:160 + t], tol, "decoded a"); close(out[1:], want_b[31 + t:32 + t], tol, "decoded b")


@pytest.mark.parametrize("dtype", DTYPES)
def test_latent_attention_finds_a_far_key(dtype):
    """Among 700 keys one, far back and at a page's last slot, is made to match the last query's rotated and plain
    parts strongly: the output must be that token's value (and not its neighbours')."""
    ops = ops_for(dtype)
    H, R, dr, page_size, n, far = 2, 16, 8, 16, 700, 127
    g = torch.Generator().manual_seed(3)
    rows = torch.randn(n, R + dr, generator=g)
    rows[far, :R] = 0.0
    rows[far, 3] = 6.0                                      # a latent no other token resembles
    rows[far, R:] = 0.0
    rows[far, R] = 5.0
    pages = torch.full((64, page_size, R + dr), float("nan"), dtype=dtype, device=DEV)
    perm = torch.randperm(64, generator=g)[:-(-n // page_size)]
    for p in range(n):
        pages[perm[p // page_size], p % page_size] = rows[p].to(dtype).to(DEV)
    qa = torch.zeros(1, H, R + dr, device=DEV)
    qa[0, 0, 3] = 4.0                                       # head 0 asks for that latent
    qa[0, 1] = torch.randn(R + dr, generator=g).to(DEV) * 0.1
    out = torch.empty(1, H, R, device=DEV)
    ops.attention_latent(qa, out, pages, perm.to(torch.int32).view(1, -1).to(DEV), page_size, i32([n - 1]), i32([0]), H, R, dr, 1.0)
    torch.cuda.synchronize()
    stored = pages.float().cpu()
    look = torch.stack([stored[perm[p // page_size], p % page_size] for p in range(n)]).double()
    for head in range(H):
        wts = torch.softmax(look @ qa[0, head].double().cpu(), 0)
        close(out[0, head], wts @ look[:, :R], 2e-5, f"head {head}")
    assert float(out[0, 0, 3]) > 5.9 and abs(float(out[0, 0, 0])) < 0.05
    # the same query one position before the far key does not see it
    ops.attention_latent(qa, out, pages, perm.to(torch.int32).view(1, -1).to(DEV), page_size, i32([far - 1]), i32([0]), H, R, dr, 1.0)
    torch.cuda.synchronize()
    assert float(out[0, 0, 3]) < 3.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, R, dr", [(16, 64, 16), (5, 32, 8), (20, 128, 32), (1, 16, 0), (3, 24, 8)])
def test_latent_attention_single_token_kernel(dtype, H, R, dr):
    """Steps of single tokens take a kernel that deals a row's keys out in runs of 256 positions and joins them: rows
    whose contexts end just inside, at and just behind a run's border, one position long, and 900 long, with a padding
    row, against the general kernel and against the softmax written out."""
    from minivllm_amd.engine.step import AttentionPlan
    ops = ops_for(dtype)
    page_size, n_pages = 16, 64
    ctx = [255, 256, 257, 1, 900, 512]
    g = torch.Generator().manual_seed(H)
    pages = torch.randn(n_pages * len(ctx), page_size, R + dr, generator=g).to(dtype).to(DEV)
    width = -(-max(ctx) // page_size)
    bt = torch.full((len(ctx), width), -1, dtype=torch.int32)
    perm = torch.randperm(n_pages * len(ctx), generator=g)
    used = 0
    for s, c in enumerate(ctx):
        need = -(-c // page_size)
        bt[s, :need] = perm[used:used + need].to(torch.int32)
        used += need
    bt = bt.to(DEV)
    n = len(ctx) + 1
    qa = (1.5 * torch.randn(n, H, R + dr, generator=g)).to(DEV)
    pos = i32([c - 1 for c in ctx] + [0]); tsq = i32(list(range(len(ctx))) + [-1])
    plan = AttentionPlan(decode_only=True, max_q_len=1, max_context_len=1024, n_seqs=len(ctx))
    fast = torch.full((n, H, R), float("nan"), device=DEV)
    slow = torch.full((n, H, R), float("nan"), device=DEV)
    ops.ledger = []
    ops.attention_latent(qa, fast, pages, bt, page_size, pos, tsq, H, R, dr, 0.2, plan=plan)
    taken = [e[0] for e in ops.ledger]
    ops.ledger = None
    ops.attention_latent(qa, slow, pages, bt, page_size, pos, tsq, H, R, dr, 0.2)
    torch.cuda.synchronize()
    assert taken == ["mv_attention_latent_split"], taken
    assert (fast[-1] == 0).all()
    stored = pages.float().cpu().double()
    for s, c in enumerate(ctx):
        rows = torch.stack([stored[bt[s, p // page_size].item(), p % page_size] for p in range(c)])
        for h in range(H):
            w = torch.softmax(rows @ qa[s, h].double().cpu() * 0.2, 0)
            close(fast[s, h], w @ rows[:, :R], 3e-5, f"context {c} head {h}")
    close(fast[:-1], slow[:-1].double(), 3e-5, "against the general kernel")


@pytest.mark.parametrize("H, R, dr", [(16, 256, 64), (5, 64, 32), (20, 128, 32), (8, 128, 64)])
@pytest.mark.parametrize("page_size", [16, 8])
def test_latent_attention_mfma_kernel(H, R, dr, page_size):
    """bfloat16 steps with prompt portions take an MFMA kernel (a row's 16 heads are the rows of its first operand, the
    values come from the slot-contiguous pages): a prompt of 100 tokens, a portion that starts in the middle of a block of
    32 keys, single rows at positions 0, 31, 32, 33 and 700, a padding row; NaN in every slot nobody wrote. Against the
    softmax written out on the stored rows."""
    from minivllm_amd.engine.step import AttentionPlan
    dtype = torch.bfloat16
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(H + R)
    ctx = [100, 77, 1, 32, 33, 34, 701]                    # contexts of the seven requests after the step
    qlens = [100, 20, 1, 1, 1, 1, 1]
    n_pages = sum(-(-c // page_size) for c in ctx) + 3
    pages = torch.full((n_pages, page_size, R + dr), float("nan"), dtype=dtype, device=DEV)
    pages_t = torch.full((n_pages, R, page_size), float("nan"), dtype=dtype, device=DEV)
    perm = torch.randperm(n_pages, generator=g).tolist()
    width = -(-max(ctx) // page_size)
    bt = torch.full((len(ctx), width), -1, dtype=torch.int32)
    rows, used = [], 0
    for s_, c in enumerate(ctx):
        need = -(-c // page_size)
        bt[s_, :need] = torch.tensor(perm[used:used + need], dtype=torch.int32)
        used += need
        data = torch.randn(c, R + dr, generator=g).to(dtype)
        rows.append(data)
        for p_ in range(c):
            pages[bt[s_, p_ // page_size], p_ % page_size] = data[p_].to(DEV)
            pages_t[bt[s_, p_ // page_size], :, p_ % page_size] = data[p_, :R].to(DEV)
    pos, tsq = [], []
    for s_, (c, ql) in enumerate(zip(ctx, qlens)):
        pos += list(range(c - ql, c)); tsq += [s_] * ql
    pos.append(0); tsq.append(-1)
    n = len(pos)
    qa = (1.2 * torch.randn(n, H, R + dr, generator=g)).to(DEV)
    plan = AttentionPlan(decode_only=False, max_q_len=100, max_context_len=1024, n_seqs=len(ctx))
    got = torch.full((n, H, R), float("nan"), device=DEV)
    ops.ledger = []
    ops.attention_latent(qa, got, pages, bt.to(DEV), page_size, i32(pos), i32(tsq), H, R, dr, 0.15, plan=plan, pages_t=pages_t)
    torch.cuda.synchronize()
    assert [e[0] for e in ops.ledger] == ["mv_attention_latent_mfma"]
    ops.ledger = None
    bad = (~torch.isfinite(got)).nonzero()
    assert bad.numel() == 0, f"non-finite outputs at (row, head, channel) {bad[:8].tolist()} ... of rows at positions {sorted({pos[i] for i in bad[:, 0].tolist()})[:12]}"
    assert (got[-1] == 0).all()
    worst = 0.0
    for t in range(n - 1):
        look = rows[tsq[t]][:pos[t] + 1].double()
        for h in range(H):
            w = torch.softmax(look @ qa[t, h].double().cpu() * 0.15, 0)
            want = w @ look[:, :R]
            worst = max(worst, float((got[t, h].double().cpu() - want).abs().max() / want.abs().max()))
    assert worst < 2e-2, worst


@pytest.mark.parametrize("H, IN, OUT, tail, n", [(16, 128, 256, 64, 300), (3, 32, 40, 8, 70), (5, 64, 128, 0, 130), (2, 96, 17, 4, 65)])
def test_per_head_maps_mfma_against_the_general_kernel(H, IN, OUT, tail, n):
    """bfloat16 steps of more than 64 rows take an MFMA kernel for the per-head maps: both directions (queries into latent
    space with the rotated tail; weighted latents into values with the gate), padding rows, against the general kernel
    and against the sums written out."""
    dtype = torch.bfloat16
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(IN + OUT)
    w = (torch.randn(H, IN, OUT, generator=g) / IN ** 0.5).to(dtype).to(DEV)
    w_rows = w.transpose(1, 2).contiguous()
    tsq = i32([0] * (n - 2) + [-1, -1])
    pos = i32(list(range(n - 2)) + [0, 0])
    table = ops.rope_table((1.0 / (10000.0 ** (torch.arange(0, tail, 2, dtype=torch.float) / tail))).to(DEV), 1024) if tail else None
    # queries -> latent space
    x = torch.randn(n, H, IN + tail, generator=g).to(dtype).to(DEV)
    outs = []
    for rows in (w_rows, None):
        out = torch.full((n, H, OUT + tail), float("nan"), device=DEV)
        ops.ledger = []
        ops.head_linear(x, w, out, tsq, tail=tail, table=table, positions=pos, w_rows=rows)
        torch.cuda.synchronize()
        assert [e[0] for e in ops.ledger] == ["mv_head_linear_mfma" if rows is not None else "mv_head_linear"]
        ops.ledger = None
        outs.append(out)
    want = torch.einsum("thi,hio->tho", x[..., :IN].double(), w.double())
    close(outs[0][:-2, :, :OUT], want[:-2], 1e-5, "queries into latent space")
    close(outs[0][:-2], outs[1][:-2].double(), 1e-5, "against the general kernel, tail included")
    assert (outs[0][-2:] == 0).all()
    # weighted latents -> values, gated
    lat = torch.randn(n, H, IN, generator=g).to(DEV)
    gate = torch.randn(n, H * OUT, generator=g).to(dtype).to(DEV)
    outs = []
    for rows in (w_rows, None):
        out = torch.full((n, H * OUT), float("nan"), dtype=dtype, device=DEV)
        ops.head_linear(lat, w, out, tsq, gate=gate, w_rows=rows)
        torch.cuda.synchronize()
        outs.append(out)
    want = (torch.einsum("thi,hio->tho", lat.double(), w.double()).reshape(n, H * OUT) * torch.sigmoid(gate.double()))
    close(outs[0][:-2], want[:-2], 1.2e-2, "weighted latents into values")
    close(outs[0][:-2], outs[1][:-2].double(), 1.2e-2, "against the general kernel")
    assert (outs[0][-2:] == 0).all()


# ---------------------------------------------------------------------------------------
# router and experts
# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("E, groups, keep, top", [(10, 5, 3, 3), (6, 1, 1, 2), (6, 3, 2, 2), (4, 1, 1, 4), (64, 8, 4, 8), (20, 4, 3, 4),
                                                   (7, 7, 2, 2), (130, 2, 1, 6)])
def test_router_against_the_plain_choice(E, groups, keep, top):
    ops = ops_for(torch.float32)
    g = torch.Generator().manual_seed(E)
    n, hid = 200, 24
    h = torch.randn(n, hid, generator=g, dtype=torch.float64)
    router = 2.0 * torch.randn(E, hid, generator=g, dtype=torch.float64) / hid ** 0.5
    correction = (0.3 * torch.randn(E, generator=g)).to(torch.bfloat16)
    logits = (h @ router.T).float().to(DEV)
    dense = torch.full((n, E), 7.0, device=DEV); ids = torch.empty(n, top, dtype=torch.int32, device=DEV)
    weights = torch.empty(n, top, device=DEV)
    ops.moe_route(logits, correction.to(DEV), groups, keep, top, plain.WEIGHT_SUM_EPS, dense, ids, weights)
    torch.cuda.synchronize()
    score = torch.softmax(logits.double().cpu(), -1)
    chosen, want = plain.route(torch.eye(E, dtype=torch.float64)[:0], None, None, 0, 1, 1) if False else (None, None)
    choice = score + correction.double()
    per = E // groups
    best = choice.view(n, groups, per).max(-1).values
    kept = torch.zeros(n, groups, dtype=torch.bool).scatter_(1, best.topk(keep, -1).indices, True)
    choice = choice.masked_fill(~kept.repeat_interleave(per, 1), float("-inf"))
    chosen = choice.topk(top, -1).indices
    picked = score.gather(1, chosen)
    want = picked / (picked.sum(-1, keepdim=True) + plain.WEIGHT_SUM_EPS)
    assert torch.equal(ids.cpu().long(), chosen), "chosen experts, in the order of choice"
    assert float((weights.cpu().double() - want).abs().max()) < 1e-6
    full = torch.zeros(n, E, dtype=torch.float64).scatter_(1, chosen, want)
    assert float((dense.cpu().double() - full).abs().max()) < 1e-6


def test_router_choice_can_be_negative_and_other_groups_stay_out():
    """A correction that makes every choice of the kept groups negative and leaves an expert of a dropped group at zero:
    the dropped group's expert must still not be chosen."""
    ops = ops_for(torch.float32)
    E, groups, keep, top = 6, 3, 1, 2
    logits = torch.zeros(1, E, device=DEV)                  # scores 1/6 each
    correction = torch.tensor([-1.0, -0.9, -0.5, -3.0, -2.0, -0.95]).to(DEV)    # group worths: -0.73, -0.33, -0.78
    dense = torch.empty(1, E, device=DEV); ids = torch.empty(1, top, dtype=torch.int32, device=DEV); weights = torch.empty(1, top, device=DEV)
    ops.moe_route(logits, correction, groups, keep, top, 1e-20, dense, ids, weights)
    torch.cuda.synchronize()
    assert ids.cpu().tolist() == [[2, 3]] and torch.allclose(weights.cpu(), torch.tensor([[0.5, 0.5]]))


@pytest.mark.parametrize("dtype", DTYPES)
def test_routed_experts_against_the_plain_mixture(dtype):
    """The feed-forward part itself, with identity experts: a tiny runtime, the part built from tensors by name."""
    from minivllm_amd.parts.base import Runtime, Workspace
    from minivllm_amd.parts.moe import RoutedExperts, RoutedExpertsSpec
    ops = ops_for(dtype)
    hid, F, E, I, top, groups, keep, n = 40, 24, 5, 3, 3, 4, 3, 70
    g = torch.Generator().manual_seed(11)
    w = {"router": 3.0 * torch.randn(E + I, hid, generator=g) / hid ** 0.5, "correction": 0.05 * torch.randn(E + I, generator=g)}
    for e in range(E):
        w[f"e{e}.gate"] = torch.randn(F, hid, generator=g) / hid ** 0.5
        w[f"e{e}.up"] = torch.randn(F, hid, generator=g) / hid ** 0.5
        w[f"e{e}.down"] = torch.randn(hid, F, generator=g) / F ** 0.5
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    spec = RoutedExpertsSpec(hidden_size=hid, expert_size=F, num_experts=E, identity_experts=I, top=top, groups=groups,
                             keep_groups=keep, correction=True)
    tensors = {"router": w["router"].to(DEV), "correction": w["correction"].to(DEV)}
    for e in range(E):
        for k in ("gate", "up", "down"):
            tensors[f"{k}.{e}"] = w[f"e{e}.{k}"].to(DEV)
    rt = Runtime(device=torch.device(DEV), dtype=dtype, ops=ops, workspace=Workspace(torch.device(DEV)), max_positions=64)
    part = RoutedExperts(spec, tensors, rt)
    x = torch.randn(n, hid, generator=g).to(dtype)
    got = part.forward(x.to(DEV), None)
    torch.cuda.synchronize()
    mlp = {"kind": "moe", "expert": {"ff": F}, "router": {"experts": E, "identity": I, "top": top, "groups": {"count": groups, "keep": keep}}}
    want = plain.mixture(x.double(), {"m." + k: v.double() for k, v in w.items()}, "m.", mlp)
    chosen, _ = plain.route(x.double(), w["router"].double(), w["correction"].double(), top, groups, keep)
    assert (chosen >= E).any() and (chosen < E).any()       # identity experts and real ones were both used
    close(got, want, 3e-5 if dtype == torch.float32 else 2e-2, "mixture")


@pytest.mark.parametrize("n", [1, 7, 70, 300])
@pytest.mark.parametrize("hid, F, E, I, top, groups, keep", [(64, 32, 5, 3, 3, 4, 3), (96, 64, 16, 0, 4, 4, 2), (32, 160, 3, 1, 4, 1, 1)])
def test_grouped_experts_against_all_experts(n, hid, F, E, I, top, groups, keep):
    """bfloat16 with sizes the MFMA kernels serve: the products over the chosen pairs only give what computing every
    expert and zeroing the others gives, and what the plain mixture gives."""
    from minivllm_amd.parts.base import Runtime, Workspace
    from minivllm_amd.parts.moe import RoutedExperts, RoutedExpertsSpec
    dtype = torch.bfloat16
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(n + E)
    w = {"router": 3.0 * torch.randn(E + I, hid, generator=g) / hid ** 0.5, "correction": 0.05 * torch.randn(E + I, generator=g)}
    for e in range(E):
        w[f"e{e}.gate"] = torch.randn(F, hid, generator=g) / hid ** 0.5
        w[f"e{e}.up"] = torch.randn(F, hid, generator=g) / hid ** 0.5
        w[f"e{e}.down"] = torch.randn(hid, F, generator=g) / F ** 0.5
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    tensors = {"router": w["router"].to(DEV), "correction": w["correction"].to(DEV)}
    for e in range(E):
        for k in ("gate", "up", "down"):
            tensors[f"{k}.{e}"] = w[f"e{e}.{k}"].to(DEV)
    x = torch.randn(n, hid, generator=g).to(dtype)
    outs = {}
    for grouped in (True, False):
        spec = RoutedExpertsSpec(hidden_size=hid, expert_size=F, num_experts=E, identity_experts=I, top=top, groups=groups,
                                 keep_groups=keep, correction=True, grouped=grouped, grouped_max_rows=1e9, grouped_min_weight=0)
        rt = Runtime(device=torch.device(DEV), dtype=dtype, ops=ops, workspace=Workspace(torch.device(DEV)), max_positions=64)
        ops.ledger = []
        outs[grouped] = RoutedExperts(spec, tensors, rt).forward(x.to(DEV), None).clone()
        torch.cuda.synchronize()
        assert ("mv_moe_grouped" in [e[0] for e in ops.ledger]) == grouped
        ops.ledger = None
    mlp = {"kind": "moe", "expert": {"ff": F}, "router": {"experts": E, "identity": I, "top": top, "groups": {"count": groups, "keep": keep}}}
    want = plain.mixture(x.double(), {"m." + k: v.double() for k, v in w.items()}, "m.", mlp)
    close(outs[True], want, 2e-2, "chosen pairs only against the plain mixture")
    close(outs[True], outs[False].double(), 2e-2, "chosen pairs only against all experts")


def test_scaled_logits():
    ops = ops_for(torch.float32)
    x = torch.randn(5, 33, device=DEV)
    want = x[:, :30] * 0.3
    view = x[:, :30]
    ops.scale_f32(view, 0.3)
    torch.cuda.synchronize()
    assert torch.allclose(view, want) and float(x[:, 30:].abs().min()) > 0
