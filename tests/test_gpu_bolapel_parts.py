"""Each mechanism of Bolapel alone, the engine's kernels against the plain functions: token shift,
the delta rule (prepare, scan, finish; any mix of requests; state carried, slots used again; long
decoding), sigmoid attention over pages (chunks, windows, key/value sizes, far keys, page and chunk
edges), the fused norms around a sublayer and the logit cap."""
import math

import numpy as np
import pytest
import torch

from plain import bolapel_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def ops_for(dtype):
    from minivllm_amd.kernels.ops import Ops
    return Ops(dtype)


def i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


def step_ints(q_lens, slots, pad_rows=0, pad_seqs=0):
    """token_seq, cu_seqlens, state_slots of a step with these requests (and padding at the end)."""
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
@pytest.mark.parametrize("dtype", DTYPES)
def test_token_shift(dtype):
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(0)
    w, q_lens, slots = 40, [5, 1, 3, 2], [2, 0, 3, 1]
    n = sum(q_lens) + 2
    h = torch.randn(n, w, generator=g).to(dtype)
    mix = torch.rand(w, generator=g).to(torch.bfloat16)
    state = torch.randn(5, w, generator=g).to(dtype)
    tsq, cu, sl = step_ints(q_lens, slots, pad_rows=2, pad_seqs=1)
    out = torch.full((n, w), 7.0, dtype=dtype, device=DEV)
    dstate = state.to(DEV).clone()
    ops.token_shift(h.to(DEV), mix.to(DEV), dstate, tsq, cu, sl, out)
    torch.cuda.synchronize()
    base = 0
    for q, slot in zip(q_lens, slots):
        want = plain.token_shift(h[base:base + q].double(), mix.double(), before=state[slot].double())
        close(out[base:base + q], want, 1e-6 if dtype == torch.float32 else 8e-3, "shifted rows")
        assert torch.equal(dstate[slot].cpu(), h[base + q - 1])          # the state is a copy of the last row
        base += q
    assert torch.equal(dstate[4].cpu(), state[4])                        # a slot nobody holds is not touched
    assert (out[base:] == 0).all()                                       # padding rows


# ---------------------------------------------------------------------------------------
def delta_inputs(n, H, D, rank, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    inner = H * D
    pad = (-rank) % 8
    packed = torch.randn(n, 5 * inner + rank + pad, generator=g)
    packed[:, inner:2 * inner] *= 1.5                                    # keys
    t = dict(w2=torch.randn(inner, rank, generator=g) / rank ** 0.5, w0=torch.randn(inner, generator=g),
             a_bias=torch.randn(inner, generator=g), norm=1 + 0.1 * torch.randn(inner, generator=g))
    return packed.to(dtype), {k: v.to(torch.bfloat16) for k, v in t.items()}


def delta_plain(packed, t, H, D, rank, eps, states):
    """What the three kernels should give for one request: (raw, gated, final states) in float64."""
    n, inner = packed.shape[0], H * D
    p = packed.double()
    blocks = [p[:, i * inner:(i + 1) * inner].view(n, H, D) for i in range(5)]
    r, k, v, gte, a = blocks
    lora = torch.tanh(p[:, 5 * inner:5 * inner + rank]) @ t["w2"].double().T + t["w0"].double()
    decay = torch.exp(-plain.DECAY_RATE * torch.sigmoid(lora)).view(n, H, D)
    rate = torch.sigmoid(a + t["a_bias"].double().view(H, D))
    raw = torch.empty(n, H, D, dtype=torch.float64)
    final = []
    for j in range(H):
        raw[:, j], S = plain.delta_rule_scan(r[:, j], k[:, j], v[:, j], decay[:, j], rate[:, j], state=states[j].double())
        final.append(S)
    gated = plain.rms_norm(raw, None, eps).reshape(n, inner) * t["norm"].double() * torch.sigmoid(gte.reshape(n, inner))
    return raw.reshape(n, inner), gated, torch.stack(final)


def run_delta(ops, packed, t, H, D, rank, eps, state, q_lens, slots, pad_rows=0, pad_seqs=0, fused=False):
    """``state`` [slots, H, D, D] holds each head's matrix column by column (the transpose of the plain S).
    ``fused``: the one kernel for steps of single tokens (every q_len must be 1); it returns no raw rows."""
    n, inner = packed.shape[0], H * D
    tsq, cu, sl = step_ints(q_lens, slots, pad_rows, pad_seqs)
    dev = {k: v.to(DEV) for k, v in t.items()}
    w2t = dev["w2"].t().contiguous()
    out = torch.empty(n, inner, dtype=packed.dtype, device=DEV)
    p = packed.to(DEV)
    if fused:
        ops.delta_step(p, H, D, rank, w2t, dev["w0"], dev["a_bias"], dev["norm"], plain.DECAY_RATE, plain.DELTA_KEY_EPS,
                       eps, state, tsq, sl, out)
        torch.cuda.synchronize()
        return None, out
    coef = torch.empty(n, H, 5, D, dtype=torch.float32, device=DEV)
    raw = torch.zeros(n, inner, dtype=torch.float32, device=DEV)
    ops.delta_prepare(p, H, D, rank, w2t, dev["w0"], dev["a_bias"], plain.DECAY_RATE, plain.DELTA_KEY_EPS, coef)
    ops.delta_scan(p, coef, state, cu, sl, len(q_lens) + pad_seqs, H, D, raw)
    ops.delta_finish(raw, p, dev["norm"], H, D, eps, out)
    torch.cuda.synchronize()
    return raw, out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, D, rank", [(2, 16, 6), (3, 24, 5), (1, 40, 3), (4, 64, 32), (2, 128, 16), (1, 200, 4),
                                        (5, 8, 1), (2, 30, 7)])
def test_delta_rule_mixed_step(dtype, H, D, rank):
    """Requests of 37, 1, 18 and 2 rows in one step, each on a state that earlier tokens left, in slots
    out of order; padding rows and a padding sequence behind them."""
    ops = ops_for(dtype)
    q_lens, slots, eps = [37, 1, 18, 2], [3, 0, 4, 1], 1e-5
    n = sum(q_lens)
    packed, t = delta_inputs(n + 3, H, D, rank, seed=H * 1000 + D, dtype=dtype)
    g = torch.Generator().manual_seed(5)
    state = torch.randn(6, H, D, D, generator=g) * 0.3
    dstate = state.transpose(-1, -2).contiguous().to(DEV)
    raw, out = run_delta(ops, packed, t, H, D, rank, eps, dstate, q_lens, slots, pad_rows=3, pad_seqs=2)
    base = 0
    for q, slot in zip(q_lens, slots):
        want_raw, want, final = delta_plain(packed[base:base + q], t, H, D, rank, eps, state[slot])
        close(raw[base:base + q], want_raw, 2e-5, f"scan of request in slot {slot}")
        close(out[base:base + q], want, 2e-5 if dtype == torch.float32 else 8e-3, "finished rows")
        close(dstate[slot].transpose(-1, -2), final, 2e-5, "state after the step")
        base += q
    for slot in (2, 5):
        assert torch.equal(dstate[slot].transpose(-1, -2).cpu(), state[slot])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, D, rank", [(2, 16, 6), (3, 24, 5), (1, 40, 3), (4, 64, 32), (2, 128, 16), (1, 200, 4),
                                        (5, 8, 1), (2, 30, 7)])
def test_delta_rule_step_of_single_tokens(dtype, H, D, rank):
    """Five requests with one token each (slots out of order, a padding row between them): the one fused
    kernel against the plain recurrence, and against the three kernels it stands for."""
    ops = ops_for(dtype)
    slots, eps = [3, 0, 4, 1, 5], 1e-5
    packed, t = delta_inputs(7, H, D, rank, seed=H * 77 + D, dtype=dtype)
    g = torch.Generator().manual_seed(6)
    state = torch.randn(7, H, D, D, generator=g) * 0.3
    fused_state = state.transpose(-1, -2).contiguous().to(DEV)
    three_state = fused_state.clone()
    _, fused = run_delta(ops, packed, t, H, D, rank, eps, fused_state, [1] * 5, slots, pad_rows=2, fused=True)
    _, three = run_delta(ops, packed, t, H, D, rank, eps, three_state, [1] * 5, slots, pad_rows=2)
    for row, slot in enumerate(slots):
        _, want, final = delta_plain(packed[row:row + 1], t, H, D, rank, eps, state[slot])
        close(fused[row:row + 1], want, 2e-5 if dtype == torch.float32 else 8e-3, f"row {row}")
        close(fused_state[slot].transpose(-1, -2), final, 2e-5, "state after the step")
    close(fused[:5], three[:5].double(), 1e-6 if dtype == torch.float32 else 8e-3, "fused against three kernels")
    close(fused_state, three_state.double(), 1e-6, "states, fused against three kernels")
    assert (fused[5:] == 0).all()
    for slot in (2, 6):
        assert torch.equal(fused_state[slot].transpose(-1, -2).cpu(), state[slot])


def test_delta_rule_token_by_token_is_the_prompt_bit_for_bit():
    """300 tokens in one step, in portions of 2 to 64, and one by one through the state: the same
    additions in the same order, so the same bits; a slot is used again after a zeroed start."""
    dtype, H, D, rank, eps = torch.bfloat16, 2, 64, 8, 1e-5
    ops = ops_for(dtype)
    n = 300
    packed, t = delta_inputs(n, H, D, rank, seed=11, dtype=dtype)
    results = []
    for cuts in ([n], [2, 64, 3, 31, 64, 64, 2, 70], [1] * n):
        state = torch.zeros(3, H, D, D, dtype=torch.float32, device=DEV)
        state[1].fill_(9.0)                                  # what a request before left in the slot
        state[1].zero_()                                     # ... is cleared when the next one starts at 0
        rows, base = [], 0
        for q in cuts:
            raw, out = run_delta(ops, packed[base:base + q], t, H, D, rank, eps, state, [q], [1])
            rows.append(out.clone())
            base += q
        results.append((torch.cat(rows), state[1].clone()))
    for rows, st in results[1:]:
        assert torch.equal(rows, results[0][0]) and torch.equal(st, results[0][1])
    want_raw, want, final = delta_plain(packed, t, H, D, rank, eps, torch.zeros(H, D, D))
    close(results[0][0], want, 8e-3, "300 tokens")
    close(results[0][1].transpose(-1, -2), final, 2e-5, "state after 300 tokens")


def test_delta_rule_full_removal_replaces_a_key():
    """rate 1 (a large bias) and decay 1 (a very negative offset): writing a key twice leaves the second value."""
    dtype, H, D, rank = torch.float32, 1, 16, 2
    ops = ops_for(dtype)
    inner = H * D
    packed = torch.zeros(2, 5 * inner + 8)
    packed[:, inner + 3] = 2.0                               # the key: 2 e_3 both times
    packed[:, 0 * inner + 3] = 1.0                           # r = e_3
    packed[0, 2 * inner:3 * inner] = 1.0                     # values 1, then 5
    packed[1, 2 * inner:3 * inner] = 5.0
    t = dict(w2=torch.zeros(inner, rank), w0=torch.full((inner,), -40.0), a_bias=torch.full((inner,), 40.0),
             norm=torch.ones(inner))
    state = torch.zeros(1, H, D, D, device=DEV)
    raw, _ = run_delta(ops, packed, t, H, D, rank, 1e-5, state, [2], [0])
    close(raw[0], torch.full((inner,), 2.0), 1e-5)           # S = k v^T, o = S^T r = 2 * 1
    close(raw[1], torch.full((inner,), 10.0), 1e-5)          # the first value is gone: 2 * 5


# ---------------------------------------------------------------------------------------
def paged(k, v, page_size, n_pages, seed):
    """k [n, G, D], v [n, G, Dv] into pages handed out in a shuffled order; pages nobody owns hold NaN."""
    n, G, D = k.shape
    Dv = v.shape[2]
    need = -(-n // page_size)
    ids = np.random.default_rng(seed).permutation(n_pages)[:need]
    kp = torch.full((n_pages, G, page_size, D), float("nan"), dtype=k.dtype)
    vp = torch.full((n_pages, G, Dv, page_size), float("nan"), dtype=v.dtype)
    for j in range(n):
        kp[ids[j // page_size], :, j % page_size, :] = k[j]
        vp[ids[j // page_size], :, :, j % page_size] = v[j]
    # slots behind the last token of the last page are never read: leave NaN there
    return kp.to(DEV), vp.to(DEV), [int(i) for i in ids]


def run_attention(ops, q, k, v, positions, scale, chunk, window, bias, gate, page_size=4, seed=0, with_plan=False,
                  variant=None):
    """``with_plan``: the step is described to the kernels' front end as the engine does (one request of
    these rows, in row 1 of the block table), which lets it pick the MFMA kernel where the sizes allow."""
    from minivllm_amd.engine.step import AttentionPlan
    n_q, H, D = q.shape
    plan = None
    if with_plan:
        plan = AttentionPlan(decode_only=n_q == 1, max_q_len=n_q, max_context_len=max(positions) + 1, n_seqs=2,
                             q_lens=[0, n_q], cu_seqlens=i32([0, 0, n_q]), prefill_variant=variant)
    Dv = v.shape[2]
    kp, vp, ids = paged(k, v, page_size, 2 * (-(-k.shape[0] // page_size)) + 3, seed)
    table = torch.full((2, len(ids) + 2), -1, dtype=torch.int32)
    table[1, :len(ids)] = torch.tensor(ids, dtype=torch.int32)          # the request is row 1 of the table
    out = torch.empty(n_q, H * Dv, dtype=q.dtype, device=DEV)
    ops.attention_sigmoid(q.reshape(n_q, H * D).to(DEV), out, kp, vp, table.to(DEV), page_size, i32(positions),
                          i32([1] * n_q), H, k.shape[1], D, Dv, scale, chunk, window,
                          None if bias is None else bias.float().to(DEV), None if gate is None else gate.to(DEV), plan=plan)
    torch.cuda.synchronize()
    return out.view(n_q, H, Dv)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, D, Dv, chunk, page", [(4, 2, 32, 24, 20, 4), (6, 1, 64, 40, 33, 16), (3, 3, 16, 16, 7, 8),
                                                      (8, 2, 128, 64, 48, 16), (2, 2, 24, 24, None, 4),
                                                      (4, 4, 128, 128, 64, 16), (8, 1, 128, 96, 300, 16)])
def test_sigmoid_attention_over_pages(dtype, H, G, D, Dv, chunk, page):
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(D + Dv)
    n = 150
    q = torch.randn(n, H, D, generator=g).to(dtype)
    k = torch.randn(n, G, D, generator=g).to(dtype)
    v = torch.randn(n, G, Dv, generator=g).to(dtype)
    bias = torch.randn(H, generator=g) - 2.0
    gate = torch.randn(n, H + 3, generator=g).to(dtype)                  # rows wider than the heads
    scale = 1.7 / math.sqrt(D)
    want = plain.chunked_sigmoid_attention(q.double(), k.double(), v.double(), scale, bias.double(), chunk)
    want = want * torch.sigmoid(gate[:, :H].double())[:, :, None]
    for with_plan in (False, True):
        got = run_attention(ops, q, k, v, list(range(n)), scale, chunk, None, bias, gate, page_size=page, with_plan=with_plan)
        close(got, want, 1e-5 if dtype == torch.float32 else 8e-3, f"every position of a prompt (plan={with_plan})")
    # a portion from the middle of the sequence, cut inside a chunk and a page
    got = run_attention(ops, q[37:101], k[:101], v[:101], list(range(37, 101)), scale, chunk, None, bias, gate[37:101],
                        page_size=page, with_plan=True)
    close(got, want[37:101], 1e-5 if dtype == torch.float32 else 8e-3, "a portion")
    # single decoded tokens: the same rows, asked for one position at a time
    for p in sorted({0, 1, n - 1} | ({chunk - 1, chunk, chunk + 1, 2 * chunk - 1, 2 * chunk} if chunk and 2 * chunk < n else set())):
        one = run_attention(ops, q[p:p + 1], k[:p + 1], v[:p + 1], [p], scale, chunk, None, bias, gate[p:p + 1],
                            page_size=page, seed=p, with_plan=bool(p % 2))
        close(one, want[p:p + 1], 1e-5 if dtype == torch.float32 else 8e-3, f"position {p} alone")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk, window, page", [(10, None, 4), (64, None, 16), (None, 9, 4), (40, 13, 8), (None, None, 16)])
def test_sigmoid_attention_sees_exactly_its_keys(dtype, chunk, window, page):
    """Zero queries give every visible key the weight sigmoid(bias) = 1/2, and value j is the j-th unit
    vector: the output row names the keys that were seen, each exactly once, whatever page they lie in."""
    ops = ops_for(dtype)
    n = 200
    q = torch.zeros(n, 2, 16, dtype=dtype)
    k = torch.randn(n, 1, 16).to(dtype)
    v = torch.eye(n, dtype=dtype)[:, None, :]
    got = run_attention(ops, q, k, v, list(range(n)), 1.0, chunk, window, torch.zeros(2), None, page_size=page).float().cpu()
    for i in range(n):
        lo = max(0 if chunk is None else i // chunk * chunk, 0 if window is None else i - window)
        want = torch.zeros(n)
        want[lo:i + 1] = 0.5
        assert torch.equal(got[i, 0], want) and torch.equal(got[i, 1], want), f"query {i} (keys {lo}..{i})"


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("chunk, window, page", [(10, None, 16), (64, None, 16), (None, 9, 32), (40, 13, 16), (None, None, 16),
                                                 (100, None, 64)])
def test_mfma_sigmoid_attention_sees_exactly_its_keys(D, chunk, window, page):
    """The same through the MFMA kernel (bfloat16, head sizes 64 and 128, values as large as keys): the
    value of key j is the unit vector j % D scaled by 1 + j // D, so a row still names its keys."""
    dtype = torch.bfloat16
    ops = ops_for(dtype)
    n = 3 * D
    q = torch.zeros(n, 4, D, dtype=dtype)
    k = torch.randn(n, 2, D).to(dtype)
    v = torch.zeros(n, 2, D)
    for j in range(n):
        v[j, :, j % D] = 1 + j // D
    for rows in (range(n), range(D + 5, n - 3)):
        rows = list(rows)
        got = run_attention(ops, q[rows], k[:rows[-1] + 1], v[:rows[-1] + 1].to(dtype), rows, 1.0, chunk, window,
                            torch.zeros(4), None, page_size=page, with_plan=True).float().cpu()
        for at, i in enumerate(rows):
            lo = max(0 if chunk is None else i // chunk * chunk, 0 if window is None else i - window)
            want = torch.zeros(D)
            for j in range(lo, i + 1):
                want[j % D] += 0.5 * (1 + j // D)
            for hd in range(4):
                assert torch.equal(got[at, hd], want), f"query {i} head {hd} (keys {lo}..{i})"


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("variant", [(1, 1), (2, 1), (1, 2), (2, 2)])
@pytest.mark.parametrize("chunk, window", [(512, None), (None, None), (300, 77)])
def test_mfma_sigmoid_attention_long_contexts_every_variant(D, variant, chunk, window):
    """1,100 tokens, so that a workgroup walks dozens of key blocks, with both column widths and with one
    and two key groups per workgroup (the two groups' sums are added at the end): rows that name their keys."""
    dtype = torch.bfloat16
    ops = ops_for(dtype)
    n = 1100
    q = torch.zeros(n, 4, D, dtype=dtype)
    k = torch.randn(n, 2, D).to(dtype)
    v = torch.zeros(n, 2, D)
    for j in range(n):
        v[j, :, j % D] = 1 + j // D
    rows = list(range(700, n))
    got = run_attention(ops, q[rows], k, v.to(dtype), rows, 1.0, chunk, window, torch.zeros(4), None, page_size=16,
                        with_plan=True, variant=variant).float().cpu()
    for at, i in enumerate(rows):
        lo = max(0 if chunk is None else i // chunk * chunk, 0 if window is None else i - window)
        want = torch.zeros(D)
        for j in range(lo, i + 1):
            want[j % D] += 0.5 * (1 + j // D)
        for hd in range(4):
            assert torch.equal(got[at, hd], want), f"query {i} head {hd} (keys {lo}..{i})"
    # random queries, keys, bias and gates over the same context, against the plain function
    g = torch.Generator().manual_seed(D)
    q = torch.randn(n, 4, D, generator=g).to(dtype)
    v = torch.randn(n, 2, D, generator=g).to(dtype)
    bias = torch.randn(4, generator=g) - 4.0
    gate = torch.randn(n, 4, generator=g).to(dtype)
    scale = 1.5 / math.sqrt(D)
    idx = torch.arange(n)
    want = plain.chunked_sigmoid_attention(q.double(), k.double(), v.double(), scale, bias.double(), chunk)
    if window is not None:                                   # the plain function has no window: apply it by hand
        seen = (idx[None, :] <= idx[:, None]) & (idx[None, :] >= idx[:, None] - window)
        if chunk is not None:
            seen &= (idx[None, :] // chunk) == (idx[:, None] // chunk)
        want = torch.empty(n, 4, D, dtype=torch.float64)
        for hd in range(4):
            wgt = torch.sigmoid((q[:, hd].double() @ k[:, hd // 2].double().T) * scale + bias[hd].double()) * seen
            want[:, hd] = wgt @ v[:, hd // 2].double()
    want = want * torch.sigmoid(gate.double())[:, :, None]
    got = run_attention(ops, q[rows], k, v, rows, scale, chunk, window, bias, gate[rows], page_size=16, with_plan=True,
                        variant=variant)
    close(got, want[rows], 1e-2, "random rows")


@pytest.mark.parametrize("dtype", DTYPES)
def test_sigmoid_attention_far_key_stands_out(dtype):
    """One key hundreds of positions back (inside the query's chunk) is the only one with a weight near
    one; a key just outside the chunk that would score as high must not show."""
    ops = ops_for(dtype)
    n, D, Dv, chunk = 700, 32, 8, 512
    g = torch.Generator().manual_seed(1)
    k = (torch.randn(n, 1, D, generator=g) * 0.1)
    v = torch.randn(n, 1, Dv, generator=g)
    q = torch.zeros(1, 1, D)
    q[0, 0, 0] = 6.0
    for far in (512, 513, 640):                              # the first keys of the chunk, and one in its middle
        kk = k.clone()
        kk[far, 0, 0] = 5.0
        kk[511, 0, 0] = 5.0                                  # just outside the chunk of position 699
        got = run_attention(ops, q.to(dtype), kk.to(dtype), v.to(dtype), [n - 1], 1.0, chunk, None,
                            torch.tensor([-15.0]), None, page_size=16, seed=far)
        want = plain.chunked_sigmoid_attention(q.double().expand(n, 1, D), kk.to(dtype).double(), v.to(dtype).double(),
                                               1.0, torch.tensor([-15.0]).double(), chunk)[n - 1:]
        close(got, want, 1e-5 if dtype == torch.float32 else 8e-3, f"far key {far}")
        assert float((got[0, 0].float().cpu() - v[far, 0].to(dtype).float()).abs().max()) < 0.05


# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("h", [48, 256, 1000])
def test_norms_around_a_sublayer(dtype, h):
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(h)
    n = 9
    y = (torch.randn(n, h, generator=g) * 3).to(dtype)
    resid = torch.randn(n, h, generator=g)
    wa = (1 + 0.1 * torch.randn(h, generator=g)).to(torch.bfloat16)
    wb = (1 + 0.1 * torch.randn(h, generator=g)).to(torch.bfloat16)
    want_resid = resid.double() + plain.rms_norm(y.double(), wa.double(), 1e-5)
    want_rows = plain.rms_norm(want_resid, wb.double(), 2e-6)
    r = resid.to(DEV).clone()
    rows = torch.empty(n, h, dtype=dtype, device=DEV)
    ops.norm_add_norm(y.to(DEV), (wa.to(DEV), 1e-5, False), r, (wb.to(DEV), 2e-6, False), rows)
    close(r, want_resid, 1e-6, "residual")
    close(rows, want_rows, 1e-6 if dtype == torch.float32 else 8e-3, "rows of the next norm")
    r2 = resid.to(DEV).clone()
    ops.norm_add_norm(y.to(DEV), (wa.to(DEV), 1e-5, False), r2, None, None)        # the add alone
    assert torch.equal(r2, r)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("h", [48, 1024, 5000, 9000])
def test_norms_with_the_next_token_shift(dtype, h):
    """A step of single tokens: the kernel that closes a sublayer also applies the next layer's token
    shift. The same bits as the two kernels it stands for; a padding row touches no state."""
    ops = ops_for(dtype)
    g = torch.Generator().manual_seed(h)
    n, slots = 5, [2, 0, 3, 1]
    y = (torch.randn(n, h, generator=g) * 3).to(dtype).to(DEV)
    resid = torch.randn(n, h, generator=g).to(DEV)
    wa = (1 + 0.1 * torch.randn(h, generator=g)).to(torch.bfloat16).to(DEV)
    wb = (1 + 0.1 * torch.randn(h, generator=g)).to(torch.bfloat16).to(DEV)
    mix = torch.rand(h, generator=g).to(torch.bfloat16).to(DEV)
    state = torch.randn(5, h, generator=g).to(dtype).to(DEV)
    tsq, cu, sl = step_ints([1, 1, 1, 1], slots, pad_rows=1)
    r1, s1 = resid.clone(), state.clone()
    rows = torch.empty(n, h, dtype=dtype, device=DEV)
    want = torch.empty(n, h, dtype=dtype, device=DEV)
    ops.norm_add_norm(y, (wa, 1e-5, False), r1, (wb, 2e-6, False), rows)
    ops.token_shift(rows, mix, s1, tsq, cu, sl, want)
    r2, s2 = resid.clone(), state.clone()
    got = torch.empty(n, h, dtype=dtype, device=DEV)
    ops.norm_add_norm(y, (wa, 1e-5, False), r2, (wb, 2e-6, False), got, shift=(mix, s2, tsq, sl))
    torch.cuda.synchronize()
    assert torch.equal(r1, r2) and torch.equal(s1, s2) and torch.equal(got, want)
    assert torch.equal(s2[4], state[4]) and (got[4] == 0).all()
    prev = state[slots[1]].double().cpu()
    hrow = rows[1].double().cpu()
    close(got[1], hrow + (prev - hrow) * mix.double().cpu(), 1e-6 if dtype == torch.float32 else 8e-3)


def test_soft_cap():
    ops = ops_for(torch.float32)
    x = torch.linspace(-90, 90, 7 * 333).view(7, 333)
    d = x.to(DEV).clone()
    ops.soft_cap(d[:, :300], 12.5)                                       # a view with a pitch of its own
    close(d[:, :300], plain.soft_cap(x[:, :300].double(), 12.5), 1e-6)
    assert torch.equal(d[:, 300:].cpu(), x[:, 300:])
