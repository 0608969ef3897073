// Kernels of mixers that carry a fixed-size state per request from token to token.
//
//   token shift      out[t] = h[t] + (h[t-1] - h[t]) * mix, the row in front of a request's first token
//                    of the step taken from the request's state, which then takes the step's last row
//   delta rule       S <- diag(w) S - (a*u)(u^T S) + k v^T,  o = S^T r,  one matrix S per head
//                    (prepare: w, a*u, u in float from the packed projection; scan: the recurrence
//                    over each request's tokens of the step; finish: per-head RMS, weight, gate)
//
// A step is any mix of requests: token_seq[t] names the request of row t (-1: a padding row),
// cu_seqlens[s] .. cu_seqlens[s+1] are the rows of request s, state_slots[s] its row of the state
// tensors. States are float (the shift's row has the activation type, it is a copy); decays,
// rates, unit keys and the recurrence are float whatever the activation type T is.
#include "dispatch.h"

// ---------------------------------------------------------------------------------------
// Token shift. One workgroup per row. The thread that serves column c of a request's first row
// is the only one that touches state[slot][c]: it reads the old value and then stores the
// request's last row of this step there.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
token_shift_kernel(const T* __restrict__ h, long ldh, T* __restrict__ out, long ldo, WeightPtr mix,
                   T* __restrict__ state, const int* __restrict__ token_seq, const int* __restrict__ cu_seqlens,
                   const int* __restrict__ state_slots, int width) {
    const int t = blockIdx.x;
    const int seq = token_seq[t];
    T* o = out + (size_t)t * ldo;
    if (seq < 0) {
        for (int c = threadIdx.x; c < width; c += blockDim.x) o[c] = from_f<T>(0.f);
        return;
    }
    const int first = cu_seqlens[seq];
    const int last = cu_seqlens[seq + 1] - 1;
    const T* cur = h + (size_t)t * ldh;
    if (t > first) {
        const T* prev = cur - ldh;
        for (int c = threadIdx.x; c < width; c += blockDim.x) {
            const float x = to_f(cur[c]);
            o[c] = from_f<T>(x + (to_f(prev[c]) - x) * mix.at(c));
        }
        return;
    }
    T* st = state + (size_t)state_slots[seq] * width;
    const T* tail = h + (size_t)last * ldh;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        const float x = to_f(cur[c]);
        const float p = to_f(st[c]);
        st[c] = tail[c];
        o[c] = from_f<T>(x + (p - x) * mix.at(c));
    }
}

extern "C" int mv_token_shift(const void* h, long ldh, void* out, long ldo, const void* mix, int mix_dtype, void* state,
                              const int* token_seq, const int* cu_seqlens, const int* state_slots, int n, int width,
                              int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && width > 0 && ldh >= width && ldo >= width, "token_shift: bad sizes n=%d width=%d", n, width);
    MV_REQUIRE(h != out, "token_shift: a row reads the row in front of it, the output must be another buffer");
    MV_REQUIRE(mv_valid_dtype(mix_dtype) && mix && state && token_seq && cu_seqlens && state_slots,
               "token_shift: missing operand");
    if (n == 0) return 0;
    WeightPtr m{mix, mix_dtype};
    MV_DISPATCH_T(dtype, "token_shift",
                  hipLaunchKernelGGL(token_shift_kernel<T>, dim3(n), dim3(256), 0, stream, (const T*)h, ldh, (T*)out, ldo,
                                     m, (T*)state, token_seq, cu_seqlens, state_slots, width));
    return mv_check_launch("token_shift");
}

// ---------------------------------------------------------------------------------------
// Delta rule, prepare. The packed rows hold [r | k | v | g | a | w1] (H*D columns each, `rank` for
// w1) from column 0 on. For DP_TOKENS rows and 256 channels a workgroup:
//   coef[0][t][c] = exp(-decay_rate * sigmoid(w0[c] + sum_j W2[c][j] tanh(w1[t][j])))
//   coef[2][t][c] = u = k[t][c] / sqrt(sum over the head of k^2 + key_eps)
//   coef[1][t][c] = sigmoid(a[t][c] + a_bias[c]) * u
// A row of W2 is read once for the workgroup's rows.
// ---------------------------------------------------------------------------------------
#define DP_TOKENS 8
#define DP_MAX_RANK 512
#define DP_MAX_HEADS 260      // heads that 256 channels can touch, for head sizes >= 1

__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }

template <typename T>
__global__ void __launch_bounds__(256)
delta_prepare_kernel(const T* __restrict__ packed, long ld, int H, int D, int rank, WeightPtr w2, WeightPtr w0,
                     WeightPtr a_bias, float decay_rate, float key_eps, const int* __restrict__ token_seq,
                     float* __restrict__ coef, int n) {
    __shared__ float th[DP_TOKENS][DP_MAX_RANK];
    __shared__ float inv_len[DP_TOKENS][DP_MAX_HEADS];
    const int inner = H * D;
    const int t0 = blockIdx.x * DP_TOKENS;
    const int c0 = blockIdx.y * 256;
    const int nt = min(DP_TOKENS, n - t0);
    const int tid = threadIdx.x;
    const int lane = tid % MV_WAVE, wave = tid / MV_WAVE;
    for (int i = tid; i < nt * rank; i += 256) {
        const int tt = i / rank, j = i % rank;
        th[tt][j] = tanhf(to_f(packed[(size_t)(t0 + tt) * ld + 5 * (size_t)inner + j]));
    }
    // lengths of the keys of the heads these channels belong to, a wave per (row, head)
    const int h_lo = c0 / D;
    const int h_hi = min(H - 1, (c0 + 255) / D);
    const int nh = h_hi - h_lo + 1;
    for (int p = wave; p < nt * nh; p += 4) {
        const int tt = p / nh, hh = p % nh;
        const T* k = packed + (size_t)(t0 + tt) * ld + inner + (size_t)(h_lo + hh) * D;
        float ss = 0.f;
        for (int d = lane; d < D; d += MV_WAVE) {
            const float v = to_f(k[d]);
            ss = fmaf(v, v, ss);
        }
        ss = wave_sum(ss);
        if (lane == 0) inv_len[tt][hh] = 1.f / sqrtf(ss + key_eps);
    }
    __syncthreads();
    const int c = c0 + tid;
    if (c >= inner) return;
    float acc[DP_TOKENS];
#pragma unroll
    for (int tt = 0; tt < DP_TOKENS; ++tt) acc[tt] = 0.f;
    for (int j = 0; j < rank; ++j) {
        const float w = w2.at((size_t)c * rank + j);
#pragma unroll
        for (int tt = 0; tt < DP_TOKENS; ++tt) acc[tt] = fmaf(w, th[tt][j], acc[tt]);
    }
    const float b0 = w0.at(c), ab = a_bias.at(c);
    const int hh = c / D - h_lo;
    const size_t plane = (size_t)n * inner;
#pragma unroll
    for (int tt = 0; tt < DP_TOKENS; ++tt) {
        if (tt >= nt) break;
        const size_t row = (size_t)(t0 + tt);
        const T* p = packed + row * ld;
        const float u = to_f(p[inner + c]) * inv_len[tt][hh];
        const float rate = sigmoid_f(to_f(p[4 * (size_t)inner + c]) + ab);
        float* o = coef + row * inner + c;
        o[0] = expf(-decay_rate * sigmoid_f(acc[tt] + b0));
        o[plane] = rate * u;
        o[2 * plane] = u;
    }
}

extern "C" int mv_delta_prepare(const void* packed, long ld, int n, int H, int D, int rank, const void* w2, const void* w0,
                                const void* a_bias, int weight_dtype, float decay_rate, float key_eps,
                                const int* token_seq, float* coef, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && D > 0 && rank > 0, "delta_prepare: bad sizes n=%d H=%d D=%d rank=%d", n, H, D, rank);
    MV_REQUIRE(rank <= DP_MAX_RANK, "delta_prepare: rank %d exceeds the supported maximum %d", rank, DP_MAX_RANK);
    MV_REQUIRE(ld >= 5L * H * D + rank, "delta_prepare: rows of %ld columns do not hold 5 x %d + %d", ld, H * D, rank);
    MV_REQUIRE(mv_valid_dtype(weight_dtype) && w2 && w0 && a_bias && coef, "delta_prepare: missing operand");
    MV_REQUIRE(key_eps > 0.f, "delta_prepare: key_eps must be positive");
    if (n == 0) return 0;
    WeightPtr pw2{w2, weight_dtype}, pw0{w0, weight_dtype}, pab{a_bias, weight_dtype};
    dim3 grid((n + DP_TOKENS - 1) / DP_TOKENS, (H * D + 255) / 256);
    MV_REQUIRE(grid.y <= 65535, "delta_prepare: too many channels");
    MV_DISPATCH_T(dtype, "delta_prepare",
                  hipLaunchKernelGGL(delta_prepare_kernel<T>, grid, dim3(256), 0, stream, (const T*)packed, ld, H, D,
                                     rank, pw2, pw0, pab, decay_rate, key_eps, token_seq, coef, n));
    return mv_check_launch("delta_prepare");
}

// ---------------------------------------------------------------------------------------
// Delta rule, scan. A workgroup of 256 threads owns 64 value columns of one head of one request:
// four neighbouring lanes share a column j, each keeps R rows of S[:, j] in registers (rows
// sub*R .. sub*R+R-1, so D <= 4R; rows beyond D stay zero). Per token
//     read = sum_i u_i S_ij            (R multiply-adds a lane, then a sum over the four lanes)
//     S_ij = w_i S_ij - (a u)_i read + k_i v_j ;   o_j = sum_i r_i S_ij
// The per-token vectors w, a*u, u, k, r (the same for every column) and v are staged in LDS,
// 16 (or 8) tokens at a time. The request's state is read at the start and written at the end.
// ---------------------------------------------------------------------------------------
// lanes 4q .. 4q+3 end with the sum of their four values: two exchanges inside the quad (data-parallel
// moves with the lane patterns [1,0,3,2] and [2,3,0,1]; nothing goes through LDS)
__device__ __forceinline__ float quad_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    return v;
}

template <typename T, int R>
__global__ void __launch_bounds__(256)
delta_scan_kernel(const T* __restrict__ packed, long ld, const float* __restrict__ coef, float* __restrict__ state,
                  const int* __restrict__ cu_seqlens, const int* __restrict__ state_slots, int H, int D,
                  float* __restrict__ out, int n) {
    constexpr int DP = 4 * R;                       // padded key size
    constexpr int DS_TOKENS = R > 32 ? 8 : 16;      // tokens staged at a time
    __shared__ __attribute__((aligned(16))) float sv[5][DS_TOKENS][DP];   // w, a*u, u, k, r
    __shared__ float svv[DS_TOKENS][64];
    const int seq = blockIdx.x, head = blockIdx.y, j0 = blockIdx.z * 64;
    const int begin = cu_seqlens[seq], end = cu_seqlens[seq + 1];
    if (end <= begin) return;
    const int tid = threadIdx.x;
    const int sub = tid & 3;
    const int col = tid >> 2;                        // 0..63
    const int j = j0 + col;
    const bool live = j < D;
    const int inner = H * D;
    const size_t plane = (size_t)n * inner;
    float* S = state + ((size_t)state_slots[seq] * H + head) * (size_t)D * D;
    float s[R];
#pragma unroll
    for (int e = 0; e < R; ++e) {
        const int i = sub * R + e;
        s[e] = (live && i < D) ? S[(size_t)i * D + j] : 0.f;
    }
    for (int base = begin; base < end; base += DS_TOKENS) {
        const int nt = min(DS_TOKENS, end - base);
        __syncthreads();
        for (int x = tid; x < nt * DP; x += 256) {
            const int tt = x / DP, i = x % DP;
            const size_t row = (size_t)(base + tt);
            float w = 0.f, au = 0.f, u = 0.f, k = 0.f, r = 0.f;
            if (i < D) {
                const size_t c = row * inner + (size_t)head * D + i;
                w = coef[c];
                au = coef[plane + c];
                u = coef[2 * plane + c];
                const T* p = packed + row * ld + (size_t)head * D + i;
                r = to_f(p[0]);
                k = to_f(p[inner]);
            }
            sv[0][tt][i] = w; sv[1][tt][i] = au; sv[2][tt][i] = u; sv[3][tt][i] = k; sv[4][tt][i] = r;
        }
        for (int x = tid; x < nt * 64; x += 256) {
            const int tt = x / 64, jj = x % 64;
            svv[tt][jj] = (j0 + jj < D) ? to_f(packed[(size_t)(base + tt) * ld + 2 * (size_t)inner + (size_t)head * D + j0 + jj])
                                        : 0.f;
        }
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const float* w = &sv[0][tt][sub * R];
            const float* au = &sv[1][tt][sub * R];
            const float* u = &sv[2][tt][sub * R];
            const float* k = &sv[3][tt][sub * R];
            const float* r = &sv[4][tt][sub * R];
            float read = 0.f;
#pragma unroll
            for (int e = 0; e < R; ++e) read = fmaf(u[e], s[e], read);
            read = quad_sum(read);
            const float vj = svv[tt][col];
            float o = 0.f;
#pragma unroll
            for (int e = 0; e < R; ++e) {
                const float x = fmaf(w[e], s[e], fmaf(k[e], vj, -au[e] * read));
                s[e] = x;
                o = fmaf(r[e], x, o);
            }
            o = quad_sum(o);
            if (live && sub == 0) out[(size_t)(base + tt) * inner + (size_t)head * D + j] = o;
        }
    }
#pragma unroll
    for (int e = 0; e < R; ++e) {
        const int i = sub * R + e;
        if (live && i < D) S[(size_t)i * D + j] = s[e];
    }
}

extern "C" int mv_delta_scan(const void* packed, long ld, const float* coef, float* state, const int* cu_seqlens,
                             const int* state_slots, int n_seqs, int n, int H, int D, float* out, int dtype,
                             hipStream_t stream) {
    MV_REQUIRE(n >= 0 && n_seqs >= 0 && H > 0 && D > 0, "delta_scan: bad sizes n=%d seqs=%d H=%d D=%d", n, n_seqs, H, D);
    MV_REQUIRE(D <= 256, "delta_scan: head size %d exceeds the supported maximum 256", D);
    MV_REQUIRE(ld >= 3L * H * D, "delta_scan: rows of %ld columns do not hold r, k and v of %d", ld, H * D);
    MV_REQUIRE(packed && coef && state && cu_seqlens && state_slots && out, "delta_scan: missing operand");
    MV_REQUIRE(H <= 65535 && (D + 63) / 64 <= 65535, "delta_scan: too many heads");
    if (n == 0 || n_seqs == 0) return 0;
    dim3 grid(n_seqs, H, (D + 63) / 64);
#define DS_LAUNCH(R)                                                                                                 \
    MV_DISPATCH_T(dtype, "delta_scan",                                                                               \
                  hipLaunchKernelGGL((delta_scan_kernel<T, R>), grid, dim3(256), 0, stream, (const T*)packed, ld, coef, \
                                     state, cu_seqlens, state_slots, H, D, out, n))
    if (D <= 16) {
        DS_LAUNCH(4);
    } else if (D <= 32) {
        DS_LAUNCH(8);
    } else if (D <= 64) {
        DS_LAUNCH(16);
    } else if (D <= 128) {
        DS_LAUNCH(32);
    } else {
        DS_LAUNCH(64);
    }
#undef DS_LAUNCH
    return mv_check_launch("delta_scan");
}

// ---------------------------------------------------------------------------------------
// Delta rule, finish. One wave per (row, head):
//   y[t][c] = o[t][c] / sqrt(mean over the head of o^2 + eps) * weight[c] * sigmoid(g[t][c])
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
delta_finish_kernel(const float* __restrict__ raw, const T* __restrict__ packed, long ld, WeightPtr weight, int H, int D,
                    float eps, T* __restrict__ out, long ldo, int n) {
    const int lane = threadIdx.x % MV_WAVE;
    const long unit = (long)blockIdx.x * 4 + threadIdx.x / MV_WAVE;
    if (unit >= (long)n * H) return;
    const int t = (int)(unit / H), head = (int)(unit % H);
    const int inner = H * D;
    const float* o = raw + (size_t)t * inner + (size_t)head * D;
    float ss = 0.f;
    for (int d = lane; d < D; d += MV_WAVE) ss = fmaf(o[d], o[d], ss);
    ss = wave_sum(ss);
    const float rinv = 1.f / sqrtf(ss / (float)D + eps);
    const T* g = packed + (size_t)t * ld + 3 * (size_t)inner + (size_t)head * D;
    T* y = out + (size_t)t * ldo + (size_t)head * D;
    for (int d = lane; d < D; d += MV_WAVE)
        y[d] = from_f<T>(o[d] * rinv * weight.at((size_t)head * D + d) * sigmoid_f(to_f(g[d])));
}

extern "C" int mv_delta_finish(const float* raw, const void* packed, long ld, const void* weight, int weight_dtype, int n,
                               int H, int D, float eps, void* out, long ldo, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && D > 0 && eps > 0.f, "delta_finish: bad sizes n=%d H=%d D=%d", n, H, D);
    MV_REQUIRE(ld >= 4L * H * D && ldo >= (long)H * D, "delta_finish: row pitches too small");
    MV_REQUIRE(mv_valid_dtype(weight_dtype) && raw && packed && weight && out, "delta_finish: missing operand");
    if (n == 0) return 0;
    const long units = (long)n * H;
    WeightPtr w{weight, weight_dtype};
    MV_DISPATCH_T(dtype, "delta_finish",
                  hipLaunchKernelGGL(delta_finish_kernel<T>, dim3((unsigned)((units + 3) / 4)), dim3(256), 0, stream, raw,
                                     (const T*)packed, ld, w, H, D, eps, (T*)out, ldo, n));
    return mv_check_launch("delta_finish");
}
