// Attention over a cached latent: every token caches one row [latent (R) | rotated key part (DR)]
// that all query heads share. A head's key is a linear map of the latent (W_uk) beside the shared
// rotated part, its value another linear map (W_uv); neither is ever materialised. With
// qa = W_uk^T q_plain (the query carried into the latent's space) the score of a key is
//     (qa . latent + q_rot . k_rot) * scale
// and the head's output is W_uv applied to the softmax-weighted sum of the latents. So the kernels are
//     latent_prepare     norms of the two down-projections, rotation of the key part, cache write
//     head_linear        per head y = W_h x (queries into latent space, rotating their rotated part on
//                        the way; weighted latents into values, times the output gate)
//     attention_latent   softmax attention with one shared key row of R + DR numbers whose first R
//                        are also the value
// Page layout: rows[page][slot][R + DR] in the activation type. Scores, weights and sums are float.
#include "dispatch.h"

// ---------------------------------------------------------------------------------------
// Prepare. Packed rows: [dq (QR) | dkv (R + DR) | ...]. One workgroup per row:
//   cq[t]           = dq / rms(dq) * wq                      (the query's latent, activation type)
//   page row of t   = [dkv[:R] / rms(dkv[:R]) * wkv | rot(dkv[R:], position)]
// rot pairs channel i with i + DR/2; table[p] = [cos (DR/2) | sin (DR/2)] of position p.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
latent_prepare_kernel(const T* __restrict__ packed, long ld, int QR, int R, int DR, WeightPtr wq, WeightPtr wkv, float eps,
                      const float* __restrict__ table, const int* __restrict__ positions, const int* __restrict__ token_seq,
                      const int* __restrict__ block_table, int bt_width, int page_size, T* __restrict__ cq, long ldq,
                      T* __restrict__ pages) {
    __shared__ float scratch[17];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int seq = token_seq[t];
    T* qo = cq + (size_t)t * ldq;
    if (seq < 0) {
        for (int c = tid; c < QR; c += 256) qo[c] = from_f<T>(0.f);
        return;
    }
    const T* p = packed + (size_t)t * ld;
    float ss = 0.f;
    for (int c = tid; c < QR; c += 256) {
        const float x = to_f(p[c]);
        ss = fmaf(x, x, ss);
    }
    ss = block_sum(ss, scratch);
    float inv = 1.f / sqrtf(ss / (float)QR + eps);
    for (int c = tid; c < QR; c += 256) qo[c] = from_f<T>(to_f(p[c]) * inv * wq.at(c));
    const T* kv = p + QR;
    ss = 0.f;
    for (int c = tid; c < R; c += 256) {
        const float x = to_f(kv[c]);
        ss = fmaf(x, x, ss);
    }
    ss = block_sum(ss, scratch);
    inv = 1.f / sqrtf(ss / (float)R + eps);
    const int pos = positions[t];
    const int page = block_table[(size_t)seq * bt_width + pos / page_size];
    T* row = pages + ((size_t)page * page_size + pos % page_size) * (size_t)(R + DR);
    for (int c = tid; c < R; c += 256) row[c] = from_f<T>(to_f(kv[c]) * inv * wkv.at(c));
    const int half = DR / 2;
    const float* cs = table + (size_t)pos * DR;
    for (int i = tid; i < half; i += 256) {
        const float a = to_f(kv[R + i]), b = to_f(kv[R + half + i]);
        const float c = cs[i], s = cs[half + i];
        row[R + i] = from_f<T>(a * c - b * s);
        row[R + half + i] = from_f<T>(b * c + a * s);
    }
}

extern "C" int mv_latent_prepare(const void* packed, long ld, int n, int QR, int R, int DR, const void* wq, const void* wkv,
                                 int weight_dtype, float eps, const float* table, int table_rows, const int* positions,
                                 const int* token_seq, const int* block_table, int bt_width, int page_size, void* cq,
                                 long ldq, void* pages, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && QR > 0 && R > 0 && DR >= 0 && DR % 2 == 0, "latent_prepare: bad sizes n=%d QR=%d R=%d DR=%d", n, QR, R, DR);
    MV_REQUIRE(ld >= (long)QR + R + DR && ldq >= QR && page_size > 0 && bt_width > 0, "latent_prepare: row pitches too small");
    MV_REQUIRE(mv_valid_dtype(weight_dtype) && packed && wq && wkv && (table || DR == 0) && table_rows >= 0 && positions && token_seq
               && block_table && cq && pages && eps > 0.f, "latent_prepare: missing operand");
    if (n == 0) return 0;
    WeightPtr a{wq, weight_dtype}, b{wkv, weight_dtype};
    MV_DISPATCH_T(dtype, "latent_prepare",
                  hipLaunchKernelGGL(latent_prepare_kernel<T>, dim3(n), dim3(256), 0, stream, (const T*)packed, ld, QR, R, DR, a,
                                     b, eps, table, positions, token_seq, block_table, bt_width, page_size, (T*)cq, ldq,
                                     (T*)pages));
    return mv_check_launch("latent_prepare");
}

// ---------------------------------------------------------------------------------------
// Per-head linear map. x rows [n][H][ldx_head] (IN inputs used), w [H][IN][OUT] (the inputs of an
// output column are a stride of OUT apart, so neighbouring threads read neighbouring words),
// y rows [n][H][ldy_head]:  y[t][h][j] = sum_i x[t][h][i] w[h][i][j], the sum in the order of i.
// A workgroup takes HL_TOKENS rows of one head; the weight is read once for them.
//   tail > 0   x[t][h][IN .. IN+tail) is copied behind the OUT outputs, rotated by the row's position
//              (pairs i, i + tail/2; table[p] = [cos | sin])
//   gate       y is multiplied by sigmoid(gate[t][h * OUT + j])
// ---------------------------------------------------------------------------------------
#define HL_TOKENS 8
#define HL_MAX_IN 1024

template <typename TIN, typename TOUT, typename TG>
__global__ void __launch_bounds__(256)
head_linear_kernel(const TIN* __restrict__ x, long ldx, int ldx_head, WeightPtr w, int IN, int OUT, TOUT* __restrict__ y, long ldy,
                   int ldy_head, int tail, const float* __restrict__ table, const int* __restrict__ positions,
                   const TG* __restrict__ gate, long ldg, const int* __restrict__ token_seq, int n) {
    __shared__ float xs[HL_TOKENS][HL_MAX_IN];
    const int t0 = blockIdx.x * HL_TOKENS, head = blockIdx.y, tid = threadIdx.x;
    const int nt = min(HL_TOKENS, n - t0);
    for (int e = tid; e < HL_TOKENS * IN; e += 256) {
        const int tt = e / IN, i = e % IN;
        xs[tt][i] = tt < nt ? to_f(x[(size_t)(t0 + tt) * ldx + (size_t)head * ldx_head + i]) : 0.f;
    }
    __syncthreads();
    for (int j = tid; j < OUT; j += 256) {
        float acc[HL_TOKENS];
#pragma unroll
        for (int tt = 0; tt < HL_TOKENS; ++tt) acc[tt] = 0.f;
        const size_t w0 = (size_t)head * IN * OUT + j;
        for (int i = 0; i < IN; ++i) {
            const float wv = w.at(w0 + (size_t)i * OUT);
#pragma unroll
            for (int tt = 0; tt < HL_TOKENS; ++tt) acc[tt] = fmaf(xs[tt][i], wv, acc[tt]);
        }
#pragma unroll
        for (int tt = 0; tt < HL_TOKENS; ++tt) {
            if (tt < nt) {
                float v = acc[tt];
                if (token_seq[t0 + tt] < 0) v = 0.f;
                else if (gate) v *= 1.f / (1.f + expf(-to_f(gate[(size_t)(t0 + tt) * ldg + (size_t)head * OUT + j])));
                y[(size_t)(t0 + tt) * ldy + (size_t)head * ldy_head + j] = from_f<TOUT>(v);
            }
        }
    }
    const int half = tail / 2;
    for (int e = tid; e < nt * half; e += 256) {
        const int tt = e / half, i = e % half;
        const int t = t0 + tt;
        const TIN* src = x + (size_t)t * ldx + (size_t)head * ldx_head + IN;
        TOUT* dst = y + (size_t)t * ldy + (size_t)head * ldy_head + OUT;
        if (token_seq[t] < 0) {
            dst[i] = from_f<TOUT>(0.f);
            dst[half + i] = from_f<TOUT>(0.f);
            continue;
        }
        const float* cs = table + (size_t)positions[t] * tail;
        const float a = to_f(src[i]), b = to_f(src[half + i]);
        dst[i] = from_f<TOUT>(a * cs[i] - b * cs[half + i]);
        dst[half + i] = from_f<TOUT>(b * cs[i] + a * cs[half + i]);
    }
}

// mode 0: x activation type -> y float (with an optional rotated tail); mode 1: x float -> y activation
// type (with an optional gate of the activation type)
extern "C" int mv_head_linear(const void* x, long ldx, int ldx_head, const void* w, int weight_dtype, int n, int H, int IN,
                              int OUT, void* y, long ldy, int ldy_head, int tail, const float* table, const int* positions,
                              const void* gate, long ldg, const int* token_seq, int mode, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && IN > 0 && OUT > 0 && tail >= 0 && tail % 2 == 0, "head_linear: bad sizes n=%d H=%d IN=%d OUT=%d", n, H, IN, OUT);
    MV_REQUIRE(IN <= HL_MAX_IN, "head_linear: %d inputs a head, at most %d are served", IN, HL_MAX_IN);
    MV_REQUIRE(ldx_head >= IN + tail && ldy_head >= OUT + tail && ldx >= (long)(H - 1) * ldx_head + IN + tail
               && ldy >= (long)(H - 1) * ldy_head + OUT + tail, "head_linear: row pitches too small");
    MV_REQUIRE(mv_valid_dtype(weight_dtype) && x && w && y && token_seq && (tail == 0 || (table && positions)) && H <= 65535
               && (!gate || ldg >= (long)H * OUT), "head_linear: missing operand");
    MV_REQUIRE((mode == 0 && !gate) || (mode == 1 && tail == 0), "head_linear: mode %d does not take these options", mode);
    if (n == 0) return 0;
    WeightPtr wp{w, weight_dtype};
    dim3 grid((n + HL_TOKENS - 1) / HL_TOKENS, H);
    if (mode == 0) {
        MV_DISPATCH_T(dtype, "head_linear",
                      hipLaunchKernelGGL((head_linear_kernel<T, float, T>), grid, dim3(256), 0, stream, (const T*)x, ldx, ldx_head,
                                         wp, IN, OUT, (float*)y, ldy, ldy_head, tail, table, positions, (const T*)nullptr, 0L,
                                         token_seq, n));
    } else {
        MV_DISPATCH_T(dtype, "head_linear",
                      hipLaunchKernelGGL((head_linear_kernel<float, T, T>), grid, dim3(256), 0, stream, (const float*)x, ldx,
                                         ldx_head, wp, IN, OUT, (T*)y, ldy, ldy_head, 0, table, positions, (const T*)gate, ldg,
                                         token_seq, n));
    }
    return mv_check_launch("head_linear");
}

// ---------------------------------------------------------------------------------------
// Attention. One workgroup per (row, group of AL_HEADS heads): the query heads of a row read the same
// key rows, so a key row that a thread has fetched serves all heads of the group. Keys are visited in
// tiles of AL_THREADS from position 0 (causal: a query at position p sees 0..p), so the order of
// additions depends on the position alone. q float [n][H][R + DR]; out float [n][H][R]: the
// weighted sum of the visible latents.
// ---------------------------------------------------------------------------------------
#define AL_THREADS 128
#define AL_HEADS 4
#define AL_MAX_KEY 640
#define AL_MAX_R 512

template <typename T>
__global__ void __launch_bounds__(AL_THREADS)
attention_latent_kernel(const float* __restrict__ q, long ldq, float* __restrict__ out, long ldo, const T* __restrict__ pages,
                        const int* __restrict__ block_table, int bt_width, int page_size, const int* __restrict__ positions,
                        const int* __restrict__ token_seq, int H, int R, int DR, float scale) {
    __shared__ float qs[AL_HEADS][AL_MAX_KEY];
    __shared__ float ps[AL_HEADS][AL_THREADS];
    __shared__ long roff[AL_THREADS];
    __shared__ float scratch[17];
    const int tok = blockIdx.x, h0 = blockIdx.y * AL_HEADS, tid = threadIdx.x;
    const int nh = min(AL_HEADS, H - h0);
    const int DK = R + DR;
    const int seq = token_seq[tok];
    if (seq < 0) {
        for (int e = tid; e < nh * R; e += AL_THREADS) out[(size_t)tok * ldo + (size_t)(h0 + e / R) * R + e % R] = 0.f;
        return;
    }
    const int hi = positions[tok];
    const int* bt = block_table + (size_t)seq * bt_width;
    for (int e = tid; e < AL_HEADS * DK; e += AL_THREADS) {
        const int hh = e / DK, d = e % DK;
        qs[hh][d] = hh < nh ? q[(size_t)tok * ldq + (size_t)(h0 + hh) * DK + d] : 0.f;
    }
    __syncthreads();
    float m[AL_HEADS], l[AL_HEADS];
    float acc[AL_HEADS][AL_MAX_R / AL_THREADS];
#pragma unroll
    for (int hh = 0; hh < AL_HEADS; ++hh) {
        m[hh] = -INFINITY;
        l[hh] = 0.f;
#pragma unroll
        for (int i = 0; i < AL_MAX_R / AL_THREADS; ++i) acc[hh][i] = 0.f;
    }
    for (int base = 0; base <= hi; base += AL_THREADS) {
        const int j = base + tid;
        const bool valid = j <= hi;
        float s[AL_HEADS];
#pragma unroll
        for (int hh = 0; hh < AL_HEADS; ++hh) s[hh] = -INFINITY;
        long ro = 0;
        if (valid) {
            ro = ((long)bt[j / page_size] * page_size + j % page_size) * DK;
            const T* row = pages + ro;
            float dot[AL_HEADS];
#pragma unroll
            for (int hh = 0; hh < AL_HEADS; ++hh) dot[hh] = 0.f;
            for (int d = 0; d < DK; ++d) {
                const float kd = to_f(row[d]);
#pragma unroll
                for (int hh = 0; hh < AL_HEADS; ++hh) dot[hh] = fmaf(qs[hh][d], kd, dot[hh]);
            }
#pragma unroll
            for (int hh = 0; hh < AL_HEADS; ++hh) s[hh] = dot[hh] * scale;
        }
        roff[tid] = ro;
        float corr[AL_HEADS];
#pragma unroll
        for (int hh = 0; hh < AL_HEADS; ++hh) {
            const float tmax = block_max(s[hh], scratch);
            const float m_new = fmaxf(m[hh], tmax);
            const float p = valid ? expf(s[hh] - m_new) : 0.f;
            ps[hh][tid] = p;
            const float tsum = block_sum(p, scratch);      // its barriers also publish ps and roff
            corr[hh] = expf(m[hh] - m_new);                // first tile: exp(-inf) = 0
            l[hh] = l[hh] * corr[hh] + tsum;
            m[hh] = m_new;
        }
        const int cnt = min(AL_THREADS, hi - base + 1);
#pragma unroll
        for (int i = 0; i < AL_MAX_R / AL_THREADS; ++i) {
            const int d = tid + i * AL_THREADS;
            if (d < R) {
                float a[AL_HEADS];
#pragma unroll
                for (int hh = 0; hh < AL_HEADS; ++hh) a[hh] = acc[hh][i] * corr[hh];
                for (int jj = 0; jj < cnt; ++jj) {
                    const float v = to_f(pages[roff[jj] + d]);
#pragma unroll
                    for (int hh = 0; hh < AL_HEADS; ++hh) a[hh] = fmaf(ps[hh][jj], v, a[hh]);
                }
#pragma unroll
                for (int hh = 0; hh < AL_HEADS; ++hh) acc[hh][i] = a[hh];
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int hh = 0; hh < AL_HEADS; ++hh) {
        if (hh < nh) {
            const float inv = 1.f / l[hh];
#pragma unroll
            for (int i = 0; i < AL_MAX_R / AL_THREADS; ++i) {
                const int d = tid + i * AL_THREADS;
                if (d < R) out[(size_t)tok * ldo + (size_t)(h0 + hh) * R + d] = acc[hh][i] * inv;
            }
        }
    }
}

extern "C" int mv_attention_latent(const float* q, long ldq, float* out, long ldo, const void* pages, const int* block_table,
                                   int bt_width, int page_size, const int* positions, const int* token_seq, int n, int H,
                                   int R, int DR, float scale, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && R > 0 && DR >= 0, "attention_latent: bad sizes n=%d H=%d R=%d DR=%d", n, H, R, DR);
    MV_REQUIRE(R <= AL_MAX_R && R + DR <= AL_MAX_KEY, "attention_latent: a latent of %d and a rotated part of %d exceed %d / %d",
               R, DR, AL_MAX_R, AL_MAX_KEY);
    MV_REQUIRE(page_size > 0 && bt_width > 0 && ldq >= (long)H * (R + DR) && ldo >= (long)H * R, "attention_latent: pitches too small");
    MV_REQUIRE(q && out && pages && block_table && positions && token_seq && (H + AL_HEADS - 1) / AL_HEADS <= 65535,
               "attention_latent: missing operand");
    if (n == 0) return 0;
    MV_DISPATCH_T(dtype, "attention_latent",
                  hipLaunchKernelGGL(attention_latent_kernel<T>, dim3(n, (H + AL_HEADS - 1) / AL_HEADS), dim3(AL_THREADS), 0,
                                     stream, q, ldq, out, ldo, (const T*)pages, block_table, bt_width, page_size, positions,
                                     token_seq, H, R, DR, scale));
    return mv_check_launch("attention_latent");
}
