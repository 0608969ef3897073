// Paged causal attention with sigmoid weights, for any mix of query portions.
//
// The query at position p of a request sees the request's keys at positions lo .. p, with
//   lo = max(start of p's chunk, p - window, 0)       chunk: positions with equal p / chunk
// (chunk <= 0: no chunks; window < 0: no window). The weight of a visible key is
// sigmoid(q.k * scale + bias[head]); weights are not normalised over the keys, so the output is
// a plain sum and the order of its additions depends only on p and lo, never on the batch.
// Head h's output is multiplied by sigmoid(gate[token][h]) when gates are given. Values may have
// another size than keys.
//
// Layouts:  K[page][kv_head][slot][D]   V[page][kv_head][Dv][slot]
// The general kernel (one workgroup per token and head) takes every size up to 512 and both
// activation types: it is the float32 path's and the fall-back of the bfloat16 path.
#include "dispatch.h"

#define AS_THREADS 128
#define AS_MAX_D 512

__device__ __forceinline__ float as_sigmoid(float z) { return 1.f / (1.f + expf(-z)); }

// q . k over D channels with the key row read 16 bytes at a time (the caller vouches for D % 8 == 0 and a
// 16-byte aligned row); the additions run in the order of the channels, as the one-by-one loop's do
__device__ __forceinline__ float as_dot8(const float* qs, const bf16* krow, int D) {
    float dot = 0.f;
    for (int d = 0; d < D; d += 8) {
        const uint4 u = *reinterpret_cast<const uint4*>(krow + d);
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            dot = fmaf(qs[d + 2 * e], __uint_as_float(w[e] << 16), dot);
            dot = fmaf(qs[d + 2 * e + 1], __uint_as_float(w[e] & 0xffff0000u), dot);
        }
    }
    return dot;
}
__device__ __forceinline__ float as_dot8(const float* qs, const float* krow, int D) {
    float dot = 0.f;
    for (int d = 0; d < D; d += 4) {
        const float4 k = *reinterpret_cast<const float4*>(krow + d);
        dot = fmaf(qs[d], k.x, dot);
        dot = fmaf(qs[d + 1], k.y, dot);
        dot = fmaf(qs[d + 2], k.z, dot);
        dot = fmaf(qs[d + 3], k.w, dot);
    }
    return dot;
}

template <typename T>
__global__ void __launch_bounds__(AS_THREADS)
attention_sigmoid_kernel(const T* __restrict__ q, long q_stride, T* __restrict__ out, long out_stride,
                         const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                         const int* __restrict__ block_table, int bt_width, int page_size,
                         const int* __restrict__ positions, const int* __restrict__ token_seq, int H, int Hkv, int D,
                         int Dv, float scale, int chunk, int window, const float* __restrict__ bias,
                         const T* __restrict__ gate, long gate_stride) {
    __shared__ float qs[AS_MAX_D];
    __shared__ float ps[AS_THREADS];
    __shared__ long voff[AS_THREADS];

    const int tok = blockIdx.x;
    const int head = blockIdx.y;
    const int tid = threadIdx.x;
    const int seq = token_seq[tok];
    T* o = out + (size_t)tok * out_stride + (size_t)head * Dv;
    if (seq < 0) {
        for (int d = tid; d < Dv; d += AS_THREADS) o[d] = from_f<T>(0.f);
        return;
    }
    const int pos = positions[tok];
    const int kvh = head / (H / Hkv);
    int lo = 0;
    if (chunk > 0) lo = pos / chunk * chunk;
    if (window >= 0 && pos - window > lo) lo = pos - window;
    const int hi = pos;
    const int* bt = block_table + (size_t)seq * bt_width;
    const float b = bias ? bias[head] : 0.f;
    const bool wide_keys = D % 8 == 0 && ((uintptr_t)k_pages % 16) == 0;      // key rows start at multiples of 16 bytes

    const T* qrow = q + (size_t)tok * q_stride + (size_t)head * D;
    for (int d = tid; d < D; d += AS_THREADS) qs[d] = to_f(qrow[d]);

    float acc[AS_MAX_D / AS_THREADS];
#pragma unroll
    for (int i = 0; i < AS_MAX_D / AS_THREADS; ++i) acc[i] = 0.f;

    for (int base = lo; base <= hi; base += AS_THREADS) {
        __syncthreads();                 // qs is written; the tile before has been consumed
        const int j = base + tid;
        float p = 0.f;
        long vo = 0;
        if (j <= hi) {
            const int page = bt[j / page_size];
            const int slot = j % page_size;
            const T* krow = k_pages + (((size_t)page * Hkv + kvh) * page_size + slot) * D;
            float dot = 0.f;
            if (wide_keys) {
                dot = as_dot8(qs, krow, D);
            } else {
                for (int d = 0; d < D; ++d) dot = fmaf(qs[d], to_f(krow[d]), dot);
            }
            p = as_sigmoid(dot * scale + b);
            vo = (long)(((size_t)page * Hkv + kvh) * Dv) * page_size + slot;
        }
        ps[tid] = p;
        voff[tid] = vo;
        __syncthreads();
        const int cnt = (hi - base + 1) < AS_THREADS ? (hi - base + 1) : AS_THREADS;
#pragma unroll
        for (int i = 0; i < AS_MAX_D / AS_THREADS; ++i) {
            const int d = tid + i * AS_THREADS;
            if (d < Dv) {
                float a = acc[i];
                for (int jj = 0; jj < cnt; ++jj)
                    a = fmaf(ps[jj], to_f(v_pages[voff[jj] + (long)d * page_size]), a);
                acc[i] = a;
            }
        }
    }
    const float g = gate ? as_sigmoid(to_f(gate[(size_t)tok * gate_stride + head])) : 1.f;
#pragma unroll
    for (int i = 0; i < AS_MAX_D / AS_THREADS; ++i) {
        const int d = tid + i * AS_THREADS;
        if (d < Dv) o[d] = from_f<T>(acc[i] * g);
    }
}

extern "C" int mv_attention_sigmoid_ref(const void* q, long q_stride, void* out, long out_stride, const void* k_pages,
                                        const void* v_pages, const int* block_table, int bt_width, int page_size,
                                        const int* positions, const int* token_seq, int n, int H, int Hkv, int D, int Dv,
                                        float scale, int chunk, int window, const float* bias, const void* gate,
                                        long gate_stride, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && H > 0 && Hkv > 0 && D > 0 && Dv > 0, "attention_sigmoid: bad sizes n=%d H=%d Hkv=%d D=%d Dv=%d",
               n, H, Hkv, D, Dv);
    MV_REQUIRE(H % Hkv == 0, "attention_sigmoid: %d query heads are not a multiple of %d key/value heads", H, Hkv);
    MV_REQUIRE(D <= AS_MAX_D && Dv <= AS_MAX_D, "attention_sigmoid: head sizes %d / %d exceed the supported maximum %d",
               D, Dv, AS_MAX_D);
    MV_REQUIRE(page_size > 0 && bt_width > 0, "attention_sigmoid: bad page size %d or block table width %d", page_size,
               bt_width);
    MV_REQUIRE(q_stride >= (long)H * D && out_stride >= (long)H * Dv, "attention_sigmoid: row strides too small");
    MV_REQUIRE(gate == nullptr || gate_stride >= H, "attention_sigmoid: gate rows too short");
    MV_REQUIRE(H <= 65535, "attention_sigmoid: too many heads %d", H);
    if (n == 0) return 0;
    MV_DISPATCH_T(dtype, "attention_sigmoid",
                  hipLaunchKernelGGL(attention_sigmoid_kernel<T>, dim3(n, H), dim3(AS_THREADS), 0, stream, (const T*)q,
                                     q_stride, (T*)out, out_stride, (const T*)k_pages, (const T*)v_pages, block_table,
                                     bt_width, page_size, positions, token_seq, H, Hkv, D, Dv, scale, chunk, window,
                                     bias, (const T*)gate, gate_stride));
    return mv_check_launch("attention_sigmoid");
}
