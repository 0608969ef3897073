// Mixture of experts: the router's choice and the kernels around the experts' products.
//
//   moe_route          from float logits [n][E] (E = real experts + identity experts): scores = softmax
//                      over all E; choice = scores + correction; the experts form `groups` equal runs of
//                      neighbours, a group's worth is its largest choice, only experts of the `keep`
//                      worthiest groups can be chosen; the `top` largest choices are chosen; the weight of
//                      a chosen expert is its score divided by the chosen scores' sum (+ sum_eps).
//                      Leaves the weights dense, [n][E] with zeros for the others, and as lists
//                      (ids [n][top], weights [n][top], in the order chosen).
//   moe_swiglu_scale   act[t][e][c] = weight[t][e] * silu(gate[t][e][c]) * up[t][e][c]: the gated pair of
//                      every expert with the router's weight applied before the one rounding, so that
//                      one product with all experts' down matrices side by side sums the chosen experts
//   moe_identity_add   y[t] += (sum of the weights of the identity experts of t) * h[t]
#include "dispatch.h"

#define MR_MAX_E 1024

// the largest value over the wave and the smallest index that holds it (index INT_MAX: nothing left)
__device__ __forceinline__ void wave_argmax(float& best, int& at) {
    for (int o = 32; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o, 64);
        const int oa = __shfl_xor(at, o, 64);
        if (ob > best || (ob == best && oa < at)) {
            best = ob;
            at = oa;
        }
    }
}

__global__ void __launch_bounds__(64)
moe_route_kernel(const float* __restrict__ logits, long ld, int E, WeightPtr correction, int has_correction, int groups, int keep,
                 int top, float sum_eps, float* __restrict__ dense, int* __restrict__ ids, float* __restrict__ weights) {
    __shared__ float score[MR_MAX_E];
    __shared__ float choice[MR_MAX_E];
    __shared__ float worth[MR_MAX_E];          // of the groups
    __shared__ int open_group[MR_MAX_E];       // 1: its experts may be chosen
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* z = logits + (size_t)t * ld;
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) {
        const float p = expf(z[e] - mx);
        score[e] = p;
        sum += p;
    }
    sum = wave_sum(sum);
    const float inv = 1.f / sum;
    for (int e = lane; e < E; e += 64) {
        const float s = score[e] * inv;
        score[e] = s;
        choice[e] = s + (has_correction ? correction.at(e) : 0.f);
        dense[(size_t)t * E + e] = 0.f;
    }
    __syncthreads();
    const int per = E / groups;
    for (int g = lane; g < groups; g += 64) {
        float w = -INFINITY;
        for (int i = 0; i < per; ++i) w = fmaxf(w, choice[g * per + i]);
        worth[g] = w;
        open_group[g] = keep >= groups ? 1 : 0;
    }
    __syncthreads();
    if (keep < groups) {
        for (int round = 0; round < keep; ++round) {          // the best group left, the first among equals
            float best = -INFINITY;
            int at = 0x7fffffff;
            for (int g = lane; g < groups; g += 64)
                if (!open_group[g] && (at == 0x7fffffff || worth[g] > best)) {
                    best = worth[g];
                    at = g;
                }
            wave_argmax(best, at);
            __syncthreads();
            if (lane == 0 && at != 0x7fffffff) open_group[at] = 1;
            __syncthreads();
        }
    }
    float picked_sum = 0.f;
    float my_w = 0.f;                                          // lane r holds the r-th chosen score (top <= 64)
    int my_id = -1;
    for (int round = 0; round < top; ++round) {
        float best = -INFINITY;
        int at = 0x7fffffff;
        for (int e = lane; e < E; e += 64)
            if (open_group[e / per] && choice[e] != -INFINITY && (at == 0x7fffffff || choice[e] > best)) {
                best = choice[e];
                at = e;
            }
        wave_argmax(best, at);
        __syncthreads();
        if (at != 0x7fffffff) {
            const float s = score[at];
            picked_sum += s;
            if (lane == round) {
                my_w = s;
                my_id = at;
            }
            if (lane == 0) choice[at] = -INFINITY;            // taken
        }
        __syncthreads();
    }
    if (lane < top) {
        const float w = my_id >= 0 ? my_w / (picked_sum + sum_eps) : 0.f;
        ids[(size_t)t * top + lane] = my_id;
        weights[(size_t)t * top + lane] = w;
        if (my_id >= 0) dense[(size_t)t * E + my_id] = w;
    }
}

extern "C" int mv_moe_route(const float* logits, long ld, int n, int E, const void* correction, int weight_dtype, int groups,
                            int keep, int top, float sum_eps, float* dense, int* ids, float* weights, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && E > 0 && E <= MR_MAX_E && ld >= E, "moe_route: bad sizes n=%d E=%d (at most %d)", n, E, MR_MAX_E);
    MV_REQUIRE(groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups, "moe_route: %d groups of which %d stay do not fit %d experts",
               groups, keep, E);
    MV_REQUIRE(top >= 1 && top <= 64 && top <= (E / groups) * keep, "moe_route: top %d does not fit", top);
    MV_REQUIRE(logits && dense && ids && weights && (!correction || mv_valid_dtype(weight_dtype)), "moe_route: missing operand");
    if (n == 0) return 0;
    WeightPtr c{correction, weight_dtype};
    hipLaunchKernelGGL(moe_route_kernel, dim3(n), dim3(64), 0, stream, logits, ld, E, c, correction ? 1 : 0, groups, keep, top,
                       sum_eps, dense, ids, weights);
    return mv_check_launch("moe_route");
}

// gate_up rows: [gate of expert 0 (F) | ... | gate of expert E-1 | up of expert 0 | ... ]; act rows [E][F]
template <typename T>
__global__ void __launch_bounds__(256)
moe_swiglu_scale_kernel(const T* __restrict__ gate_up, long ld, const float* __restrict__ dense, int ld_dense, int E, int F,
                        T* __restrict__ act, long total) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const long EF = (long)E * F;
    const long t = i / EF, c = i % EF;
    const float w = dense[t * ld_dense + c / F];
    float v = 0.f;
    if (w != 0.f) {
        const float g = to_f(gate_up[t * ld + c]), u = to_f(gate_up[t * ld + EF + c]);
        v = w * (g / (1.f + expf(-g))) * u;
    }
    act[t * EF + c] = from_f<T>(v);
}

extern "C" int mv_moe_swiglu_scale(const void* gate_up, long ld, const float* dense, int ld_dense, int n, int E, int F, void* act,
                                   int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && E > 0 && F > 0 && ld >= 2L * E * F && ld_dense >= E, "moe_swiglu_scale: bad sizes n=%d E=%d F=%d", n, E, F);
    MV_REQUIRE(gate_up && dense && act, "moe_swiglu_scale: missing operand");
    const long total = (long)n * E * F;
    if (total == 0) return 0;
    MV_DISPATCH_T(dtype, "moe_swiglu_scale",
                  hipLaunchKernelGGL(moe_swiglu_scale_kernel<T>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                                     (const T*)gate_up, ld, dense, ld_dense, E, F, (T*)act, total));
    return mv_check_launch("moe_swiglu_scale");
}

template <typename T>
__global__ void __launch_bounds__(256)
moe_identity_add_kernel(T* __restrict__ y, long ldy, const T* __restrict__ h, long ldh, const float* __restrict__ dense,
                        int ld_dense, int first, int count, int width, int set) {
    const int t = blockIdx.x;
    float w = 0.f;
    for (int e = 0; e < count; ++e) w += dense[(size_t)t * ld_dense + first + e];
    if (w == 0.f && !set) return;
    for (int c = threadIdx.x; c < width; c += 256) {
        T* p = y + (size_t)t * ldy + c;
        *p = from_f<T>((set ? 0.f : to_f(*p)) + w * to_f(h[(size_t)t * ldh + c]));
    }
}

// y[t] (+)= (dense[t][first .. first+count) summed) * h[t]; `set` writes instead of adding
extern "C" int mv_moe_identity_add(void* y, long ldy, const void* h, long ldh, const float* dense, int ld_dense, int first,
                                   int count, int n, int width, int set, int dtype, hipStream_t stream) {
    MV_REQUIRE(n >= 0 && width > 0 && ldy >= width && ldh >= width && first >= 0 && count >= 0 && ld_dense >= first + count,
               "moe_identity_add: bad sizes n=%d width=%d", n, width);
    MV_REQUIRE(y && h && dense, "moe_identity_add: missing operand");
    if (n == 0 || (count == 0 && !set)) return 0;
    MV_DISPATCH_T(dtype, "moe_identity_add",
                  hipLaunchKernelGGL(moe_identity_add_kernel<T>, dim3(n), dim3(256), 0, stream, (T*)y, ldy, (const T*)h, ldh, dense,
                                     ld_dense, first, count, width, set));
    return mv_check_launch("moe_identity_add");
}

// float rows in place: x <- x * factor
__global__ void scale_f32_kernel(float* __restrict__ x, long ld, int cols, long total, float factor) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    x[(i / cols) * ld + (i % cols)] *= factor;
}

extern "C" int mv_scale_f32(float* x, long ld, int rows, int cols, float factor, hipStream_t stream) {
    MV_REQUIRE(rows >= 0 && cols > 0 && ld >= cols && x, "scale: bad sizes rows=%d cols=%d", rows, cols);
    const long total = (long)rows * cols;
    if (total == 0) return 0;
    hipLaunchKernelGGL(scale_f32_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, x, ld, cols, total, factor);
    return mv_check_launch("scale");
}
