// Router: one wavefront per token.  Lane e holds the logit of expert e; the
// softmax statistics and the k arg-max rounds are wave-wide butterfly
// reductions, so no LDS and no block barrier is needed.
//
// Semantics follow src/topk_softmax_kernels.hip:23-64 of the reference
// (selection on raw logits, strict '>' in ascending expert order, hence ties go
// to the lowest index; weight = exp(x - max) / sum) and, when renorm is set,
// fused_moe.py:161-162 (weights divided by the sum of the selected ones).
#include "common.h"

namespace em {
namespace {

constexpr int kRouterWaves = 4;  // tokens per workgroup

template <typename Elem>
__global__ __launch_bounds__(kRouterWaves* kWave) void router_kernel(
    const typename Elem::storage* __restrict__ logits, int64_t T, int E, int k, int renorm,
    float* __restrict__ out_w, int32_t* __restrict__ out_ids) {
    const int lane = lane_id();
    const int64_t t = static_cast<int64_t>(blockIdx.x) * kRouterWaves + (threadIdx.x / kWave);
    if (t >= T) return;  // whole wave leaves together

    float v = -INFINITY;
    if (lane < E) {
        v = Elem::load(logits[t * E + lane]);
        if (v != v) v = -INFINITY;  // a NaN logit can never be selected
    }

    // row max and softmax denominator
    float mx = v;
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    const float ex = (lane < E) ? expf(v - mx) : 0.0f;
    float denom = ex;
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) denom += __shfl_xor(denom, off);

    // k rounds of arg-max over the lanes still alive.  (alive desc, value desc,
    // index asc) is a total order, so every lane ends a round with the same
    // winner; retired lanes and lanes >= E can never win while k <= E, which
    // keeps the k indices distinct and in [0, E) even for rows of -inf.
    int alive = (lane < E) ? 1 : 0;
    float my_w = 0.0f;  // lane j < k keeps the j-th selected weight
    int my_id = 0;
    float sel_sum = 0.0f;
    for (int j = 0; j < k; ++j) {
        int ba = alive;
        float bv = v;
        int bi = lane;
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) {
            const int oa = __shfl_xor(ba, off);
            const float ov = __shfl_xor(bv, off);
            const int oi = __shfl_xor(bi, off);
            const bool better = (oa > ba) || (oa == ba && (ov > bv || (ov == bv && oi < bi)));
            if (better) { ba = oa; bv = ov; bi = oi; }
        }
        const float p = __shfl(ex, bi) / denom;
        sel_sum += p;
        if (lane == j) { my_w = p; my_id = bi; }
        if (lane == bi) alive = 0;
    }
    if (lane < k) {
        out_w[t * k + lane] = renorm ? my_w / sel_sum : my_w;
        out_ids[t * k + lane] = my_id;
    }
}

}  // namespace

int launch_router(const void* logits, int logits_dtype, int64_t T, int E, int k, int renorm,
                  float* w, int32_t* ids, hipStream_t s) {
    if (T == 0) return 0;
    const dim3 grid(static_cast<unsigned>(ceil_div(T, kRouterWaves)));
    const dim3 block(kRouterWaves * kWave);
    switch (logits_dtype) {
        case EM_DTYPE_F32:
            hipLaunchKernelGGL(router_kernel<F32Elem>, grid, block, 0, s,
                               static_cast<const float*>(logits), T, E, k, renorm, w, ids);
            break;
        case EM_DTYPE_BF16:
            hipLaunchKernelGGL(router_kernel<BF16Elem>, grid, block, 0, s,
                               static_cast<const uint16_t*>(logits), T, E, k, renorm, w, ids);
            break;
        case EM_DTYPE_F16:
            hipLaunchKernelGGL(router_kernel<F16Elem>, grid, block, 0, s,
                               static_cast<const uint16_t*>(logits), T, E, k, renorm, w, ids);
            break;
        default:
            return EM_ERR_BAD_DTYPE;
    }
    return launch_status();
}

}  // namespace em
