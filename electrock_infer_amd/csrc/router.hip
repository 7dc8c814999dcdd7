// Router: one wavefront per token.  Lane e holds the logit of expert e; the
// softmax statistics and the k arg-max rounds are wave-wide butterfly
// reductions, so no LDS and no block barrier is needed.
//
// Semantics follow src/topk_softmax_kernels.hip:23-64 of the reference
// (selection on raw logits, strict '>' in ascending expert order, hence ties go
// to the lowest index; weight = exp(x - max) / sum) and, when renorm is set,
// fused_moe.py:161-162 (weights divided by the sum of the selected ones).
#include "router_device.h"

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
    route_from_logit(v, lane, t, E, k, renorm, out_w, out_ids);
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
