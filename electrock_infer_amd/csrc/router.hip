// Router: a group of G adjacent lanes per token (G = 8 for up to eight experts: eight tokens per
// wavefront).  Lane e of a group holds the logit of expert e; the softmax statistics and the k arg-max
// rounds are butterfly reductions inside the group, so no LDS and no block barrier is needed.
//
// Semantics follow src/topk_softmax_kernels.hip:23-64 of the reference
// (selection on raw logits, strict '>' in ascending expert order, hence ties go
// to the lowest index; weight = exp(x - max) / sum) and, when renorm is set,
// fused_moe.py:161-162 (weights divided by the sum of the selected ones).
#include "router_device.h"

namespace em {
namespace {

constexpr int kRouterWaves = 4;  // wavefronts per workgroup

// G lanes per token (G = the smallest power of two >= E, at least 8): 64 / G tokens per wavefront
template <typename Elem, int G>
__global__ __launch_bounds__(kRouterWaves* kWave) void router_kernel(
    const typename Elem::storage* __restrict__ logits, int64_t T, int E, int k, int renorm,
    float* __restrict__ out_w, int32_t* __restrict__ out_ids) {
    constexpr int kTokens = kWave / G;
    const int lane = lane_id();
    const int sub = lane & (G - 1);
    const int64_t t = (static_cast<int64_t>(blockIdx.x) * kRouterWaves + (threadIdx.x / kWave)) * kTokens + lane / G;
    const bool valid = t < T;

    float v = -INFINITY;
    if (valid && sub < E) {
        v = Elem::load(logits[t * E + sub]);
        if (v != v) v = -INFINITY;  // a NaN logit can never be selected
    }
    route_group<G>(v, lane, t, valid, E, k, renorm, out_w, out_ids);
}

template <typename Elem>
void launch_typed(const void* logits, int64_t T, int E, int k, int renorm, float* w, int32_t* ids, hipStream_t s) {
    const typename Elem::storage* lp = static_cast<const typename Elem::storage*>(logits);
    const dim3 block(kRouterWaves * kWave);
    auto go = [&](auto kernel, int g) {
        const dim3 grid(static_cast<unsigned>(ceil_div(T, static_cast<int64_t>(kRouterWaves) * (kWave / g))));
        launch(kernel, grid, block, 0, s, lp, T, E, k, renorm, w, ids);
    };
    if (E <= 8) go(router_kernel<Elem, 8>, 8);
    else if (E <= 16) go(router_kernel<Elem, 16>, 16);
    else if (E <= 32) go(router_kernel<Elem, 32>, 32);
    else go(router_kernel<Elem, 64>, 64);
}

}  // namespace

int launch_router(const void* logits, int logits_dtype, int64_t T, int E, int k, int renorm,
                  float* w, int32_t* ids, hipStream_t s) {
    if (T == 0) return 0;
    switch (logits_dtype) {
        case EM_DTYPE_F32: launch_typed<F32Elem>(logits, T, E, k, renorm, w, ids, s); break;
        case EM_DTYPE_BF16: launch_typed<BF16Elem>(logits, T, E, k, renorm, w, ids, s); break;
        case EM_DTYPE_F16: launch_typed<F16Elem>(logits, T, E, k, renorm, w, ids, s); break;
        default: return EM_ERR_BAD_DTYPE;
    }
    return launch_status();
}

}  // namespace em
