// Router selection shared by the stand-alone router and by the kernel that computes the logits itself.
#pragma once
#include "common.h"

namespace em {

// One token per aligned group of G lanes (G a power of two, E <= G <= 64): lane `sub` < E of the group brings
// the logit of expert `sub` in `v` (a NaN logit must already be -inf), the k selected weights and ids go to
// out_w / out_ids [t*k .. t*k+k) when `valid`.  All 64 lanes of the wavefront must call it together.
// Selection on the raw logits, strict '>' in ascending expert order, hence ties go to the lowest index
// (src/topk_softmax_kernels.hip:23-64); weight = exp(x - max) / sum, divided by the sum of the selected
// ones when renorm is set (fused_moe.py:161-162).
template <int G>
__device__ __forceinline__ void route_group(float v, int lane, int64_t t, bool valid, int E, int k, int renorm,
                                            float* __restrict__ out_w, int32_t* __restrict__ out_ids) {
    const int sub = lane & (G - 1);
    const int group_base = lane - sub;
    // row max and softmax denominator
    float mx = v;
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
    const float ex = (sub < E) ? expf(v - mx) : 0.0f;
    float denom = ex;
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) denom += __shfl_xor(denom, off);

    // k rounds of arg-max over the lanes still alive.  (alive desc, value desc,
    // index asc) is a total order, so every lane of a group ends a round with the same
    // winner; retired lanes and lanes >= E can never win while k <= E, which
    // keeps the k indices distinct and in [0, E) even for rows of -inf.
    int alive = (sub < E) ? 1 : 0;
    float my_w = 0.0f;  // lane j < k keeps the j-th selected weight
    int my_id = 0;
    float sel_sum = 0.0f;
    for (int j = 0; j < k; ++j) {
        int ba = alive;
        float bv = v;
        int bi = sub;
#pragma unroll
        for (int off = G / 2; off > 0; off >>= 1) {
            const int oa = __shfl_xor(ba, off);
            const float ov = __shfl_xor(bv, off);
            const int oi = __shfl_xor(bi, off);
            const bool better = (oa > ba) || (oa == ba && (ov > bv || (ov == bv && oi < bi)));
            if (better) { ba = oa; bv = ov; bi = oi; }
        }
        const float p = __shfl(ex, group_base + bi) / denom;
        sel_sum += p;
        if (sub == j) { my_w = p; my_id = bi; }
        if (sub == bi) alive = 0;
    }
    if (valid && sub < k) {
        out_w[t * k + sub] = renorm ? my_w / sel_sum : my_w;
        out_ids[t * k + sub] = my_id;
    }
}

// One token per wavefront: lane e < E brings the logit of expert e.
__device__ __forceinline__ void route_from_logit(float v, int lane, int64_t t, int E, int k, int renorm,
                                                 float* __restrict__ out_w, int32_t* __restrict__ out_ids) {
    route_group<kWave>(v, lane, t, true, E, k, renorm, out_w, out_ids);
}

// Tail of the kernels that compute the logits of 16 tokens per workgroup on the MFMA, the waves splitting H:
// `acc` is the wave's partial 16x16 tile (lane l: token l % 16, experts 4 * (l / 16) .. + 3).  The partial
// tiles meet in LDS and are added in wave order; optional rounding to bf16 as the reference's linear does
// (layers/linear.py:53-54); then E adjacent lanes per token run the selection, 64 / E tokens per wavefront.
// Contains a block barrier: all waves of the workgroup must call it.
template <int E_, int WAVES>
__device__ __forceinline__ void reduce_tiles_and_route(f32x4_t acc, float (*partial)[16][E_], int wave, int lane,
                                                       int64_t t0, int64_t T, int k, int renorm, int round_bf16,
                                                       void* __restrict__ logits_out, float* __restrict__ out_w,
                                                       int32_t* __restrict__ out_ids) {
    const int r16 = lane & 15, kq = lane >> 4;
    if (4 * kq < E_) *reinterpret_cast<f32x4_t*>(&partial[wave][r16][4 * kq]) = acc;
    __syncthreads();
    constexpr int kTokPerWave = kWave / E_;
    if (wave * kTokPerWave < 16) {  // whole waves leave together
        const int tok = wave * kTokPerWave + lane / E_;
        const int e = lane % E_;
        const int64_t t = t0 + tok;
        const bool valid = (t < T);
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) v += partial[w][tok][e];
        if (round_bf16) {
            const uint16_t b = f32_to_bf16_bits(v);
            v = bf16_bits_to_f32(b);
            if (valid && logits_out != nullptr) static_cast<uint16_t*>(logits_out)[t * E_ + e] = b;
        } else if (valid && logits_out != nullptr) {
            static_cast<float*>(logits_out)[t * E_ + e] = v;
        }
        if (v != v) v = -INFINITY;  // a NaN logit can never be selected
        route_group<E_>(v, lane, t, valid, E_, k, renorm, out_w, out_ids);
    }
}

}  // namespace em
