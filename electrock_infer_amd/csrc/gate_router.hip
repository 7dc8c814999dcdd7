// Router gate fused with the router: logits[t, e] = sum_h x[t, h] * gate_w[e, h], then the
// top-k softmax of router.hip, in one launch.
//
// The reference computes the logits with a bf16 linear layer in the model
// (models/mixtral.py:40-42,59; layers/linear.py:53-54: F.linear(x, weight) -> bf16 [T, E]) and
// hands them to the MoE layer.  Here a workgroup of 8 wavefronts owns 16 tokens and the waves split H:
// each wave runs v_mfma_f32_16x16x32_bf16 over its slice with the gate rows as the M operand (expert
// e in row e; for E = 8 rows 8..15 repeat them and are ignored) and the token rows as the N operand,
// both read straight from global memory in operand layout (the gate matrix, 64 KB for 8 x 4096, stays
// in L2; x streams from HBM once).  The eight partial 16 x E tiles meet in LDS, are added in wave order,
// and E adjacent lanes per token run the router's selection -- 64 / E tokens per wavefront at once.
// With round_bf16 the fp32 sum is rounded to bf16 first, as the reference's linear does (ties then exist
// and go to the lowest expert index); without it the fp32 logits are used as they are.
// The kernel is bound by reading x once (T * H * 2 bytes).
#include "router_device.h"

namespace em {
namespace {

constexpr int kGateWaves = 8;
constexpr int kGateThreads = kGateWaves * kWave;
constexpr int kGateTokens = 16;  // tokens per workgroup: the N extent of the MFMA
constexpr int kGateBatch = 8;    // K steps of 32 whose loads are in flight together

template <int E_>
__global__ __launch_bounds__(kGateThreads) void gate_router_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ gate_w, int64_t T, int H, int k, int renorm,
    int round_bf16, void* __restrict__ logits_out, float* __restrict__ out_w, int32_t* __restrict__ out_ids) {
    static_assert(E_ == 8 || E_ == 16, "experts sit in the 16 rows of one MFMA");
    __shared__ __attribute__((aligned(16))) float partial[kGateWaves][kGateTokens][E_];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int r16 = lane & 15;  // operand row: expert (M) resp. token (N)
    const int kq = lane >> 4;   // which 8 of the 32 K values of a step
    const int64_t t0 = static_cast<int64_t>(blockIdx.x) * kGateTokens;

    // this wave's K steps
    const int nsteps = (H + 31) / 32;
    const int per_wave = (nsteps + kGateWaves - 1) / kGateWaves;
    const int s_begin = wave * per_wave;
    const int s_end = (s_begin + per_wave < nsteps) ? s_begin + per_wave : nsteps;

    const bool tok_ok = (t0 + r16 < T);
    const uint16_t* xrow = x + (tok_ok ? t0 + r16 : 0) * H;
    const uint16_t* grow = gate_w + static_cast<int64_t>(r16 % E_) * H;

    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = s_begin; s0 < s_end; s0 += kGateBatch) {
        u32x4_t xa[kGateBatch], ga[kGateBatch];
#pragma unroll
        for (int i = 0; i < kGateBatch; ++i) {
            const int h = (s0 + i) * 32 + kq * 8;
            const bool ok = (s0 + i < s_end) && (h < H);  // H is a multiple of 8: a piece is inside or outside
            xa[i] = (ok && tok_ok) ? *reinterpret_cast<const u32x4_t*>(xrow + h) : u32x4_t{0u, 0u, 0u, 0u};
            ga[i] = ok ? *reinterpret_cast<const u32x4_t*>(grow + h) : u32x4_t{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int i = 0; i < kGateBatch; ++i)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ga[i]),
                                                          __builtin_bit_cast(bf16x8_t, xa[i]), acc, 0, 0, 0);
    }
    // the lane holds token r16, experts 4 * kq .. 4 * kq + 3
    if (4 * kq < E_) *reinterpret_cast<f32x4_t*>(&partial[wave][r16][4 * kq]) = acc;
    __syncthreads();

    // E adjacent lanes per token: 64 / E tokens per wavefront
    constexpr int kTokPerWave = kWave / E_;
    if (wave * kTokPerWave < kGateTokens) {  // whole waves leave together
        const int tok = wave * kTokPerWave + lane / E_;
        const int e = lane % E_;
        const int64_t t = t0 + tok;
        const bool valid = (t < T);
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < kGateWaves; ++w) v += partial[w][tok][e];
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

}  // namespace

bool gate_router_supported(int H, int E) {
    return (E == 8 || E == 16) && H % 8 == 0 && H > 0;
}

int launch_gate_router(const void* x, const void* gate_w, int64_t T, int H, int E, int k, int renorm,
                       int round_bf16, void* logits_out, float* w, int32_t* ids, hipStream_t s) {
    if (T == 0) return 0;
    if (!gate_router_supported(H, E)) return EM_ERR_UNSUPPORTED;
    const unsigned grid = static_cast<unsigned>(ceil_div(T, static_cast<int64_t>(kGateTokens)));
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    const uint16_t* gp = static_cast<const uint16_t*>(gate_w);
    if (E == 8)
        hipLaunchKernelGGL(gate_router_kernel<8>, dim3(grid), dim3(kGateThreads), 0, s, xp, gp, T, H, k, renorm,
                           round_bf16, logits_out, w, ids);
    else
        hipLaunchKernelGGL(gate_router_kernel<16>, dim3(grid), dim3(kGateThreads), 0, s, xp, gp, T, H, k, renorm,
                           round_bf16, logits_out, w, ids);
    return launch_status();
}

}  // namespace em
