// Router gate fused with the router: logits[t, e] = sum_h x[t, h] * gate_w[e, h], then the
// top-k softmax of router.hip, in one launch.
//
// The reference computes the logits with a bf16 linear layer in the model
// (models/mixtral.py:40-42,59; layers/linear.py:53-54: F.linear(x, weight) -> bf16 [T, E]) and
// hands them to the MoE layer.  Here a workgroup keeps the E x H gate matrix in LDS (64 KB for
// 8 x 4096) and every wavefront owns whole tokens: the 64 lanes split the row of x into 16-byte
// pieces, accumulate E partial dot products in fp32, and a butterfly
// leaves logit e in lane e -- exactly what the router's selection expects.  With round_bf16 the
// fp32 sum is rounded to bf16 first, as the reference's linear does (ties then exist and go to
// the lowest expert index); without it the fp32 logits are used as they are.
// The kernel is bound by reading x once (T * H * 2 bytes).
#include "router_device.h"

namespace em {
namespace {

constexpr int kGateWaves = 8;
constexpr int kGateThreads = kGateWaves * kWave;
constexpr int kChunk = 8;  // 16-byte pieces of x a lane holds at once: one chunk = 4096 elements per wave

// fp32 dot product of 8 values of x with a 16-byte piece (8 bf16) of a gate row, added to acc
__device__ __forceinline__ float dot8(const u32x4_t a, const u32x4_t b, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        acc = fmaf(bf16_lo(a[i]), bf16_lo(b[i]), acc);
        acc = fmaf(bf16_hi(a[i]), bf16_hi(b[i]), acc);
    }
    return acc;
}

// pieces [chunk * 512, chunk * 512 + 512) of one row of x, piece i * 64 + lane in reg[i]
__device__ __forceinline__ void load_chunk(u32x4_t (&reg)[kChunk], const uint16_t* __restrict__ x, int64_t t, int H,
                                           int chunk, int lane, int pieces) {
    const u32x4_t* xrow = reinterpret_cast<const u32x4_t*>(x + t * H);
#pragma unroll
    for (int i = 0; i < kChunk; ++i) {
        const int c = (chunk * kChunk + i) * kWave + lane;
        if (c < pieces) reg[i] = xrow[c];
    }
}

template <int E_>
__global__ __launch_bounds__(kGateThreads) void gate_router_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ gate_w, int64_t T, int H, int k, int renorm,
    int round_bf16, void* __restrict__ logits_out, float* __restrict__ out_w, int32_t* __restrict__ out_ids,
    int tokens_per_wave) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];  // gate_w, E_ rows of H bf16
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int pieces = H / 8;  // 16-byte pieces per row
    const int nchunks = (pieces + kChunk * kWave - 1) / (kChunk * kWave);

    const int64_t t_begin = (static_cast<int64_t>(blockIdx.x) * kGateWaves + wave) * tokens_per_wave;
    int64_t t_end = t_begin + tokens_per_wave;
    if (t_end > T) t_end = T;

    // the first chunk of x is on its way while the workgroup copies gate_w into LDS
    u32x4_t cur[kChunk], nxt[kChunk];
    if (t_begin < t_end) load_chunk(cur, x, t_begin, H, 0, lane, pieces);
    for (int c = tid; c < E_ * pieces; c += kGateThreads)
        reinterpret_cast<u32x4_t*>(smem)[c] = reinterpret_cast<const u32x4_t*>(gate_w)[c];
    __syncthreads();

    float acc[E_];
#pragma unroll
    for (int e = 0; e < E_; ++e) acc[e] = 0.0f;
    int chunk = 0;
    for (int64_t t = t_begin; t < t_end;) {
        // request the next chunk (of this token or of the next one) before working on the current one
        const bool last_chunk = (chunk + 1 == nchunks);
        const int64_t t_next = last_chunk ? t + 1 : t;
        const int chunk_next = last_chunk ? 0 : chunk + 1;
        if (t_next < t_end) load_chunk(nxt, x, t_next, H, chunk_next, lane, pieces);
#pragma unroll
        for (int i = 0; i < kChunk; ++i) {
            const int c = (chunk * kChunk + i) * kWave + lane;
            if (c < pieces) {
#pragma unroll
                for (int e = 0; e < E_; ++e)
                    acc[e] = dot8(cur[i], reinterpret_cast<const u32x4_t*>(smem)[e * pieces + c], acc[e]);
            }
        }
        if (last_chunk) {
            // every lane ends with all E sums; lane e keeps sum e
            float v = -INFINITY;
#pragma unroll
            for (int e = 0; e < E_; ++e) {
                float s = acc[e];
#pragma unroll
                for (int off = kWave / 2; off > 0; off >>= 1) s += __shfl_xor(s, off);
                if (lane == e) v = s;
                acc[e] = 0.0f;
            }
            if (lane < E_) {
                if (round_bf16) {
                    const uint16_t b = f32_to_bf16_bits(v);
                    v = bf16_bits_to_f32(b);
                    if (logits_out != nullptr) static_cast<uint16_t*>(logits_out)[t * E_ + lane] = b;
                } else if (logits_out != nullptr) {
                    static_cast<float*>(logits_out)[t * E_ + lane] = v;
                }
                if (v != v) v = -INFINITY;  // a NaN logit can never be selected
            }
            route_from_logit(v, lane, t, E_, k, renorm, out_w, out_ids);
        }
#pragma unroll
        for (int i = 0; i < kChunk; ++i) cur[i] = nxt[i];
        t = t_next;
        chunk = chunk_next;
    }
}

}  // namespace

bool gate_router_supported(int H, int E) {
    return (E == 8 || E == 16) && H % 8 == 0 && static_cast<int64_t>(E) * H * 2 <= 160 * 1024;
}

int launch_gate_router(const void* x, const void* gate_w, int64_t T, int H, int E, int k, int renorm,
                       int round_bf16, void* logits_out, float* w, int32_t* ids, hipStream_t s) {
    if (T == 0) return 0;
    if (!gate_router_supported(H, E)) return EM_ERR_UNSUPPORTED;
    // enough workgroups to fill the GPU, few enough that copying gate_w into LDS stays small next to reading x
    int tpw = static_cast<int>(ceil_div(T, static_cast<int64_t>(kGateWaves) * 512));
    tpw = tpw < 1 ? 1 : (tpw > 16 ? 16 : tpw);
    const unsigned grid = static_cast<unsigned>(ceil_div(T, static_cast<int64_t>(kGateWaves) * tpw));
    const int lds = E * H * 2;
    const void* kernel = (E == 8) ? reinterpret_cast<const void*>(gate_router_kernel<8>)
                                  : reinterpret_cast<const void*>(gate_router_kernel<16>);
    // Opt in to the dynamic LDS size (idempotent runtime call; gate matrices beyond 64 KB need it).
    hipError_t attr = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (attr != hipSuccess) return static_cast<int>(attr);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    const uint16_t* gp = static_cast<const uint16_t*>(gate_w);
    if (E == 8)
        hipLaunchKernelGGL(gate_router_kernel<8>, dim3(grid), dim3(kGateThreads), lds, s, xp, gp, T, H, k, renorm,
                           round_bf16, logits_out, w, ids, tpw);
    else
        hipLaunchKernelGGL(gate_router_kernel<16>, dim3(grid), dim3(kGateThreads), lds, s, xp, gp, T, H, k, renorm,
                           round_bf16, logits_out, w, ids, tpw);
    return launch_status();
}

}  // namespace em
