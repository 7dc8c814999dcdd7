// Shape-generic grouped expert GEMM on bf16 MFMA (v_mfma_f32_16x16x32_bf16).
// This is the always-correct path: any H, I that are multiples of 8, any
// sorted-block size in {16, 32} or a multiple of 64.  The tuned decode / prefill kernels replace it
// for the shapes they support.
//
//   MODE 1  act[p, j] = bf16( silu(x[tok(p)] . w13[e, j]) * (x[tok(p)] . w13[e, I + j]) )
//           (reference: Triton GEMM #1 + _C.silu_and_mul, fused_moe.py:250-272, with
//           gate and up kept in fp32 until the single rounding of the product)
//   MODE 2  y[z, slot(p), n] = sum over the z-th K slice of act[p, :] . w2[e, n, :]
//           (reference: Triton GEMM #2, fused_moe.py:282-287; the routing weight and
//           the top-k sum are applied in fp32 by the combine kernel)
// p runs over sorted (padded) positions; one workgroup owns one sorted block
// (= one expert) times 128 weight rows and walks K in steps of 64 through a
// double-buffered LDS tile.  Four waves split the weight rows, all share the
// token rows.
#include "common.h"

namespace em {
namespace {

constexpr int kThreads = 256;
constexpr int kBR = 128;              // weight rows per tile
constexpr int kBK = 64;               // K elements per stage
constexpr int kPitch = kBK * 2 + 16;  // LDS row pitch in bytes; /16 is odd -> conflict-free b128 reads
constexpr int kChunksPerRow = kBK / 8;

__device__ __forceinline__ u32x4_t ld16(const void* p) { return *reinterpret_cast<const u32x4_t*>(p); }

template <int MODE, int MF>
__global__ __launch_bounds__(kThreads) void gemm_generic_kernel(MoeProblem p) {
    constexpr int BM = MF * 16;
    constexpr int kAChunks = BM * kChunksPerRow;                  // 16-byte chunks of the A tile
    constexpr int kAPerThread = (kAChunks + kThreads - 1) / kThreads;
    constexpr int kBPerThread = kBR * kChunksPerRow / kThreads;   // 4
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[2][BM * kPitch];
    __shared__ __attribute__((aligned(16))) uint8_t lds_b[2][kBR * kPitch];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int64_t m0 = static_cast<int64_t>(blockIdx.y) * BM;
    if (m0 >= p.post_pad[0]) return;
    const int expert = p.expert_ids[m0 / p.block];

    const int K = (MODE == 1) ? p.H : p.I;
    const int Nw = (MODE == 1) ? p.I : p.H;  // output columns of this stage
    const int n0 = blockIdx.x * ((MODE == 1) ? kBR / 2 : kBR);
    int k_begin = 0, k_end = K;
    if (MODE == 2 && p.ksplit > 1) {
        const int per = static_cast<int>(round_up(ceil_div(K, p.ksplit), kBK));
        k_begin = blockIdx.z * per;
        k_end = (k_begin + per < K) ? k_begin + per : K;
        if (k_begin >= k_end) k_end = k_begin;  // empty slice still writes zeros below
    }

    // ---- per-thread source rows (loop invariant) ----
    const uint16_t* a_src[kAPerThread];
    int a_row[kAPerThread], a_kc[kAPerThread];
#pragma unroll
    for (int i = 0; i < kAPerThread; ++i) {
        const int c = tid + i * kThreads;
        a_row[i] = c / kChunksPerRow;
        a_kc[i] = (c % kChunksPerRow) * 8;
        a_src[i] = nullptr;
        if (c < kAChunks) {
            if (MODE == 1) {
                const int slot = p.sorted_ids[m0 + a_row[i]];
                if (slot >= 0) a_src[i] = p.x + static_cast<int64_t>(slot / p.top_k) * p.H;
            } else {
                a_src[i] = p.act + (m0 + a_row[i]) * static_cast<int64_t>(p.I);
            }
        }
    }
    const uint16_t* b_src[kBPerThread];
    int b_row[kBPerThread], b_kc[kBPerThread];
    const uint16_t* wbase = (MODE == 1) ? p.w13 + static_cast<int64_t>(expert) * 2 * p.I * p.H
                                        : p.w2 + static_cast<int64_t>(expert) * p.H * p.I;
#pragma unroll
    for (int i = 0; i < kBPerThread; ++i) {
        const int c = tid + i * kThreads;
        b_row[i] = c / kChunksPerRow;
        b_kc[i] = (c % kChunksPerRow) * 8;
        int64_t grow;
        bool ok;
        if (MODE == 1) {
            const int half = kBR / 2;
            const int j = n0 + (b_row[i] % half);
            ok = j < Nw;
            grow = (b_row[i] < half) ? j : static_cast<int64_t>(p.I) + j;
        } else {
            grow = n0 + b_row[i];
            ok = grow < Nw;
        }
        b_src[i] = ok ? wbase + grow * K : nullptr;
    }

    u32x4_t a_reg[kAPerThread], b_reg[kBPerThread];
    auto load_global = [&](int k0) {
#pragma unroll
        for (int i = 0; i < kAPerThread; ++i) {
            const int k = k0 + a_kc[i];
            a_reg[i] = (a_src[i] != nullptr && k < k_end) ? ld16(a_src[i] + k) : u32x4_t{0, 0, 0, 0};
        }
#pragma unroll
        for (int i = 0; i < kBPerThread; ++i) {
            const int k = k0 + b_kc[i];
            b_reg[i] = (b_src[i] != nullptr && k < k_end) ? ld16(b_src[i] + k) : u32x4_t{0, 0, 0, 0};
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < kAPerThread; ++i)
            if (tid + i * kThreads < kAChunks)
                *reinterpret_cast<u32x4_t*>(&lds_a[buf][a_row[i] * kPitch + a_kc[i] * 2]) = a_reg[i];
#pragma unroll
        for (int i = 0; i < kBPerThread; ++i)
            *reinterpret_cast<u32x4_t*>(&lds_b[buf][b_row[i] * kPitch + b_kc[i] * 2]) = b_reg[i];
    };

    f32x4_t acc[MF][2];
#pragma unroll
    for (int f = 0; f < MF; ++f) acc[f][0] = acc[f][1] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // weight rows of this wave inside the LDS tile
    const int frow0 = (MODE == 1) ? wave * 16 : wave * 32;
    const int frow1 = (MODE == 1) ? kBR / 2 + wave * 16 : wave * 32 + 16;
    const int r16 = lane & 15;
    const int kq = lane >> 4;

    const int nk = static_cast<int>(ceil_div(k_end - k_begin, kBK));
    if (nk > 0) {
        load_global(k_begin);
        store_lds(0);
    }
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < nk) load_global(k_begin + (kt + 1) * kBK);
#pragma unroll
        for (int ks = 0; ks < kBK / 32; ++ks) {
            const int koff = ks * 64 + kq * 16;
            const bf16x8_t b0 = *reinterpret_cast<const bf16x8_t*>(&lds_b[buf][(frow0 + r16) * kPitch + koff]);
            const bf16x8_t b1 = *reinterpret_cast<const bf16x8_t*>(&lds_b[buf][(frow1 + r16) * kPitch + koff]);
#pragma unroll
            for (int f = 0; f < MF; ++f) {
                const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(&lds_a[buf][(f * 16 + r16) * kPitch + koff]);
                acc[f][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b0, acc[f][0], 0, 0, 0);
                acc[f][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b1, acc[f][1], 0, 0, 0);
            }
        }
        if (kt + 1 < nk) store_lds(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: lane holds column r16, rows 4*kq + v of every 16x16 fragment ----
    if (MODE == 1) {
        const int j = n0 + wave * 16 + r16;
        if (j < Nw) {
#pragma unroll
            for (int f = 0; f < MF; ++f)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float g = acc[f][0][v];
                    const float u = acc[f][1][v];
                    store_act(p, (m0 + f * 16 + kq * 4 + v) * static_cast<int64_t>(p.I) + j, silu_mul(g, u));
                }
        }
    } else {
        float* ybase = p.y + static_cast<int64_t>(blockIdx.z) * p.T * p.top_k * p.H;
#pragma unroll
        for (int f = 0; f < MF; ++f)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int slot = p.sorted_ids[m0 + f * 16 + kq * 4 + v];
                if (slot < 0) continue;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int n = n0 + wave * 32 + h * 16 + r16;
                    if (n < Nw) {
                        float* dst = ybase + static_cast<int64_t>(slot) * p.H + n;
                        *dst = p.y_accumulate ? *dst + acc[f][h][v] : acc[f][h][v];
                    }
                }
            }
    }
}

// out[t, :] = sum_j w[t, j] * sum_z y[z, t*k + j, :]   (fp32, one final rounding)
// kStream: the partial results are too many to still sit in the caches when they are read (exactly once):
// streaming loads.  Small sets are read back out of L2, where streaming loads of just-written lines are slower.
template <bool kOutF32, bool kStream>
__global__ __launch_bounds__(256) void combine_kernel(const float* __restrict__ y, const float* __restrict__ w,
                                                      void* __restrict__ out, int64_t T, int H, int top_k,
                                                      int ksplit) {
    const int64_t t = blockIdx.x;
    const int64_t zstride = T * top_k * static_cast<int64_t>(H);
    for (int h = (blockIdx.y * 256 + threadIdx.x) * 4; h < H; h += gridDim.y * 256 * 4) {
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
        for (int j = 0; j < top_k; ++j) {
            const float wj = w[t * top_k + j];
            const float* row = y + (t * top_k + j) * static_cast<int64_t>(H) + h;
            auto load = [](const float* ptr) {
                return kStream ? __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(ptr))
                               : *reinterpret_cast<const f32x4_t*>(ptr);
            };
            f32x4_t s = load(row);
            for (int z = 1; z < ksplit; ++z) s += load(row + z * zstride);
            acc += wj * s;
        }
        if (kOutF32) {
            *reinterpret_cast<f32x4_t*>(static_cast<float*>(out) + t * H + h) = acc;
        } else {
            u32x2_t o = {pack_bf16(acc[0], acc[1]), pack_bf16(acc[2], acc[3])};
            *reinterpret_cast<u32x2_t*>(static_cast<uint16_t*>(out) + t * H + h) = o;
        }
    }
}

// The same sum over fp16 partial results: eight columns per thread (16-byte loads).  An fp16 infinity marks a value
// that did not fit the format; it stands as float32 at the same index of `wide` (rare: looked for only when a sum over
// the K slices is not finite).
template <bool kOutF32, bool kStream>
__global__ __launch_bounds__(256) void combine_f16_kernel(const uint16_t* __restrict__ y, const float* __restrict__ wide,
                                                          const float* __restrict__ w, void* __restrict__ out, int64_t T,
                                                          int H, int top_k, int ksplit) {
    const int64_t t = blockIdx.x;
    const int64_t zstride = T * top_k * static_cast<int64_t>(H);
    for (int h = (blockIdx.y * 256 + threadIdx.x) * 8; h < H; h += gridDim.y * 256 * 8) {
        float acc[8] = {};
        for (int j = 0; j < top_k; ++j) {
            const float wj = w[t * top_k + j];
            const int64_t at = (t * top_k + j) * static_cast<int64_t>(H) + h;
            const uint16_t* row = y + at;
            float s[8] = {};
            for (int z = 0; z < ksplit; ++z) {
                const u32x4_t* ptr = reinterpret_cast<const u32x4_t*>(row + z * zstride);
                const u32x4_t v = kStream ? __builtin_nontemporal_load(ptr) : *ptr;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    s[2 * i] += f16_bits_to_f32(static_cast<uint16_t>(v[i]));
                    s[2 * i + 1] += f16_bits_to_f32(static_cast<uint16_t>(v[i] >> 16));
                }
            }
            uint32_t seen = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t mag = __float_as_uint(s[i]) & 0x7fffffffu;
                seen = mag > seen ? mag : seen;
            }
            if (seen >= 0x7f800000u) {  // an infinity or a NaN among the sums: add again, escaped values from `wide`
#pragma unroll
                for (int i = 0; i < 8; ++i) s[i] = 0.0f;
                for (int z = 0; z < ksplit; ++z)
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const uint16_t bits = row[z * zstride + i];
                        s[i] += ((bits & 0x7fffu) == 0x7c00u) ? wide[at + z * zstride + i] : f16_bits_to_f32(bits);
                    }
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[i] += wj * s[i];
        }
        if (kOutF32) {
            float* o = static_cast<float*>(out) + t * H + h;
            *reinterpret_cast<f32x4_t*>(o) = f32x4_t{acc[0], acc[1], acc[2], acc[3]};
            *reinterpret_cast<f32x4_t*>(o + 4) = f32x4_t{acc[4], acc[5], acc[6], acc[7]};
        } else {
            const u32x4_t o = {pack_bf16(acc[0], acc[1]), pack_bf16(acc[2], acc[3]), pack_bf16(acc[4], acc[5]),
                               pack_bf16(acc[6], acc[7])};
            *reinterpret_cast<u32x4_t*>(static_cast<uint16_t*>(out) + t * H + h) = o;
        }
    }
}

}  // namespace

int launch_gemm_generic(const MoeProblem& p, int mode, hipStream_t s) {
    // one row tile never spans experts: tile height = the sort block (16 or 32) or 64 for larger blocks
    if (p.block != 16 && p.block != 32 && p.block % 64 != 0) return EM_ERR_UNSUPPORTED;
    const int tile_rows = (p.block < 64) ? p.block : 64;
    const unsigned mblocks = static_cast<unsigned>(p.sorted_len / tile_rows);
    if (mblocks == 0) return 0;
    const dim3 blk(kThreads);
    const dim3 grid = (mode == 1) ? dim3(static_cast<unsigned>(ceil_div(p.I, kBR / 2)), mblocks, 1)
                                  : dim3(static_cast<unsigned>(ceil_div(p.H, kBR)), mblocks,
                                         static_cast<unsigned>(p.ksplit));
#define EM_LAUNCH_GENERIC(MODE)                                                             \
    do {                                                                                    \
        if (tile_rows == 16) launch((gemm_generic_kernel<MODE, 1>), grid, blk, 0, s, p);      \
        else if (tile_rows == 32) launch((gemm_generic_kernel<MODE, 2>), grid, blk, 0, s, p); \
        else launch((gemm_generic_kernel<MODE, 4>), grid, blk, 0, s, p);                      \
    } while (0)
    if (mode == 1) EM_LAUNCH_GENERIC(1);
    else EM_LAUNCH_GENERIC(2);
#undef EM_LAUNCH_GENERIC
    return launch_status();
}

int launch_combine(const MoeProblem& p, void* out, int out_f32, hipStream_t s) {
    if (p.T == 0) return 0;
    // beyond the memory-side cache (256 MB) the partial results come back from HBM
    const bool stream = static_cast<int64_t>(p.ksplit) * p.T * p.top_k * p.H * (p.y_f16 ? 2 : 4) > (int64_t{256} << 20);
    if (p.y_f16) {
        if (p.H % 8 != 0) return EM_ERR_UNSUPPORTED;
        const unsigned cols = static_cast<unsigned>(ceil_div(p.H, 2048));
        const dim3 grid(static_cast<unsigned>(p.T), cols < 8 ? cols : 8);
        auto go = [&](auto kernel) {
            launch(kernel, grid, dim3(256), 0, s, reinterpret_cast<const uint16_t*>(p.y), p.y_wide, p.topk_w, out, p.T,
                   p.H, p.top_k, p.ksplit);
        };
        if (out_f32) { if (stream) go(combine_f16_kernel<true, true>); else go(combine_f16_kernel<true, false>); }
        else { if (stream) go(combine_f16_kernel<false, true>); else go(combine_f16_kernel<false, false>); }
        return launch_status();
    }
    const unsigned cols = static_cast<unsigned>(ceil_div(p.H, 1024));
    const dim3 grid(static_cast<unsigned>(p.T), cols < 8 ? cols : 8);
    auto go = [&](auto kernel) {
        launch(kernel, grid, dim3(256), 0, s, p.y, p.topk_w, out, p.T, p.H, p.top_k, p.ksplit);
    };
    if (out_f32) { if (stream) go(combine_kernel<true, true>); else go(combine_kernel<true, false>); }
    else { if (stream) go(combine_kernel<false, true>); else go(combine_kernel<false, false>); }
    return launch_status();
}

}  // namespace em
