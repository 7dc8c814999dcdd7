// Weight-streaming expert GEMM for decode batches (at most a few 16-row MFMA
// fragments of tokens per expert).  The layer is HBM-bound there: every byte
// of the active experts' w13 / w2 has to cross the memory bus once, the
// arithmetic is almost free.  The kernel is therefore organised around the
// weight stream:
//
//   * one workgroup = (expert, 64 weight rows, K slice); its four waves split
//     the K slice, so inside the main loop the waves never synchronise;
//   * each wave pulls 64 rows x 128 B per step with 16-byte loads, eight lanes
//     on one row (full 128-byte lines), keeps two steps in flight in registers,
//     and turns the rows into MFMA operand layout through a wave-private LDS
//     tile (pitch 144 B: conflict-free b128 reads);
//   * the few token rows (A operand) are read straight from L2 into operand
//     layout, prefetched as deep as the weights;
//   * the four partial accumulators meet once, at the end, in LDS.
//
//   MODE 1  64 rows = 32 gate rows j and the 32 up rows I + j of w13[e]; epilogue
//           act[p, j] = silu(g) * u with g, u still in fp32, rounded once (fp16, or bf16 with EM_FLAG_BF16_ACT)
//           (reference: Triton GEMM #1 + _C.silu_and_mul, fused_moe.py:250-272)
//   MODE 2  64 rows n of w2[e], K slice z of I; epilogue y[z, slot, n] = partial sum
//           (reference: Triton GEMM #2, fused_moe.py:282-287)
//
// Needs the sort done with 16-row blocks and the per-expert segment offsets.
#include "common.h"

namespace em {
namespace {

constexpr int kWaves = 4;
constexpr int kStep = 64;                 // K elements per step (128 B per weight row)
constexpr int kRows = 64;                 // weight rows per workgroup
constexpr int kPitch = kStep * 2 + 16;    // 144 B
constexpr int kMaxF = 2;                  // 16-row token fragments of a pass whose rows are fetched two steps ahead
// further fragments of the same pass, fetched in the step that uses them (w13 GEMM: up to 64 tokens an expert has at
// most 64 rows; the w2 GEMM runs here up to 8 tokens only, one fragment per expert, and keeps its registers)
template <int MODE> struct Extra { static constexpr int kMaxX = MODE == 1 ? 2 : 0; };

__device__ __forceinline__ u32x4_t ld16(const uint16_t* p) { return *reinterpret_cast<const u32x4_t*>(p); }
// Weights are read exactly once per call: a non-temporal load keeps the stream from
// displacing the token rows in L2 / Infinity Cache and measures ~15% faster than a
// plain load for this access pattern (7.0 vs 6.0 TB/s on a pure read of w13).
__device__ __forceinline__ u32x4_t ld16_stream(const uint16_t* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
}

// F16 (fp16 activations, MODE 2 only): the token rows are fp16 (MoeProblem::act_f16); the weight fragments are turned
// into fp16 between the LDS tile and the MFMA (not when they are fp16 in memory, MoeProblem::w2_f16), which costs
// this HBM-bound kernel nothing.
template <int MODE, bool F16>
__global__ __launch_bounds__(kWaves * 64, 2) void gemm_stream_kernel(MoeProblem p,
                                                                     const int32_t* __restrict__ seg_begin,
                                                                     int tiles_per_expert, int kslice) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[kWaves][kRows * kPitch];
    constexpr int kMaxX = Extra<MODE>::kMaxX;
    constexpr int kPassF = kMaxF + kMaxX;  // fragments per pass over the weight rows

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int expert = blockIdx.x / tiles_per_expert;
    const int tile = blockIdx.x - expert * tiles_per_expert;
    const int seg = seg_begin[expert];
    const int nfrag_total = (seg_begin[expert + 1] - seg) >> 4;
    if (nfrag_total == 0) return;  // expert without tokens: its weights are never read

    const int K = (MODE == 1) ? p.H : p.I;
    const int per_wave = kslice / kWaves;
    const int k_begin = blockIdx.y * kslice + wave * per_wave;
    const int nsteps = per_wave / kStep;

    // weight rows this lane loads: rows i*8 + lane/8 (i = 0..7), 16-byte chunk lane%8
    const int lrow = lane >> 3;
    const int lchunk = lane & 7;
    const uint16_t* brow[8];
    {
        const uint16_t* wbase;
        if (MODE == 1) {
            wbase = p.w13 + static_cast<int64_t>(expert) * 2 * p.I * p.H;
            const int j0 = tile * 32;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int r = i * 8 + lrow;
                const int64_t grow = (r < 32) ? (j0 + r) : (static_cast<int64_t>(p.I) + j0 + (r - 32));
                brow[i] = wbase + grow * K + k_begin + lchunk * 8;
            }
        } else {
            wbase = p.w2 + static_cast<int64_t>(expert) * p.H * p.I;
            const int n0 = tile * kRows;
#pragma unroll
            for (int i = 0; i < 8; ++i)
                brow[i] = wbase + static_cast<int64_t>(n0 + i * 8 + lrow) * K + k_begin + lchunk * 8;
        }
    }
    uint8_t* my = lds[wave];
    const int r16 = lane & 15;
    const int kq = lane >> 4;

    // A pass streams the workgroup's weight rows once for up to kPassF fragments.  With even routing a decode batch
    // has one or two fragments per expert: their token rows are prefetched as deep as the weights.  An expert that the
    // routing favours brings a third and fourth; their rows (L2 hits) are fetched in the step that multiplies them, which
    // costs that workgroup part of its prefetch distance but not a second pass over the weights.
    for (int f0 = 0; f0 < nfrag_total; f0 += kPassF) {
        const int nall = (nfrag_total - f0 < kPassF) ? nfrag_total - f0 : kPassF;
        const int nf = nall < kMaxF ? nall : kMaxF;
        const int nx = nall - nf;  // workgroup-uniform

        // token rows of this lane (operand layout: row r16 of each fragment)
        const uint16_t* arow[kPassF];
#pragma unroll
        for (int f = 0; f < kPassF; ++f) {
            arow[f] = nullptr;
            if (f < nall) {
                const int pos = seg + (f0 + f) * 16 + r16;
                if (MODE == 1) {
                    const int slot = p.sorted_ids[pos];
                    if (slot >= 0) arow[f] = p.x + static_cast<int64_t>(slot / p.top_k) * p.H + k_begin + kq * 8;
                } else {
                    arow[f] = p.act + static_cast<int64_t>(pos) * p.I + k_begin + kq * 8;
                }
            }
        }

        f32x4_t acc[kPassF][4];
#pragma unroll
        for (int f = 0; f < kPassF; ++f)
#pragma unroll
            for (int g = 0; g < 4; ++g) acc[f][g] = f32x4_t{0.f, 0.f, 0.f, 0.f};

        constexpr int kAW = 2;  // per fragment: two 32-wide K halves
        u32x4_t b0[8], b1[8], a0[kMaxF][kAW], a1[kMaxF][kAW];
        auto issue = [&](int s, u32x4_t(&b)[8], u32x4_t(&a)[kMaxF][kAW]) {
            const int koff = s * kStep;
#pragma unroll
            for (int i = 0; i < 8; ++i) b[i] = ld16_stream(brow[i] + koff);
#pragma unroll
            for (int f = 0; f < kMaxF; ++f)
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    a[f][ks] = (arow[f] != nullptr) ? ld16(arow[f] + koff + ks * 32) : u32x4_t{0, 0, 0, 0};
                }
        };
        auto consume = [&](int s, u32x4_t(&b)[8], u32x4_t(&a)[kMaxF][kAW]) {
            u32x4_t ax[kMaxX > 0 ? kMaxX : 1][kAW];
            if (kMaxX > 0 && nx > 0) {
#pragma unroll
                for (int f = 0; f < kMaxX; ++f)
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks)
                        ax[f][ks] = (arow[kMaxF + f] != nullptr) ? ld16(arow[kMaxF + f] + s * kStep + ks * 32) : u32x4_t{0, 0, 0, 0};
            }
#pragma unroll
            for (int i = 0; i < 8; ++i)
                *reinterpret_cast<u32x4_t*>(my + (i * 8 + lrow) * kPitch + lchunk * 16) = b[i];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                bf16x8_t bf[4];
                f16x8_t hf[4];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    bf[g] = *reinterpret_cast<const bf16x8_t*>(my + (g * 16 + r16) * kPitch + ks * 64 + kq * 16);
                    if (F16) {
                        if (p.w2_f16) __builtin_memcpy(&hf[g], &bf[g], 16);
                        else hf[g] = bf16x8_to_f16x8(bf[g]);
                    }
                }
#pragma unroll
                for (int f = 0; f < kMaxF; ++f) {
                    if (f < nf) {
                        if (F16) {
                            f16x8_t af;
                            __builtin_memcpy(&af, &a[f][ks], 16);
#pragma unroll
                            for (int g = 0; g < 4; ++g)
                                acc[f][g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, hf[g], acc[f][g], 0, 0, 0);
                        } else {
                            bf16x8_t af;
                            __builtin_memcpy(&af, &a[f][ks], 16);
#pragma unroll
                            for (int g = 0; g < 4; ++g)
                                acc[f][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, bf[g], acc[f][g], 0, 0, 0);
                        }
                    }
                }
                if (kMaxX > 0 && nx > 0) {
#pragma unroll
                    for (int f = 0; f < kMaxX; ++f) {
                        if (f < nx) {
                            if (F16) {
                                f16x8_t af;
                                __builtin_memcpy(&af, &ax[f][ks], 16);
#pragma unroll
                                for (int g = 0; g < 4; ++g)
                                    acc[kMaxF + f][g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, hf[g], acc[kMaxF + f][g], 0, 0, 0);
                            } else {
                                bf16x8_t af;
                                __builtin_memcpy(&af, &ax[f][ks], 16);
#pragma unroll
                                for (int g = 0; g < 4; ++g)
                                    acc[kMaxF + f][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, bf[g], acc[kMaxF + f][g], 0, 0, 0);
                            }
                        }
                    }
                }
            }
        };

        if (nsteps > 0) issue(0, b0, a0);
        if (nsteps > 1) issue(1, b1, a1);
        for (int s = 0; s < nsteps; s += 2) {
            consume(s, b0, a0);
            if (s + 2 < nsteps) issue(s + 2, b0, a0);
            if (s + 1 < nsteps) {
                consume(s + 1, b1, a1);
                if (s + 3 < nsteps) issue(s + 3, b1, a1);
            }
        }

        // ---- meet the four K-slice partials in LDS (reusing the staging tiles), kMaxF fragments at a time ----
        for (int h0 = 0; h0 < nall; h0 += kMaxF) {
            const int nh = (nall - h0 < kMaxF) ? nall - h0 : kMaxF;
            __syncthreads();
            f32x4_t* red = reinterpret_cast<f32x4_t*>(&lds[0][0]);  // [wave][f][g][lane]
#pragma unroll
            for (int f = 0; f < kMaxF; ++f)
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    red[((wave * kMaxF + f) * 4 + g) * 64 + lane] = (kMaxX == 0 || h0 == 0) ? acc[f][g] : acc[(kMaxF + f) % kPassF][g];
            __syncthreads();
            auto total = [&](int f, int g) {
                f32x4_t t = red[((0 * kMaxF + f) * 4 + g) * 64 + lane];
#pragma unroll
                for (int w = 1; w < kWaves; ++w) t += red[((w * kMaxF + f) * 4 + g) * 64 + lane];
                return t;
            };
            if (MODE == 1) {
                if (wave < 2) {
                    const int j = tile * 32 + wave * 16 + r16;
                    for (int f = 0; f < nh; ++f) {
                        const f32x4_t g = total(f, wave);
                        const f32x4_t u = total(f, 2 + wave);
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            const int64_t row = seg + (f0 + h0 + f) * 16 + kq * 4 + v;
                            store_act(p, row * p.I + j, silu_mul(g[v], u[v]));
                        }
                    }
                }
            } else {
                float* ybase = p.y + static_cast<int64_t>(blockIdx.y) * p.T * p.top_k * p.H;
                const int n = tile * kRows + wave * 16 + r16;
                for (int f = 0; f < nh; ++f) {
                    const f32x4_t t = total(f, wave);
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int slot = p.sorted_ids[seg + (f0 + h0 + f) * 16 + kq * 4 + v];
                        if (slot >= 0) ybase[static_cast<int64_t>(slot) * p.H + n] = t[v];
                    }
                }
            }
        }
        __syncthreads();  // staging tiles are reused by the next pass
    }
}

}  // namespace

bool stream_supported(const MoeProblem& p) {
    return p.block == 16 && p.H % 256 == 0 && p.I % 32 == 0 && p.H % kRows == 0 && p.ksplit >= 1 &&
           p.I % (p.ksplit * kWaves * kStep) == 0;
}

int launch_gemm_stream(const MoeProblem& p, const int32_t* seg_begin, int mode, hipStream_t s) {
    if (!stream_supported(p)) return EM_ERR_UNSUPPORTED;
    static_assert(kWaves * kMaxF * 4 * 64 * 16 <= kWaves * kRows * kPitch, "reduction buffer must fit the staging tiles");
    const dim3 blk(kWaves * 64);
    if (mode == 1) {
        const int tiles = p.I / 32;
        launch((gemm_stream_kernel<1, false>), dim3(static_cast<unsigned>(p.E * tiles), 1), blk, 0, s, p,
                           seg_begin, tiles, p.H);
    } else {
        const int tiles = p.H / kRows;
        const dim3 grid(static_cast<unsigned>(p.E * tiles), static_cast<unsigned>(p.ksplit));
        if (p.act_f16)
            launch((gemm_stream_kernel<2, true>), grid, blk, 0, s, p, seg_begin, tiles, p.I / p.ksplit);
        else
            launch((gemm_stream_kernel<2, false>), grid, blk, 0, s, p, seg_begin, tiles, p.I / p.ksplit);
    }
    return launch_status();
}

}  // namespace em
