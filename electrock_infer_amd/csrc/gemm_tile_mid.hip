// Tiled grouped expert GEMM for batches between decode and prefill size (a few dozen
// rows per expert).  The weights still have to be streamed once from HBM, as in decode,
// but there are too many token rows for the streaming kernel's operand-from-L2 scheme and
// its half-rate 16x16x32 MFMA.  This kernel is the 256-row tiled kernel cut down in M so
// that LDS holds a deeper copy ring:
//
//   workgroup  512 threads = 8 waves as 2 (M) x 4 (N); tile of up to 64 (MI = 1) or 128 (MI = 2)
//              sorted rows x 256 weight rows; wave sub-tile (32 MI) x 64 on
//              v_mfma_f32_32x32x16_bf16
//   ring       three stages of 8 MI KB of token rows + 32 KB of weight rows (K step 64),
//              two of them in flight while the third is multiplied: 80-96 KB per CU on the
//              way from HBM, which is what covers its latency at this CU's share of 8 TB/s
//   tiles      experts are padded to 32 rows by the sort and cut into tiles; the last tile
//              of an expert holds what is left (a multiple of 32) and waves without rows
//              do not multiply.  The copy count per wave and stage stays fixed (rows that do not
//              exist re-read row 0), so completion can be counted with s_waitcnt vmcnt.
//   the rest   LDS swizzle, operand pipelining across the barrier, gate/up pairing in one
//              lane, XCD-aware tile order, split-K for w2 and the LDS-turned epilogues are
//              those of the 256-row kernel.
#include "common.h"
#include "lds_copy.h"

namespace em {
namespace {

constexpr int kTN = 256, kTK = 64;
constexpr int kThreads = 512;
constexpr int kNStage = 3;
constexpr int kBBytes = kTN * kTK * 2;               // 32 KB
template <int MI> struct Geo {
    static constexpr int kTM = 64 * MI;                          // rows per tile
    static constexpr int kABytes = kTM * kTK * 2;                // 8 or 16 KB
    static constexpr int kStageBytes = kABytes + kBBytes;        // 40 or 48 KB
    static constexpr int kLdsBytes = kNStage * kStageBytes;      // 120 or 144 KB
    static constexpr int kCopies = kStageBytes / (kThreads * 16);  // per thread and stage: MI of A, 4 of B
};
constexpr int kGroupM = 4;
constexpr int kXcds = 8;
constexpr int kRowBlock = 32;

template <int MODE, int MI>
__global__ __launch_bounds__(kThreads, 1) void gemm_tile_mid_kernel(MoeProblem p, const int32_t* __restrict__ seg_begin,
                                                                   int ntiles_n, int kslice) {
    constexpr int kTM = Geo<MI>::kTM, kABytes = Geo<MI>::kABytes, kStageBytes = Geo<MI>::kStageBytes,
                  kCopies = Geo<MI>::kCopies;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    int mtiles = 0;
    for (int e = 0; e < p.E; ++e) mtiles += (seg_begin[e + 1] - seg_begin[e] + kTM - 1) / kTM;
    const int total = mtiles * ntiles_n;
    const int per_xcd = (total + kXcds - 1) / kXcds;
    const int xcd = blockIdx.x % kXcds;
    const int local = blockIdx.x / kXcds;
    const int logical = xcd * per_xcd + local;
    if (local >= per_xcd || logical >= total) return;
    const int group_sz = kGroupM * ntiles_n;
    const int group = logical / group_sz;
    const int in_group = logical - group * group_sz;
    const int rows_in_group = (mtiles - group * kGroupM < kGroupM) ? mtiles - group * kGroupM : kGroupM;
    const int nt = in_group / rows_in_group;
    int mt = group * kGroupM + in_group % rows_in_group;
    int expert = 0;
    for (; expert < p.E - 1; ++expert) {
        const int t = (seg_begin[expert + 1] - seg_begin[expert] + kTM - 1) / kTM;
        if (mt < t) break;
        mt -= t;
    }
    const int64_t m0 = seg_begin[expert] + static_cast<int64_t>(mt) * kTM;
    const int rows_left = seg_begin[expert + 1] - static_cast<int>(m0);
    const int valid = rows_left < kTM ? rows_left : kTM;  // multiple of 32

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 2;
    const int wn = wave & 3;
    const int K = (MODE == 1) ? p.H : p.I;
    const int k_begin = blockIdx.y * kslice;

    // ---- copy plan (per stage): copies 0..MI-1 = 8 token rows each, the other four = weight rows.
    // Byte o of a region holds piece q ^ (u & 7) of 2-row group u = o / 256, q = (row & 1) * 8 + piece.
    const uint16_t* src[kCopies];
    const uint16_t* wbase = (MODE == 1) ? p.w13 + static_cast<int64_t>(expert) * 2 * p.I * p.H
                                        : p.w2 + static_cast<int64_t>(expert) * p.H * p.I;
#pragma unroll
    for (int n = 0; n < kCopies; ++n) {
        const int o = (n < MI ? n : n - MI) * 8192 + wave * 1024 + lane * 16;
        const int u = o >> 8;
        const int q = ((o >> 4) & 15) ^ (u & 7);
        const int r = u * 2 + (q >> 3);
        const int piece = q & 7;
        if (n < MI) {
            const int rr = (r < valid) ? r : 0;
            if (MODE == 1) {
                const int slot = p.sorted_ids[m0 + rr];
                const int tok = (slot >= 0) ? slot / p.top_k : 0;  // pad rows multiply token 0; never stored
                src[n] = p.x + static_cast<int64_t>(tok) * p.H + k_begin + piece * 8;
            } else {
                src[n] = p.act + (m0 + rr) * static_cast<int64_t>(p.I) + k_begin + piece * 8;
            }
        } else {
            int64_t grow;
            if (MODE == 1)  // LDS row r of the B tile: wave column r/64, gate (0) or up (1) half, j offset r%32
                grow = static_cast<int64_t>((r >> 5) & 1) * p.I + nt * 128 + (r >> 6) * 32 + (r & 31);
            else
                grow = static_cast<int64_t>(nt) * kTN + r;
            src[n] = wbase + grow * K + k_begin + piece * 8;
        }
    }
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem));
    const uint32_t dma_base = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
    auto issue = [&](int stage_k, int buf) {
        const int k0 = stage_k * kTK;
#pragma unroll
        for (int n = 0; n < kCopies; ++n)
            if (n < MI) dma16(src[n] + k0, dma_base + buf * kStageBytes + n * 8192);                             // token rows: shared
            else dma16_stream(src[n] + k0, dma_base + buf * kStageBytes + kABytes + (n - MI) * 8192);   // weight rows: read once
    };

    f32x16_t acc[MI][2];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.f;

    const int r32 = lane & 31;
    const int kh = lane >> 5;
    const int sw = (r32 >> 1) & 7;
    int a_off[4], b_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        const int piece = (ks * 2 + kh) ^ sw;
        const int ra = wm * (32 * MI) + r32, rb = wn * 64 + r32;
        a_off[ks] = (ra >> 1) * 256 + ((ra & 1) * 8 + piece) * 16;
        b_off[ks] = kABytes + (rb >> 1) * 256 + ((rb & 1) * 8 + piece) * 16;
    }
    int nmi = (valid - wm * (32 * MI) + 31) / 32;  // 32-row fragments of this wave that exist (wave-uniform)
    nmi = __builtin_amdgcn_readfirstlane(nmi < 0 ? 0 : (nmi > MI ? MI : nmi));
    const bool work = nmi > 0;

    bf16x8_t fa[2][MI], fb[2][2];
    auto read_frags = [&](const uint8_t* s, int ks, int set) {
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
            if (mi < nmi) fa[set][mi] = *reinterpret_cast<const bf16x8_t*>(s + a_off[ks] + mi * 4096);
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) fb[set][ni] = *reinterpret_cast<const bf16x8_t*>(s + b_off[ks] + ni * 4096);
    };
    auto multiply = [&](int set) {
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
            if (mi < nmi) {
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][mi], fb[set][ni], acc[mi][ni], 0, 0, 0);
            }
    };

    const int nk = kslice / kTK;
    issue(0, 0);
    if (1 < nk) issue(1, 1);
    if (1 < nk) wait_dma<kCopies>(); else wait_dma<0>();  // stage 0 has landed; stage 1 may still fly
    block_barrier();
    if (2 < nk) issue(2, 2);
    if (work) read_frags(smem, 0, 0);
    int buf = 0;  // ring slot of stage kt
    for (int kt = 0; kt + 1 < nk; ++kt) {
        const uint8_t* s = smem + buf * kStageBytes;
        if (work) {
            read_frags(s, 1, 1); multiply(0);
            read_frags(s, 2, 0); multiply(1);
            read_frags(s, 3, 1); multiply(0);
        }
        if (kt + 2 < nk) wait_dma<kCopies>(); else wait_dma<0>();  // stage kt+1 landed; kt+2 may still fly
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");        // this wave's last reads of stage kt are done
        block_barrier();
        if (kt + 3 < nk) issue(kt + 3, buf);                        // stage kt's slot is free again
        buf = (buf + 1 == kNStage) ? 0 : buf + 1;
        if (work) {
            read_frags(smem + buf * kStageBytes, 0, 0);
            multiply(1);
        }
    }
    if (work) {
        const uint8_t* s = smem + buf * kStageBytes;
        read_frags(s, 1, 1); multiply(0);
        read_frags(s, 2, 0); multiply(1);
        read_frags(s, 3, 1); multiply(0);
        multiply(1);
    }

    // ---- epilogue through LDS (see the 256-row kernel) ----
    block_barrier();
    if (MODE == 1) {
        constexpr int kPitchC = 128 * 2 + 16;
        auto store_tile = [&](bool low_part) {
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
                if (mi >= nmi) break;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = wm * (32 * MI) + mi * 32 + 8 * (v >> 2) + 4 * kh + (v & 3);
                    const float g = acc[mi][0][v];
                    const float u = acc[mi][1][v];
                    const float val = silu_mul(g, u);
                    uint16_t bits = f32_to_bf16_bits(val);
                    if (low_part) bits = f32_to_bf16_bits(val - bf16_bits_to_f32(bits));
                    *reinterpret_cast<uint16_t*>(smem + row * kPitchC + (wn * 32 + r32) * 2) = bits;
                }
            }
            __syncthreads();
            uint16_t* dst = low_part ? p.act_lo : p.act;
#pragma unroll
            for (int i = 0; i < 2 * MI; ++i) {
                const int c = tid + i * kThreads;  // 16-byte piece: row c/16, columns (c%16)*8..+8
                const int row = c >> 4;
                if (row < valid)
                    *reinterpret_cast<u32x4_t*>(dst + (m0 + row) * static_cast<int64_t>(p.I) + nt * 128 + (c & 15) * 8) =
                        *reinterpret_cast<const u32x4_t*>(smem + row * kPitchC + (c & 15) * 16);
            }
        };
        store_tile(false);
        if (p.act_lo != nullptr) {
            __syncthreads();
            store_tile(true);
        }
    } else {
        constexpr int kPitchY = 64 * 4 + 16;
        int32_t* slots = reinterpret_cast<int32_t*>(smem);
        uint8_t* ytile = smem + 1024 + wave * (32 * kPitchY);
        if (tid < kTM) slots[tid] = (tid < valid) ? p.sorted_ids[m0 + tid] : -1;
        __syncthreads();
        float* ybase = p.y + static_cast<int64_t>(blockIdx.y) * p.T * p.top_k * p.H + nt * kTN + wn * 64;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi) {
            if (mi >= nmi) break;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = 8 * (v >> 2) + 4 * kh + (v & 3);
                *reinterpret_cast<float*>(ytile + row * kPitchY + r32 * 4) = acc[mi][0][v];
                *reinterpret_cast<float*>(ytile + row * kPitchY + (32 + r32) * 4) = acc[mi][1][v];
            }
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int it = 0; it < 8; ++it) {
                const int row = it * 4 + (lane >> 4);
                const int slot = slots[wm * (32 * MI) + mi * 32 + row];
                f32x4_t val = *reinterpret_cast<const f32x4_t*>(ytile + row * kPitchY + (lane & 15) * 16);
                if (slot >= 0) {
                    f32x4_t* dst = reinterpret_cast<f32x4_t*>(ybase + static_cast<int64_t>(slot) * p.H + (lane & 15) * 4);
                    if (p.y_accumulate) val += *dst;
                    *dst = val;
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
}

template <int MI>
int launch_mid(const MoeProblem& p, const int32_t* seg_begin, int mode, hipStream_t s) {
    constexpr int kTM = Geo<MI>::kTM, kLdsBytes = Geo<MI>::kLdsBytes;
    const int ntiles_n = (mode == 1) ? p.I / 128 : p.H / kTN;
    const int64_t max_mtiles = ceil_div(p.T * p.top_k + static_cast<int64_t>(p.E) * (kRowBlock - 1), kTM) + p.E;
    const unsigned grid = static_cast<unsigned>(round_up(max_mtiles * ntiles_n, kXcds));
    if (grid == 0) return 0;
    static bool attr_set[64] = {};  // caches an idempotent runtime call per device
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    if (!attr_set[dev]) {
        hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tile_mid_kernel<1, MI>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
        hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tile_mid_kernel<2, MI>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
        if (e1 != hipSuccess) return static_cast<int>(e1);
        if (e2 != hipSuccess) return static_cast<int>(e2);
        attr_set[dev] = true;
    }
    if (mode == 1)
        hipLaunchKernelGGL((gemm_tile_mid_kernel<1, MI>), dim3(grid, 1), dim3(kThreads), kLdsBytes, s, p, seg_begin,
                           ntiles_n, p.H);
    else
        hipLaunchKernelGGL((gemm_tile_mid_kernel<2, MI>), dim3(grid, static_cast<unsigned>(p.ksplit)), dim3(kThreads),
                           kLdsBytes, s, p, seg_begin, ntiles_n, p.I / p.ksplit);
    return launch_status();
}

}  // namespace

// rows_per_tile: 64 or 128
int launch_gemm_tile_mid(const MoeProblem& p, const int32_t* seg_begin, int mode, int rows_per_tile, hipStream_t s) {
    if (!tile_supported(p)) return EM_ERR_UNSUPPORTED;  // same shape rules and sort block as the 256-row kernel
    return rows_per_tile == 64 ? launch_mid<1>(p, seg_begin, mode, s) : launch_mid<2>(p, seg_begin, mode, s);
}

}  // namespace em
