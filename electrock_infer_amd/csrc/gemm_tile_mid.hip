// Tiled grouped expert GEMM for batches between decode and prefill size (a few dozen
// rows per expert).  The weights still have to be streamed once from HBM, as in decode,
// but there are too many token rows for the streaming kernel's operand-from-L2 scheme.
// This kernel is the 256-row tiled kernel cut down in M, and where it pays in N, so that
// LDS holds a deeper copy ring and the tiles fill whole rounds of CUs:
//
//   workgroup  512 threads = 8 waves as 2 (M) x 4 (N); tile of up to 128 (MI = 2) or, for the w2 GEMM of decode
//              batches, 64 (MI = 1) sorted rows x NT = 128 or 256 weight rows; wave sub-tile (32 MI) x (NT / 4) as
//              2 MI x NT / 64 accumulators of v_mfma_f32_16x16x32_bf16
//   ring       S stages of 8 MI KB of token rows + NT / 8 KB of weight rows (K step 64), as many
//              as fit 160 KB (3 .. 6), all but one in flight while that one is multiplied:
//              80-120 KB per CU on the way from HBM, which is what covers its latency at this
//              CU's share of 8 TB/s
//   NT         every tile streams its weight rows once, so the time is the number of rounds of
//              256 CUs that the tiles make.  For the w13 GEMM of the 8x7B shape 256-row tiles give
//              8 x 112 = 896 tiles = 3.5 rounds: the launch takes 256-row tiles for the whole rounds
//              (768) and cuts the rest into 256 tiles of 128 weight rows, a round of half the length
//              (128-row tiles everywhere measured slower: the token rows are read twice as often)
//   tiles      experts are padded to a multiple of 16 rows by the sort (16- or 32-row blocks) and cut
//              into tiles of equal height (a multiple of 16); fragments without rows are not
//              multiplied.  The copy count per wave and stage stays fixed (rows that do not exist
//              re-read row 0), so completion can be counted with s_waitcnt vmcnt.
//   K order    every tile starts at its own K offset and wraps around (see `rot` below)
//   the rest   LDS swizzle, gate/up pairing in one lane, XCD-aware tile order, split-K for w2
//              and the LDS-turned epilogues are those of the 256-row kernel.
#include <atomic>

#include "common.h"
#include "lds_copy.h"

namespace em {
namespace {

constexpr int kTK = 64;
constexpr int kThreads = 512;
constexpr int kLdsMax = 160 * 1024;
constexpr int kMaxStages = 6;
template <int MI, int NT> struct Geo {
    static constexpr int kTM = 64 * MI;                          // rows per tile
    static constexpr int kABytes = kTM * kTK * 2;                // 8 or 16 KB
    static constexpr int kBBytes = NT * kTK * 2;                 // 16 or 32 KB
    static constexpr int kStageBytes = kABytes + kBBytes;
    static constexpr int kStages = (kLdsMax / kStageBytes) < kMaxStages ? (kLdsMax / kStageBytes) : kMaxStages;
    static constexpr int kLdsBytes = kStages * kStageBytes;
    static constexpr int kCopiesA = kABytes / (kThreads * 16);   // per thread and stage
    static constexpr int kCopiesB = kBBytes / (kThreads * 16);
    static constexpr int kCopies = kCopiesA + kCopiesB;
    static constexpr int kRF = 2 * MI;                           // 16-row fragments per wave
    static constexpr int kCF = NT / 64;                          // 16-column fragments per wave
};
constexpr int kGroupM = 4;
constexpr int kXcds = 8;
constexpr int kRowUnit = 16;  // rows of an MFMA fragment: sorted blocks are multiples of it

// at most `stages` x COPIES of this wave's copies still in flight
template <int COPIES>
__device__ __forceinline__ void wait_stages(int stages) {
    static_assert((kMaxStages - 1) * COPIES < 64, "vmcnt is a 6-bit count");
    switch (stages) {
        case 0: wait_dma<0>(); break;
        case 1: wait_dma<COPIES>(); break;
        case 2: wait_dma<2 * COPIES>(); break;
        case 3: wait_dma<3 * COPIES>(); break;
        case 4: wait_dma<4 * COPIES>(); break;
        default: wait_dma<5 * COPIES>(); break;
    }
}

// One tile: `block` is the workgroup's index among those of its tile width, `col0` the first weight row
// (MODE 1: first gate row) of the range that this width covers, `ntiles_n` the tiles across that range.
// F16, w2 GEMM: the token rows are fp16 (MoeProblem::act_f16); the weight fragments are converted on their
// way from LDS to the MFMA (not when they are fp16 in memory, MoeProblem::w2_f16), which costs this HBM-bound kernel
// nothing.  F16, w13 GEMM: the SiLU*mul activations are stored as fp16 (clamped), else as bf16.
template <int MODE, int MI, int NT, bool F16>
__device__ __forceinline__ void tile_body(const MoeProblem& p, const int32_t* __restrict__ seg_begin, int block, int col0,
                                          int ntiles_n, int kslice, uint8_t* smem) {
    typedef Geo<MI, NT> G;
    constexpr int kTM = G::kTM, kABytes = G::kABytes, kStageBytes = G::kStageBytes, kCopies = G::kCopies,
                  kCopiesA = G::kCopiesA, kStages = G::kStages, kRF = G::kRF, kCF = G::kCF;
    static_assert(kStages >= 3, "ring depth");

    int mtiles = 0;
    for (int e = 0; e < p.E; ++e) mtiles += (seg_begin[e + 1] - seg_begin[e] + kTM - 1) / kTM;
    const int total = mtiles * ntiles_n;
    const int per_xcd = (total + kXcds - 1) / kXcds;
    const int xcd = block % kXcds;
    const int local = block / kXcds;
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
    // the expert's 16-row fragments are dealt evenly to its tiles
    const int e_rows = seg_begin[expert + 1] - seg_begin[expert];
    const int e_tiles = (e_rows + kTM - 1) / kTM;
    const int e_frags = e_rows / kRowUnit;
    const int frag_base = e_frags / e_tiles, frag_rem = e_frags % e_tiles;
    const int64_t m0 = seg_begin[expert] + static_cast<int64_t>(mt * frag_base + (mt < frag_rem ? mt : frag_rem)) * kRowUnit;
    const int valid = (frag_base + (mt < frag_rem ? 1 : 0)) * kRowUnit;  // multiple of 16, at most kTM

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 2;
    const int wn = wave & 3;
    const int K = (MODE == 1) ? p.H : p.I;
    const int k_begin = blockIdx.y * kslice;

    // ---- copy plan (per stage): copies 0 .. kCopiesA - 1 = 8 token rows each per wave, the others = weight rows.
    // Byte o of a region holds piece q ^ (u & 7) of 2-row group u = o / 256, q = (row & 1) * 8 + piece.
    const uint16_t* src[kCopies];
    const uint16_t* wbase = (MODE == 1) ? p.w13 + static_cast<int64_t>(expert) * 2 * p.I * p.H
                                        : p.w2 + static_cast<int64_t>(expert) * p.H * p.I;
#pragma unroll
    for (int n = 0; n < kCopies; ++n) {
        const int o = (n < kCopiesA ? n : n - kCopiesA) * 8192 + wave * 1024 + lane * 16;
        const int u = o >> 8;
        const int q = ((o >> 4) & 15) ^ (u & 7);
        const int r = u * 2 + (q >> 3);
        const int piece = q & 7;
        if (n < kCopiesA) {
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
            if (MODE == 1) {  // LDS row r of the B tile: wave column, gate (0) or up (1) half, offset inside the half
                constexpr int kWaveCols = NT / 4, kHalf = NT / 8;
                const int idx = r % kWaveCols;
                grow = static_cast<int64_t>(idx / kHalf) * p.I + col0 + nt * (NT / 2) + (r / kWaveCols) * kHalf + idx % kHalf;
            } else {
                grow = static_cast<int64_t>(col0) + nt * NT + r;
            }
            src[n] = wbase + grow * K + k_begin + piece * 8;
        }
    }
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem));
    const uint32_t dma_base = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
    const int nk = kslice / kTK;
    // Tiles that run side by side start at different K offsets and wrap around: with every tile of a round at the
    // same offset, all rows of all tiles ask for the same 128 bytes of their rows (one every 2 K bytes) at a time and
    // load the memory channels unevenly (w13 GEMM of the 8x7B shape: 319 -> 299 us).  The offset depends on the
    // expert and the column tile only, so a row's sum keeps one order whatever batch it arrives in.  w2 tiles next
    // to each other share act rows through L2 and move apart by a few steps only (larger strides: 150 -> 178 us).
    const int rot = ((MODE == 1) ? nt * 9 + expert * 3 : nt * 5 + expert * 8) % nk;
    auto issue = [&](int stage_k, int buf) {
        int kk = stage_k + rot;
        kk = (kk >= nk) ? kk - nk : kk;
        const int k0 = kk * kTK;
#pragma unroll
        for (int n = 0; n < kCopies; ++n)
            if (n < kCopiesA) dma16(src[n] + k0, dma_base + buf * kStageBytes + n * 8192);  // token rows: shared
            else dma16_stream(src[n] + k0, dma_base + buf * kStageBytes + kABytes + (n - kCopiesA) * 8192);  // weights: read once
    };

    // accumulator (f, g): rows wm * 32 MI + f * 16 .. + 16 of the tile, weight rows wn * NT / 4 + g * 16 .. + 16
    f32x4_t acc[kRF][kCF];
#pragma unroll
    for (int f = 0; f < kRF; ++f)
#pragma unroll
        for (int g = 0; g < kCF; ++g) acc[f][g] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // operand reads: lane (r16, kq) takes row r16 of a 16-row fragment, piece k32 * 4 + kq of the 128-byte row
    const int r16 = lane & 15;
    const int kq = lane >> 4;
    const int sw = (r16 >> 1) & 7;
    int a_off[2], b_off[2];
#pragma unroll
    for (int k32 = 0; k32 < 2; ++k32) {
        const int piece = (k32 * 4 + kq) ^ sw;
        const int ra = wm * (32 * MI) + r16, rb = wn * (NT / 4) + r16;
        a_off[k32] = (ra >> 1) * 256 + ((ra & 1) * 8 + piece) * 16;
        b_off[k32] = kABytes + (rb >> 1) * 256 + ((rb & 1) * 8 + piece) * 16;
    }
    int nfr = (valid - wm * (32 * MI)) / kRowUnit;  // fragments of this wave that hold rows (wave-uniform)
    nfr = __builtin_amdgcn_readfirstlane(nfr < 0 ? 0 : (nfr > kRF ? kRF : nfr));
    const bool work = nfr > 0;

    bf16x8_t fa[2][kRF], fb[2][kCF];
    auto read_frags = [&](const uint8_t* s, int k32, int set) {
#pragma unroll
        for (int f = 0; f < kRF; ++f)
            if (f < nfr) fa[set][f] = *reinterpret_cast<const bf16x8_t*>(s + a_off[k32] + f * 2048);
#pragma unroll
        for (int g = 0; g < kCF; ++g) fb[set][g] = *reinterpret_cast<const bf16x8_t*>(s + b_off[k32] + g * 2048);
    };
    auto multiply = [&](int set) {
#pragma unroll
        for (int f = 0; f < kRF; ++f)
            if (f < nfr) {
#pragma unroll
                for (int g = 0; g < kCF; ++g)
                    acc[f][g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[set][f], fb[set][g], acc[f][g], 0, 0, 0);
            }
    };
    auto multiply_f16 = [&](int set) {
        f16x8_t hb[kCF];
#pragma unroll
        for (int g = 0; g < kCF; ++g) {
            if (p.w2_f16) __builtin_memcpy(&hb[g], &fb[set][g], 16);
            else hb[g] = bf16x8_to_f16x8(fb[set][g]);
        }
#pragma unroll
        for (int f = 0; f < kRF; ++f)
            if (f < nfr) {
                f16x8_t ha;
                __builtin_memcpy(&ha, &fa[set][f], 16);
#pragma unroll
                for (int g = 0; g < kCF; ++g)
                    acc[f][g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ha, hb[g], acc[f][g], 0, 0, 0);
            }
    };

    // Stage st lives in ring slot st % kStages.  Stages are queued in order, so "at most n stages' worth of
    // copies in flight" means every stage but the n newest has landed.
    for (int st = 0; st < kStages && st < nk; ++st) issue(st, st);
    wait_stages<kCopies>((nk < kStages ? nk : kStages) - 1);  // stage 0 has landed
    block_barrier();
    if (work) read_frags(smem, 0, 0);
    int buf = 0;  // ring slot of stage kt
    for (int kt = 0; kt + 1 < nk; ++kt) {
        if (work) {
            read_frags(smem + buf * kStageBytes, 1, 1);
            if (MODE == 2 && F16) multiply_f16(0); else multiply(0);
        }
        {
            const int newer = nk - 2 - kt;  // stages queued after kt + 1: up to kt + kStages - 1, or the last one
            wait_stages<kCopies>(newer < kStages - 2 ? newer : kStages - 2);  // stage kt + 1 has landed
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this wave's last reads of stage kt are done
        block_barrier();
        if (kt + kStages < nk) issue(kt + kStages, buf);  // stage kt's slot is free again
        buf = (buf + 1 == kStages) ? 0 : buf + 1;
        if (work) {
            read_frags(smem + buf * kStageBytes, 0, 0);
            if (MODE == 2 && F16) multiply_f16(1); else multiply(1);
        }
    }
    if (work) {
        read_frags(smem + buf * kStageBytes, 1, 1);
        if (MODE == 2 && F16) { multiply_f16(0); multiply_f16(1); } else { multiply(0); multiply(1); }
    }

    // ---- epilogue through LDS (see the 256-row kernel).  Element i of lane (r16, kq) of a 16x16 accumulator is
    // row 4 * kq + i, column r16.
    block_barrier();
    if (MODE == 1) {
        constexpr int kColsC = NT / 2;  // act columns of the tile
        constexpr int kPitchC = kColsC * 2 + 16;
        {
            // SiLU(gate) * up in float32, rounded once to the storage type, four rows of one column at a time
            uint32_t seen = 0;  // largest magnitude bit pattern stored as fp16 (a NaN's is larger than any number's)
#pragma unroll
            for (int f = 0; f < kRF; ++f) {
                if (f >= nfr) break;
#pragma unroll
                for (int gg = 0; gg < kCF / 2; ++gg) {
                    float v[4];
                    uint16_t bits[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) v[i] = silu_mul(acc[f][gg][i], acc[f][gg + kCF / 2][i]);
                    if (F16) {
                        clamp_to_f16x4(v, seen, bits);
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i) bits[i] = f32_to_bf16_bits(v[i]);
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int row = wm * (32 * MI) + f * 16 + 4 * kq + i;
                        *reinterpret_cast<uint16_t*>(smem + row * kPitchC + (wn * (NT / 8) + gg * 16 + r16) * 2) = bits[i];
                    }
                }
            }
            if (F16 && seen > kF16MaxAsF32Bits) {
                // rare: put the NaNs back (the clamp made numbers of them) and count the clamped values of rows
                // that hold a routed slot (pad rows repeat token 0)
                int n = 0;
#pragma unroll
                for (int f = 0; f < kRF; ++f) {
                    if (f >= nfr) break;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int row = wm * (32 * MI) + f * 16 + 4 * kq + i;
                        const bool routed = p.sorted_ids[m0 + row] >= 0;
#pragma unroll
                        for (int gg = 0; gg < kCF / 2; ++gg) {
                            const float val = silu_mul(acc[f][gg][i], acc[f][gg + kCF / 2][i]);
                            if (val != val)
                                *reinterpret_cast<uint16_t*>(smem + row * kPitchC + (wn * (NT / 8) + gg * 16 + r16) * 2) = 0x7e00;
                            else if (routed && fabsf(val) > 65504.0f)
                                ++n;
                        }
                    }
                }
                if (n > 0) atomicAdd(p.saturated, n);
            }
            __syncthreads();
            uint16_t* dst = p.act;
            constexpr int kPiecesRow = kColsC / 8;  // 16-byte pieces per row
#pragma unroll
            for (int i = 0; i < kTM * kPiecesRow / kThreads; ++i) {
                const int c = tid + i * kThreads;
                const int row = c / kPiecesRow, pc = c % kPiecesRow;
                if (row < valid)
                    // (non-temporal, as in the 256-row kernel: -2 to -3 % from 128 to 352 tokens; the same hint on the
                    // partial sums of the w2 GEMM, which the combine reads at once, costs 1 %)
                    __builtin_nontemporal_store(
                        *reinterpret_cast<const u32x4_t*>(smem + row * kPitchC + pc * 16),
                        reinterpret_cast<u32x4_t*>(dst + (m0 + row) * static_cast<int64_t>(p.I) + col0 + nt * kColsC + pc * 8));
            }
        }
    } else {
        constexpr int kColsY = NT / 4;          // fp32 columns of a wave
        constexpr int kPitchY = kColsY * 4 + 16;
        constexpr int kLanesRow = kColsY / 4;   // lanes that store one row, 16 bytes each
        constexpr int kRowsIt = 64 / kLanesRow;
        int32_t* slots = reinterpret_cast<int32_t*>(smem);
        uint8_t* ytile = smem + 1024 + wave * (16 * kPitchY);
        // (Fetching the slots before the main loop, to hide the latency, measured 30 % slower: an ordinary load
        // in flight ahead of the copies slows every step of this kernel.)
        if (tid < kTM) slots[tid] = (tid < valid) ? p.sorted_ids[m0 + tid] : -1;
        __syncthreads();
        float* ybase = p.y + static_cast<int64_t>(blockIdx.y) * p.T * p.top_k * p.H + col0 + nt * NT + wn * kColsY;
#pragma unroll
        for (int f = 0; f < kRF; ++f) {
            if (f >= nfr) break;
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int g = 0; g < kCF; ++g)
                    *reinterpret_cast<float*>(ytile + (4 * kq + i) * kPitchY + (g * 16 + r16) * 4) = acc[f][g][i];
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int it = 0; it < 16 / kRowsIt; ++it) {
                const int row = it * kRowsIt + lane / kLanesRow;
                const int slot = slots[wm * (32 * MI) + f * 16 + row];
                f32x4_t val = *reinterpret_cast<const f32x4_t*>(ytile + row * kPitchY + (lane % kLanesRow) * 16);
                if (slot >= 0) {
                    f32x4_t* dst = reinterpret_cast<f32x4_t*>(ybase + static_cast<int64_t>(slot) * p.H + (lane % kLanesRow) * 4);
                    *dst = val;
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
}

template <int MODE, int MI, bool F16>
__global__ __launch_bounds__(kThreads, 1) void gemm_tile_mid_kernel(MoeProblem p, const int32_t* __restrict__ seg_begin,
                                                                   int wide_blocks, int ntn_wide, int col0n,
                                                                   int ntn_narrow, int kslice) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int b = blockIdx.x;
    if (b < wide_blocks) tile_body<MODE, MI, 256, F16>(p, seg_begin, b, 0, ntn_wide, kslice, smem);
    else tile_body<MODE, MI, 128, F16>(p, seg_begin, b - wide_blocks, col0n, ntn_narrow, kslice, smem);
}

template <int MODE, int MI, bool F16>
int launch_mid(const MoeProblem& p, const int32_t* seg_begin, hipStream_t s) {
    constexpr int kTM = 64 * MI;
    constexpr int kLdsBytes = Geo<MI, 256>::kLdsBytes > Geo<MI, 128>::kLdsBytes ? Geo<MI, 256>::kLdsBytes : Geo<MI, 128>::kLdsBytes;
    constexpr int kCus = 256;
    // Every tile streams its weight rows once, so the launch takes as many rounds of the CUs as its tiles make.
    // With routing near uniform there are `row_tiles` row tiles; 256-row tiles that fill whole rounds come first,
    // and what would be a partial round of them is cut into 128-row tiles, which take about half as long.
    const int units = (MODE == 1) ? p.I / 128 : p.H / 256;   // 256-row tiles across all weight rows
    const int slices = (MODE == 1) ? 1 : p.ksplit;
    const int64_t row_tiles = p.E * ceil_div(ceil_div(p.T * p.top_k, p.E), kTM);
    const int64_t wide_all = row_tiles * units * slices;
    int ntn_wide = units;
    if (wide_all % kCus != 0) ntn_wide = static_cast<int>((wide_all / kCus) * kCus / (row_tiles * slices));
    const int ntn_narrow = 2 * (units - ntn_wide);
    const int col0n = ntn_wide * ((MODE == 1) ? 128 : 256);
    // upper bound of the sum over experts of ceil(padded rows_e / rows per tile)
    const int64_t max_mtiles = ceil_div(p.T * p.top_k + static_cast<int64_t>(p.E) * (p.block - 1), kTM) + p.E;
    const int wide_blocks = static_cast<int>(round_up(max_mtiles * ntn_wide, kXcds));
    const unsigned grid = static_cast<unsigned>(wide_blocks + round_up(max_mtiles * ntn_narrow, kXcds));
    if (grid == 0) return 0;
    static std::atomic<bool> attr_set[64];  // caches an idempotent runtime call per device
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    if (!attr_set[dev].load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tile_mid_kernel<MODE, MI, F16>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
        if (e != hipSuccess) return static_cast<int>(e);
        attr_set[dev].store(true, std::memory_order_release);
    }
    launch((gemm_tile_mid_kernel<MODE, MI, F16>), dim3(grid, static_cast<unsigned>(slices)), dim3(kThreads),
                       kLdsBytes, s, p, seg_begin, wide_blocks, ntn_wide, col0n, ntn_narrow,
                       (MODE == 1) ? p.H : p.I / p.ksplit);
    return launch_status();
}

}  // namespace

// Shape rules of the 256-row kernel; the sort may use 16- or 32-row blocks.
bool tile_mid_supported(const MoeProblem& p) {
    return (p.block == 16 || p.block == 32) && tile_shape_ok(p.H, p.I) && p.T > 0 && p.ksplit >= 1 &&
           p.I % (p.ksplit * kTK) == 0;
}

// rows_per_tile: 128, or 64 for the w2 GEMM (decode batches; the w13 GEMM has no use for 64-row tiles: above the
// streaming kernel's range they are no faster than 128-row tiles with even routing and slower with uneven routing)
int launch_gemm_tile_mid(const MoeProblem& p, const int32_t* seg_begin, int mode, int rows_per_tile, hipStream_t s) {
    if (!tile_mid_supported(p) || (rows_per_tile != 128 && !(mode == 2 && rows_per_tile == 64))) return EM_ERR_UNSUPPORTED;
    if (mode == 1) return p.act_f16 ? launch_mid<1, 2, true>(p, seg_begin, s) : launch_mid<1, 2, false>(p, seg_begin, s);
    if (p.act_f16) return rows_per_tile == 64 ? launch_mid<2, 1, true>(p, seg_begin, s) : launch_mid<2, 2, true>(p, seg_begin, s);
    return rows_per_tile == 64 ? launch_mid<2, 1, false>(p, seg_begin, s) : launch_mid<2, 2, false>(p, seg_begin, s);
}

}  // namespace em
