// Tiled grouped expert GEMM for batches beyond decode size (tens to thousands of rows
// per expert), where the layer moves from HBM-bound to bound by the bf16 MFMA rate.
//
//   workgroup  512 threads = 8 waves as 2 (M) x 4 (N); tile of up to 256 sorted rows x 256
//              weight rows; K in steps of 64 through two 64 KB LDS stages
//   tiles      the sort pads experts to 32 rows only; every expert is cut into 256-row
//              tiles and its last tile is as high as the rows that are left (a multiple
//              of 32).  A wave multiplies only the 32-row fragments that exist, so a
//              short tile costs its share of MFMA time, and its missing A rows are not
//              fetched.  The tile list is rebuilt by every workgroup from the per-expert
//              segment starts (at most 64 scalar loads).
//   loads      global -> LDS directly (global_load_lds_dwordx4), no registers in
//              between; eight lanes fetch one full 128-byte line of a row (measured
//              L2 -> CU feed: ~23 TB/s with 128 B per row against ~16 TB/s with 64 B);
//              the copy of stage k+1 runs while stage k is multiplied; completion is
//              tracked by hand with s_waitcnt vmcnt + one s_barrier per stage
//   prefetch   a stage only completes when its slowest line has arrived, and the first
//              workgroup of an XCD to ask for a line pays HBM latency; so every
//              workgroup also touches (one dword per line, into a dummy LDS area) its
//              share of the lines that the workgroups sharing its A and B tiles will
//              need six stages later, which turns those misses into L2 hits
//   LDS        rows are 128 B; the 16-byte pieces of every 2-row group are XOR-
//              swizzled so that the 16 lanes of a b128 operand read hit 16 bank groups
//   wave       128 x 64 sub-tile = 4 x 2 v_mfma_f32_32x32x16_bf16 accumulators (the
//              16x16x32 form runs at half this rate on gfx950); operand fragments are
//              double-buffered in registers and their LDS reads are woven between the
//              MFMAs of the previous 16-wide K step, also across the stage barrier
//   MODE 1     the wave's two N fragments are 32 gate rows j and the matching 32
//              up rows I + j, so SiLU(g) * u is lane-local in the epilogue
//   MODE 2     256 rows of w2[e], optionally one of `ksplit` K slices; fp32 partial rows
//              are scattered to y[z, slot]
//   order      workgroup ids are dealt to the 8 XCDs round-robin by the hardware;
//              they are re-mapped so that each XCD walks one contiguous range of
//              tiles, ordered 4 row tiles x all column tiles, which lets the 32
//              CUs of an XCD share A and B tiles through their own L2.
#include "common.h"
#include "lds_copy.h"
#include <type_traits>

namespace em {
namespace {

constexpr int kTM = 256, kTN = 256, kTK = 64;
constexpr int kThreads = 512;
constexpr int kStages = 2;
constexpr int kRegionBytes = kTM * kTK * 2;          // 32 KB: A rows, then 32 KB of B rows
constexpr int kStageBytes = 2 * kRegionBytes;        // 64 KB
constexpr int kLdsBytes = kStages * kStageBytes;     // 128 KB
constexpr int kTouchBytes = 8 * 256;                 // dummy landing area of the L2 touches
constexpr int kTouchAhead = 6;                       // stages between a touch and its use
constexpr int kRowBlock = 32;                        // sort padding this kernel needs
constexpr int kGroupM = 4;
constexpr int kXcds = 8;
constexpr int kDmaPerStage = kStageBytes / (kThreads * 16);  // 8 per thread
constexpr int kDmaHalf = kDmaPerStage / 2;                   // first half A rows, second half B rows

template <int MODE>
__global__ __launch_bounds__(kThreads, 1) void gemm_tile_kernel(MoeProblem p, const int32_t* __restrict__ seg_begin,
                                                               int ntiles_n, int kslice) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    // ---- tile list: expert e owns ceil(rows_e / 256) row tiles ----
    int mtiles = 0;
    for (int e = 0; e < p.E; ++e) mtiles += (seg_begin[e + 1] - seg_begin[e] + kTM - 1) / kTM;
    // ---- which tile: XCD-aware re-mapping over the ACTUAL number of row tiles ----
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
    const int m_in_group = in_group % rows_in_group;
    const int nt = in_group / rows_in_group;
    int mt = group * kGroupM + m_in_group;  // global row-tile index -> (expert, tile inside the expert)
    int expert = 0;
    for (; expert < p.E - 1; ++expert) {
        const int t = (seg_begin[expert + 1] - seg_begin[expert] + kTM - 1) / kTM;
        if (mt < t) break;
        mt -= t;
    }
    const int64_t m0 = seg_begin[expert] + static_cast<int64_t>(mt) * kTM;
    const int rows_left = seg_begin[expert + 1] - static_cast<int>(m0);
    const int valid = rows_left < kTM ? rows_left : kTM;  // multiple of 32, >= 32

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 2;  // 0..1
    const int wn = wave & 3;   // 0..3
    const int K = (MODE == 1) ? p.H : p.I;
    const int k_begin = blockIdx.y * kslice;

    // ---- copy plan: copy n of a stage lands at region n / 4, byte (n % 4) * 8 KB + wave * 1 KB + lane * 16.
    // Byte o of a region holds piece q ^ (u & 7) of 2-row group u = o / 256, q = (row & 1) * 8 + piece.
    // One copy covers 8 whole rows; copies of A rows beyond `valid` are skipped.
    const uint16_t* src[kDmaPerStage];
    bool live[kDmaPerStage];
    const uint16_t* wbase = (MODE == 1) ? p.w13 + static_cast<int64_t>(expert) * 2 * p.I * p.H
                                        : p.w2 + static_cast<int64_t>(expert) * p.H * p.I;
#pragma unroll
    for (int n = 0; n < kDmaPerStage; ++n) {
        const int o = (n % kDmaHalf) * 8192 + wave * 1024 + lane * 16;
        const int u = o >> 8;
        const int q = ((o >> 4) & 15) ^ (u & 7);
        const int r = u * 2 + (q >> 3);
        const int piece = q & 7;
        if (n < kDmaHalf) {
            live[n] = ((n % kDmaHalf) * 64 + wave * 8) < valid;  // wave-uniform
            const int rr = (r < valid) ? r : 0;
            if (MODE == 1) {
                const int slot = p.sorted_ids[m0 + rr];
                const int tok = (slot >= 0) ? slot / p.top_k : 0;  // pad rows multiply token 0; never stored
                src[n] = p.x + static_cast<int64_t>(tok) * p.H + k_begin + piece * 8;
            } else {
                src[n] = p.act + (m0 + rr) * static_cast<int64_t>(p.I) + k_begin + piece * 8;
            }
        } else {
            live[n] = true;
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
    auto issue = [&](int stage_k, int buf) {  // stage_k: K step index, buf: ring slot
        const int k0 = stage_k * kTK;
#pragma unroll
        for (int n = 0; n < kDmaPerStage; ++n)
            if (live[n])
                dma16(src[n] + k0, dma_base + buf * kStageBytes + (n / kDmaHalf) * kRegionBytes + (n % kDmaHalf) * 8192);
    };

    // ---- L2 touch plan: line id = wave * 64 + lane, 0..255 = A rows, 256..511 = B rows.  The up to 8 column
    // tiles that run next to this one share its A tile and the 4 row tiles of its group share its B tile, so
    // this workgroup touches every 8th A line and every 4th B line; other lanes repeat line 0 (coalesced away).
    // Every wave issues exactly one touch per stage, which keeps the vmcnt bookkeeping uniform.
    const uint16_t* touch_src;
    {
        const int tl = wave * 64 + lane;
        const int trow = tl & 255;
        if (tl < 256) {
            const bool mine = (trow & 7) == (nt & 7) && trow < valid;
            const int rr = mine ? trow : 0;
            if (MODE == 1) {
                const int slot = p.sorted_ids[m0 + rr];
                touch_src = p.x + static_cast<int64_t>(slot >= 0 ? slot / p.top_k : 0) * p.H + k_begin;
            } else {
                touch_src = p.act + (m0 + rr) * static_cast<int64_t>(p.I) + k_begin;
            }
        } else {
            const bool mine = (trow & 3) == m_in_group;
            const int r = mine ? trow : 0;
            const int64_t grow = (MODE == 1)
                                     ? static_cast<int64_t>((r >> 5) & 1) * p.I + nt * 128 + (r >> 6) * 32 + (r & 31)
                                     : static_cast<int64_t>(nt) * kTN + r;
            touch_src = wbase + grow * K + k_begin;
        }
    }
    const uint32_t touch_dst = __builtin_amdgcn_readfirstlane(lds0 + kLdsBytes + wave * 256);
    const int nk = kslice / kTK;
    auto touch = [&](int stage_k) {
        dma4(touch_src + (stage_k < nk ? stage_k : nk - 1) * kTK, touch_dst);
    };

    f32x16_t acc[4][2];
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.f;

    // ---- operand reads: lane (r32, kh) takes row r32 of a 32-row fragment, piece ks*2 + kh ----
    const int r32 = lane & 31;
    const int kh = lane >> 5;
    const int sw = (r32 >> 1) & 7;  // (row / 2) & 7 is the same for every fragment of this lane
    int a_off[4], b_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        const int piece = (ks * 2 + kh) ^ sw;
        const int ra = wm * 128 + r32, rb = wn * 64 + r32;
        a_off[ks] = (ra >> 1) * 256 + ((ra & 1) * 8 + piece) * 16;
        b_off[ks] = kRegionBytes + (rb >> 1) * 256 + ((rb & 1) * 8 + piece) * 16;
    }
    // 32-row fragments of this wave that hold rows of the tile (wave-uniform)
    int nmi = (valid - wm * 128 + 31) / 32;
    nmi = nmi < 0 ? 0 : (nmi > 4 ? 4 : nmi);
    nmi = __builtin_amdgcn_readfirstlane(nmi);

    bf16x8_t fa[2][4], fb[2][2];
    // FULL: all four fragments exist (the common case) -> fixed instruction mix with scheduling hints
    auto main_loop = [&](auto full_tag) {
        constexpr bool FULL = decltype(full_tag)::value;
        auto read_frags = [&](const uint8_t* s, int ks, int set) {
#pragma unroll
            for (int mi = 0; mi < 4; ++mi)
                if (FULL || mi < nmi) fa[set][mi] = *reinterpret_cast<const bf16x8_t*>(s + a_off[ks] + mi * 4096);
#pragma unroll
            for (int ni = 0; ni < 2; ++ni) fb[set][ni] = *reinterpret_cast<const bf16x8_t*>(s + b_off[ks] + ni * 4096);
        };
        auto multiply = [&](int set) {
#pragma unroll
            for (int mi = 0; mi < 4; ++mi)
                if (FULL || mi < nmi) {
#pragma unroll
                    for (int ni = 0; ni < 2; ++ni)
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][mi], fb[set][ni], acc[mi][ni], 0, 0, 0);
                }
            if (FULL) {  // scheduling hint: one LDS read after each of the first six MFMAs, then the last two
#pragma unroll
                for (int i = 0; i < 6; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
                __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            }
        };
        const bool work = FULL || nmi > 0;  // waves without rows still copy, touch and meet the barriers
        issue(0, 0);
        touch(1);
        wait_dma<1>();  // everything but the touch
        block_barrier();
        if (1 < nk) issue(1, 1);
        touch(2);
        if (work) read_frags(smem, 0, 0);
        for (int kt = 0; kt + 1 < nk; ++kt) {
            const uint8_t* s = smem + (kt & 1) * kStageBytes;
            if (work) {
                read_frags(s, 1, 1); multiply(0);
                read_frags(s, 2, 0); multiply(1);
                read_frags(s, 3, 1); multiply(0);
            }
            wait_dma<1>();                                      // this wave's part of stage kt+1 is in LDS
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // its last reads of stage kt are in registers
            block_barrier();                                    // ... and so are everyone else's
            if (kt + 2 < nk) issue(kt + 2, kt & 1);             // stage kt's buffer is free again
            touch(kt + 2 + kTouchAhead);
            if (work) {
                read_frags(smem + ((kt + 1) & 1) * kStageBytes, 0, 0);
                multiply(1);
            }
        }
        if (work) {  // last stage: nothing left to copy
            const uint8_t* s = smem + ((nk - 1) & 1) * kStageBytes;
            read_frags(s, 1, 1); multiply(0);
            read_frags(s, 2, 0); multiply(1);
            read_frags(s, 3, 1); multiply(0);
            multiply(1);
        }
        wait_dma<0>();  // the last touches must not outlive the workgroup's LDS
    };
    if (nmi == 4) main_loop(std::true_type{});
    else main_loop(std::false_type{});

    // ---- epilogue.  Element v of lane l of a 32x32 accumulator sits at row 8*(v/4) + 4*(l/32) + v%4,
    // column l%32: one column per lane.  Results are turned through LDS (free after the last stage) so
    // that global stores are 16 bytes per lane on full 128-byte lines.
    block_barrier();  // every wave has read its last operands: the stage buffers can be reused
    if (MODE == 1) {
        // act tile [256 rows][128 columns] bf16, row pitch 272 B
        constexpr int kPitchC = 128 * 2 + 16;
        auto store_tile = [&](bool low_part) {
#pragma unroll
            for (int mi = 0; mi < 4; ++mi) {
                if (mi >= nmi) break;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = wm * 128 + mi * 32 + 8 * (v >> 2) + 4 * kh + (v & 3);
                    const float g = acc[mi][0][v];
                    const float u = acc[mi][1][v];
                    const float val = g / (1.0f + __expf(-g)) * u;
                    uint16_t bits = f32_to_bf16_bits(val);
                    if (low_part) bits = f32_to_bf16_bits(val - bf16_bits_to_f32(bits));
                    *reinterpret_cast<uint16_t*>(smem + row * kPitchC + (wn * 32 + r32) * 2) = bits;
                }
            }
            __syncthreads();
            uint16_t* dst = low_part ? p.act_lo : p.act;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int c = tid + i * kThreads;  // 16-byte piece c of the tile: row c/16, columns (c%16)*8..+8
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
        // slots of the tile's rows -> LDS; then per wave and 32-row fragment a private [32][64] fp32 tile, pitch 272 B
        constexpr int kPitchY = 64 * 4 + 16;
        int32_t* slots = reinterpret_cast<int32_t*>(smem);
        uint8_t* ytile = smem + 1024 + wave * (32 * kPitchY);
        if (tid < kTM) slots[tid] = (tid < valid) ? p.sorted_ids[m0 + tid] : -1;
        __syncthreads();
        float* ybase = p.y + static_cast<int64_t>(blockIdx.y) * p.T * p.top_k * p.H + nt * kTN + wn * 64;
#pragma unroll
        for (int mi = 0; mi < 4; ++mi) {
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
                const int slot = slots[wm * 128 + mi * 32 + row];
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

}  // namespace

bool tile_shape_ok(int H, int I) { return H % kTN == 0 && I % 128 == 0 && H % kTK == 0 && I % kTK == 0; }
int tile_row_block() { return kRowBlock; }

bool tile_supported(const MoeProblem& p) {
    return p.block == kRowBlock && tile_shape_ok(p.H, p.I) && p.T > 0 && p.ksplit >= 1 &&
           p.I % (p.ksplit * kTK) == 0;
}

int launch_gemm_tile(const MoeProblem& p, const int32_t* seg_begin, int mode, hipStream_t s) {
    if (!tile_supported(p)) return EM_ERR_UNSUPPORTED;
    const int ntiles_n = (mode == 1) ? p.I / 128 : p.H / kTN;
    // upper bound of the sum over experts of ceil(padded rows_e / 256)
    const int64_t max_mtiles = ceil_div(p.T * p.top_k + static_cast<int64_t>(p.E) * (kRowBlock - 1), kTM) + p.E;
    const int64_t total = max_mtiles * ntiles_n;
    const unsigned grid = static_cast<unsigned>(round_up(total, kXcds));
    if (grid == 0) return 0;
    constexpr int lds_bytes = kLdsBytes + kTouchBytes;
    // Opt in to more than 64 KB of dynamic LDS once per device.  The flags only cache an
    // idempotent runtime call; a race between threads at worst repeats it.
    static bool attr_set[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    if (!attr_set[dev]) {
        hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tile_kernel<1>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tile_kernel<2>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (e1 != hipSuccess) return static_cast<int>(e1);
        if (e2 != hipSuccess) return static_cast<int>(e2);
        attr_set[dev] = true;
    }
    if (mode == 1)
        hipLaunchKernelGGL(gemm_tile_kernel<1>, dim3(grid, 1), dim3(kThreads), lds_bytes, s, p, seg_begin, ntiles_n, p.H);
    else
        hipLaunchKernelGGL(gemm_tile_kernel<2>, dim3(grid, static_cast<unsigned>(p.ksplit)), dim3(kThreads), lds_bytes,
                           s, p, seg_begin, ntiles_n, p.I / p.ksplit);
    return launch_status();
}

}  // namespace em
