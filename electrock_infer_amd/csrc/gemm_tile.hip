// Tiled grouped expert GEMM for prefill batches (hundreds of rows per expert),
// where the layer is bound by the bf16 MFMA rate.
//
//   workgroup  512 threads = 8 waves as 2 (M) x 4 (N); tile 256 sorted rows x 256
//              weight rows; K in steps of 64 through two 64 KB LDS stages
//   loads      global -> LDS directly (global_load_lds_dwordx4), no registers in
//              between; eight lanes fetch one full 128-byte line of a row (measured
//              L2 -> CU feed: ~23 TB/s with 128 B per row against ~16 TB/s with 64 B);
//              the copy of stage k+1 runs while stage k is multiplied; completion is
//              tracked by hand with s_waitcnt vmcnt + one s_barrier per stage
//   LDS        rows are 128 B; the 16-byte pieces of every 2-row group are XOR-
//              swizzled so that the 16 lanes of a b128 operand read hit 16 bank groups
//   wave       128 x 64 sub-tile = 4 x 2 v_mfma_f32_32x32x16_bf16 accumulators (the
//              16x16x32 form runs at half this rate on gfx950); operand fragments are
//              double-buffered in registers and their LDS reads are woven between the
//              MFMAs of the previous 16-wide K step, also across the stage barrier
//   MODE 1     the wave's two N fragments are 32 gate rows j and the matching 32
//              up rows I + j, so SiLU(g) * u is lane-local in the epilogue
//   MODE 2     256 rows of w2[e]; fp32 partial rows are scattered to y[slot]
//   rows       A rows are gathered through sorted_token_ids (MODE 1) or read in
//              sorted order from act (MODE 2); the sort pads every expert to 256.
//              Pad rows read token 0: their products only reach pad rows of act,
//              which no output row depends on.
//   order      workgroup ids are dealt to the 8 XCDs round-robin by the hardware;
//              they are re-mapped so that each XCD walks one contiguous range of
//              tiles, ordered 4 row blocks x all column tiles, which lets the 32
//              CUs of an XCD share A and B tiles through their own L2.
#include "common.h"

namespace em {
namespace {

constexpr int kTM = 256, kTN = 256, kTK = 64;
constexpr int kThreads = 512;
constexpr int kStages = 2;
constexpr int kRegionBytes = kTM * kTK * 2;          // 32 KB: A rows, then 32 KB of B rows
constexpr int kStageBytes = 2 * kRegionBytes;        // 64 KB
constexpr int kLdsBytes = kStages * kStageBytes;     // 128 KB
constexpr int kGroupM = 4;
constexpr int kXcds = 8;
constexpr int kDmaPerStage = kStageBytes / (kThreads * 16);  // 8 per thread
constexpr int kDmaHalf = kDmaPerStage / 2;                   // first half A rows, second half B rows

// M0 is a reserved register that the compiler never keeps live values in here (the
// kernel has no dynamically indexed register arrays); naming it as a clobber documents
// the write and only triggers an advisory warning.
#pragma clang diagnostic ignored "-Winline-asm"

// One wave copies 64 x 16 B from per-lane global addresses to 1 KB of LDS starting at
// the wave-uniform byte address `lds_addr`.  The compiler does not see the LDS write:
// every consumer sits behind wait_dma<>() + block_barrier().
__device__ __forceinline__ void dma16(const void* gptr, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :: "v"(gptr), "s"(lds_addr) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void wait_dma() {  // at most N of this wave's copies still in flight
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}
__device__ __forceinline__ void block_barrier() { asm volatile("s_barrier" ::: "memory"); }

template <int MODE>
__global__ __launch_bounds__(kThreads, 1) void gemm_tile_kernel(MoeProblem p, int ntiles_n) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    // ---- which tile: XCD-aware re-mapping over the ACTUAL number of row blocks ----
    const int mblocks = p.post_pad[0] / kTM;
    const int total = mblocks * ntiles_n;
    const int per_xcd = (total + kXcds - 1) / kXcds;
    const int xcd = blockIdx.x % kXcds;
    const int local = blockIdx.x / kXcds;
    const int logical = xcd * per_xcd + local;
    if (local >= per_xcd || logical >= total) return;
    const int group_sz = kGroupM * ntiles_n;
    const int group = logical / group_sz;
    const int in_group = logical - group * group_sz;
    const int rows_in_group = (mblocks - group * kGroupM < kGroupM) ? mblocks - group * kGroupM : kGroupM;
    const int mb = group * kGroupM + in_group % rows_in_group;
    const int nt = in_group / rows_in_group;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 2;  // 0..1
    const int wn = wave & 3;   // 0..3
    const int64_t m0 = static_cast<int64_t>(mb) * kTM;
    const int expert = p.expert_ids[m0 / p.block];
    const int K = (MODE == 1) ? p.H : p.I;

    // ---- copy plan: copy n of a stage lands at region n / 4, byte (n % 4) * 8 KB + wave * 1 KB + lane * 16.
    // Byte o of a region holds piece q ^ (u & 7) of 2-row group u = o / 256, q = (row & 1) * 8 + piece.
    const uint16_t* src[kDmaPerStage];
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
            if (MODE == 1) {
                const int slot = p.sorted_ids[m0 + r];
                const int tok = (slot >= 0) ? slot / p.top_k : 0;
                src[n] = p.x + static_cast<int64_t>(tok) * p.H + piece * 8;
            } else {
                src[n] = p.act + (m0 + r) * static_cast<int64_t>(p.I) + piece * 8;
            }
        } else {
            int64_t grow;
            if (MODE == 1)  // LDS row r of the B tile: wave column r/64, gate (0) or up (1) half, j offset r%32
                grow = static_cast<int64_t>((r >> 5) & 1) * p.I + nt * 128 + (r >> 6) * 32 + (r & 31);
            else
                grow = static_cast<int64_t>(nt) * kTN + r;
            src[n] = wbase + grow * K + piece * 8;
        }
    }
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem));
    const uint32_t dma_base = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
    auto issue = [&](int stage_k, int buf) {  // stage_k: K step index, buf: ring slot
        const int k0 = stage_k * kTK;
#pragma unroll
        for (int n = 0; n < kDmaPerStage; ++n)
            dma16(src[n] + k0, dma_base + buf * kStageBytes + (n / kDmaHalf) * kRegionBytes + (n % kDmaHalf) * 8192);
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
    bf16x8_t fa[2][4], fb[2][2];
    auto read_frags = [&](const uint8_t* s, int ks, int set) {
#pragma unroll
        for (int mi = 0; mi < 4; ++mi) fa[set][mi] = *reinterpret_cast<const bf16x8_t*>(s + a_off[ks] + mi * 4096);
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) fb[set][ni] = *reinterpret_cast<const bf16x8_t*>(s + b_off[ks] + ni * 4096);
    };
    auto multiply = [&](int set) {
#pragma unroll
        for (int mi = 0; mi < 4; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
                acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][mi], fb[set][ni], acc[mi][ni], 0, 0, 0);
        // scheduling hint: one LDS read after each of the first six MFMAs, then the last two MFMAs
#pragma unroll
        for (int i = 0; i < 6; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
    };

    const int nk = K / kTK;
    issue(0, 0);
    wait_dma<0>();
    block_barrier();
    if (1 < nk) issue(1, 1);
    read_frags(smem, 0, 0);
    for (int kt = 0; kt < nk; ++kt) {
        const uint8_t* s = smem + (kt & 1) * kStageBytes;
        read_frags(s, 1, 1); multiply(0);
        read_frags(s, 2, 0); multiply(1);
        read_frags(s, 3, 1); multiply(0);
        if (kt + 1 < nk) {
            wait_dma<0>();                                   // this wave's part of stage kt+1 is in LDS
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // its last reads of stage kt are in registers
            block_barrier();                                 // ... and so are everyone else's
            if (kt + 2 < nk) issue(kt + 2, kt & 1);          // stage kt's buffer is free again
            read_frags(smem + ((kt + 1) & 1) * kStageBytes, 0, 0);
        }
        multiply(1);
    }

    // ---- epilogue: element v of lane l sits at row 8*(v/4) + 4*(l/32) + v%4, column l%32 ----
    if (MODE == 1) {
        const int j = nt * 128 + wn * 32 + r32;
#pragma unroll
        for (int mi = 0; mi < 4; ++mi)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = wm * 128 + mi * 32 + 8 * (v >> 2) + 4 * kh + (v & 3);
                const float g = acc[mi][0][v];
                const float u = acc[mi][1][v];
                const float sg = g / (1.0f + __expf(-g));
                store_act(p, (m0 + row) * static_cast<int64_t>(p.I) + j, sg * u);
            }
    } else {
#pragma unroll
        for (int mi = 0; mi < 4; ++mi)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = wm * 128 + mi * 32 + 8 * (v >> 2) + 4 * kh + (v & 3);
                const int slot = p.sorted_ids[m0 + row];
                if (slot < 0) continue;
                float* yrow = p.y + static_cast<int64_t>(slot) * p.H + nt * kTN + wn * 64 + r32;
                yrow[0] = p.y_accumulate ? yrow[0] + acc[mi][0][v] : acc[mi][0][v];
                yrow[32] = p.y_accumulate ? yrow[32] + acc[mi][1][v] : acc[mi][1][v];
            }
    }
}

}  // namespace

bool tile_supported(const MoeProblem& p) {
    return p.block == kTM && p.ksplit == 1 && p.H % kTN == 0 && p.I % 128 == 0 && p.H % kTK == 0 &&
           p.I % kTK == 0 && p.T > 0;
}

int launch_gemm_tile(const MoeProblem& p, int mode, hipStream_t s) {
    if (!tile_supported(p)) return EM_ERR_UNSUPPORTED;
    const int ntiles_n = (mode == 1) ? p.I / 128 : p.H / kTN;
    const int64_t max_mblocks = p.sorted_len / kTM;
    const int64_t total = max_mblocks * ntiles_n;
    const unsigned grid = static_cast<unsigned>(round_up(total, kXcds));
    if (grid == 0) return 0;
    // Opt in to more than 64 KB of dynamic LDS once per device.  The flags only cache an
    // idempotent runtime call; a race between threads at worst repeats it.
    static bool attr_set[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    if (!attr_set[dev]) {
        hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tile_kernel<1>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
        hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tile_kernel<2>),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
        if (e1 != hipSuccess) return static_cast<int>(e1);
        if (e2 != hipSuccess) return static_cast<int>(e2);
        attr_set[dev] = true;
    }
    if (mode == 1)
        hipLaunchKernelGGL(gemm_tile_kernel<1>, dim3(grid), dim3(kThreads), kLdsBytes, s, p, ntiles_n);
    else
        hipLaunchKernelGGL(gemm_tile_kernel<2>, dim3(grid), dim3(kThreads), kLdsBytes, s, p, ntiles_n);
    return launch_status();
}

}  // namespace em
