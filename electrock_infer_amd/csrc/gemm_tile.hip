// Tiled grouped expert GEMM for prefill batches (hundreds of rows per expert),
// where the layer is bound by the bf16 MFMA rate.
//
//   workgroup  512 threads = 8 waves as 2 (M) x 4 (N); tile 256 sorted rows x 256
//              weight rows, K in steps of 64 through a double-buffered LDS tile
//              (2 x 72 KB with the 144-byte row pitch that keeps b128 reads
//              conflict-free)
//   wave       128 x 64 sub-tile = 4 x 2 v_mfma_f32_32x32x16_bf16 accumulators
//   MODE 1     the wave's two N fragments are 32 gate rows j and the matching 32
//              up rows I + j, so SiLU(g) * u is lane-local in the epilogue
//   MODE 2     256 rows of w2[e]; fp32 partial rows are scattered to y[slot]
//   rows       A rows are gathered through sorted_token_ids (MODE 1) or read in
//              sorted order from act (MODE 2); the sort pads every expert to 256
//   order      workgroup ids are dealt to the 8 XCDs round-robin by the hardware;
//              they are re-mapped so that each XCD walks one contiguous range of
//              tiles, ordered 4 row blocks x all column tiles, which lets the 32
//              CUs of an XCD share A and B tiles through their own L2.
#include "common.h"

namespace em {
namespace {

constexpr int kTM = 256, kTN = 256, kTK = 64;
constexpr int kThreads = 512;
constexpr int kPitch = kTK * 2 + 16;                 // 144 B
constexpr int kStageBytes = (kTM + kTN) * kPitch;    // 73,728 B
constexpr int kLdsBytes = 2 * kStageBytes;           // 147,456 B
constexpr int kGroupM = 4;
constexpr int kXcds = 8;

__device__ __forceinline__ u32x4_t ld16(const uint16_t* p) { return *reinterpret_cast<const u32x4_t*>(p); }

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

    // ---- per-thread global sources: chunk c = tid + i*512 -> row c/8, 16-byte piece c%8 ----
    const int lrow = tid >> 3;
    const int lkc = (tid & 7) * 8;
    const uint16_t* a_src[4];
    const uint16_t* b_src[4];
    const uint16_t* wbase = (MODE == 1) ? p.w13 + static_cast<int64_t>(expert) * 2 * p.I * p.H
                                        : p.w2 + static_cast<int64_t>(expert) * p.H * p.I;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = lrow + i * 64;
        if (MODE == 1) {
            const int slot = p.sorted_ids[m0 + r];
            a_src[i] = (slot >= 0) ? p.x + static_cast<int64_t>(slot / p.top_k) * p.H + lkc : nullptr;
            // LDS row r of the B tile: wave column r/64, gate (0) or up (1) half, j offset r%32
            const int64_t grow = static_cast<int64_t>((r >> 5) & 1) * p.I + nt * 128 + (r >> 6) * 32 + (r & 31);
            b_src[i] = wbase + grow * K + lkc;
        } else {
            a_src[i] = p.act + (m0 + r) * static_cast<int64_t>(p.I) + lkc;
            b_src[i] = wbase + static_cast<int64_t>(nt * kTN + r) * K + lkc;
        }
    }

    u32x4_t a_reg[4], b_reg[4];
    auto load_global = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) a_reg[i] = (a_src[i] != nullptr) ? ld16(a_src[i] + k0) : u32x4_t{0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 4; ++i) b_reg[i] = ld16(b_src[i] + k0);
    };
    auto store_lds = [&](int buf) {
        uint8_t* sa = smem + buf * kStageBytes;
        uint8_t* sb = sa + kTM * kPitch;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<u32x4_t*>(sa + (lrow + i * 64) * kPitch + lkc * 2) = a_reg[i];
            *reinterpret_cast<u32x4_t*>(sb + (lrow + i * 64) * kPitch + lkc * 2) = b_reg[i];
        }
    };

    f32x16_t acc[4][2];
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[mi][ni][v] = 0.f;

    const int r32 = lane & 31;
    const int kh = lane >> 5;  // which 8-element half of a 16-wide K step
    const int a_off = (wm * 128 + r32) * kPitch + kh * 16;
    const int b_off = kTM * kPitch + (wn * 64 + r32) * kPitch + kh * 16;

    const int nk = K / kTK;
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < nk) load_global((kt + 1) * kTK);
        const uint8_t* s = smem + buf * kStageBytes;
#pragma unroll
        for (int ks = 0; ks < kTK / 16; ++ks) {
            bf16x8_t af[4], bfr[2];
#pragma unroll
            for (int mi = 0; mi < 4; ++mi)
                af[mi] = *reinterpret_cast<const bf16x8_t*>(s + a_off + mi * 32 * kPitch + ks * 32);
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
                bfr[ni] = *reinterpret_cast<const bf16x8_t*>(s + b_off + ni * 32 * kPitch + ks * 32);
#pragma unroll
            for (int mi = 0; mi < 4; ++mi)
#pragma unroll
                for (int ni = 0; ni < 2; ++ni)
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[mi], bfr[ni], acc[mi][ni], 0, 0, 0);
        }
        if (kt + 1 < nk) store_lds(buf ^ 1);
        __syncthreads();
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
                p.act[(m0 + row) * static_cast<int64_t>(p.I) + j] = f32_to_bf16_bits(sg * u);
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
                yrow[0] = acc[mi][0][v];
                yrow[32] = acc[mi][1][v];
            }
    }
}

}  // namespace

bool tile_supported(const MoeProblem& p) {
    return p.block == kTM && p.ksplit == 1 && p.H % kTN == 0 && p.I % 128 == 0 && p.H % kTK == 0 &&
           p.I % kTK == 0;
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
