// Tiled grouped expert GEMM for batches beyond decode size (tens to thousands of rows
// per expert), where the layer moves from HBM-bound to bound by the bf16 MFMA rate.
//
//   workgroup  512 threads = 8 waves as 2 (M) x 4 (N); tile of up to 256 sorted rows x 256
//              weight rows; K in steps of 64; LDS (all 160 KB) holds a ring of two 32 KB
//              slots of token rows (A) and a ring of three 32 KB slots of weight rows (B)
//   tiles      the sort pads experts to 32 rows only; an expert with r rows gets ceil(r / 256)
//              row tiles and its 32-row blocks are dealt evenly to them (heights differ by
//              one block at most): every tile streams the same weight bytes whatever its
//              height, so a full-height tiling with a nearly empty last tile cost a full
//              tile's time for a few rows, and equal tiles stay in step and share through
//              L2.  A wave multiplies only the blocks it has -- its main loop is instantiated
//              for 1 .. 4 blocks -- and missing A rows are not fetched.  The tile list is
//              rebuilt by every workgroup from the per-expert segment starts (at most 64
//              scalar loads).
//   loads      global -> LDS directly (global_load_lds_dwordx4), no registers in
//              between; eight lanes fetch one full 128-byte line of a row (measured
//              L2 -> CU feed: ~26 TB/s with 128 B per row against ~17 TB/s with 64 B).
//              Weight rows stream from HBM and are requested two K steps before their
//              use (w2 GEMM: one and a half, see the main loop), token rows (L2 / memory-side
//              cache hits) one step before; with a single stage in flight the slowest line of
//              a stage, at HBM latency, sat on the critical path of every step.  Completion is
//              tracked by hand with s_waitcnt vmcnt + one s_barrier per step.
//   issue      the eight copy instructions of a wave are issued one by one between the
//              MFMAs that follow the barrier: issued back to back (by both waves of
//              a SIMD at once) they left the matrix pipe idle for a fifth of every step
//   LDS        rows are 128 B; the 16-byte pieces of every 2-row group are XOR-
//              swizzled so that the 16 lanes of a b128 operand read hit 16 bank groups
//   wave       128 x 64 sub-tile = 8 x 4 v_mfma_f32_16x16x32_bf16 accumulators.  Both bf16
//              shapes run at the same rate, but with real operand values the board's power
//              limit, not the issue rate, sets the speed, and this shape needs less power
//              per flop (registers-only loop, N(0,1) x N(0,0.02) operands: 2.08 against
//              1.85 PFLOP/s for 32x32x16).  A K step of 64 is walked in four units of 16
//              MFMAs (first / second two 32-row blocks of the wave x first / second 32 of K); operand fragments are
//              double-buffered in registers and their LDS reads are woven between the
//              MFMAs of the previous unit, also across the stage barrier
//   MODE 1     N fragments 0, 1 of a wave are 32 gate rows j and fragments 2, 3 the matching
//              32 up rows I + j, so SiLU(g) * u is lane-local in the epilogue
//   MODE 2     256 rows of w2[e], optionally one of `ksplit` K slices; fp32 partial rows
//              are scattered to y[z, slot]
//   order      workgroup ids are dealt to the 8 XCDs round-robin by the hardware; each XCD
//              takes an eighth of the column tiles of every expert and walks them expert by
//              expert, column by column, row tile fastest, so that the 32 CUs of an XCD share
//              weight and token tiles through their own L2 and weights leave HBM once.  In the
//              w2 GEMM an XCD also stays on one K slice, so it fetches that slice of the
//              activation rows only.
#include <atomic>

#include "common.h"
#include "lds_copy.h"
#include <type_traits>

namespace em {
namespace {

constexpr int kTM = 256, kTN = 256, kTK = 64;
constexpr int kThreads = 512;
constexpr int kSlotBytes = kTM * kTK * 2;            // 32 KB: 256 rows x 64 K of one operand
constexpr int kSlotsA = 2, kSlotsB = 3;
constexpr int kOffB = kSlotsA * kSlotBytes;          // B ring behind the A ring
constexpr int kLdsBytes = (kSlotsA + kSlotsB) * kSlotBytes;  // 160 KB
constexpr int kRowBlock = 32;                        // sort padding this kernel needs
constexpr int kGroupM = 4;
constexpr int kMaxGroupRows = 12;                  // row tiles of one expert that share a pass over its weights
constexpr int kXcds = 8;
constexpr int kDmaHalf = kSlotBytes / (kThreads * 16);  // 4 copies per thread and operand slot
constexpr int kDmaPerStage = 2 * kDmaHalf;              // first half A rows, second half B rows

// STREAM: the weight rows are copied with the non-temporal hint.  Right when most experts fit one row tile
// (every weight byte is then read by one workgroup only); wrong when several row tiles share them through L2.
// F16, w2 GEMM (on fp16 activations): the activation rows are fp16 (MoeProblem::act_f16); every weight fragment is turned
// into fp16 once, before its first MFMA, and the fp16 MFMA of the same shape and rate runs instead.  F16 = 1 converts
// bf16 weights, F16 = 2 takes weights that are fp16 in memory (MoeProblem::w2_f16) as they come.
// F16, w13 GEMM: 1 = the SiLU*mul activations are stored as fp16 (clamped; MoeProblem::act_f16), 0 = as bf16.
// PERSIST: the launch has one workgroup per CU (or fewer) and every workgroup walks tiles until none is left: its
// first tile is the one its id names, the following ones come from a ticket counter per XCD (`tickets[8]`, zero
// before the launch), so that tile i still runs on XCD i % 8 and tiles are handed out in the order above.  Nothing
// but the ticket is shared between workgroups: a workgroup never waits for another one.
template <int MODE, bool STREAM, int F16, bool PERSIST>
__global__ __launch_bounds__(kThreads, 1) void gemm_tile_kernel(MoeProblem p, const int32_t* __restrict__ seg_begin,
                                                               int ntiles_n, int kslice, int ids_x, int nz,
                                                               int* __restrict__ tickets) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    // ---- tile list: expert e owns ceil(rows_e / 256) row tiles ----
    int mtiles = 0;
    for (int e = 0; e < p.E; ++e) mtiles += (seg_begin[e + 1] - seg_begin[e] + kTM - 1) / kTM;
    // Tile ids: [0, ids_x) for K slice 0, [ids_x, 2 * ids_x) for slice 1, ...; ids_x is a multiple of 8.
    const int my_xcd = blockIdx.x % kXcds;
    const int first_ticket = gridDim.x / kXcds;  // tiles 0 .. gridDim.x - 1 are the workgroups' first ones
    int tile_n = blockIdx.x / kXcds;              // this XCD's tile_n-th tile comes next (PERSIST)
    int next_n = -1;                              // thread 0: ticket drawn ahead, while the current tile runs
    for (bool first_tile = true;; first_tile = false) {
    int id_x, id_z;
    if (PERSIST) {
        if (!first_tile) {
            // hand the next ticket to all waves through LDS (every byte of it belongs to the copy rings, which are
            // idle between two tiles: the barriers fence the last reads of the tile before and the first copies of
            // the next one)
            __syncthreads();
            if (threadIdx.x == 0) {
                if (next_n < 0) next_n = first_ticket + atomicAdd(&tickets[my_xcd], 1);
                *reinterpret_cast<volatile int*>(smem) = next_n;
                next_n = -1;
            }
            __syncthreads();
            tile_n = __builtin_amdgcn_readfirstlane(*reinterpret_cast<volatile int*>(smem));
            __syncthreads();
        }
        const int id = tile_n * kXcds + my_xcd;
        if (tile_n >= (1 << 26) || id >= ids_x * nz) break;  // every wave of the workgroup leaves here together
        id_z = id / ids_x;
        id_x = id - id_z * ids_x;
    } else {
        if (!first_tile) break;
        id_x = blockIdx.x;
        id_z = blockIdx.y;
    }
    int nt, mt, expert = 0;
    if (MODE == 2 && kXcds % nz == 0 && (ntiles_n * nz) % kXcds == 0) {
        // w2 GEMM: an XCD works on one K slice only (slice xcd % nz), so its L2 fetches that slice of the activation
        // rows instead of all of them, and on ntiles_n * nz / 8 of the column tiles of every expert
        const int cols = ntiles_n * nz / kXcds;
        const int xcd = id_x % kXcds;
        int local = (id_z * ids_x + id_x) / kXcds;
        if (local >= mtiles * cols) { if (PERSIST) continue; return; }
        id_z = xcd % nz;
        for (; expert < p.E - 1; ++expert) {
            const int t = ((seg_begin[expert + 1] - seg_begin[expert] + kTM - 1) / kTM) * cols;
            if (local < t) break;
            local -= t;
        }
        const int rows_e = (seg_begin[expert + 1] - seg_begin[expert] + kTM - 1) / kTM;
        const int ngroups = (rows_e + kMaxGroupRows - 1) / kMaxGroupRows;
        const int grows = (rows_e + ngroups - 1) / ngroups;
        int g0 = 0, gr = grows;
        for (;; g0 += grows) {
            gr = (rows_e - g0 < grows) ? rows_e - g0 : grows;
            if (local < gr * cols) break;
            local -= gr * cols;
        }
        nt = (xcd / nz) * cols + local / gr;
        mt = g0 + local % gr;
    } else if (ntiles_n % kXcds == 0) {
        const int cols = ntiles_n / kXcds;
        const int xcd = id_x % kXcds;
        int local = id_x / kXcds;
        if (local >= mtiles * cols) { if (PERSIST) continue; return; }
        for (; expert < p.E - 1; ++expert) {
            const int t = ((seg_begin[expert + 1] - seg_begin[expert] + kTM - 1) / kTM) * cols;
            if (local < t) break;
            local -= t;
        }
        const int rows_e = (seg_begin[expert + 1] - seg_begin[expert] + kTM - 1) / kTM;
        // experts with many row tiles are walked in groups of at most kMaxGroupRows row tiles (else the CUs of
        // an XCD would share one weight tile but no token rows)
        const int ngroups = (rows_e + kMaxGroupRows - 1) / kMaxGroupRows;
        const int grows = (rows_e + ngroups - 1) / ngroups;
        int g0 = 0, gr = grows;
        for (;; g0 += grows) {
            gr = (rows_e - g0 < grows) ? rows_e - g0 : grows;
            if (local < gr * cols) break;
            local -= gr * cols;
        }
        nt = xcd * cols + local / gr;
        mt = g0 + local % gr;
    } else {
        // column count not divisible: contiguous ranges of 4 row tiles x all column tiles per XCD
        const int total = mtiles * ntiles_n;
        const int per_xcd = (total + kXcds - 1) / kXcds;
        const int xcd = id_x % kXcds;
        const int local = id_x / kXcds;
        const int logical = xcd * per_xcd + local;
        if (local >= per_xcd || logical >= total) { if (PERSIST) continue; return; }
        const int group_sz = kGroupM * ntiles_n;
        const int group = logical / group_sz;
        const int in_group = logical - group * group_sz;
        const int rows_in_group = (mtiles - group * kGroupM < kGroupM) ? mtiles - group * kGroupM : kGroupM;
        nt = in_group / rows_in_group;
        mt = group * kGroupM + in_group % rows_in_group;  // global row-tile index -> (expert, tile inside the expert)
        for (; expert < p.E - 1; ++expert) {
            const int t = (seg_begin[expert + 1] - seg_begin[expert] + kTM - 1) / kTM;
            if (mt < t) break;
            mt -= t;
        }
    }
    // The expert's 32-row blocks are dealt evenly to its row tiles (heights differ by at most one block): every
    // tile streams the same weight bytes, so a nearly empty last tile would cost a full tile's time.
    const int e_rows = seg_begin[expert + 1] - seg_begin[expert];
    const int e_tiles = (e_rows + kTM - 1) / kTM;
    const int e_blocks = e_rows / kRowBlock;
    const int blk_base = e_blocks / e_tiles, blk_rem = e_blocks % e_tiles;
    const int64_t m0 = seg_begin[expert] + static_cast<int64_t>(mt * blk_base + (mt < blk_rem ? mt : blk_rem)) * kRowBlock;
    const int valid = (blk_base + (mt < blk_rem ? 1 : 0)) * kRowBlock;  // multiple of 32, >= 32

    // (PERSIST: the thread index is made opaque once per tile, so that everything derived from it -- copy plans,
    // operand offsets -- is worked out again for every tile instead of being kept in registers across the tile loop:
    // the loop body needs all 256 registers a wave has here)
    int tid_once = threadIdx.x;
    if (PERSIST) asm volatile("" : "+v"(tid_once));
    const int tid = tid_once;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 2;  // 0..1
    const int wn = wave & 3;   // 0..3
    const int K = (MODE == 1) ? p.H : p.I;
    const int k_begin = id_z * kslice;

    // ---- copy plan: copy n of a stage lands at region n / 4, byte (n % 4) * 8 KB + wave * 1 KB + lane * 16.
    // Byte o of a region holds piece q ^ (u & 7) of 2-row group u = o / 256, q = (row & 1) * 8 + piece.
    // One copy covers 8 whole rows; copies of A rows beyond `valid` are skipped.
    // Addresses are a wave-uniform base per operand plus a 32-bit byte offset per lane.
    uint32_t voff[kDmaPerStage];
    bool live[kDmaPerStage];
    const uint16_t* wbase = (MODE == 1) ? p.w13 + static_cast<int64_t>(expert) * 2 * p.I * p.H
                                        : p.w2 + static_cast<int64_t>(expert) * p.H * p.I;
    // (wave-uniform addresses, said so to the compiler: the copies take their base from scalar registers)
    auto uniform_ptr = [](const void* ptr) {
        const uint64_t v = reinterpret_cast<uint64_t>(ptr);
        const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
        const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
        return reinterpret_cast<const uint8_t*>((static_cast<uint64_t>(hi) << 32) | lo);
    };
    const uint8_t* base_a = uniform_ptr(((MODE == 1) ? p.x : p.act + m0 * static_cast<int64_t>(p.I)) + k_begin);
    const uint8_t* base_b = uniform_ptr(wbase + k_begin);
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
                voff[n] = static_cast<uint32_t>(tok) * static_cast<uint32_t>(p.H * 2) + piece * 16;
            } else {
                voff[n] = static_cast<uint32_t>(rr) * static_cast<uint32_t>(p.I * 2) + piece * 16;
            }
        } else {
            live[n] = true;
            uint32_t grow;
            if (MODE == 1)  // LDS row r of the B tile: wave column r/64, gate (0) or up (1) half, j offset r%32
                grow = static_cast<uint32_t>((r >> 5) & 1) * p.I + nt * 128 + (r >> 6) * 32 + (r & 31);
            else
                grow = static_cast<uint32_t>(nt) * kTN + r;
            voff[n] = grow * static_cast<uint32_t>(K * 2) + piece * 16;
        }
    }
    // MODE 2 scatters its rows by slot in the epilogue: fetch the slot of row `tid` now, not at the end of the tile
    int my_slot = -1;
    if (MODE == 2 && tid < kTM && tid < valid) my_slot = p.sorted_ids[m0 + tid];
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem));
    const uint32_t dma_base = __builtin_amdgcn_readfirstlane(lds0 + wave * 1024);
    const int nk = kslice / kTK;
    // While every weight byte is read by one workgroup only (STREAM) the w13 tiles start at different K offsets and
    // wrap around, as in the 64- / 128-row kernel: tiles in step ask for the same 128 bytes of all their rows at once
    // and load the memory channels unevenly (T=512: 401 -> 353 us, T=768: 433 -> 416 us).  Larger batches keep the
    // tiles of an XCD in step, they share token rows and weights through L2; the w2 tiles share act rows at every size.
    // The offset depends on expert and column tile only, so a row's sum keeps one order whatever batch it comes in.
    constexpr bool kRotate = STREAM && MODE == 1;
    const int rot = kRotate ? __builtin_amdgcn_readfirstlane((nt * 9 + expert * 3) % nk) : 0;
    auto krot = [&](int stage_k) {
        if (!kRotate) return stage_k;
        const int k = stage_k + rot;
        return __builtin_amdgcn_readfirstlane(k >= nk ? k - nk : k);
    };
    // copy n (0..3) of the token rows / weight rows of K step stage_k
    auto copy_a = [&](int n, int stage_k) {
        dma16(voff[n], base_a + static_cast<int64_t>(krot(stage_k)) * (kTK * 2),
              dma_base + (stage_k & 1) * kSlotBytes + n * 8192);
    };
    auto copy_b = [&](int n, int stage_k, int slot) {
        if (STREAM)
            dma16_stream(voff[kDmaHalf + n], base_b + static_cast<int64_t>(krot(stage_k)) * (kTK * 2),
                         dma_base + kOffB + slot * kSlotBytes + n * 8192);
        else
            dma16(voff[kDmaHalf + n], base_b + static_cast<int64_t>(krot(stage_k)) * (kTK * 2),
                  dma_base + kOffB + slot * kSlotBytes + n * 8192);
    };
    auto issue_a = [&](int stage_k) {
#pragma unroll
        for (int n = 0; n < kDmaHalf; ++n)
            if (live[n]) copy_a(n, stage_k);
    };
    auto issue_b = [&](int stage_k, int slot) {
#pragma unroll
        for (int n = 0; n < kDmaHalf; ++n) copy_b(n, stage_k, slot);
    };

    // accumulator (f, g): rows frag_row(f) .. +16 of the tile (see below), weight rows wn*64 + g*16 .. +16
    f32x4_t acc[8][4];
#pragma unroll
    for (int f = 0; f < 8; ++f)
#pragma unroll
        for (int g = 0; g < 4; ++g) acc[f][g] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // ---- operand reads: lane (r16, kq) takes row r16 of a 16-row fragment, piece k32*4 + kq of the 128-byte row ----
    const int r16 = lane & 15;
    const int kq = lane >> 4;
    const int sw = (r16 >> 1) & 7;  // (row / 2) & 7 is the same for every fragment of this lane
    // (K half 1 reads piece (4 + kq) ^ sw = (kq ^ sw) ^ 4: its offsets are those of K half 0 with bit 6 flipped, formed
    // where they are used instead of being kept in two more registers)
    int a_off0, b_off0;
    {
        const int piece = kq ^ sw;
        const int ra = wm * 32 + r16, rb = wn * 64 + r16;
        a_off0 = (ra >> 1) * 256 + ((ra & 1) * 8 + piece) * 16;
        b_off0 = kOffB + (rb >> 1) * 256 + ((rb & 1) * 8 + piece) * 16;
    }
    struct HalfOffset {
        int base;
        __device__ __forceinline__ int operator[](int k32) const { return k32 ? (base ^ 64) : base; }
    };
    const HalfOffset a_off{a_off0}, b_off{b_off0};
    // The 32-row blocks of a tile are dealt alternately to the two wave rows: block b belongs to wave row b % 2, so a
    // tile of nb blocks gives them ceil(nb / 2) and floor(nb / 2) (the two wave rows of a wave column share a SIMD,
    // so the MFMA time of a short tile is the same either way; the even split evens out their LDS reads and waits).  16-row fragment f of wave row wm
    // (f < 2 * nmi, nmi = the wave's blocks, wave-uniform) starts at tile row frag_row(f).
    const int nblocks = valid / kRowBlock;
    int nmi = (wm == 0) ? (nblocks + 1) / 2 : nblocks / 2;
    nmi = __builtin_amdgcn_readfirstlane(nmi);
    auto frag_row = [&](int f) { return (f >> 1) * 64 + wm * 32 + (f & 1) * 16; };
    auto frag_off = [](int f) { return (f >> 1) * 8192 + (f & 1) * 2048; };  // bytes in a slot of token rows, from fragment 0

    // Unit u = 0..3 of a K step: row half h = u & 1 (fragments 4h .. 4h+3), K half k32 = u >> 1.
    // Token fragments live in register set u & 1, weight fragments (shared by both row halves) in set k32.
    // (defined values at the start of every tile: a wave with fewer than four blocks never reads the fragments it
    // does not load, but the compiler cannot see that, and would carry all sixteen from one tile to the next)
    bf16x8_t fa[2][4], fb[2][4];
    if (PERSIST) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                fa[i][j] = bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
                fb[i][j] = bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
            }
    }
    auto mma = [](const bf16x8_t& a, const bf16x8_t& b, f32x4_t c) {
        if (MODE == 2 && F16) {
            f16x8_t ha, hb;  // the registers already hold fp16 bits
            __builtin_memcpy(&ha, &a, 16);
            __builtin_memcpy(&hb, &b, 16);
            return __builtin_amdgcn_mfma_f32_16x16x32_f16(ha, hb, c, 0, 0, 0);
        }
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    };
    auto convert_weights = [&](int k32) {  // bf16 -> fp16 in place, once per fragment
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const f16x8_t h = bf16x8_to_f16x8(fb[k32][g]);
            __builtin_memcpy(&fb[k32][g], &h, 16);
        }
    };
    // operand fragments of unit u of K step stage_k (weight rows in ring slot bslot)
    // (nmi_tag: the wave's number of 32-row blocks as a constant, 0 = use the runtime value)
    auto read_frags = [&](int stage_k, int bslot, int u, auto nmi_tag) {
        constexpr int NMI = decltype(nmi_tag)::value;
        const int h = u & 1, k32 = u >> 1;
        const uint8_t* sa = smem + (stage_k & 1) * kSlotBytes;
        const uint8_t* sb = smem + bslot * kSlotBytes;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (NMI ? (h * 4 + j < 2 * NMI) : (h * 4 + j < 2 * nmi))
                fa[h][j] = *reinterpret_cast<const bf16x8_t*>(sa + a_off[k32] + frag_off(h * 4 + j));
        if (h == 0) {
#pragma unroll
            for (int g = 0; g < 4; ++g) fb[k32][g] = *reinterpret_cast<const bf16x8_t*>(sb + b_off[k32] + g * 2048);
        }
    };
    // the 16 MFMAs of unit u; `reads` LDS reads issued just before the call are spread one behind each of the first MFMAs
    auto multiply = [&](int u, auto reads_tag, auto nmi_tag) {
        constexpr int NMI = decltype(nmi_tag)::value;
        constexpr bool FULL = NMI == 4;
        constexpr int reads = decltype(reads_tag)::value;
        const int h = u & 1, k32 = u >> 1;
        if (MODE == 2 && F16 == 1 && h == 0) convert_weights(k32);  // unit u is the first to use the fragments of this K half
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (NMI ? (h * 4 + j < 2 * NMI) : (h * 4 + j < 2 * nmi)) {
#pragma unroll
                for (int gi = 0; gi < 4; ++gi) {
                    const int g = (j & 1) ? 3 - gi : gi;  // serpentine: one operand changes between neighbours
                    acc[h * 4 + j][g] = mma(fa[h][j], fb[k32][g], acc[h * 4 + j][g]);
                }
            }
        if (FULL) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (i < reads) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
            __builtin_amdgcn_sched_group_barrier(0x008, 16 - reads, 0);
        }
    };
    const std::integral_constant<int, 0> r0;
    const std::integral_constant<int, 4> r4;
    const std::integral_constant<int, 8> r8;
    auto next_slot = [](int slot) { return slot == kSlotsB - 1 ? 0 : slot + 1; };

    // Copies are queued per wave in the order  A(0) B(0) B(1) | A(1) B(2) | A(2) B(3) | ...  so that at the end
    // of step kt everything but the newest four copies (B(kt+2)) has to be in LDS: vmcnt(4), vmcnt(0) at the end.
    issue_a(0);
    issue_b(0, 0);
    if (1 < nk) {
        issue_b(1, 1);
        wait_dma<kDmaHalf>();
    } else {
        wait_dma<0>();
    }
    block_barrier();
    if (1 < nk) issue_a(1);
    if (2 < nk) issue_b(2, 2);
    // the next tile's ticket is drawn now and looked at when this tile is done (the atomic counts as one more
    // memory operation in flight for thread 0's wave, which can only make that wave's waits stricter)
    if (PERSIST && threadIdx.x == 0) next_n = first_ticket + atomicAdd(&tickets[my_xcd], 1);
    int bs = 0;  // ring slot of the weight rows of step kt
    // The main loop for a wave with NMI = 1 .. 4 blocks of 32 rows (a compile-time constant: fixed instruction
    // mix).  After the barrier that ends step kt, the MFMAs of its last unit alternate with the copies of A(kt+2)
    // and B(kt+3) (the slots step kt has just freed) and with the first operand reads of step kt+1.
    // w2 GEMM (kSpreadB): only the copies of A follow the barrier; the four of B(kt+3) are issued one step later,
    // between the units of step kt+1.  All eight waves hand their copies to the address unit at the same moment, which
    // works them off at one per 16 cycles: with half as many queued behind the barrier the activation rows, which
    // have one step to arrive, are in LDS sooner (w2 kernel -2 % at 8192 tokens, -5 % at 1024), and the weight rows
    // still have a step and a half.  The w13 GEMM is 1 % slower that way at 4096 tokens and more, and keeps its order.
    // Either way the wait at the end of a step leaves exactly the newest four copies, B's, in flight.
    constexpr bool kSpreadB = MODE == 2;
    auto main_loop = [&](auto nmi_tag) {
        constexpr int NMI = decltype(nmi_tag)::value;
        read_frags(0, 0, 0, nmi_tag);
        auto step = [&](int kt, auto copy_a_tag, auto copy_b_tag) {
            constexpr bool CA = decltype(copy_a_tag)::value, CB = decltype(copy_b_tag)::value;
            // (kSpreadB: B(kt+2) goes to the slot that step kt-1 has freed, in between the units of this step)
            const int bfree = bs == 0 ? kSlotsB - 1 : bs - 1;
            if (kSpreadB && CB) { copy_b(0, kt + 2, bfree); copy_b(1, kt + 2, bfree); }
            read_frags(kt, bs, 1, nmi_tag); multiply(0, r4, nmi_tag);
            if (kSpreadB && CB) copy_b(2, kt + 2, bfree);
            read_frags(kt, bs, 2, nmi_tag); multiply(1, r8, nmi_tag);
            if (kSpreadB && CB) copy_b(3, kt + 2, bfree);
            read_frags(kt, bs, 3, nmi_tag); multiply(2, r4, nmi_tag);
            if (CA) wait_dma<kDmaHalf>(); else wait_dma<0>();   // this wave's parts of A(kt+1), B(kt+1) are in LDS
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // its last reads of step kt are in registers
            block_barrier();                                    // ... and so are everyone else's
            __builtin_amdgcn_sched_barrier(0);
            const int bn = next_slot(bs);
            const uint8_t* sa = smem + ((kt + 1) & 1) * kSlotBytes;
            const uint8_t* sb = smem + bn * kSlotBytes;
            // unit 3 of step kt; behind every second MFMA a copy, behind the others a read of unit 0 of step kt+1
            // (weight fragment 0 and token fragment 0 first: the next unit starts with them).  A wave with fewer
            // than four blocks has fewer (or no) MFMAs here; its copies and reads keep their places.
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int j = i >> 2, g = (j & 1) ? 3 - (i & 3) : (i & 3);  // serpentine, as in multiply()
                if (4 + j < 2 * NMI)
                    acc[4 + j][g] = mma(fa[1][j], fb[1][g], acc[4 + j][g]);
                const int n = i >> 1;
                if ((i & 1) == 0) {
                    if (n < 4) { if (CA && (NMI == 4 || live[n])) copy_a(n, kt + 2); }
                    else { if (!kSpreadB && CB) copy_b(n - 4, kt + 3, bs); }
                } else if (n == 0) {
                    fb[0][0] = *reinterpret_cast<const bf16x8_t*>(sb + b_off[0]);
                } else if (n == 1) {
                    fa[0][0] = *reinterpret_cast<const bf16x8_t*>(sa + a_off[0]);
                } else if (n < 5) {
                    fb[0][n - 1] = *reinterpret_cast<const bf16x8_t*>(sb + b_off[0] + (n - 1) * 2048);
                } else if (n - 4 < 2 * NMI) {
                    fa[0][n - 4] = *reinterpret_cast<const bf16x8_t*>(sa + a_off[0] + frag_off(n - 4));
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            bs = bn;
        };
        int kt = 0;
        if (kSpreadB) {
            // step kt requests B(kt+2) while it multiplies (the prologue requested B(2)) and A(kt+2) behind its barrier
            if (kt + 2 < nk) { step(kt, std::true_type{}, std::false_type{}); ++kt; }
            for (; kt + 2 < nk; ++kt) step(kt, std::true_type{}, std::true_type{});
        } else {
            for (; kt + 3 < nk; ++kt) step(kt, std::true_type{}, std::true_type{});
            for (; kt + 2 < nk; ++kt) step(kt, std::true_type{}, std::false_type{});
        }
        for (; kt + 1 < nk; ++kt) step(kt, std::false_type{}, std::false_type{});
        read_frags(nk - 1, bs, 1, nmi_tag); multiply(0, r4, nmi_tag);
        read_frags(nk - 1, bs, 2, nmi_tag); multiply(1, r8, nmi_tag);
        read_frags(nk - 1, bs, 3, nmi_tag); multiply(2, r4, nmi_tag);
        multiply(3, r0, nmi_tag);
    };
    if (nmi == 4) {
        main_loop(std::integral_constant<int, 4>{});
    } else if (nmi == 3) {
        main_loop(std::integral_constant<int, 3>{});
    } else if (nmi == 2) {
        main_loop(std::integral_constant<int, 2>{});
    } else if (nmi == 1) {
        main_loop(std::integral_constant<int, 1>{});
    } else {
        // A wave without rows (the tile is one block high) still copies and meets the barriers.
        // Skipped copies of missing token rows do not change the counts: the newest four are B's.
        const std::integral_constant<int, 0> part;
        const bool work = nmi > 0;
        if (work) read_frags(0, 0, 0, part);
        for (int kt = 0; kt + 1 < nk; ++kt) {
            if (work) {
                read_frags(kt, bs, 1, part); multiply(0, r0, part);
                read_frags(kt, bs, 2, part); multiply(1, r0, part);
                read_frags(kt, bs, 3, part); multiply(2, r0, part);
            }
            if (kt + 2 < nk) wait_dma<kDmaHalf>(); else wait_dma<0>();
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            block_barrier();
            if (kt + 2 < nk) issue_a(kt + 2);
            if (kt + 3 < nk) issue_b(kt + 3, bs);
            bs = next_slot(bs);
            if (work) {
                read_frags(kt + 1, bs, 0, part);  // unit 0 of the next step lands in set 0 ...
                multiply(3, r0, part);            // ... while unit 3 multiplies set 1 of both operands
            }
        }
        if (work) {
            read_frags(nk - 1, bs, 1, part); multiply(0, r0, part);
            read_frags(nk - 1, bs, 2, part); multiply(1, r0, part);
            read_frags(nk - 1, bs, 3, part); multiply(2, r0, part);
            multiply(3, r0, part);
        }
    }

    // ---- epilogue.  Element i of lane l of a 16x16 accumulator sits at row 4*(l/16) + i, column l%16: one
    // column per lane.  Results are turned through LDS (free after the last stage) so that global stores
    // are 16 bytes per lane on full 128-byte lines.
    block_barrier();  // every wave has read its last operands: the stage buffers can be reused
    // (the lane's position in the tile, worked out again from the thread index instead of being kept through the
    // main loop, which has no register to spare)
    int tid_epi = threadIdx.x;
    if (PERSIST) asm volatile("" : "+v"(tid_epi));
    const int e_tid = tid_epi, e_lane = tid_epi & 63, e_r16 = tid_epi & 15, e_kq = (tid_epi >> 4) & 3;
    if (MODE == 1) {
        // act tile [256 rows][128 columns] bf16, row pitch 272 B
        constexpr int kPitchC = 128 * 2 + 16;
        {
            // SiLU(gate) * up in float32, rounded once to the storage type, four rows of one column at a time
            constexpr bool kAct16 = F16 != 0;
            uint32_t seen = 0;  // largest magnitude bit pattern stored as fp16 (a NaN's is larger than any number's)
#pragma unroll
            for (int f = 0; f < 8; ++f) {
                if (f >= 2 * nmi) break;
#pragma unroll
                for (int gg = 0; gg < 2; ++gg) {
                    float v[4];
                    uint16_t bits[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) v[i] = silu_mul(acc[f][gg][i], acc[f][gg + 2][i]);
                    if (kAct16) {
                        clamp_to_f16x4(v, seen, bits);
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i) bits[i] = f32_to_bf16_bits(v[i]);
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int row = frag_row(f) + 4 * e_kq + i;
                        *reinterpret_cast<uint16_t*>(smem + row * kPitchC + (wn * 32 + gg * 16 + e_r16) * 2) = bits[i];
                    }
                }
            }
            if (kAct16 && seen > kF16MaxAsF32Bits) {
                // rare: put the NaNs back (the clamp made numbers of them) and count the clamped values of rows
                // that hold a routed slot (pad rows repeat token 0)
                int n = 0;
#pragma unroll
                for (int f = 0; f < 8; ++f) {
                    if (f >= 2 * nmi) break;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int row = frag_row(f) + 4 * e_kq + i;
                        const bool routed = p.sorted_ids[m0 + row] >= 0;
#pragma unroll
                        for (int gg = 0; gg < 2; ++gg) {
                            const float val = silu_mul(acc[f][gg][i], acc[f][gg + 2][i]);
                            if (val != val)
                                *reinterpret_cast<uint16_t*>(smem + row * kPitchC + (wn * 32 + gg * 16 + e_r16) * 2) = 0x7e00;
                            else if (routed && fabsf(val) > 65504.0f)
                                ++n;
                        }
                    }
                }
                if (n > 0) atomicAdd(p.saturated, n);
            }
            __syncthreads();
            uint16_t* dst = p.act;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int c = e_tid + i * kThreads;  // 16-byte piece c of the tile: row c/16, columns (c%16)*8..+8
                const int row = c >> 4;
                if (row < valid)
                    // (non-temporal: the tile is not read again before the w2 GEMM; as ordinary stores the activations
                    // displace weight and token lines, T=400-512: +3 % on this kernel)
                    __builtin_nontemporal_store(
                        *reinterpret_cast<const u32x4_t*>(smem + row * kPitchC + (c & 15) * 16),
                        reinterpret_cast<u32x4_t*>(dst + (m0 + row) * static_cast<int64_t>(p.I) + nt * 128 + (c & 15) * 8));
            }
        }
    } else {
        // slots of the tile's rows -> LDS; then per wave and 32-row fragment a private [32][64] fp32 tile, pitch 272 B
        constexpr int kPitchY = 64 * 4 + 16;
        int32_t* slots = reinterpret_cast<int32_t*>(smem);
        uint8_t* ytile = smem + 1024 + wave * (32 * kPitchY);
        if (e_tid < kTM) slots[e_tid] = my_slot;
        __syncthreads();
        const int64_t yoff = static_cast<int64_t>(id_z) * p.T * p.top_k * p.H + nt * kTN + wn * 64;
        float* ybase = p.y + yoff;
        uint16_t* ybase_h = reinterpret_cast<uint16_t*>(p.y) + yoff;  // the same partial results as fp16 (p.y_f16)
        // kHalf: the partial sums go out as fp16.  A value beyond the fp16 range becomes the fp16 infinity (the plain
        // rounding) and is stored again as float32 at the same index of y_wide, where the combine looks when it meets
        // an infinity: the rows of a 32-row block whose e_lane saw such a value are walked a second time (rare).
        float* wbase_y = p.y_wide + yoff;
        auto store_rows = [&](auto half_tag) {
            constexpr bool kHalf = decltype(half_tag)::value;
#pragma unroll
            for (int mi = 0; mi < 4; ++mi) {
                if (mi >= nmi) break;
#pragma unroll
                for (int hh = 0; hh < 2; ++hh)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int row = hh * 16 + 4 * e_kq + i;
#pragma unroll
                        for (int g = 0; g < 4; ++g)
                            *reinterpret_cast<float*>(ytile + row * kPitchY + (g * 16 + e_r16) * 4) = acc[mi * 2 + hh][g][i];
                    }
                __builtin_amdgcn_wave_barrier();
                uint32_t seen = 0;  // largest magnitude bit pattern this e_lane stored as fp16
#pragma unroll
                for (int it = 0; it < 8; ++it) {
                    const int row = it * 4 + (e_lane >> 4);
                    const int slot = slots[(2 * mi + wm) * 32 + row];
                    f32x4_t val = *reinterpret_cast<const f32x4_t*>(ytile + row * kPitchY + (e_lane & 15) * 16);
                    if (slot >= 0) {
                        const int64_t at = static_cast<int64_t>(slot) * p.H + (e_lane & 15) * 4;
                        if (kHalf) {
                            const f16x2_t lo = __builtin_convertvector(f32x2_t{val[0], val[1]}, f16x2_t);
                            const f16x2_t hi = __builtin_convertvector(f32x2_t{val[2], val[3]}, f16x2_t);
                            uint32_t plo, phi;
                            __builtin_memcpy(&plo, &lo, 4);
                            __builtin_memcpy(&phi, &hi, 4);
                            __builtin_nontemporal_store(u32x2_t{plo, phi}, reinterpret_cast<u32x2_t*>(ybase_h + at));
#pragma unroll
                            for (int c = 0; c < 4; ++c) {
                                const uint32_t mag = __float_as_uint(val[c]) & 0x7fffffffu;
                                seen = mag > seen ? mag : seen;
                            }
                        } else {
                            __builtin_nontemporal_store(val, reinterpret_cast<f32x4_t*>(ybase + at));
                        }
                    }
                }
                if (kHalf && seen >= kF16InfAsF32Bits) {
#pragma unroll
                    for (int it = 0; it < 8; ++it) {
                        const int row = it * 4 + (e_lane >> 4);
                        const int slot = slots[(2 * mi + wm) * 32 + row];
                        const f32x4_t val = *reinterpret_cast<const f32x4_t*>(ytile + row * kPitchY + (e_lane & 15) * 16);
                        if (slot >= 0)
                            *reinterpret_cast<f32x4_t*>(wbase_y + static_cast<int64_t>(slot) * p.H + (e_lane & 15) * 4) = val;
                    }
                }
                __builtin_amdgcn_wave_barrier();
            }
        };
        if (p.y_f16) store_rows(std::true_type{});
        else store_rows(std::false_type{});
    }
    }  // next tile
}

}  // namespace

bool tile_shape_ok(int H, int I) { return H % kTN == 0 && I % 128 == 0 && H % kTK == 0 && I % kTK == 0; }
int tile_row_block() { return kRowBlock; }

bool tile_supported(const MoeProblem& p) {
    // copy addresses are 32-bit byte offsets from x, from an expert's weights and from a tile of act
    const int64_t lim = int64_t{1} << 32;
    return p.block == kRowBlock && tile_shape_ok(p.H, p.I) && p.T > 0 && p.ksplit >= 1 &&
           p.I % (p.ksplit * kTK) == 0 && p.T * p.H * 2 < lim && int64_t{4} * p.I * p.H < lim &&
           int64_t{kTM} * p.I * 2 < lim;
}

namespace {
__global__ void zero_tickets_kernel(int* tickets) {
    if (threadIdx.x < kXcds) tickets[threadIdx.x] = 0;
}
}  // namespace

// tickets: kXcds ints of device memory of this launch's own, zero when the kernel starts (cleared by the sort kernel in
// front of the GEMMs, or here, on the stream, with clear_tickets); nullptr: one workgroup per tile, handed out by the
// hardware.
int launch_gemm_tile(const MoeProblem& p, const int32_t* seg_begin, int mode, int* tickets, bool clear_tickets,
                     hipStream_t s) {
    if (!tile_supported(p)) return EM_ERR_UNSUPPORTED;
    const int ntiles_n = (mode == 1) ? p.I / 128 : p.H / kTN;
    // upper bound of the sum over experts of ceil(padded rows_e / 256)
    const int64_t max_mtiles = ceil_div(p.T * p.top_k + static_cast<int64_t>(p.E) * (kRowBlock - 1), kTM) + p.E;
    const int64_t total = max_mtiles * ntiles_n;
    const unsigned grid = static_cast<unsigned>(round_up(total, kXcds));
    if (grid == 0) return 0;
    constexpr int lds_bytes = kLdsBytes;
    // Opt in to more than 64 KB of dynamic LDS once per device.  The flags only cache an
    // idempotent runtime call; a race between threads at worst repeats it.
    static std::atomic<bool> attr_set[64];
    static std::atomic<int> num_cus[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    if (!attr_set[dev].load(std::memory_order_acquire)) {
        const void* kernels[18] = {reinterpret_cast<const void*>(gemm_tile_kernel<1, false, 1, false>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<1, true, 1, false>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<1, false, 1, true>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<1, true, 1, true>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<1, false, 0, false>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<1, true, 0, false>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<2, false, 0, false>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<2, true, 0, false>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<2, false, 1, false>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<2, true, 1, false>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<2, false, 2, false>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<2, true, 2, false>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<1, false, 0, true>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<1, true, 0, true>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<2, false, 0, true>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<2, true, 0, true>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<2, false, 2, true>),
                                   reinterpret_cast<const void*>(gemm_tile_kernel<2, true, 2, true>)};
        for (const void* k : kernels) {
            hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
            if (e != hipSuccess) return static_cast<int>(e);
        }
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < kXcds) cus = 256;
        num_cus[dev].store(cus, std::memory_order_relaxed);
        attr_set[dev].store(true, std::memory_order_release);
    }
    // one row tile per expert on average up to 7/8 full: weights are read once -> streaming copies.  The w2 GEMM keeps
    // them up to 1.25 row tiles per expert (T=1024-1280: -7 % on the kernel); the w13 GEMM does not: its streaming form
    // also starts the tiles at different K offsets, which costs 8 % once most experts have two row tiles that share weights.
    const bool stream_b = p.T * p.top_k * 8 <= static_cast<int64_t>(p.E) * kTM * (mode == 1 ? 7 : 10);
    const int nz = (mode == 1) ? 1 : p.ksplit;
    const int kslice = (mode == 1) ? p.H : p.I / p.ksplit;
    // (the w2 kernel that converts bf16 weight fragments on the way has no register left for the tile queue: it runs
    // one workgroup per tile; the loader's float16 w2 and bf16 activations take the queue)
    const bool converts = mode == 2 && p.act_f16 && !p.w2_f16;
    const bool persist = tickets != nullptr && !converts;
    dim3 g(grid, static_cast<unsigned>(nz));
    if (persist) {
        // one workgroup per CU (a workgroup takes all of a CU's LDS), a multiple of 8 so that ids map to XCDs
        const int64_t ids = static_cast<int64_t>(grid) * nz;
        const int64_t cus = num_cus[dev].load(std::memory_order_relaxed) / kXcds * kXcds;
        g = dim3(static_cast<unsigned>(ids < cus ? ids : cus), 1);
        if (clear_tickets) launch(zero_tickets_kernel, dim3(1), dim3(64), 0, s, tickets);
    }
    auto go = [&](auto kernel) {
        launch(kernel, g, dim3(kThreads), lds_bytes, s, p, seg_begin, ntiles_n, kslice, static_cast<int>(grid), nz, tickets);
    };
#define EM_TILE_GO(MODE, F16)                                              \
    do {                                                                   \
        if (persist) {                                                     \
            if (stream_b) go(gemm_tile_kernel<MODE, true, F16, true>);     \
            else go(gemm_tile_kernel<MODE, false, F16, true>);             \
        } else {                                                           \
            if (stream_b) go(gemm_tile_kernel<MODE, true, F16, false>);    \
            else go(gemm_tile_kernel<MODE, false, F16, false>);            \
        }                                                                  \
    } while (0)
    if (mode == 1 && p.act_f16) EM_TILE_GO(1, 1);
    else if (mode == 1) EM_TILE_GO(1, 0);
    else if (p.act_f16 && p.w2_f16) EM_TILE_GO(2, 2);
    else if (p.act_f16) {
        if (stream_b) go(gemm_tile_kernel<2, true, 1, false>);
        else go(gemm_tile_kernel<2, false, 1, false>);
    } else EM_TILE_GO(2, 0);
#undef EM_TILE_GO
    return launch_status();
}

}  // namespace em
