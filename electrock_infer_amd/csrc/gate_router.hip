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
    reduce_tiles_and_route<E_, kGateWaves>(acc, partial, wave, lane, t0, T, k, renorm, round_bf16, logits_out, out_w,
                                           out_ids);
}

// The same with RMSNorm, optionally behind a residual add, in front (models/mixtral.py:194-197:
// post_attention_layernorm, then block_sparse_moe): the workgroup takes the sum of squares of its 16 rows of
// x (+ residual), writing the new residual, then normalises them, writes the normalised rows for the expert
// GEMMs and feeds them to the MFMA as it goes.  RESIDENT (H <= 4096): a lane keeps its 128 values of the
// summed rows in registers between the two passes; else the rows are read a second time, out of L2.
// Rounding points as in norm.hip (LAYER: the module's, else the native op's).  bf16 rows only.
constexpr int kNormGateWaves = 16;   // 1024 threads: 64 kept values per lane leave room for four waves per SIMD
constexpr int kNormGateThreads = kNormGateWaves * kWave;
constexpr int kNormBatch = 4;        // K steps whose loads are in flight together (8 would spill)
constexpr int64_t kFusedNormMaxT = 16;  // up to here norm + gate + router share one launch
constexpr int kResidentSteps = 8;    // K steps of 32 a wave keeps in registers: 16 waves x 8 x 32 = 4096
template <int E_, typename WElem, bool ADD, bool LAYER, bool RESIDENT>
__global__ __launch_bounds__(kNormGateThreads) void norm_gate_router_kernel(
    // h_out may be x_in (plain norm, or norm of the sum with the residual written elsewhere): no __restrict__ on the rows
    const uint16_t* x_in, const uint16_t* res_in,
    const typename WElem::storage* __restrict__ norm_w, float eps, uint16_t* h_out,
    uint16_t* res_out, const uint16_t* __restrict__ gate_w, int64_t T, int H, int k, int renorm,
    int round_bf16, void* __restrict__ logits_out, float* __restrict__ out_w, int32_t* __restrict__ out_ids) {
    static_assert(E_ == 8 || E_ == 16, "experts sit in the 16 rows of one MFMA");
    __shared__ __attribute__((aligned(16))) float partial[kNormGateWaves][kGateTokens][E_];
    __shared__ float sumsq[kNormGateWaves][kGateTokens];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int r16 = lane & 15;
    const int kq = lane >> 4;
    const int64_t t0 = static_cast<int64_t>(blockIdx.x) * kGateTokens;
    const int nsteps = (H + 31) / 32;
    const int per_wave = (nsteps + kNormGateWaves - 1) / kNormGateWaves;
    const int s_begin = wave * per_wave;
    const int s_end = (s_begin + per_wave < nsteps) ? s_begin + per_wave : nsteps;
    const bool tok_ok = (t0 + r16 < T);
    const int64_t row = (tok_ok ? t0 + r16 : 0) * H;
    const uint16_t* grow = gate_w + static_cast<int64_t>(r16 % E_) * H;

    // the 8 values of one piece of the (summed) row in float32; with ADD the rounded sum goes to `rounded`
    auto row_piece = [&](const u32x4_t xv, const u32x4_t rv, float (&s)[8], u32x4_t& rounded) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float lo = bf16_lo(xv[j]), hi = bf16_hi(xv[j]);
            if (ADD) {
                lo += bf16_lo(rv[j]);
                hi += bf16_hi(rv[j]);
                rounded[j] = pack_bf16(lo, hi);
                if (!LAYER) {
                    lo = bf16_lo(rounded[j]);
                    hi = bf16_hi(rounded[j]);
                }
            }
            s[2 * j] = lo;
            s[2 * j + 1] = hi;
        }
    };

    // ---- pass 1: sum of squares of this wave's slice of the 16 rows; the new residual ----
    float kept[RESIDENT ? kResidentSteps : 1][8];
    float sq = 0.0f;
#pragma unroll
    for (int b = 0; b < (RESIDENT ? kResidentSteps / kNormBatch : 1 << 30); ++b) {
        const int s0 = s_begin + b * kNormBatch;
        if (s0 >= s_end) break;
        u32x4_t xa[kNormBatch], ra[kNormBatch];
#pragma unroll
        for (int i = 0; i < kNormBatch; ++i) {
            const int h = (s0 + i) * 32 + kq * 8;
            const bool ok = (s0 + i < s_end) && (h < H) && tok_ok;
            xa[i] = ok ? *reinterpret_cast<const u32x4_t*>(x_in + row + h) : u32x4_t{0u, 0u, 0u, 0u};
            if (ADD) ra[i] = ok ? *reinterpret_cast<const u32x4_t*>(res_in + row + h) : u32x4_t{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int i = 0; i < kNormBatch; ++i) {
            const int h = (s0 + i) * 32 + kq * 8;
            const bool ok = (s0 + i < s_end) && (h < H) && tok_ok;
            float sv[8];
            u32x4_t rounded;
            row_piece(xa[i], ra[i], sv, rounded);
#pragma unroll
            for (int j = 0; j < 8; ++j) sq = fmaf(sv[j], sv[j], sq);
            if (RESIDENT) {
#pragma unroll
                for (int j = 0; j < 8; ++j) kept[b * kNormBatch + i][j] = sv[j];
            }
            if (ADD && ok) *reinterpret_cast<u32x4_t*>(res_out + row + h) = rounded;
        }
    }
    sq += __shfl_xor(sq, 16);
    sq += __shfl_xor(sq, 32);
    if (kq == 0) sumsq[wave][r16] = sq;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < kNormGateWaves; ++w) total += sumsq[w][r16];
    const float rstd = 1.0f / sqrtf(total / static_cast<float>(H) + eps);

    // ---- pass 2: normalise (the rows come out of L2 this time), store, multiply with the gate rows ----
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int b = 0; b < (RESIDENT ? kResidentSteps / kNormBatch : 1 << 30); ++b) {
        const int s0 = s_begin + b * kNormBatch;
        if (s0 >= s_end) break;
        u32x4_t xa[kNormBatch], ra[kNormBatch], ga[kNormBatch];
#pragma unroll
        for (int i = 0; i < kNormBatch; ++i) {
            const int h = (s0 + i) * 32 + kq * 8;
            const bool okk = (s0 + i < s_end) && (h < H);
            const bool ok = okk && tok_ok;
            if (!RESIDENT) {
                xa[i] = ok ? *reinterpret_cast<const u32x4_t*>(x_in + row + h) : u32x4_t{0u, 0u, 0u, 0u};
                if (ADD) ra[i] = ok ? *reinterpret_cast<const u32x4_t*>(res_in + row + h) : u32x4_t{0u, 0u, 0u, 0u};
            }
            ga[i] = okk ? *reinterpret_cast<const u32x4_t*>(grow + h) : u32x4_t{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int i = 0; i < kNormBatch; ++i) {
            const int h = (s0 + i) * 32 + kq * 8;
            const bool okk = (s0 + i < s_end) && (h < H);
            float sv[8], wv[8];
            if (RESIDENT) {
#pragma unroll
                for (int j = 0; j < 8; ++j) sv[j] = kept[b * kNormBatch + i][j];
            } else {
                u32x4_t rounded;
                row_piece(xa[i], ra[i], sv, rounded);
            }
            if (sizeof(typename WElem::storage) == 2) {   // 8 bf16 weights: one 16-byte piece
                const u32x4_t w4 = okk ? *reinterpret_cast<const u32x4_t*>(norm_w + h) : u32x4_t{0u, 0u, 0u, 0u};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    wv[2 * j] = bf16_lo(w4[j]);
                    wv[2 * j + 1] = bf16_hi(w4[j]);
                }
            } else {                                      // 8 fp32 weights: two pieces
                const f32x4_t z = {0.f, 0.f, 0.f, 0.f};
                const f32x4_t wa = okk ? *reinterpret_cast<const f32x4_t*>(norm_w + h) : z;
                const f32x4_t wb = okk ? *reinterpret_cast<const f32x4_t*>(norm_w + h + 4) : z;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    wv[j] = wa[j];
                    wv[4 + j] = wb[j];
                }
            }
            u32x4_t yb;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float lo, hi;
                if (LAYER) {
                    const uint32_t tpair = pack_bf16(sv[2 * j] * rstd, sv[2 * j + 1] * rstd);
                    lo = bf16_lo(tpair) * wv[2 * j];
                    hi = bf16_hi(tpair) * wv[2 * j + 1];
                } else {
                    lo = (sv[2 * j] * wv[2 * j]) * rstd;
                    hi = (sv[2 * j + 1] * wv[2 * j + 1]) * rstd;
                }
                yb[j] = pack_bf16(lo, hi);
            }
            if (okk && tok_ok) *reinterpret_cast<u32x4_t*>(h_out + row + h) = yb;
            if (!(okk && tok_ok)) yb = u32x4_t{0u, 0u, 0u, 0u};  // rows / columns that do not exist multiply as zero
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, ga[i]),
                                                          __builtin_bit_cast(bf16x8_t, yb), acc, 0, 0, 0);
        }
    }
    reduce_tiles_and_route<E_, kNormGateWaves>(acc, partial, wave, lane, t0, T, k, renorm, round_bf16, logits_out, out_w,
                                           out_ids);
}

template <int E_, typename WElem, bool RESIDENT>
void launch_norm_gate(bool add, bool layer, unsigned grid, hipStream_t s, const uint16_t* x, const uint16_t* r,
                      const void* nw, float eps, uint16_t* h, uint16_t* ro, const uint16_t* g, int64_t T, int H, int k,
                      int renorm, int round_bf16, void* lo, float* w, int32_t* ids) {
    typedef typename WElem::storage WS;
    const WS* nwp = static_cast<const WS*>(nw);
    const dim3 gd(grid), bd(kNormGateThreads);
    if (add && layer)
        launch((norm_gate_router_kernel<E_, WElem, true, true, RESIDENT>), gd, bd, 0, s, x, r, nwp, eps, h, ro, g, T, H, k, renorm, round_bf16, lo, w, ids);
    else if (add)
        launch((norm_gate_router_kernel<E_, WElem, true, false, RESIDENT>), gd, bd, 0, s, x, r, nwp, eps, h, ro, g, T, H, k, renorm, round_bf16, lo, w, ids);
    else if (layer)
        launch((norm_gate_router_kernel<E_, WElem, false, true, RESIDENT>), gd, bd, 0, s, x, r, nwp, eps, h, ro, g, T, H, k, renorm, round_bf16, lo, w, ids);
    else
        launch((norm_gate_router_kernel<E_, WElem, false, false, RESIDENT>), gd, bd, 0, s, x, r, nwp, eps, h, ro, g, T, H, k, renorm, round_bf16, lo, w, ids);
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
        launch(gate_router_kernel<8>, dim3(grid), dim3(kGateThreads), 0, s, xp, gp, T, H, k, renorm,
                           round_bf16, logits_out, w, ids);
    else
        launch(gate_router_kernel<16>, dim3(grid), dim3(kGateThreads), 0, s, xp, gp, T, H, k, renorm,
                           round_bf16, logits_out, w, ids);
    return launch_status();
}

}  // namespace em

namespace em {

int launch_norm_gate_router(const void* x_in, const void* res_in, const void* norm_w, int norm_w_dtype, float eps,
                            bool layer_semantics, void* h_out, void* res_out, const void* gate_w, int64_t T, int H,
                            int E, int k, int renorm, int round_bf16, void* logits_out, float* w, int32_t* ids,
                            hipStream_t s) {
    if (T == 0) return 0;
    if (!gate_router_supported(H, E)) return EM_ERR_UNSUPPORTED;
    if (norm_w_dtype != EM_DTYPE_BF16 && norm_w_dtype != EM_DTYPE_F32) return EM_ERR_BAD_DTYPE;
    // One launch pays while the launch itself is what costs (a single workgroup: 14 against 9 + 9 us at T = 1).
    // Beyond that the row-per-workgroup norm kernel followed by the gate kernel is as fast or faster (the fused
    // workgroup is a chain of load, reduce, barrier, scale and store, with one workgroup per CU), so those run.
    if (T > kFusedNormMaxT && rms_norm_supported(H, EM_DTYPE_BF16, norm_w_dtype)) {
        const int rc = launch_rms_norm(x_in, res_in, norm_w, h_out, res_out, T, H, eps, EM_DTYPE_BF16, norm_w_dtype,
                                       layer_semantics, s);
        if (rc != 0) return rc;
        return launch_gate_router(h_out, gate_w, T, H, E, k, renorm, round_bf16, logits_out, w, ids, s);
    }
    const unsigned grid = static_cast<unsigned>(ceil_div(T, static_cast<int64_t>(kGateTokens)));
    const uint16_t* xp = static_cast<const uint16_t*>(x_in);
    const uint16_t* rp = static_cast<const uint16_t*>(res_in);
    uint16_t* hp = static_cast<uint16_t*>(h_out);
    uint16_t* rop = static_cast<uint16_t*>(res_out);
    const uint16_t* gp = static_cast<const uint16_t*>(gate_w);
    const bool add = res_in != nullptr;
    const bool w32 = norm_w_dtype == EM_DTYPE_F32;
    const bool resident = ceil_div(ceil_div(H, 32), kNormGateWaves) <= kResidentSteps;
#define EM_NORM_GATE(E_, W_, R_) launch_norm_gate<E_, W_, R_>(add, layer_semantics, grid, s, xp, rp, norm_w, eps, hp, rop, gp, T, H, k, renorm, round_bf16, logits_out, w, ids)
    if (E == 8) {
        if (w32) { if (resident) EM_NORM_GATE(8, F32Elem, true); else EM_NORM_GATE(8, F32Elem, false); }
        else { if (resident) EM_NORM_GATE(8, BF16Elem, true); else EM_NORM_GATE(8, BF16Elem, false); }
    } else {
        if (w32) { if (resident) EM_NORM_GATE(16, F32Elem, true); else EM_NORM_GATE(16, F32Elem, false); }
        else { if (resident) EM_NORM_GATE(16, BF16Elem, true); else EM_NORM_GATE(16, BF16Elem, false); }
    }
#undef EM_NORM_GATE
    return launch_status();
}

}  // namespace em
