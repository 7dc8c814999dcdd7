// RMSNorm and residual-add + RMSNorm: the step in front of the MoE block
// (models/mixtral.py:194-197: post_attention_layernorm, then block_sparse_moe).
//
// One workgroup per token row; every thread keeps its 16-byte pieces of the row in registers
// between the sum of squares and the scaling, so a row is read once and written once:
// the kernel is an HBM stream of 2 (norm) or 4 (add + norm) rows of H elements per token.
//
// Two sets of rounding points exist in the reference and both are offered:
//   EM_NORM_LAYER  what the model runs (layers/layernorm.py:17-41): s = f32(x) + f32(residual);
//                  residual' = T(s); var = mean(s^2) on the un-rounded sum;
//                  y = T( f32(T(s * rsqrt(var + eps))) * f32(w) )
//   EM_NORM_OP     the native op (src/add_rms_norm.hip:24-84, 87-140): r = T(x + residual);
//                  residual' = r; var = mean(f32(r)^2); y = T( (f32(r) * f32(w)) * rsqrt(var + eps) )
// with T the rounding to the element type (identity for fp32).
#include "common.h"

namespace em {
namespace {

constexpr int kNormThreads = 256;
constexpr int kNormWaves = kNormThreads / kWave;
constexpr int kNormMaxVec = 8;  // 16-byte pieces of a row per thread: H <= 16384 (16-bit) / 8192 (fp32)

template <typename Elem> struct NormVec { static constexpr int n = 16 / sizeof(typename Elem::storage); };

template <typename Elem, typename WElem, bool ADD, bool LAYER>
__global__ __launch_bounds__(kNormThreads) void rms_norm_kernel(
    // x_out may be x_in and res_out may be res_in (the native op works in place): no __restrict__ on those four
    const typename Elem::storage* x_in, const typename Elem::storage* res_in,
    const typename WElem::storage* __restrict__ weight, typename Elem::storage* x_out,
    typename Elem::storage* res_out, int H, float eps) {
    typedef typename Elem::storage S;
    typedef typename WElem::storage WS;
    constexpr int V = NormVec<Elem>::n;
    __shared__ float wave_sum[kNormWaves];
    const int tid = threadIdx.x;
    const int nvec = H / V;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * H;

    float s[kNormMaxVec][V];
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < kNormMaxVec; ++i) {
        const int c = tid + i * kNormThreads;
        if (c < nvec) {
            u32x4_t xv = reinterpret_cast<const u32x4_t*>(x_in + row)[c];
            S xs[V];
            __builtin_memcpy(xs, &xv, 16);
            if (ADD) {
                u32x4_t rv = reinterpret_cast<const u32x4_t*>(res_in + row)[c];
                S rs[V], ro[V];
                __builtin_memcpy(rs, &rv, 16);
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    const float a = Elem::load(xs[j]) + Elem::load(rs[j]);
                    ro[j] = Elem::store(a);
                    s[i][j] = LAYER ? a : Elem::load(ro[j]);
                }
                u32x4_t ov;
                __builtin_memcpy(&ov, ro, 16);
                reinterpret_cast<u32x4_t*>(res_out + row)[c] = ov;
            } else {
#pragma unroll
                for (int j = 0; j < V; ++j) s[i][j] = Elem::load(xs[j]);
            }
#pragma unroll
            for (int j = 0; j < V; ++j) sum = fmaf(s[i][j], s[i][j], sum);
        }
    }
    // every thread ends with the same total, added in the same order
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    if ((tid & (kWave - 1)) == 0) wave_sum[tid / kWave] = sum;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < kNormWaves; ++w) total += wave_sum[w];
    const float rstd = 1.0f / sqrtf(total / static_cast<float>(H) + eps);

#pragma unroll
    for (int i = 0; i < kNormMaxVec; ++i) {
        const int c = tid + i * kNormThreads;
        if (c < nvec) {
            WS ws[V];
            if (sizeof(WS) * V == 16) {
                u32x4_t wv = reinterpret_cast<const u32x4_t*>(weight)[c];
                __builtin_memcpy(ws, &wv, 16);
            } else {  // fp32 weight with a 16-bit row: two pieces
                u32x4_t w0 = reinterpret_cast<const u32x4_t*>(weight)[2 * c];
                u32x4_t w1 = reinterpret_cast<const u32x4_t*>(weight)[2 * c + 1];
                __builtin_memcpy(ws, &w0, 16);
                __builtin_memcpy(reinterpret_cast<char*>(ws) + 16, &w1, 16);
            }
            S ys[V];
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const float w = WElem::load(ws[j]);
                if (LAYER) {
                    const S t = Elem::store(s[i][j] * rstd);
                    ys[j] = Elem::store(Elem::load(t) * w);
                } else {
                    ys[j] = Elem::store((s[i][j] * w) * rstd);
                }
            }
            u32x4_t yv;
            __builtin_memcpy(&yv, ys, 16);
            reinterpret_cast<u32x4_t*>(x_out + row)[c] = yv;
        }
    }
}

template <typename Elem, typename WElem>
int launch_typed(const void* x_in, const void* res_in, const void* weight, void* x_out, void* res_out,
                 int64_t T, int H, float eps, bool add, bool layer, hipStream_t s) {
    typedef typename Elem::storage S;
    typedef typename WElem::storage WS;
    const dim3 grid(static_cast<unsigned>(T)), block(kNormThreads);
    const S* xi = static_cast<const S*>(x_in);
    const S* ri = static_cast<const S*>(res_in);
    const WS* w = static_cast<const WS*>(weight);
    S* xo = static_cast<S*>(x_out);
    S* ro = static_cast<S*>(res_out);
    if (add && layer)
        launch((rms_norm_kernel<Elem, WElem, true, true>), grid, block, 0, s, xi, ri, w, xo, ro, H, eps);
    else if (add)
        launch((rms_norm_kernel<Elem, WElem, true, false>), grid, block, 0, s, xi, ri, w, xo, ro, H, eps);
    else if (layer)
        launch((rms_norm_kernel<Elem, WElem, false, true>), grid, block, 0, s, xi, ri, w, xo, ro, H, eps);
    else
        launch((rms_norm_kernel<Elem, WElem, false, false>), grid, block, 0, s, xi, ri, w, xo, ro, H, eps);
    return launch_status();
}

}  // namespace

bool rms_norm_supported(int H, int dtype, int weight_dtype) {
    const int v = (dtype == EM_DTYPE_F32) ? 4 : 8;
    if (H <= 0 || H % v != 0 || H / v > kNormThreads * kNormMaxVec) return false;
    return weight_dtype == dtype || weight_dtype == EM_DTYPE_F32;
}

int launch_rms_norm(const void* x_in, const void* res_in, const void* weight, void* x_out, void* res_out,
                    int64_t T, int H, float eps, int dtype, int weight_dtype, bool layer, hipStream_t s) {
    if (T == 0) return 0;
    if (!rms_norm_supported(H, dtype, weight_dtype)) return EM_ERR_UNSUPPORTED;
    const bool add = res_in != nullptr;
    const bool w32 = weight_dtype == EM_DTYPE_F32;
    switch (dtype) {
        case EM_DTYPE_F32:
            return launch_typed<F32Elem, F32Elem>(x_in, res_in, weight, x_out, res_out, T, H, eps, add, layer, s);
        case EM_DTYPE_BF16:
            return w32 ? launch_typed<BF16Elem, F32Elem>(x_in, res_in, weight, x_out, res_out, T, H, eps, add, layer, s)
                       : launch_typed<BF16Elem, BF16Elem>(x_in, res_in, weight, x_out, res_out, T, H, eps, add, layer, s);
        case EM_DTYPE_F16:
            return w32 ? launch_typed<F16Elem, F32Elem>(x_in, res_in, weight, x_out, res_out, T, H, eps, add, layer, s)
                       : launch_typed<F16Elem, F16Elem>(x_in, res_in, weight, x_out, res_out, T, H, eps, add, layer, s);
        default:
            return EM_ERR_BAD_DTYPE;
    }
}

}  // namespace em
