// Stand-alone element-wise ops of the reference `_C` surface: silu_and_mul and
// moe_sum.  Both are pure HBM streams: 16-byte loads/stores per lane, lanes on
// consecutive addresses, a 2-D grid (row, column block) so that any (rows, width) fills the chip.
// The fused layer path does not use them (SiLU*mul lives in the first expert
// GEMM's epilogue, the top-k sum in the combine kernel).
#include "common.h"

namespace em {
namespace {

constexpr int kEwThreads = 256;

template <typename Elem> struct VecOf;          // elements per 16-byte vector
template <> struct VecOf<F32Elem> { static constexpr int n = 4; };
template <> struct VecOf<BF16Elem> { static constexpr int n = 8; };
template <> struct VecOf<F16Elem> { static constexpr int n = 8; };

template <typename Elem, bool kFastExp>
__device__ __forceinline__ typename Elem::storage silu_mul_one(typename Elem::storage g,
                                                              typename Elem::storage u) {
    // reference: SiLU in fp32, rounded to the element type, then a multiply in
    // the element type (src/activation_kernels.hip:40-45)
    const float gf = Elem::load(g);
    const float s = gf / (1.0f + (kFastExp ? __expf(-gf) : expf(-gf)));
    const typename Elem::storage sr = Elem::store(s);
    return Elem::store(Elem::load(sr) * Elem::load(u));
}

template <typename Elem, bool kVec>
__global__ __launch_bounds__(kEwThreads) void silu_and_mul_kernel(
    typename Elem::storage* __restrict__ out, const typename Elem::storage* __restrict__ in, int64_t d) {
    typedef typename Elem::storage S;
    constexpr bool kFast = sizeof(S) == 2;  // the reference uses __expf for 16-bit types, expf for fp32
    constexpr int V = VecOf<Elem>::n;
    const int64_t row = blockIdx.x;
    const S* gate = in + row * 2 * d;
    const S* up = gate + d;
    S* o = out + row * d;
    if (kVec) {
        const int64_t nvec = d / V;
        for (int64_t v = static_cast<int64_t>(blockIdx.y) * kEwThreads + threadIdx.x; v < nvec;
             v += static_cast<int64_t>(gridDim.y) * kEwThreads) {
            u32x4_t gv = reinterpret_cast<const u32x4_t*>(gate)[v];
            u32x4_t uv = reinterpret_cast<const u32x4_t*>(up)[v];
            u32x4_t ov;
            S gs[V], us[V], os[V];
            __builtin_memcpy(gs, &gv, 16);
            __builtin_memcpy(us, &uv, 16);
#pragma unroll
            for (int i = 0; i < V; ++i) os[i] = silu_mul_one<Elem, kFast>(gs[i], us[i]);
            __builtin_memcpy(&ov, os, 16);
            reinterpret_cast<u32x4_t*>(o)[v] = ov;
        }
    } else {
        for (int64_t j = static_cast<int64_t>(blockIdx.y) * kEwThreads + threadIdx.x; j < d;
             j += static_cast<int64_t>(gridDim.y) * kEwThreads)
            o[j] = silu_mul_one<Elem, kFast>(gate[j], up[j]);
    }
}

template <typename Elem, bool kVec>
__global__ __launch_bounds__(kEwThreads) void moe_sum_kernel(
    const typename Elem::storage* __restrict__ in, typename Elem::storage* __restrict__ out, int topk,
    int64_t H) {
    typedef typename Elem::storage S;
    constexpr int V = VecOf<Elem>::n;
    const int64_t t = blockIdx.x;
    const S* src = in + t * topk * H;
    S* dst = out + t * H;
    if (kVec) {
        const int64_t nvec = H / V;
        for (int64_t v = static_cast<int64_t>(blockIdx.y) * kEwThreads + threadIdx.x; v < nvec;
             v += static_cast<int64_t>(gridDim.y) * kEwThreads) {
            S acc[V];
#pragma unroll
            for (int i = 0; i < V; ++i) acc[i] = Elem::store(0.0f);
            for (int kk = 0; kk < topk; ++kk) {
                u32x4_t xv = reinterpret_cast<const u32x4_t*>(src + kk * H)[v];
                S xs[V];
                __builtin_memcpy(xs, &xv, 16);
                // accumulate in the element type, one rounding per add (src/moe_sum.hip:38-44)
#pragma unroll
                for (int i = 0; i < V; ++i) acc[i] = Elem::store(Elem::load(acc[i]) + Elem::load(xs[i]));
            }
            u32x4_t ov;
            __builtin_memcpy(&ov, acc, 16);
            reinterpret_cast<u32x4_t*>(dst)[v] = ov;
        }
    } else {
        for (int64_t j = static_cast<int64_t>(blockIdx.y) * kEwThreads + threadIdx.x; j < H;
             j += static_cast<int64_t>(gridDim.y) * kEwThreads) {
            S acc = Elem::store(0.0f);
            for (int kk = 0; kk < topk; ++kk) acc = Elem::store(Elem::load(acc) + Elem::load(src[kk * H + j]));
            dst[j] = acc;
        }
    }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <typename Elem>
int run_silu(void* out, const void* in, int64_t rows, int64_t d, hipStream_t s) {
    typedef typename Elem::storage S;
    constexpr int V = VecOf<Elem>::n;
    const bool vec = (d % V == 0) && aligned16(out) && aligned16(in);
    const int64_t work = vec ? d / V : d;
    const dim3 grid(static_cast<unsigned>(rows),
                    static_cast<unsigned>(ceil_div(work, kEwThreads) < 64 ? ceil_div(work, kEwThreads) : 64));
    if (vec)
        launch((silu_and_mul_kernel<Elem, true>), grid, dim3(kEwThreads), 0, s,
                           static_cast<S*>(out), static_cast<const S*>(in), d);
    else
        launch((silu_and_mul_kernel<Elem, false>), grid, dim3(kEwThreads), 0, s,
                           static_cast<S*>(out), static_cast<const S*>(in), d);
    return launch_status();
}

template <typename Elem>
int run_sum(const void* in, void* out, int64_t T, int topk, int64_t H, hipStream_t s) {
    typedef typename Elem::storage S;
    constexpr int V = VecOf<Elem>::n;
    const bool vec = (H % V == 0) && aligned16(out) && aligned16(in);
    const int64_t work = vec ? H / V : H;
    const dim3 grid(static_cast<unsigned>(T),
                    static_cast<unsigned>(ceil_div(work, kEwThreads) < 64 ? ceil_div(work, kEwThreads) : 64));
    if (vec)
        launch((moe_sum_kernel<Elem, true>), grid, dim3(kEwThreads), 0, s,
                           static_cast<const S*>(in), static_cast<S*>(out), topk, H);
    else
        launch((moe_sum_kernel<Elem, false>), grid, dim3(kEwThreads), 0, s,
                           static_cast<const S*>(in), static_cast<S*>(out), topk, H);
    return launch_status();
}

}  // namespace

int launch_silu_and_mul(void* out, const void* in, int64_t rows, int64_t d, int dtype, hipStream_t s) {
    if (rows == 0 || d == 0) return 0;
    switch (dtype) {
        case EM_DTYPE_F32: return run_silu<F32Elem>(out, in, rows, d, s);
        case EM_DTYPE_BF16: return run_silu<BF16Elem>(out, in, rows, d, s);
        case EM_DTYPE_F16: return run_silu<F16Elem>(out, in, rows, d, s);
        default: return EM_ERR_BAD_DTYPE;
    }
}

int launch_moe_sum(const void* in, void* out, int64_t T, int topk, int64_t H, int dtype, hipStream_t s) {
    if (T == 0 || H == 0) return 0;
    switch (dtype) {
        case EM_DTYPE_F32: return run_sum<F32Elem>(in, out, T, topk, H, s);
        case EM_DTYPE_BF16: return run_sum<BF16Elem>(in, out, T, topk, H, s);
        case EM_DTYPE_F16: return run_sum<F16Elem>(in, out, T, topk, H, s);
        default: return EM_ERR_BAD_DTYPE;
    }
}

}  // namespace em
