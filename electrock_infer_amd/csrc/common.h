// Shared device/host helpers for the gfx950 MoE kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <tuple>
#include <utility>
#include "../../include/electrock_moe.h"

namespace em {

constexpr int kWave = 64;          // CDNA wavefront width
constexpr int kMaxExperts = 64;    // one lane per expert in the router / sort
constexpr int kMaxTopK = 8;
// Counters of one layer call, one int32 each, cleared by the sort in front of the GEMMs: [0, 8) tile tickets of the
// w13 launch, [8, 16) of the w2 launch (one per XCD), [16] activations clamped to the fp16 range.
constexpr int kLayerCounters = 17;
constexpr int kSaturatedCounter = 16;

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

__host__ __device__ constexpr int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
__host__ __device__ constexpr int64_t round_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }

// ---- bf16 / f16 <-> f32 on raw bits (round to nearest even) -----------------
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) {
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    const __bf16 b = static_cast<__bf16>(f);  // v_cvt_pk_bf16_f32: round to nearest even, NaN stays NaN
    uint16_t h;
    __builtin_memcpy(&h, &b, 2);
    return h;
}
// SiLU(g) * u in fp32 for the fused GEMM epilogues; the reciprocal is the hardware's (1 ulp)
__device__ __forceinline__ float silu_mul(float g, float u) {
    return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u;
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return static_cast<float>(v);
}
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
    _Float16 v = static_cast<_Float16>(f);
    uint16_t h;
    __builtin_memcpy(&h, &v, 2);
    return h;
}
// fp16 with out-of-range values clamped to the largest finite one (a NaN stays a NaN)
__device__ __forceinline__ uint16_t f32_to_f16_bits_sat(float f) {
    const float c = fminf(fmaxf(f, -65504.0f), 65504.0f);
    return f32_to_f16_bits(f != f ? f : c);
}
// two packed bf16 in one dword
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
// Eight bf16 as fp16: exact for every bf16 value of magnitude 2^-14 .. 65504 (fp16 has the longer mantissa); smaller
// ones keep an absolute error below 2^-25, larger ones become the largest finite fp16.
__device__ __forceinline__ f16x8_t bf16x8_to_f16x8(bf16x8_t v) {
    u32x4_t w;
    __builtin_memcpy(&w, &v, 16);
    f16x8_t out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const auto h = __builtin_amdgcn_cvt_pkrtz(bf16_lo(w[i]), bf16_hi(w[i]));
        out[2 * i] = h[0];
        out[2 * i + 1] = h[1];
    }
    return out;
}
// Four SiLU*mul results as fp16 bits, clamped to +-65504, for the GEMM epilogues; `seen` keeps the largest magnitude
// bit pattern that went through (a NaN's is larger than every number's), so that the caller can tell afterwards, with
// one compare, whether anything was clamped or was a NaN -- a NaN comes out of the clamp as a number and has to be put
// back by the caller.  v_med3 + a packed conversion: a third of the instructions of a compare-and-select clamp.
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
constexpr uint32_t kF16MaxAsF32Bits = 0x477fe000u;  // 65504.0f
constexpr uint32_t kF16InfAsF32Bits = 0x477ff000u;  // 65520.0f: from here on a float32 rounds to the fp16 infinity
__device__ __forceinline__ void clamp_to_f16x4(const float (&v)[4], uint32_t& seen, uint16_t (&out)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t mag = __float_as_uint(v[i]) & 0x7fffffffu;
        seen = mag > seen ? mag : seen;
    }
#pragma unroll
    for (int i = 0; i < 4; i += 2) {
        const f32x2_t c = {__builtin_amdgcn_fmed3f(v[i], -65504.0f, 65504.0f),
                           __builtin_amdgcn_fmed3f(v[i + 1], -65504.0f, 65504.0f)};
        const f16x2_t h = __builtin_convertvector(c, f16x2_t);  // round to nearest even
        uint32_t w;
        __builtin_memcpy(&w, &h, 4);
        out[i] = static_cast<uint16_t>(w);
        out[i + 1] = static_cast<uint16_t>(w >> 16);
    }
}
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    bf16x2_t v;
    v[0] = static_cast<__bf16>(lo);
    v[1] = static_cast<__bf16>(hi);
    uint32_t w;
    __builtin_memcpy(&w, &v, 4);
    return w;
}

// Element traits for the three storage types the ops accept.
struct F32Elem {
    typedef float storage;
    static __device__ __forceinline__ float load(const storage& v) { return v; }
    static __device__ __forceinline__ storage store(float f) { return f; }
};
struct BF16Elem {
    typedef uint16_t storage;
    static __device__ __forceinline__ float load(const storage& v) { return bf16_bits_to_f32(v); }
    static __device__ __forceinline__ storage store(float f) { return f32_to_bf16_bits(f); }
};
struct F16Elem {
    typedef uint16_t storage;
    static __device__ __forceinline__ float load(const storage& v) { return f16_bits_to_f32(v); }
    static __device__ __forceinline__ storage store(float f) { return f32_to_f16_bits(f); }
};

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// Kernel launches report through the return value of hipLaunchKernel, not through the runtime's sticky
// "last error": that one may hold an error of unrelated earlier work of the caller, and reading it clears it.
// launch() notes a failed launch for the calling thread, launch_status() returns the first one noted since it
// was last asked (0 = every launch was queued).
inline int& launch_rc() {
    static thread_local int rc = 0;
    return rc;
}
template <typename... KArgs, size_t... Is>
inline hipError_t launch_tuple(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds, hipStream_t s,
                               std::tuple<KArgs...>& vals, std::index_sequence<Is...>) {
    void* ptrs[] = {static_cast<void*>(&std::get<Is>(vals))...};
    return hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs, lds, s);
}
template <typename... KArgs, typename... Args>
inline void launch(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds, hipStream_t s, Args&&... args) {
    static_assert(sizeof...(KArgs) == sizeof...(Args), "argument count does not match the kernel's");
    std::tuple<KArgs...> vals(static_cast<KArgs>(std::forward<Args>(args))...);
    const hipError_t e = launch_tuple(kernel, grid, block, lds, s, vals, std::index_sequence_for<KArgs...>{});
    if (e != hipSuccess && launch_rc() == 0) launch_rc() = static_cast<int>(e);
}
inline int launch_status() {
    const int rc = launch_rc();
    launch_rc() = 0;
    return rc;
}

// ---- stage launchers (defined in the .hip files, called from capi.hip) ------
int launch_router(const void* logits, int logits_dtype, int64_t T, int E, int k, int renorm,
                  float* w, int32_t* ids, hipStream_t s);
bool gate_router_supported(int H, int E);
int launch_gate_router(const void* x, const void* gate_w, int64_t T, int H, int E, int k, int renorm,
                       int round_bf16, void* logits_out, float* w, int32_t* ids, hipStream_t s);
// RMSNorm (behind a residual add when res_in != nullptr) + gate + router in one launch; bf16 rows,
// norm weight bf16 or fp32; h_out receives the normalised rows, res_out the new residual
int launch_norm_gate_router(const void* x_in, const void* res_in, const void* norm_w, int norm_w_dtype, float eps,
                            bool layer_semantics, void* h_out, void* res_out, const void* gate_w, int64_t T, int H,
                            int E, int k, int renorm, int round_bf16, void* logits_out, float* w, int32_t* ids,
                            hipStream_t s);
int launch_align(const void* ids, int itype, int64_t numel, int E, int block,
                 int32_t* sorted, int64_t sorted_len, int32_t* expert_ids, int64_t eid_len,
                 int32_t* post_pad, int32_t* seg_out /* [E+1] padded segment starts, may be null */,
                 int32_t* counters /* the kLayerCounters counters of a layer call to clear, may be null */,
                 hipStream_t s);
// The same sort on several workgroups (two launches); needs align_scratch_ints(numel, E) int32 of scratch.
int64_t align_scratch_ints(int64_t numel, int E);
int launch_align_multi(const int32_t* ids, int64_t numel, int E, int block, int32_t* sorted, int64_t sorted_len,
                       int32_t* expert_ids, int64_t eid_len, int32_t* post_pad, int32_t* seg_out, int32_t* counters,
                       int32_t* scratch, hipStream_t s);
// Router + sort in one launch (eight experts, k * T slots within the kernel's LDS table).
bool route_align_supported(int64_t T, int E, int k);
int launch_route_align(const void* logits, int logits_dtype, int64_t T, int k, int renorm, float* w, int32_t* ids,
                       int block, int32_t* sorted, int64_t sorted_len, int32_t* expert_ids, int64_t eid_len,
                       int32_t* post_pad, int32_t* seg_out, int32_t* counters, hipStream_t s);
int launch_silu_and_mul(void* out, const void* in, int64_t rows, int64_t d, int dtype, hipStream_t s);
int launch_moe_sum(const void* in, void* out, int64_t T, int topk, int64_t H, int dtype, hipStream_t s);
bool rms_norm_supported(int H, int dtype, int weight_dtype);
// res_in == nullptr: plain RMSNorm; x_out / res_out may alias their inputs
int launch_rms_norm(const void* x_in, const void* res_in, const void* weight, void* x_out, void* res_out,
                    int64_t T, int H, float eps, int dtype, int weight_dtype, bool layer_semantics, hipStream_t s);

// Problem description shared by the expert GEMM stages.
struct MoeProblem {
    const uint16_t* x;        // [T, H] bf16
    const uint16_t* w13;      // [E, 2I, H] bf16
    const uint16_t* w2;       // [E, H, I] bf16 (fp16 when w2_f16)
    uint16_t* act;            // [sorted_len, I] bf16 (fp16 when act_f16), rows in sorted (padded) order
    uint16_t* act_lo;         // same shape: bf16(value - act) in the two-term form of the generic kernels, else null
    int act_f16;              // act holds fp16 values (default form of the tuned kernels; act_lo is null then)
    int w2_f16;               // w2 holds fp16 values already: the fp16 w2 kernels skip their conversion
    int y_accumulate;         // generic w2 GEMM adds to y instead of overwriting it (second pass over act_lo)
    float* y;                 // [ksplit, T*top_k, H] f32, rows by flat slot
    int y_f16;                // y holds fp16 values instead (256-row kernel); a value beyond the fp16 range is the
                              // fp16 infinity there and stands as float32 in y_wide at the same index
    float* y_wide;            // [ksplit, T*top_k, H] f32, written only where y holds an escaped value
    int32_t* saturated;       // counter of activations clamped to the fp16 range (act_f16), cleared by the sort
    const int32_t* sorted_ids;
    const int32_t* expert_ids;
    const int32_t* post_pad;
    const float* topk_w;      // [T*top_k]
    int64_t T;
    int H, I, E, top_k;
    int block;                // rows per sorted block
    int64_t sorted_len;       // worst-case padded length
    int ksplit;
};
// SiLU*mul result -> act (and the rounding residual -> act_lo in the two-term form)
__device__ __forceinline__ void store_act(const MoeProblem& p, int64_t idx, float v) {
    if (p.act_f16) {
        p.act[idx] = f32_to_f16_bits_sat(v);
        if (fabsf(v) > 65504.0f) atomicAdd(p.saturated, 1);  // rare; a NaN is not a clamped value
        return;
    }
    const uint16_t hi = f32_to_bf16_bits(v);
    p.act[idx] = hi;
    if (p.act_lo != nullptr) p.act_lo[idx] = f32_to_bf16_bits(v - bf16_bits_to_f32(hi));
}

int launch_gemm_generic(const MoeProblem& p, int mode, hipStream_t s);  // mode 1: w13+SiLU*mul, 2: w2
bool stream_supported(const MoeProblem& p);
int launch_gemm_stream(const MoeProblem& p, const int32_t* seg_begin, int mode, hipStream_t s);
bool tile_shape_ok(int H, int I);
int tile_row_block();
bool tile_supported(const MoeProblem& p);
int launch_gemm_tile(const MoeProblem& p, const int32_t* seg_begin, int mode, int* tickets /* 8 ints or null */,
                     bool clear_tickets /* they were not cleared by the sort in front */, hipStream_t s);                                                               // 256-row tiles
bool tile_mid_supported(const MoeProblem& p);                                                      // 128- / 64-row tiles
int launch_gemm_tile_mid(const MoeProblem& p, const int32_t* seg_begin, int mode, int rows_per_tile /* 128 | w2: 64 */,
                         hipStream_t s);
int launch_combine(const MoeProblem& p, void* out, int out_f32, hipStream_t s);

}  // namespace em
