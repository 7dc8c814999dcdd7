// extern "C" surface of libelectrock_moe.so: argument checks, workspace layout
// and stage sequencing.  No kernel code lives here.
#include <atomic>

#include "common.h"
#include "../../include/electrock_moe_diag.h"

using namespace em;

namespace {

constexpr int kVersion = 300;

inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }
inline bool dtype_ok(int d) { return d == EM_DTYPE_F32 || d == EM_DTYPE_BF16 || d == EM_DTYPE_F16; }
inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// Up to this many tokens the weight-streaming GEMM runs (16-row sorted blocks, a
// couple of MFMA fragments per expert); above it the tiled kernels take over.
constexpr int64_t kStreamMaxT = 64;
// Above this many tokens the w2 GEMM of a streaming-size batch runs on the 64-row tiled kernel (same sorted
// layout): it holds its speed when experts get a second MFMA fragment of rows, where the streaming kernel loses
// 10 % (8x7B; T=16: 138 against 146 us, T=12: 121 against 126, T=8: equal, T=5: 98 against 90) and is 20 % ahead
// throughout on the 8x22B shape.
constexpr int64_t kStreamW2MaxT = 8;
// Tile height of the tiled kernels above the streaming range (8 experts, top-2: T/4 rows per expert on average).
// Every tile streams the weight rows of its columns once, whatever its height, so a launch takes as many rounds of
// the CUs as its tiles make.  The 256-row kernel hands its tiles out through a queue and has one row tile per expert
// up to about 1000 tokens: E x (column tiles) x (K slices) tiles.
//   * Where these fill their last round (w2 of 8x7B: 256 tiles on 256 CUs; w13 of 8x22B: 1024) it is the kernel from
//     65 tokens on: as fast as the 128-row tiles with even routing (8x7B w2, T=128 / 224 / 320 / 448: 147 / 145 / 150 /
//     158 us against 146 / 145 / 154 / 170; 8x22B w13, T=128: 480 against 478 us) and far ahead with uneven routing,
//     where experts outgrow a 128-row tile long before the average does (router logits with a Zipf bias per expert,
//     8x7B w2 T=160 / 224 / 448: 164 / 170 / 230 us against 243 / 264 / 259; 8x22B w13 T=128: 490 against 525).
//   * Where they leave a round part empty (w13 of 8x7B: 896 tiles, three and a half rounds; w2 of 8x22B: 384) the
//     128-row kernel stays: it cuts the rest of a round into narrower tiles, a round of half the length (8x7B w13
//     T=128 / 256: 291 / 293 us against 308 / 309), up to the batch sizes where most experts still fit one of its
//     tiles: 352 tokens for the w13 GEMM (with even routing it would stay ahead up to 470 tokens, 318 against 334 us
//     at 448; with the Zipf bias the 256-row tiles win from 200 tokens, 313 against 359 us at 224: the earlier switch
//     is kept), 448 for the w2 GEMM (8x22B T=352: 270 against 299 us).
// 64-row tiles are as fast as 128-row tiles with even routing from 65 to 192 tokens and a fifth slower with the Zipf
// bias (8x7B layer, T=128: 0.451 / 0.451 ms even, 0.597 / 0.491 ms uneven): the large-batch path does not use them.
constexpr int kCus = 256;  // of the GPU this library is tuned for
constexpr int64_t kTile128MaxT = 352, kTile128W2MaxT = 448;
inline bool tiles_fill_rounds(int64_t tiles) {
    const int64_t rounds = ceil_div(tiles, static_cast<int64_t>(kCus));
    return tiles > 0 && tiles * 10 >= rounds * kCus * 9;
}
// mode 1: w13 GEMM, 2: w2 GEMM; batches up to the returned size run on 128-row tiles
inline int64_t tile128_max_tokens(int mode, int H, int I, int E, int ksplit) {
    const int64_t tiles = static_cast<int64_t>(E) * (mode == 1 ? I / 128 : static_cast<int64_t>(H / 256) * ksplit);
    if (tiles_fill_rounds(tiles)) return kStreamMaxT;
    return mode == 1 ? kTile128MaxT : kTile128W2MaxT;
}
// Above this many tokens the w2 partial sums are stored as fp16 with a float32 escape (the 256-row w2 kernel's form)
constexpr int64_t kF32PartialsMaxT = 448;
// Up to this many tokens router and sort share one launch (a single workgroup, whose time grows with the batch);
// above, the two kernels (the router on many workgroups) are faster than the launch they save (8x7B layer, fused
// against separate: T=256 473.4 / 473.9 us, T=512 552.9 / 550.0, T=1024 929 / 920, T=2048 1428 / 1408).
constexpr int64_t kFusedFrontMaxT = 256;
// From this many routed slots (T * top_k) the sort of a layer call runs on several workgroups (two launches whose
// histogram lives in the workspace); below, the one-workgroup kernel is as fast and one launch (timed alone, one
// workgroup / several: 4096 slots 7.7 / 10.3 us, 16384 slots 18.5 / 10.7 us, 65536 slots 62 / 12 us).
constexpr int64_t kMultiSortMinSlots = 8192;

// Rows per sorted block, the counterpart of _get_moe_config (fused_moe.py:327-339):
// 16 (one MFMA fragment) for the streaming kernel, 32 for the tiled kernel, which cuts
// experts into tiles of up to 256 rows itself, 64 for the generic kernel.
inline int choose_block(int64_t T, int H, int I) {
    if (T <= kStreamMaxT) return 16;
    return tile_shape_ok(H, I) ? tile_row_block() : 64;
}
// Split of the w2 reduction (K = I) across workgroups: (row tiles) x (H / 256 column tiles)
// alone leaves CUs idle for small batches and ends in a ragged last round for large ones.
inline int choose_ksplit(int64_t T, int H, int I) {
    if (T > kStreamMaxT) {
        const int want = 2;  // two K slices measure fastest from 128 to 8192 tokens
        if (!tile_shape_ok(H, I)) return want;
        for (int ks = want; ks >= 1; --ks)  // the tiled kernel needs I / ksplit to be a multiple of 64
            if (I % (ks * 64) == 0) return ks;
        return 1;
    }
    // Streaming kernel: (active experts) x (H / 64) row tiles should give every CU
    // work; up to 8 tokens the reduction is split four ways.  Above that the 64-row tiled
    // kernel takes the w2 GEMM with two K slices where the shape allows it, else the streaming
    // kernel with one.  The streaming kernel needs I / ksplit to be a multiple of 256, which
    // covers the tiled kernel's 64.
    const int want = T <= kStreamW2MaxT ? 4 : (tile_shape_ok(H, I) ? 2 : 1);
    for (int ks = want; ks >= 1; --ks)
        if (I % (ks * 256) == 0) return ks;
    return want;
}

bool shapes_ok(int64_t T, int H, int I, int E, int top_k) {
    return T >= 0 && H > 0 && I > 0 && E >= 1 && E <= kMaxExperts && top_k >= 1 && top_k <= kMaxTopK &&
           top_k <= E && H % 8 == 0 && I % 8 == 0 && T * top_k < (int64_t(1) << 30);
}

constexpr unsigned kKnownFlags = EM_FLAG_OUT_F32 | EM_FLAG_GATE_F32_LOGITS | EM_FLAG_W2_F16 | EM_FLAG_BF16_ACT |
                                 EM_FLAG_F32_PARTIALS | EM_FLAG_SKIP_ROUTER | EM_FLAG_SKIP_ALIGN | EM_FLAG_SKIP_GEMM1 |
                                 EM_FLAG_SKIP_GEMM2 | EM_FLAG_SKIP_COMBINE | EM_FLAG_FORCE_GENERIC | EM_FLAG_NO_PERSIST |
                                 EM_FLAG_ONE_GROUP_SORT;

// What a layer call of these shapes and flags runs: which kernels, which storage types between them.  The
// workspace layout and the stage sequencing both follow from it.
struct Plan {
    int block;
    int ksplit;
    int64_t sorted_len;
    bool use_stream, use_tile;  // neither: the shape-generic kernels
    bool w2_on_mid;             // streaming-size batch whose w2 GEMM runs on the 64-row tiled kernel
    bool act_f16;               // SiLU*mul activations stored as fp16 (tuned kernels, default)
    bool act_pair;              // ... as a bf16 pair (value, rounding residual): generic kernels, default
    bool y_f16;                 // w2 partial sums stored as fp16 with a float32 escape (256-row kernel)
};

Plan make_plan(int64_t T, int H, int I, int E, int top_k, unsigned flags) {
    Plan pl{};
    pl.block = choose_block(T, H, I);
    pl.ksplit = choose_ksplit(T, H, I);
    pl.sorted_len = round_up(T * top_k + static_cast<int64_t>(E) * (pl.block - 1), pl.block);
    MoeProblem q{};  // the fields the kernels' own shape checks read
    q.T = T;
    q.H = H;
    q.I = I;
    q.E = E;
    q.top_k = top_k;
    q.block = pl.block;
    q.ksplit = pl.ksplit;
    q.sorted_len = pl.sorted_len;
    const bool tuned = !(flags & EM_FLAG_FORCE_GENERIC);
    pl.use_stream = tuned && T <= kStreamMaxT && stream_supported(q);
    pl.use_tile = tuned && T > kStreamMaxT && tile_supported(q);
    pl.w2_on_mid = pl.use_stream && T > kStreamW2MaxT && pl.ksplit >= 2 && tile_mid_supported(q);
    const bool bf16_act = (flags & EM_FLAG_BF16_ACT) != 0;
    pl.act_f16 = !bf16_act && (pl.use_stream || pl.use_tile);
    pl.act_pair = !bf16_act && !pl.act_f16;
    static_assert(kF32PartialsMaxT >= kTile128W2MaxT, "fp16 partial sums are the 256-row w2 kernel's");  // (at most)
    pl.y_f16 = !(flags & EM_FLAG_F32_PARTIALS) && pl.use_tile && T > kF32PartialsMaxT;
    return pl;
}

int layout_from_plan(const Plan& pl, int64_t T, int H, int I, int E, int top_k, em_moe_layout* L) {
    const int64_t slots = T * top_k;
    int64_t off = 0;
    auto take = [&off](int64_t bytes) {
        const int64_t at = off;
        off += round_up(bytes > 0 ? bytes : 1, 256);
        return at;
    };
    L->block_size = pl.block;
    L->topk_weights_off = take(slots * 4);
    L->topk_ids_off = take(slots * 4);
    L->sorted_ids_off = take(pl.sorted_len * 4);
    L->sorted_len = pl.sorted_len;
    L->expert_ids_len = pl.sorted_len / pl.block;
    L->expert_ids_off = take(L->expert_ids_len * 4);
    L->post_pad_off = take(4);
    L->seg_begin_off = take((E + 1) * 4);
    // the call's counters, cleared by the sort: tile tickets of the persistent w13 and w2 launches (one per XCD
    // each), then the count of clamped activations
    L->tickets_off = take(32 * 4);
    L->saturated_off = L->tickets_off + kSaturatedCounter * 4;
    L->sort_scratch_off = take(align_scratch_ints(slots, E) * 4);
    L->act_off = take(pl.sorted_len * static_cast<int64_t>(I) * 2);
    // the rounding residuals exist only where the shape-generic kernels run in the default (two-term) form
    L->act_lo_off = pl.act_pair ? take(pl.sorted_len * static_cast<int64_t>(I) * 2) : -1;
    L->ksplit = pl.ksplit;
    L->y_off = take(pl.ksplit * slots * static_cast<int64_t>(H) * (pl.y_f16 ? 2 : 4));
    L->y_wide_off = pl.y_f16 ? take(pl.ksplit * slots * static_cast<int64_t>(H) * 4) : -1;
    L->total_bytes = off;
    return 0;
}

}  // namespace

extern "C" {

int em_version(void) { return kVersion; }

const char* em_error_string(int code) {
    switch (code) {
        case 0: return "success";
        case EM_ERR_NULL_POINTER: return "null pointer argument";
        case EM_ERR_BAD_SHAPE: return "invalid shape argument";
        case EM_ERR_BAD_DTYPE: return "unsupported element type";
        case EM_ERR_UNSUPPORTED: return "configuration not supported by this build";
        case EM_ERR_WORKSPACE: return "workspace too small";
        case EM_ERR_BUFFER_SIZE: return "output buffer too small";
        case EM_ERR_ALIGNMENT: return "pointer not sufficiently aligned";
        case EM_ERR_STATIC_LIMIT:
            return "shapes need more scratch memory than the fixed buffer of em_moe_forward_static (EM_STATIC_SCRATCH_BYTES)";
        default: return code > 0 ? hipGetErrorString(static_cast<hipError_t>(code)) : "unknown error";
    }
}

int em_topk_softmax(const void* logits, int logits_dtype, int64_t T, int E, int k, int renormalize,
                    float* topk_weights, int32_t* topk_ids, void* stream) {
    if (T < 0 || E < 1 || E > kMaxExperts || k < 1 || k > E) return EM_ERR_BAD_SHAPE;
    if (!dtype_ok(logits_dtype)) return EM_ERR_BAD_DTYPE;
    if (T == 0) return 0;
    if (!logits || !topk_weights || !topk_ids) return EM_ERR_NULL_POINTER;
    return launch_router(logits, logits_dtype, T, E, k, renormalize, topk_weights, topk_ids, as_stream(stream));
}

int em_moe_align_block_size(const void* topk_ids, int ids_itype, int64_t numel, int num_experts,
                            int block_size, int32_t* sorted_token_ids, int64_t sorted_len,
                            int32_t* expert_ids, int64_t expert_ids_len, int32_t* num_tokens_post_pad,
                            void* stream) {
    if (numel < 0 || num_experts < 1 || num_experts > kMaxExperts || block_size < 1 ||
        numel >= (int64_t(1) << 30))
        return EM_ERR_BAD_SHAPE;
    if (ids_itype != EM_ITYPE_I32 && ids_itype != EM_ITYPE_I64) return EM_ERR_BAD_DTYPE;
    if (!sorted_token_ids || !expert_ids || !num_tokens_post_pad || (numel > 0 && !topk_ids))
        return EM_ERR_NULL_POINTER;
    if (sorted_len < 0 || expert_ids_len < 0) return EM_ERR_BUFFER_SIZE;
    return launch_align(topk_ids, ids_itype, numel, num_experts, block_size, sorted_token_ids, sorted_len,
                        expert_ids, expert_ids_len, num_tokens_post_pad, nullptr, nullptr, as_stream(stream));
}

int em_silu_and_mul(void* out, const void* in, int64_t rows, int64_t d, int dtype, void* stream) {
    if (rows < 0 || d < 0 || rows >= (int64_t(1) << 31)) return EM_ERR_BAD_SHAPE;
    if (!dtype_ok(dtype)) return EM_ERR_BAD_DTYPE;
    if (rows == 0 || d == 0) return 0;
    if (!out || !in) return EM_ERR_NULL_POINTER;
    return launch_silu_and_mul(out, in, rows, d, dtype, as_stream(stream));
}

int em_moe_sum(const void* in, void* out, int64_t T, int topk, int64_t H, int dtype, void* stream) {
    if (T < 0 || H < 0 || topk < 1 || T >= (int64_t(1) << 31)) return EM_ERR_BAD_SHAPE;
    if (!dtype_ok(dtype)) return EM_ERR_BAD_DTYPE;
    if (T == 0 || H == 0) return 0;
    if (!out || !in) return EM_ERR_NULL_POINTER;
    return launch_moe_sum(in, out, T, topk, H, dtype, as_stream(stream));
}

int em_rms_norm(const void* x_in, void* x_out, const void* weight, int64_t T, int H, double eps, int dtype,
                int weight_dtype, int semantics, void* stream) {
    if (T < 0 || H <= 0 || T >= (int64_t(1) << 31)) return EM_ERR_BAD_SHAPE;
    if (!dtype_ok(dtype) || !dtype_ok(weight_dtype)) return EM_ERR_BAD_DTYPE;
    if (semantics != EM_NORM_LAYER && semantics != EM_NORM_OP) return EM_ERR_BAD_SHAPE;
    if (!rms_norm_supported(H, dtype, weight_dtype)) return EM_ERR_UNSUPPORTED;
    if (T == 0) return 0;
    if (!x_in || !x_out || !weight) return EM_ERR_NULL_POINTER;
    return launch_rms_norm(x_in, nullptr, weight, x_out, nullptr, T, H, static_cast<float>(eps), dtype, weight_dtype,
                           semantics == EM_NORM_LAYER, as_stream(stream));
}

int em_add_rms_norm(const void* x_in, const void* residual_in, void* x_out, void* residual_out, const void* weight,
                    int64_t T, int H, double eps, int dtype, int weight_dtype, int semantics, void* stream) {
    if (T < 0 || H <= 0 || T >= (int64_t(1) << 31)) return EM_ERR_BAD_SHAPE;
    if (!dtype_ok(dtype) || !dtype_ok(weight_dtype)) return EM_ERR_BAD_DTYPE;
    if (semantics != EM_NORM_LAYER && semantics != EM_NORM_OP) return EM_ERR_BAD_SHAPE;
    if (!rms_norm_supported(H, dtype, weight_dtype)) return EM_ERR_UNSUPPORTED;
    if (T == 0) return 0;
    if (!x_in || !residual_in || !x_out || !residual_out || !weight) return EM_ERR_NULL_POINTER;
    return launch_rms_norm(x_in, residual_in, weight, x_out, residual_out, T, H, static_cast<float>(eps), dtype,
                           weight_dtype, semantics == EM_NORM_LAYER, as_stream(stream));
}

int em_moe_workspace_layout(int64_t T, int H, int I, int E, int top_k, unsigned flags, em_moe_layout* L) {
    if (!L) return EM_ERR_NULL_POINTER;
    if (!shapes_ok(T, H, I, E, top_k)) return EM_ERR_BAD_SHAPE;
    if (flags & ~kKnownFlags) return EM_ERR_UNSUPPORTED;
    return layout_from_plan(make_plan(T, H, I, E, top_k, flags), T, H, I, E, top_k, L);
}

int64_t em_moe_w2_f16_max_tokens(int H, int I, int E, int top_k) {
    if (!shapes_ok(1, H, I, E, top_k)) return 0;
    // every batch size must land on kernels with an fp16 w2 GEMM: the streaming kernel up to kStreamMaxT tokens
    // (with the 64-row tiled kernel for its w2 GEMM), the tiled kernels above
    for (int64_t T : {int64_t{1}, kStreamW2MaxT + 1, kStreamMaxT, kStreamMaxT + 1})
        if (!make_plan(T, H, I, E, top_k, 0).act_f16) return 0;
    // the tiled kernels address token rows with 32-bit byte offsets; the slot count is bounded as in shapes_ok
    const int64_t by_offsets = ((int64_t{1} << 32) - 1) / (static_cast<int64_t>(H) * 2);
    const int64_t by_slots = ((int64_t{1} << 30) - 1) / top_k;
    const int64_t t = by_offsets < by_slots ? by_offsets : by_slots;
    return (t > kStreamMaxT && make_plan(t, H, I, E, top_k, 0).act_f16) ? t : kStreamMaxT;
}

size_t em_moe_workspace_bytes(int64_t T, int H, int I, int E, int top_k, unsigned flags) {
    em_moe_layout L;
    if (em_moe_workspace_layout(T, H, I, E, top_k, flags, &L) != 0) return 0;
    return static_cast<size_t>(L.total_bytes);
}

}  // extern "C"

namespace {

// Scratch memory of em_moe_forward_static: one array per GPU, held from the moment the library is loaded on a
// device until the process ends.  In host code the name is only a handle for hipGetSymbolAddress; the device
// address is looked up once per device and passed to the kernels like any caller-provided workspace.
constexpr size_t kStaticScratchBytes = EM_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[kStaticScratchBytes];

int static_scratch(void** out) {
    static std::atomic<void*> ptrs[64];
    int dev = -1;
    const hipError_t de = hipGetDevice(&dev);
    if (de != hipSuccess) return static_cast<int>(de);
    if (dev < 0 || dev >= 64) return EM_ERR_UNSUPPORTED;
    void* ptr = ptrs[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {  // first call on this device (a race between threads at worst repeats the lookup)
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return static_cast<int>(e);
        if (ptr == nullptr || reinterpret_cast<uintptr_t>(ptr) % 256 != 0) return EM_ERR_ALIGNMENT;
        ptrs[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return 0;
}

// RMSNorm in front of the block: x of the layer is then the buffer the normalised rows are written to
struct NormFront {
    const void* x_in;
    const void* residual_in;  // may be null: plain RMSNorm
    const void* weight;
    int weight_dtype;
    float eps;
    bool layer_semantics;
    void* residual_out;
};

// The layer behind the entry points: the routing comes either from caller-provided logits or from the
// gate matrix (gate_w != nullptr: logits = x . gate_w^T computed in the router's launch), which may have
// the RMSNorm of the rows in front (norm != nullptr: that launch also writes x).
int moe_forward_impl(const void* x, const void* router_logits, int logits_dtype, const void* gate_w, const void* w13,
                     const void* w2, void* out, int64_t T, int H, int I, int E, int top_k, int renormalize,
                     void* workspace, size_t workspace_bytes, unsigned flags, void* stream,
                     const NormFront* norm = nullptr) {
    if (!shapes_ok(T, H, I, E, top_k)) return EM_ERR_BAD_SHAPE;
    if (gate_w == nullptr && !dtype_ok(logits_dtype)) return EM_ERR_BAD_DTYPE;
    if (gate_w != nullptr && !gate_router_supported(H, E)) return EM_ERR_UNSUPPORTED;
    if (T == 0) return 0;
    if (!x || (!router_logits && !gate_w) || !w13 || !w2 || !out || !workspace) return EM_ERR_NULL_POINTER;
    if (gate_w != nullptr && !aligned(gate_w, 16)) return EM_ERR_ALIGNMENT;
    if (!aligned(x, 16) || !aligned(w13, 16) || !aligned(w2, 16) || !aligned(out, 16) ||
        !aligned(workspace, 256))
        return EM_ERR_ALIGNMENT;
    if (flags & ~kKnownFlags) return EM_ERR_UNSUPPORTED;
    const Plan pl = make_plan(T, H, I, E, top_k, flags);
    // fp16 w2: only the tuned kernels have an fp16 w2 GEMM, and it multiplies fp16 activations
    if ((flags & EM_FLAG_W2_F16) && (!pl.act_f16)) return EM_ERR_UNSUPPORTED;
    em_moe_layout L;
    int rc = layout_from_plan(pl, T, H, I, E, top_k, &L);
    if (rc != 0) return rc;
    if (workspace_bytes < static_cast<size_t>(L.total_bytes)) return EM_ERR_WORKSPACE;

    uint8_t* ws = static_cast<uint8_t*>(workspace);
    hipStream_t s = as_stream(stream);
    MoeProblem p;
    p.x = static_cast<const uint16_t*>(x);
    p.w13 = static_cast<const uint16_t*>(w13);
    p.w2 = static_cast<const uint16_t*>(w2);
    p.act = reinterpret_cast<uint16_t*>(ws + L.act_off);
    // The rounding of the SiLU*mul activations stays out of the result unless EM_FLAG_BF16_ACT asks for the
    // reference's bf16 storage.  With the tuned kernels the activations are stored as fp16 (three more mantissa bits
    // than bf16; clamped to the fp16 range) and the w2 kernel turns its bf16 weight fragments into fp16 on their way
    // to the MFMA: no extra traffic and no second pass.  The shape-generic kernels store a bf16 pair (value, residual)
    // and multiply the residual in a second accumulating pass.
    p.act_lo = pl.act_pair ? reinterpret_cast<uint16_t*>(ws + L.act_lo_off) : nullptr;
    p.act_f16 = pl.act_f16 ? 1 : 0;
    p.w2_f16 = (flags & EM_FLAG_W2_F16) ? 1 : 0;
    // The partial results of the w2 GEMM (one per routed slot and K slice, before the routing weight) are float32 up
    // to 448 tokens.  Above, the 256-row kernel stores them as fp16 (their rounding, 2^-12, is far below a bf16
    // output's, 2^-9, and of the size of the fp16 activations'): half the bytes written by the kernel's epilogues,
    // which all fall into the same moments of a launch, and half the bytes read by the combine (T=8192: -1 % of the
    // layer).  A value beyond the fp16 range is stored as the fp16 infinity and, as float32, in y_wide, where the
    // combine finds it: nothing is clamped.  EM_FLAG_F32_PARTIALS keeps float32 at every size.
    p.y_f16 = pl.y_f16 ? 1 : 0;
    p.saturated = reinterpret_cast<int32_t*>(ws + L.saturated_off);
    p.y_accumulate = 0;
    p.y = reinterpret_cast<float*>(ws + L.y_off);
    p.y_wide = pl.y_f16 ? reinterpret_cast<float*>(ws + L.y_wide_off) : nullptr;
    int32_t* sorted = reinterpret_cast<int32_t*>(ws + L.sorted_ids_off);
    int32_t* eids = reinterpret_cast<int32_t*>(ws + L.expert_ids_off);
    int32_t* post_pad = reinterpret_cast<int32_t*>(ws + L.post_pad_off);
    int32_t* seg_begin = reinterpret_cast<int32_t*>(ws + L.seg_begin_off);
    float* topk_w = reinterpret_cast<float*>(ws + L.topk_weights_off);
    int32_t* topk_ids = reinterpret_cast<int32_t*>(ws + L.topk_ids_off);
    p.sorted_ids = sorted;
    p.expert_ids = eids;
    p.post_pad = post_pad;
    p.topk_w = topk_w;
    p.T = T;
    p.H = H;
    p.I = I;
    p.E = E;
    p.top_k = top_k;
    p.block = static_cast<int>(L.block_size);
    p.sorted_len = L.sorted_len;
    p.ksplit = static_cast<int>(L.ksplit);

    int32_t* counters = reinterpret_cast<int32_t*>(ws + L.tickets_off);
    const bool fused_front = !(flags & (EM_FLAG_SKIP_ROUTER | EM_FLAG_SKIP_ALIGN)) && norm == nullptr &&
                             gate_w == nullptr && T <= kFusedFrontMaxT && route_align_supported(T, E, top_k);
    if (fused_front) {
        rc = launch_route_align(router_logits, logits_dtype, T, top_k, renormalize, topk_w, topk_ids, p.block, sorted,
                                L.sorted_len, eids, L.expert_ids_len, post_pad, seg_begin, counters, s);
        if (rc != 0) return rc;
    }
    if (!fused_front && !(flags & EM_FLAG_SKIP_ROUTER)) {
        const int round_logits = (flags & EM_FLAG_GATE_F32_LOGITS) ? 0 : 1;
        if (norm != nullptr)
            rc = launch_norm_gate_router(norm->x_in, norm->residual_in, norm->weight, norm->weight_dtype, norm->eps,
                                         norm->layer_semantics, const_cast<void*>(x), norm->residual_out, gate_w, T, H,
                                         E, top_k, renormalize, round_logits, nullptr, topk_w, topk_ids, s);
        else if (gate_w != nullptr)
            rc = launch_gate_router(x, gate_w, T, H, E, top_k, renormalize, round_logits, nullptr, topk_w, topk_ids, s);
        else
            rc = launch_router(router_logits, logits_dtype, T, E, top_k, renormalize, topk_w, topk_ids, s);
        if (rc != 0) return rc;
    }
    if (!fused_front && !(flags & EM_FLAG_SKIP_ALIGN)) {
        if (T * top_k >= kMultiSortMinSlots && !(flags & EM_FLAG_ONE_GROUP_SORT))
            rc = launch_align_multi(topk_ids, T * top_k, E, p.block, sorted, L.sorted_len, eids, L.expert_ids_len, post_pad,
                                    seg_begin, counters, reinterpret_cast<int32_t*>(ws + L.sort_scratch_off), s);
        else
            rc = launch_align(topk_ids, EM_ITYPE_I32, T * top_k, E, p.block, sorted, L.sorted_len, eids,
                              L.expert_ids_len, post_pad, seg_begin, counters, s);
        if (rc != 0) return rc;
    }
    const bool use_stream = pl.use_stream, use_tile = pl.use_tile;
    auto tile_gemm = [&](const MoeProblem& q, int mode) {
        if (T <= tile128_max_tokens(mode, H, I, E, q.ksplit)) return launch_gemm_tile_mid(q, seg_begin, mode, 128, s);
        int* tickets = (flags & EM_FLAG_NO_PERSIST) ? nullptr : reinterpret_cast<int*>(ws + L.tickets_off) + (mode - 1) * 8;
        // the sort kernel clears both launches' counters; a call that skips it (stage timing) clears them here
        return launch_gemm_tile(q, seg_begin, mode, tickets, (flags & EM_FLAG_SKIP_ALIGN) != 0, s);
    };
    if (!(flags & EM_FLAG_SKIP_GEMM1)) {
        rc = use_stream ? launch_gemm_stream(p, seg_begin, 1, s)
             : use_tile ? tile_gemm(p, 1) : launch_gemm_generic(p, 1, s);
        if (rc != 0) return rc;
    }
    if (!(flags & EM_FLAG_SKIP_GEMM2)) {
        if (pl.w2_on_mid) {
            rc = launch_gemm_tile_mid(p, seg_begin, 2, 64, s);
        } else if (use_stream) {
            rc = launch_gemm_stream(p, seg_begin, 2, s);
        } else {
            rc = use_tile ? tile_gemm(p, 2) : launch_gemm_generic(p, 2, s);
            if (rc == 0 && pl.act_pair) {  // second pass: y += act_lo . w2
                MoeProblem lo = p;
                lo.act = p.act_lo;
                lo.act_lo = nullptr;
                lo.y_accumulate = 1;
                rc = launch_gemm_generic(lo, 2, s);
            }
        }
        if (rc != 0) return rc;
    }
    if (!(flags & EM_FLAG_SKIP_COMBINE)) {
        rc = launch_combine(p, out, (flags & EM_FLAG_OUT_F32) ? 1 : 0, s);
        if (rc != 0) return rc;
    }
    return 0;
}

}  // namespace

extern "C" {

int em_moe_forward(const void* x, const void* router_logits, int logits_dtype, const void* w13,
                   const void* w2, void* out, int64_t T, int H, int I, int E, int top_k, int renormalize,
                   void* workspace, size_t workspace_bytes, unsigned flags, void* stream) {
    return moe_forward_impl(x, router_logits, logits_dtype, nullptr, w13, w2, out, T, H, I, E, top_k, renormalize,
                            workspace, workspace_bytes, flags, stream);
}

int em_moe_forward_static(const void* x, const void* router_logits, int logits_dtype, const void* w13,
                          const void* w2, void* out, int64_t T, int H, int I, int E, int top_k, int renormalize,
                          unsigned flags, void* stream) {
    if (!shapes_ok(T, H, I, E, top_k)) return EM_ERR_BAD_SHAPE;
    if (flags & ~kKnownFlags) return EM_ERR_UNSUPPORTED;
    em_moe_layout L;
    const int rc = layout_from_plan(make_plan(T, H, I, E, top_k, flags), T, H, I, E, top_k, &L);
    if (rc != 0) return rc;
    if (static_cast<size_t>(L.total_bytes) > kStaticScratchBytes) return EM_ERR_STATIC_LIMIT;
    void* ws = nullptr;
    const int src = static_scratch(&ws);
    if (src != 0) return src;
    return moe_forward_impl(x, router_logits, logits_dtype, nullptr, w13, w2, out, T, H, I, E, top_k, renormalize, ws,
                            kStaticScratchBytes, flags, stream);
}

int em_moe_forward_gated(const void* x, const void* gate_w, const void* w13, const void* w2, void* out,
                         int64_t T, int H, int I, int E, int top_k, int renormalize, void* workspace,
                         size_t workspace_bytes, unsigned flags, void* stream) {
    if (!gate_w && T > 0 && shapes_ok(T, H, I, E, top_k)) return EM_ERR_NULL_POINTER;
    return moe_forward_impl(x, nullptr, EM_DTYPE_BF16, gate_w, w13, w2, out, T, H, I, E, top_k, renormalize, workspace,
                            workspace_bytes, flags, stream);
}

int em_moe_forward_normed(const void* x_in, const void* residual_in, const void* norm_weight, int norm_weight_dtype,
                          double eps, int semantics, void* h_buf, void* residual_out, const void* gate_w,
                          const void* w13, const void* w2, void* out, int64_t T, int H, int I, int E, int top_k,
                          int renormalize, void* workspace, size_t workspace_bytes, unsigned flags, void* stream) {
    if (!shapes_ok(T, H, I, E, top_k)) return EM_ERR_BAD_SHAPE;
    if (norm_weight_dtype != EM_DTYPE_BF16 && norm_weight_dtype != EM_DTYPE_F32) return EM_ERR_BAD_DTYPE;
    if (semantics != EM_NORM_LAYER && semantics != EM_NORM_OP) return EM_ERR_BAD_SHAPE;
    if (T == 0) return 0;
    if (!x_in || !norm_weight || !h_buf || !gate_w || (residual_in && !residual_out)) return EM_ERR_NULL_POINTER;
    if (!aligned(x_in, 16) || !aligned(norm_weight, 16) || (residual_in && !aligned(residual_in, 16)) ||
        (residual_out && !aligned(residual_out, 16)))
        return EM_ERR_ALIGNMENT;
    // the rows are read twice: the new residual must not land on either input
    if (residual_in && (residual_out == residual_in || residual_out == x_in || h_buf == residual_in))
        return EM_ERR_UNSUPPORTED;
    const NormFront norm{x_in, residual_in, norm_weight, norm_weight_dtype, static_cast<float>(eps),
                         semantics == EM_NORM_LAYER, residual_out};
    return moe_forward_impl(h_buf, nullptr, EM_DTYPE_BF16, gate_w, w13, w2, out, T, H, I, E, top_k, renormalize, workspace,
                            workspace_bytes, flags, stream, &norm);
}

int em_norm_gate_topk_softmax(const void* x_in, const void* residual_in, const void* norm_weight, int norm_weight_dtype,
                              double eps, int semantics, void* h_out, void* residual_out, const void* gate_w, int64_t T,
                              int H, int E, int k, int renormalize, int round_logits_bf16, void* logits_out,
                              float* topk_weights, int32_t* topk_ids, void* stream) {
    if (T < 0 || H <= 0 || H % 8 != 0 || E < 1 || E > kMaxExperts || k < 1 || k > E) return EM_ERR_BAD_SHAPE;
    if (norm_weight_dtype != EM_DTYPE_BF16 && norm_weight_dtype != EM_DTYPE_F32) return EM_ERR_BAD_DTYPE;
    if (semantics != EM_NORM_LAYER && semantics != EM_NORM_OP) return EM_ERR_BAD_SHAPE;
    if (!gate_router_supported(H, E)) return EM_ERR_UNSUPPORTED;
    if (T == 0) return 0;
    if (!x_in || !norm_weight || !h_out || !gate_w || !topk_weights || !topk_ids || (residual_in && !residual_out))
        return EM_ERR_NULL_POINTER;
    if (!aligned(x_in, 16) || !aligned(h_out, 16) || !aligned(gate_w, 16) || !aligned(norm_weight, 16) ||
        (residual_in && (!aligned(residual_in, 16) || !aligned(residual_out, 16))))
        return EM_ERR_ALIGNMENT;
    if (residual_in && (residual_out == residual_in || residual_out == x_in || h_out == residual_in))
        return EM_ERR_UNSUPPORTED;  // the rows are read twice: the new residual must not land on either input
    return launch_norm_gate_router(x_in, residual_in, norm_weight, norm_weight_dtype, static_cast<float>(eps),
                                   semantics == EM_NORM_LAYER, h_out, residual_out, gate_w, T, H, E, k, renormalize,
                                   round_logits_bf16 ? 1 : 0, logits_out, topk_weights, topk_ids, as_stream(stream));
}

int em_gate_topk_softmax(const void* x, const void* gate_w, int64_t T, int H, int E, int k, int renormalize,
                         int round_logits_bf16, void* logits_out, float* topk_weights, int32_t* topk_ids,
                         void* stream) {
    if (T < 0 || H <= 0 || H % 8 != 0 || E < 1 || E > kMaxExperts || k < 1 || k > E) return EM_ERR_BAD_SHAPE;
    if (!gate_router_supported(H, E)) return EM_ERR_UNSUPPORTED;
    if (T == 0) return 0;
    if (!x || !gate_w || !topk_weights || !topk_ids) return EM_ERR_NULL_POINTER;
    if (!aligned(x, 16) || !aligned(gate_w, 16)) return EM_ERR_ALIGNMENT;
    return launch_gate_router(x, gate_w, T, H, E, k, renormalize, round_logits_bf16 ? 1 : 0, logits_out, topk_weights,
                              topk_ids, as_stream(stream));
}

}  // extern "C"
