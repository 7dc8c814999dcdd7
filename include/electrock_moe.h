/*
 * electrock_moe.h — C ABI of libelectrock_moe.so (MI355X / gfx950).
 *
 * Drop-in boundary for the Mixtral MoE layer of RouteTrace/electrock-infer.
 * Every entry point takes raw DEVICE pointers, plain sizes and a HIP stream
 * (passed as void* so that this header needs no HIP include), launches
 * asynchronously on that stream, never allocates, frees or retains memory and
 * keeps no state between calls (but per-device notes that a kernel attribute has
 * been set and where em_moe_forward_static's scratch array lives).  The caller guarantees that the device owning the pointers is current.
 *
 * Return value of every function returning int:
 *     0   success (work is queued on `stream`)
 *   < 0   argument error, nothing was launched (EM_ERR_*)
 *   > 0   a hipError_t reported by the runtime after the launch
 *
 * Citations are relative to the reference tree (RouteTrace/electrock-infer).
 */
#ifndef ELECTROCK_MOE_H
#define ELECTROCK_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type codes */
#define EM_DTYPE_F32  0
#define EM_DTYPE_BF16 1
#define EM_DTYPE_F16  2
/* index type codes (topk_ids) */
#define EM_ITYPE_I32  0
#define EM_ITYPE_I64  1

/* argument errors */
#define EM_ERR_NULL_POINTER   (-1)
#define EM_ERR_BAD_SHAPE      (-2)
#define EM_ERR_BAD_DTYPE      (-3)
#define EM_ERR_UNSUPPORTED    (-4)
#define EM_ERR_WORKSPACE      (-5)
#define EM_ERR_BUFFER_SIZE    (-6)
#define EM_ERR_ALIGNMENT      (-7)
#define EM_ERR_STATIC_LIMIT   (-8)

/* em_moe_forward flags (0 = the defaults described at em_moe_forward) */
#define EM_FLAG_OUT_F32        (1u << 0)  /* `out` is float32 [T,H] instead of bf16                        */
#define EM_FLAG_GATE_F32_LOGITS (1u << 2) /* em_moe_forward_gated: route on the fp32 logits,              */
                                          /* not on their bf16 rounding                                   */
#define EM_FLAG_W2_F16         (1u << 3)  /* `w2` holds fp16 values (converted once by the caller)        */
#define EM_FLAG_BF16_ACT       (1u << 5)  /* SiLU*mul activations rounded to bf16 between the two GEMMs,  */
                                          /* as the reference stores them (default: kept finer, see below) */
#define EM_FLAG_F32_PARTIALS   (1u << 7)  /* w2 partial sums stored as float32 at every batch size        */
                                          /* (default: fp16 with a float32 escape above 448 tokens)       */
/* (bits 8 .. 17 are the diagnostic switches of electrock_moe_diag.h: stage masks and kernel choice) */

/* Library version, e.g. 100 = 0.1.0. */
int em_version(void);

/* Human-readable text for a return code of this library (static storage). */
const char* em_error_string(int code);

/*
 * Router: row-wise softmax + top-k (+ optional renormalisation).
 * Replaces  _C.topk_softmax(topk_weights, topk_indices, gating_output)
 *   (pytorch_bind.cpp:24-29, src/topk_softmax_kernels.hip:11-114) and, with
 *   renormalize=1, fused_topk (electrock_infer/layers/moe/fused_moe.py:130-164).
 * Selection compares raw logits; ties go to the LOWEST expert index
 * (strict '>' scan, topk_softmax_kernels.hip:42-55).  topk_ids[:,0] is the arg-max.
 *   logits        [T, E]  logits_dtype in {F32, BF16, F16}, row-major
 *   topk_weights  [T, k]  float32   softmax probability (divided by the sum of
 *                                   the k selected ones when renormalize != 0)
 *   topk_ids      [T, k]  int32
 * Limits: 1 <= k <= E <= 64.
 */
int em_topk_softmax(const void* logits, int logits_dtype, int64_t T, int E, int k,
                    int renormalize, float* topk_weights, int32_t* topk_ids,
                    void* stream);

/*
 * Router gate and router in one launch: logits = x . gate_w^T, then em_topk_softmax.
 * Replaces the gate of the model's MoE block plus the router call behind it:
 *   router_logits = self.gate(hidden_states)        (models/mixtral.py:40-42,59;
 *   ReplicatedLinear = F.linear(x, weight), layers/linear.py:31-54), followed by
 *   fused_topk (layers/moe/fused_moe.py:130-164).
 * The dot products are accumulated in fp32.  With round_logits_bf16 != 0 each logit is then
 * rounded to bf16, as the reference's bf16 linear layer returns it (equal logits exist in
 * that case and go to the lowest expert index); with 0 the fp32 sums are used directly.
 *   x             [T, H]  bf16, 16-byte aligned
 *   gate_w        [E, H]  bf16, 16-byte aligned (nn.Linear weight layout)
 *   logits_out    [T, E]  optional (may be NULL): the logits that were routed on, bf16 when
 *                         round_logits_bf16 != 0, float32 otherwise
 *   topk_weights  [T, k]  float32, topk_ids [T, k] int32, as em_topk_softmax
 * Limits: E in {8, 16}, H % 8 == 0 (the gate matrix is read from global memory: it stays in L2).
 */
int em_gate_topk_softmax(const void* x, const void* gate_w, int64_t T, int H, int E, int k,
                         int renormalize, int round_logits_bf16, void* logits_out,
                         float* topk_weights, int32_t* topk_ids, void* stream);

/*
 * RMSNorm of the rows (behind a residual add when residual_in is not NULL), router gate and top-k softmax in
 * one launch: the two lines in front of the expert GEMMs in the reference's decoder layer
 * (models/mixtral.py:194-197: post_attention_layernorm, then block_sparse_moe -> gate, models/mixtral.py:59).
 *   x_in, residual_in [T, H] bf16; norm_weight [H] bf16 or F32; gate_w [E, H] bf16 (E of 8 or 16);
 *   h_out [T, H] bf16 receives the normalised rows (the input of the experts), residual_out [T, H] bf16 the
 *   sum x_in + residual_in.  h_out may be x_in; residual_out must be a buffer of its own (the rows are read
 *   twice), else EM_ERR_UNSUPPORTED.  semantics: EM_NORM_LAYER / EM_NORM_OP.
 *   logits_out may be NULL; else [T, E] bf16 (round_logits_bf16) or F32.
 */
int em_norm_gate_topk_softmax(const void* x_in, const void* residual_in, const void* norm_weight,
                              int norm_weight_dtype, double eps, int semantics, void* h_out,
                              void* residual_out, const void* gate_w, int64_t T, int H, int E, int k,
                              int renormalize, int round_logits_bf16, void* logits_out,
                              float* topk_weights, int32_t* topk_ids, void* stream);

/*
 * em_moe_forward_gated with that launch in front: (x_in, residual_in) -> out = MoE(norm(x_in + residual_in)),
 * residual_out = x_in + residual_in.  h_buf [T, H] bf16 is scratch for the normalised rows (it may be x_in,
 * and out may be h_buf); everything else as em_moe_forward_gated.
 */
int em_moe_forward_normed(const void* x_in, const void* residual_in, const void* norm_weight,
                          int norm_weight_dtype, double eps, int semantics, void* h_buf, void* residual_out,
                          const void* gate_w, const void* w13, const void* w2, void* out, int64_t T, int H,
                          int I, int E, int top_k, int renormalize, void* workspace, size_t workspace_bytes,
                          unsigned flags, void* stream);

/*
 * Expert sort with padding to the GEMM block size.
 * Replaces  _C.moe_align_block_size(topk_ids, num_experts, block_size,
 *                                   sorted_token_ids, expert_ids, num_tokens_post_pad)
 *   (pytorch_bind.cpp:43-51, src/moe_align_block_size.hip:61-233) together with
 *   the buffer conventions of its wrapper
 *   (electrock_infer/layers/moe/moe_align_block_size.py:32-60):
 *   sorted_token_ids  [sorted_len]  int32, flat slot indices i = t*k + j grouped by
 *                     expert, ascending inside an expert, every expert segment padded
 *                     to a multiple of block_size with -1; everything after
 *                     num_tokens_post_pad is -1 too
 *   expert_ids        [expert_ids_len] int32, expert of each block; unused tail = 0
 *   num_tokens_post_pad [1] int32, sum over experts of ceil(cnt/block)*block
 * The kernel writes EVERY element of the three outputs, so it needs no
 * pre-filled buffers and yields identical bytes on pre-filled ones.
 * sorted_len >= numel + E*(block_size-1) and expert_ids_len >= ceil(that / block_size)
 * always suffice (the wrapper's sizes); shorter buffers are legal when the caller
 * knows the padded total (the reference's own test sizes them exactly,
 * test/example/test_align_block.py:142-147): writes never go past the given lengths.
 * Entries of topk_ids outside [0, E) are ignored.   Limits: 1 <= E <= 64.
 */
int em_moe_align_block_size(const void* topk_ids, int ids_itype, int64_t numel,
                            int num_experts, int block_size,
                            int32_t* sorted_token_ids, int64_t sorted_len,
                            int32_t* expert_ids, int64_t expert_ids_len,
                            int32_t* num_tokens_post_pad, void* stream);

/*
 * out[r, j] = T( T(silu_f32(in[r, j])) * in[r, d + j] ),  r < rows, j < d.
 * Replaces  _C.silu_and_mul(out, input)
 *   (pytorch_bind.cpp:18-22, src/activation_kernels.hip:23-47,99-152).
 *   in [rows, 2d], out [rows, d], same dtype in {F32, BF16, F16}.
 */
int em_silu_and_mul(void* out, const void* in, int64_t rows, int64_t d, int dtype,
                    void* stream);

/*
 * out[t, j] = sum over kk < topk of in[t, kk, j], accumulated in the element
 * type in ascending kk.
 * Replaces  _C.moe_sum(input, output)
 *   (pytorch_bind.cpp:31-35, src/moe_sum.hip:30-77).
 *   in [T, topk, H], out [T, H], same dtype in {F32, BF16, F16}.
 */
int em_moe_sum(const void* in, void* out, int64_t T, int topk, int64_t H, int dtype,
               void* stream);

/* Rounding points of the two RMSNorm definitions the reference holds (T = rounding to the element type):
 *   EM_NORM_LAYER  layers/layernorm.py:17-41, what the model runs:
 *                  s = f32(x) + f32(residual); residual' = T(s); var = mean(s^2);
 *                  y = T( f32(T(s * rsqrt(var + eps))) * f32(weight) )
 *   EM_NORM_OP     src/add_rms_norm.hip:24-84,87-140, the native op:
 *                  r = T(x + residual); residual' = r; var = mean(f32(r)^2);
 *                  y = T( (f32(r) * f32(weight)) * rsqrt(var + eps) )
 */
#define EM_NORM_LAYER 0
#define EM_NORM_OP 1

/*
 * RMSNorm over the last dimension of x [T, H]; x_out may be x_in.
 * Replaces  _C.rms_norm(input, epsilon, weight)  (pytorch_bind.cpp:53-58, src/include/ops.h:31-34)
 * and RMSNorm.rms_forward (layers/layernorm.py:17-27).
 *   dtype in {F32, BF16, F16}; weight [H] of the same dtype or F32; H a multiple of 8 (4 for F32),
 *   at most 16384 (8192 for F32), else EM_ERR_UNSUPPORTED.
 */
int em_rms_norm(const void* x_in, void* x_out, const void* weight, int64_t T, int H, double eps,
                int dtype, int weight_dtype, int semantics, void* stream);

/*
 * Residual add + RMSNorm: x_out = norm(x_in + residual_in) * weight, residual_out = x_in + residual_in;
 * outputs may alias their inputs (the native op works in place).
 * Replaces  _C.add_rms_norm(input, residual, epsilon, weight)
 *   (pytorch_bind.cpp:60-66, src/include/ops.h:36-40) and RMSNorm.add_rms_forward
 *   (layers/layernorm.py:29-41), the step in front of the MoE block (models/mixtral.py:194-197).
 */
int em_add_rms_norm(const void* x_in, const void* residual_in, void* x_out, void* residual_out,
                    const void* weight, int64_t T, int H, double eps, int dtype, int weight_dtype,
                    int semantics, void* stream);

/*
 * Largest batch size T up to which every call of em_moe_forward with these weight shapes accepts
 * EM_FLAG_W2_F16 (0: none).  The fp16 form of w2 exists in the tuned kernels only, so a caller that wants to
 * keep w2 as fp16 (a loader deciding the storage type once, before it knows any batch size) asks here first.
 * No counterpart in the reference, which keeps w2 in params_dtype (mixtral_moe.py:75-79).
 */
int64_t em_moe_w2_f16_max_tokens(int H, int I, int E, int top_k);

/*
 * Bytes of device workspace em_moe_forward needs for these shapes and flags
 * (0 for invalid shapes).  The workspace must be 256-byte aligned.  The size depends on
 * EM_FLAG_BF16_ACT, EM_FLAG_F32_PARTIALS (and the kernel-choice switch of electrock_moe_diag.h) only; pass the flags of the call.
 * A larger buffer than asked for is always valid: a caller that serves many batch sizes can
 * keep one workspace sized for its largest.
 */
size_t em_moe_workspace_bytes(int64_t T, int H, int I, int E, int top_k, unsigned flags);

/*
 * The whole layer:  out[t] = sum_j w[t,j] * W2[e_tj] ( silu(W1[e_tj] x_t) * (W3[e_tj] x_t) ).
 * Replaces  fused_experts(hidden_states, w1, w2, gating_output, topk, renormalize,
 *                         inplace, "silu")
 *   (electrock_infer/layers/moe/fused_moe.py:170-293) as called by FusedMoE.forward
 *   (electrock_infer/layers/moe/mixtral_moe.py:100-109).
 *   x             [T, H]      bf16
 *   router_logits [T, E]      logits_dtype in {F32, BF16, F16}
 *   w13           [E, 2I, H]  bf16, rows [0,I) = gate (w1), rows [I,2I) = up (w3)
 *                             (mixtral_moe.py:64-70,137-143)
 *   w2            [E, H, I]   bf16 (mixtral_moe.py:75-79); fp16 with EM_FLAG_W2_F16
 *   out           [T, H]      bf16 (float32 with EM_FLAG_OUT_F32); may alias x
 *   workspace     >= em_moe_workspace_bytes(T,H,I,E,top_k,flags), 256-byte aligned
 * Arithmetic (flags = 0): bf16 operands, float32 accumulation in both GEMMs, SiLU*mul in
 * float32, routing weight and top-k sum in float32, one rounding of the result to bf16.
 * Between the GEMMs the activations are stored as fp16 (clamped to +-65504) and the w2
 * GEMM runs on the fp16 MFMA with its bf16 weight fragments converted on the way (exactly,
 * for every weight of magnitude 2^-14 .. 65504): mean relative error 2e-4 against the fp32
 * definition, i.e. max-abs 2e-2 / mean relative 1e-3 are met with EM_FLAG_OUT_F32 (a bf16
 * output adds its own rounding, 1.4e-3).  For shapes only the generic kernels take, the
 * activations are kept as a bf16 pair (value, rounding residual) and the residual is
 * multiplied in a second pass over w2, to the same bar.
 * EM_FLAG_BF16_ACT stores the activations as bf16 instead, the reference's storage type
 * (fused_moe.py:223-239: cache2), with its range and its rounding: mean relative error
 * 1.7e-3; no conversions in the w2 GEMM (8192 tokens: -10 % on that kernel, no difference
 * up to 64 tokens).
 * EM_FLAG_W2_F16: the caller keeps w2 as fp16 (converted once, e.g. when the weights
 * are loaded; what the FusedMoE module of this package does for bfloat16 parameters).  Same
 * results as flags = 0 without the conversion (8192 tokens: -2.3 % of the layer) and with the tile
 * queue in the w2 launch, which the converting kernel has no register left for.  Only shapes the
 * tuned kernels take (em_moe_w2_f16_max_tokens) and not together with EM_FLAG_BF16_ACT; others
 * return EM_ERR_UNSUPPORTED.
 * Partial sums of the w2 GEMM (one per routed slot and K slice, before the routing weight): float32 up to 448
 * tokens; above, the 256-row kernel stores them as fp16 (half the bytes in its epilogues and in the top-k sum;
 * one more rounding of relative size 2^-12 per partial sum: mean relative error of a float32 output 2.1e-4 -> 2.9e-4).
 * No value is clamped: a partial sum beyond the fp16 range (and an infinity) is marked by the fp16 infinity and
 * kept as float32 in a second array of the workspace, from where the top-k sum takes it, so the layer follows the
 * definition at any magnitude bf16 holds.  What fp16 cannot keep is relative precision below 2^-14: partial sums
 * smaller than that in magnitude carry an absolute error of up to 2^-25.
 * EM_FLAG_F32_PARTIALS stores float32 partial sums at every batch size (8192 tokens: +1.4 % in time).
 * After the call the workspace holds topk_weights, topk_ids, sorted_token_ids,
 * expert_ids and num_tokens_post_pad (see em_moe_workspace_layout), and `saturated`: the number of
 * SiLU*mul values of routed rows whose magnitude exceeded 65504 and was clamped when they were
 * stored as fp16 (always 0 with EM_FLAG_BF16_ACT and for shapes only the generic kernels take).
 * A caller of the default arithmetic that cannot rule such activations out reads it after the
 * call and repeats the call with EM_FLAG_BF16_ACT when it is not 0.
 * Limits: E <= 64, top_k <= 8, H % 8 == 0, I % 8 == 0.  Unknown flag bits: EM_ERR_UNSUPPORTED.
 */
int em_moe_forward(const void* x, const void* router_logits, int logits_dtype,
                   const void* w13, const void* w2, void* out,
                   int64_t T, int H, int I, int E, int top_k, int renormalize,
                   void* workspace, size_t workspace_bytes, unsigned flags,
                   void* stream);

/*
 * em_moe_forward without a workspace argument, for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the
 * scratch memory is a fixed array inside the library, EM_STATIC_SCRATCH_BYTES per GPU, held
 * from the time the library is loaded until the process ends.  No counterpart in the
 * reference, which allocates its intermediate tensors on every call (fused_moe.py:223-239).
 * Arguments, flags, results and return codes as em_moe_forward; in addition
 *   EM_ERR_STATIC_LIMIT  em_moe_workspace_bytes(T,H,I,E,top_k,flags) exceeds
 *                        EM_STATIC_SCRATCH_BYTES (nothing is launched); the limit admits the
 *                        decode batches of both Mixtral shapes (up to 64 tokens at 8x22B,
 *                        about 190 at 8x7B).
 * The call allocates and frees nothing.  Its first call on a device looks up the array's
 * device address (hipGetSymbolAddress; the runtime may place the array in device memory only
 * at that moment): make that call outside graph capture.
 * All calls on one GPU share the one array, which keeps the last call's contents (the kernels
 * write every element they read, nothing has to start at zero): calls that overlap on one GPU,
 * on different streams or from different threads, race -- order them on one stream.
 * The routing results are not readable through this entry point.
 */
#define EM_STATIC_SCRATCH_BYTES ((size_t)32 << 20)
int em_moe_forward_static(const void* x, const void* router_logits, int logits_dtype,
                          const void* w13, const void* w2, void* out,
                          int64_t T, int H, int I, int E, int top_k, int renormalize,
                          unsigned flags, void* stream);

/*
 * The same layer with the router gate inside: replaces MixtralMoE.forward
 * (models/mixtral.py:53-63: gate -> experts) in one call.  Arguments as em_moe_forward, with
 * gate_w [E, H] bf16 in place of router_logits; EM_FLAG_GATE_F32_LOGITS routes on the fp32
 * logits instead of their bf16 rounding.  Limits of em_gate_topk_softmax apply.
 */
int em_moe_forward_gated(const void* x, const void* gate_w, const void* w13, const void* w2,
                         void* out, int64_t T, int H, int I, int E, int top_k, int renormalize,
                         void* workspace, size_t workspace_bytes, unsigned flags, void* stream);

/*
 * Byte offsets and element counts of the routing results em_moe_forward leaves
 * in its workspace, plus the GEMM row-block size it sorts for (the counterpart
 * of _get_moe_config, fused_moe.py:327-339).  All fields are int64.
 */
typedef struct em_moe_layout {
    int64_t block_size;
    int64_t topk_weights_off, topk_ids_off;        /* [T*top_k] f32 / i32      */
    int64_t sorted_ids_off, sorted_len;            /* [sorted_len] i32         */
    int64_t expert_ids_off, expert_ids_len;        /* [expert_ids_len] i32     */
    int64_t post_pad_off;                          /* [1] i32                  */
    int64_t seg_begin_off;                         /* [E+1] i32 padded segment starts */
    int64_t tickets_off;                           /* [2][8] i32 tile counters of the large-batch GEMM launches */
    int64_t saturated_off;                         /* [1] i32: activations of routed rows that the call clamped to the fp16 range */
    int64_t sort_scratch_off;                      /* i32 histogram rows of the sort on several workgroups */
    int64_t act_off;                               /* [sorted_len, I] fp16 (bf16 with EM_FLAG_BF16_ACT and in the generic kernels) */
    int64_t act_lo_off;                            /* [sorted_len, I] bf16 rounding residuals of the generic kernels; -1: not reserved */
    int64_t y_off, ksplit;                         /* [ksplit, T*top_k, H] f32, or fp16 (large batches without EM_FLAG_F32_PARTIALS) */
    int64_t y_wide_off;                            /* [ksplit, T*top_k, H] f32 holding the partial sums that fp16 marks as escaped; -1: y is f32 */
    int64_t total_bytes;
} em_moe_layout;

int em_moe_workspace_layout(int64_t T, int H, int I, int E, int top_k, unsigned flags,
                            em_moe_layout* layout);

#ifdef __cplusplus
}
#endif
#endif /* ELECTROCK_MOE_H */
