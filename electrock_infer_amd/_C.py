"""Counterpart of the reference's pybind module ``electrock_infer._C``
(pytorch_bind.cpp:11-99): same function names, positional order and keyword
names for the four ops on the MoE path, all writing caller-allocated outputs
in place and returning None.  Each call goes straight to the C ABI of
libelectrock_moe.so.
"""
import torch

from . import _lib


def silu_and_mul(out: torch.Tensor, input: torch.Tensor) -> None:
    """out[..., j] = silu(input[..., j]) * input[..., d + j]
    (pytorch_bind.cpp:18-22, src/activation_kernels.hip:99-152)."""
    _lib.require_device(out, input)
    if input.dim() < 2:
        raise RuntimeError("Input must have at least 2 dimensions!")
    d = input.size(-1) // 2
    if input.size(-1) != 2 * d:
        raise RuntimeError("Input last dimension must be 2*d!")
    if out.size(-1) != d:
        raise RuntimeError("Output last dimension must be d!")
    if out.dtype != input.dtype:
        raise RuntimeError("out and input must have the same dtype")
    rows = input.numel() // (2 * d) if d else 0
    if out.numel() != rows * d:
        raise RuntimeError("out has the wrong number of elements")
    code = _lib.load().em_silu_and_mul(out.data_ptr(), input.data_ptr(), rows, d,
                                       _lib.dtype_code(input.dtype), _lib.current_stream(input.device))
    _lib.check(code, "silu_and_mul")


def topk_softmax(topk_weights: torch.Tensor, topk_indices: torch.Tensor,
                 gating_output: torch.Tensor) -> None:
    """Row softmax + top-2, no renormalisation, ties to the lowest expert index
    (pytorch_bind.cpp:24-29, src/topk_softmax_kernels.hip:88-114)."""
    _lib.require_device(topk_weights, topk_indices, gating_output)
    num_experts = gating_output.size(-1)
    num_tokens = gating_output.numel() // num_experts
    topk = topk_weights.size(-1)
    # the reference op is specialised the same way (topk_softmax_kernels.hip:98-99)
    if num_experts != 8:
        raise RuntimeError("This function is compiled for num_experts=8")
    if topk != 2:
        raise RuntimeError("This function assumes top_k=2 for Mixtral")
    if gating_output.dtype != torch.float32:
        raise RuntimeError("expected scalar type Float for gating_output")
    if topk_weights.dtype != torch.float32 or topk_indices.dtype != torch.int32:
        raise RuntimeError("topk_weights must be float32 and topk_indices int32")
    if topk_weights.numel() != num_tokens * topk or topk_indices.numel() != num_tokens * topk:
        raise RuntimeError("topk outputs must hold num_tokens * topk elements")
    code = _lib.load().em_topk_softmax(gating_output.data_ptr(), _lib.DTYPE_F32, num_tokens, num_experts,
                                       topk, 0, topk_weights.data_ptr(), topk_indices.data_ptr(),
                                       _lib.current_stream(gating_output.device))
    _lib.check(code, "topk_softmax")


def moe_sum(input: torch.Tensor, output: torch.Tensor) -> None:
    """output[t] = input[t, 0] + input[t, 1]
    (pytorch_bind.cpp:31-35, src/moe_sum.hip:53-77)."""
    _lib.require_device(input, output)
    hidden = input.size(-1)
    num_tokens = output.numel() // hidden if hidden else 0
    topk = input.size(1)
    if topk != 2:
        raise RuntimeError("This simplified function is for top_k=2")  # moe_sum.hip:61
    if input.dtype != output.dtype:
        raise RuntimeError("input and output must have the same dtype")
    if input.numel() != num_tokens * topk * hidden:
        raise RuntimeError("input must be [num_tokens, topk, hidden_size]")
    code = _lib.load().em_moe_sum(input.data_ptr(), output.data_ptr(), num_tokens, topk, hidden,
                                  _lib.dtype_code(input.dtype), _lib.current_stream(input.device))
    _lib.check(code, "moe_sum")


def moe_align_block_size(topk_ids: torch.Tensor, num_experts: int, block_size: int,
                         sorted_token_ids: torch.Tensor, expert_ids: torch.Tensor,
                         num_tokens_post_pad: torch.Tensor) -> None:
    """Stable expert sort padded to block_size
    (pytorch_bind.cpp:43-51, src/moe_align_block_size.hip:143-233)."""
    _lib.require_device(topk_ids, sorted_token_ids, expert_ids, num_tokens_post_pad)
    if topk_ids.dtype == torch.int32:
        itype = _lib.ITYPE_I32
    elif topk_ids.dtype == torch.int64:
        itype = _lib.ITYPE_I64
    elif topk_ids.dtype in (torch.int8, torch.uint8, torch.int16):
        topk_ids, itype = topk_ids.to(torch.int32), _lib.ITYPE_I32
    else:
        raise RuntimeError("topk_ids must have an integer dtype")
    for name, t in (("sorted_token_ids", sorted_token_ids), ("expert_ids", expert_ids),
                    ("num_tokens_post_pad", num_tokens_post_pad)):
        if t.dtype != torch.int32:
            raise RuntimeError(f"{name} must be int32")
    code = _lib.load().em_moe_align_block_size(
        topk_ids.data_ptr(), itype, topk_ids.numel(), int(num_experts), int(block_size),
        sorted_token_ids.data_ptr(), sorted_token_ids.numel(), expert_ids.data_ptr(), expert_ids.numel(),
        num_tokens_post_pad.data_ptr(), _lib.current_stream(topk_ids.device))
    _lib.check(code, "moe_align_block_size")


def _norm_args(input: torch.Tensor, weight: torch.Tensor):
    hidden = input.size(-1)
    if weight.numel() != hidden:
        raise RuntimeError("weight must be [hidden_size]")
    if weight.dtype not in (input.dtype, torch.float32):
        raise RuntimeError("weight must have the input's dtype or float32")
    return hidden, (input.numel() // hidden if hidden else 0)


def rms_norm(input: torch.Tensor, epsilon: float, weight: torch.Tensor) -> None:
    """In-place RMSNorm with the native op's rounding: input = T((input * weight) * rsqrt(mean(input^2) + eps))
    (pytorch_bind.cpp:53-58, src/add_rms_norm.hip:87-140)."""
    _lib.require_device(input, weight)
    hidden, rows = _norm_args(input, weight)
    code = _lib.load().em_rms_norm(input.data_ptr(), input.data_ptr(), weight.data_ptr(), rows, hidden, float(epsilon),
                                   _lib.dtype_code(input.dtype), _lib.dtype_code(weight.dtype), _lib.NORM_OP,
                                   _lib.current_stream(input.device))
    _lib.check(code, "rms_norm")


def add_rms_norm(input: torch.Tensor, residual: torch.Tensor, epsilon: float, weight: torch.Tensor) -> None:
    """In place: residual = T(input + residual); input = T((residual * weight) * rsqrt(mean(residual^2) + eps))
    (pytorch_bind.cpp:60-66, src/add_rms_norm.hip:24-84)."""
    _lib.require_device(input, residual, weight)
    hidden, rows = _norm_args(input, weight)
    if residual.shape != input.shape or residual.dtype != input.dtype:
        raise RuntimeError("residual must match input")
    code = _lib.load().em_add_rms_norm(input.data_ptr(), residual.data_ptr(), input.data_ptr(), residual.data_ptr(),
                                       weight.data_ptr(), rows, hidden, float(epsilon), _lib.dtype_code(input.dtype),
                                       _lib.dtype_code(weight.dtype), _lib.NORM_OP, _lib.current_stream(input.device))
    _lib.check(code, "add_rms_norm")
