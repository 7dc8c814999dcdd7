"""ctypes binding of libelectrock_moe.so (the C ABI declared in include/electrock_moe.h).

Nothing here computes: each wrapper turns torch tensors into raw device
pointers plus the current HIP stream and raises RuntimeError on a non-zero
status.  There is deliberately no CPU or eager-PyTorch fallback.
"""
import ctypes
import os

from ._build import LIB_PATH

# element / index type codes of the C ABI
DTYPE_F32, DTYPE_BF16, DTYPE_F16 = 0, 1, 2
ITYPE_I32, ITYPE_I64 = 0, 1

NORM_LAYER, NORM_OP = 0, 1   # rounding points of layers/layernorm.py resp. of the native add_rms_norm op

FLAG_OUT_F32 = 1 << 0
FLAG_GATE_F32_LOGITS = 1 << 2
FLAG_W2_F16 = 1 << 3
FLAG_BF16_ACT = 1 << 5        # SiLU*mul activations stored as bf16 between the GEMMs (the reference's storage type)
FLAG_F32_PARTIALS = 1 << 7    # w2 partial sums stored as float32 at every batch size (default: fp16 + escape above 448 tokens)
# diagnostic switches (include/electrock_moe_diag.h): benchmarks and tests only
FLAG_SKIP_ROUTER = 1 << 8
FLAG_SKIP_ALIGN = 1 << 9
FLAG_SKIP_GEMM1 = 1 << 10
FLAG_SKIP_GEMM2 = 1 << 11
FLAG_SKIP_COMBINE = 1 << 12
FLAG_FORCE_GENERIC = 1 << 16
FLAG_NO_PERSIST = 1 << 17      # one workgroup per tile in the 256-row kernels
FLAG_ONE_GROUP_SORT = 1 << 18  # the layer's sort on one workgroup at every batch size

ERR_STATIC_LIMIT = -8
STATIC_SCRATCH_BYTES = 32 << 20   # EM_STATIC_SCRATCH_BYTES

# every symbol include/electrock_moe.h declares
EXPORTED_SYMBOLS = (
    "em_version", "em_error_string", "em_topk_softmax", "em_moe_align_block_size",
    "em_silu_and_mul", "em_moe_sum", "em_moe_workspace_bytes", "em_moe_workspace_layout",
    "em_moe_forward", "em_moe_forward_gated", "em_gate_topk_softmax", "em_rms_norm", "em_add_rms_norm",
    "em_norm_gate_topk_softmax", "em_moe_forward_normed", "em_moe_forward_static", "em_moe_w2_f16_max_tokens",
)


class MoeLayout(ctypes.Structure):
    """Mirror of struct em_moe_layout."""
    _fields_ = [(n, ctypes.c_int64) for n in (
        "block_size", "topk_weights_off", "topk_ids_off", "sorted_ids_off", "sorted_len",
        "expert_ids_off", "expert_ids_len", "post_pad_off", "seg_begin_off", "tickets_off", "saturated_off",
        "sort_scratch_off", "act_off", "act_lo_off", "y_off", "ksplit", "y_wide_off",
        "total_bytes")]


_lib = None


def load() -> ctypes.CDLL:
    """Load the built library; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m electrock_infer_amd._build` "
            "(there is no fallback implementation)")
    lib = ctypes.CDLL(LIB_PATH)
    vp, i32, i64, u32, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_uint, ctypes.c_size_t
    lib.em_version.restype = i32
    lib.em_version.argtypes = []
    lib.em_error_string.restype = ctypes.c_char_p
    lib.em_error_string.argtypes = [i32]
    lib.em_topk_softmax.restype = i32
    lib.em_topk_softmax.argtypes = [vp, i32, i64, i32, i32, i32, vp, vp, vp]
    lib.em_moe_align_block_size.restype = i32
    lib.em_moe_align_block_size.argtypes = [vp, i32, i64, i32, i32, vp, i64, vp, i64, vp, vp]
    lib.em_silu_and_mul.restype = i32
    lib.em_silu_and_mul.argtypes = [vp, vp, i64, i64, i32, vp]
    lib.em_moe_sum.restype = i32
    lib.em_moe_sum.argtypes = [vp, vp, i64, i32, i64, i32, vp]
    lib.em_moe_w2_f16_max_tokens.restype = i64
    lib.em_moe_w2_f16_max_tokens.argtypes = [i32, i32, i32, i32]
    lib.em_moe_workspace_bytes.restype = sz
    lib.em_moe_workspace_bytes.argtypes = [i64, i32, i32, i32, i32, u32]
    lib.em_moe_workspace_layout.restype = i32
    lib.em_moe_workspace_layout.argtypes = [i64, i32, i32, i32, i32, u32, ctypes.POINTER(MoeLayout)]
    lib.em_moe_forward.restype = i32
    lib.em_moe_forward.argtypes = [vp, vp, i32, vp, vp, vp, i64, i32, i32, i32, i32, i32, vp, sz, u32, vp]
    lib.em_moe_forward_static.restype = i32
    lib.em_moe_forward_static.argtypes = [vp, vp, i32, vp, vp, vp, i64, i32, i32, i32, i32, i32, u32, vp]
    lib.em_moe_forward_gated.restype = i32
    lib.em_moe_forward_gated.argtypes = [vp, vp, vp, vp, vp, i64, i32, i32, i32, i32, i32, vp, sz, u32, vp]
    lib.em_gate_topk_softmax.restype = i32
    lib.em_gate_topk_softmax.argtypes = [vp, vp, i64, i32, i32, i32, i32, i32, vp, vp, vp, vp]
    lib.em_rms_norm.restype = i32
    lib.em_rms_norm.argtypes = [vp, vp, vp, i64, i32, ctypes.c_double, i32, i32, i32, vp]
    lib.em_add_rms_norm.restype = i32
    lib.em_add_rms_norm.argtypes = [vp, vp, vp, vp, vp, i64, i32, ctypes.c_double, i32, i32, i32, vp]
    lib.em_norm_gate_topk_softmax.restype = i32
    lib.em_norm_gate_topk_softmax.argtypes = [vp, vp, vp, i32, ctypes.c_double, i32, vp, vp, vp, i64, i32, i32, i32, i32,
                                              i32, vp, vp, vp, vp]
    lib.em_moe_forward_normed.restype = i32
    lib.em_moe_forward_normed.argtypes = [vp, vp, vp, i32, ctypes.c_double, i32, vp, vp, vp, vp, vp, vp, i64, i32, i32,
                                          i32, i32, i32, vp, sz, u32, vp]
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().em_error_string(code).decode()
        raise RuntimeError(f"{what} failed: {msg} (status {code})")


def dtype_code(dtype) -> int:
    import torch
    try:
        return {torch.float32: DTYPE_F32, torch.bfloat16: DTYPE_BF16, torch.float16: DTYPE_F16}[dtype]
    except KeyError:
        raise RuntimeError(f"unsupported element type {dtype}") from None


def current_stream(device) -> int:
    import torch
    return torch.cuda.current_stream(device).cuda_stream


def require_device(*tensors) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("tensor must be on a GPU device (no CPU path exists)")
        if not t.is_contiguous():
            raise RuntimeError("tensor must be contiguous")


def workspace_layout(T: int, H: int, I: int, E: int, top_k: int, flags: int = 0) -> MoeLayout:
    L = MoeLayout()
    check(load().em_moe_workspace_layout(T, H, I, E, top_k, flags, ctypes.byref(L)), "em_moe_workspace_layout")
    return L
