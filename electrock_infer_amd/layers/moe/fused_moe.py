"""Host side of the MoE hot path, mirroring
electrock_infer/layers/moe/fused_moe.py of the reference.

``fused_topk`` and ``fused_experts`` keep the reference's names, argument
meaning and return values; behind them sits one call into the C ABI
(``em_topk_softmax`` / ``em_moe_forward``) instead of torch ops + Triton.
"""
import ctypes
from typing import Dict, List, Optional, Tuple

import torch

from ... import _lib


def _get_moe_config(num_tokens: int, num_experts: int, intermediate_size: int, topk: int) -> dict:
    """Row-block size of the expert sort as the reference picks it
    (fused_moe.py:327-339).  Kept for callers that run the ops one by one; the
    fused entry point chooses its own tiling (see ``workspace_layout``)."""
    if num_tokens <= num_experts:
        return {"BLOCK_SIZE_M": 16, "BLOCK_SIZE_N": 32, "BLOCK_SIZE_K": 64, "GROUP_SIZE_M": 1}
    return {"BLOCK_SIZE_M": 64, "BLOCK_SIZE_N": 64, "BLOCK_SIZE_K": 32, "GROUP_SIZE_M": 8}


def fused_topk(hidden_states: torch.Tensor, gating_output: torch.Tensor, topk: int,
               renormalize: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """Softmax + top-k (+ renormalise) of the router logits
    (fused_moe.py:130-164).  Returns float32 weights and int32 expert ids;
    ties go to the lowest expert index."""
    assert hidden_states.shape[0] == gating_output.shape[0], "Number of tokens mismatch"
    _lib.require_device(gating_output)
    M, E = gating_output.shape
    topk_weights = torch.empty(M, topk, dtype=torch.float32, device=gating_output.device)
    topk_ids = torch.empty(M, topk, dtype=torch.int32, device=gating_output.device)
    code = _lib.load().em_topk_softmax(gating_output.data_ptr(), _lib.dtype_code(gating_output.dtype), M, E,
                                       topk, 1 if renormalize else 0, topk_weights.data_ptr(),
                                       topk_ids.data_ptr(), _lib.current_stream(gating_output.device))
    _lib.check(code, "fused_topk")
    return topk_weights, topk_ids


class MoeWorkspace:
    """Device scratch of one ``em_moe_forward`` call shape: a 256-byte aligned buffer plus the layout of the
    call in it.

    The reference allocates its three intermediate caches and the sort buffers
    on every call (fused_moe.py:223-239, moe_align_block_size.py:32-48); here one
    buffer is kept and reused, and views of the routing results
    the kernels leave in it can be read back for inspection.  ``buffer`` may be any
    uint8 device tensor of at least ``layout.total_bytes`` (several shapes can share one).
    """

    def __init__(self, device, T: int, H: int, I: int, E: int, top_k: int, flags: int = 0,
                 buffer: Optional[torch.Tensor] = None):
        self.shape = (T, H, I, E, top_k)
        self.layout = _lib.workspace_layout(T, H, I, E, top_k, flags & _LAYOUT_FLAGS)
        if buffer is None:
            buffer = torch.empty(self.layout.total_bytes, dtype=torch.uint8, device=device)
        if buffer.numel() < self.layout.total_bytes or buffer.data_ptr() % 256 != 0:
            raise RuntimeError("workspace buffer too small or not 256-byte aligned")
        self.buffer = buffer

    def _view(self, off: int, count: int, dtype: torch.dtype) -> torch.Tensor:
        nbytes = count * torch.empty((), dtype=dtype).element_size()
        return self.buffer[off:off + nbytes].view(dtype)

    @property
    def block_size(self) -> int:
        return self.layout.block_size

    def topk_weights(self) -> torch.Tensor:
        T, _, _, _, k = self.shape
        return self._view(self.layout.topk_weights_off, T * k, torch.float32).view(T, k)

    def topk_ids(self) -> torch.Tensor:
        T, _, _, _, k = self.shape
        return self._view(self.layout.topk_ids_off, T * k, torch.int32).view(T, k)

    def sorted_token_ids(self) -> torch.Tensor:
        return self._view(self.layout.sorted_ids_off, self.layout.sorted_len, torch.int32)

    def expert_ids(self) -> torch.Tensor:
        return self._view(self.layout.expert_ids_off, self.layout.expert_ids_len, torch.int32)

    def num_tokens_post_pad(self) -> torch.Tensor:
        return self._view(self.layout.post_pad_off, 1, torch.int32)

    def saturated(self) -> torch.Tensor:
        """[1] int32: how many SiLU*mul values of routed rows the last call clamped to the fp16 range (+-65504).
        Always 0 with ``bf16_act``; reading it (``int(ws.saturated())``) synchronises with the device."""
        return self._view(self.layout.saturated_off, 1, torch.int32)


# the flags the workspace size depends on
_LAYOUT_FLAGS = _lib.FLAG_BF16_ACT | _lib.FLAG_FORCE_GENERIC | _lib.FLAG_F32_PARTIALS

# One grow-only buffer per device.  A buffer that has been handed out is never freed behind the caller's back:
# a HIP graph captured through the layer calls holds its address, so when a larger batch makes the buffer grow,
# the old one is kept (``_retired``) until ``release_workspaces``.  Growth is geometric, so the retired buffers
# together stay below twice the live one; an engine that knows its largest batch calls ``reserve_workspace`` once.
_buffers: Dict[int, torch.Tensor] = {}
_retired: Dict[int, List[torch.Tensor]] = {}


def _device_index(device) -> int:
    d = torch.device(device)
    return d.index if d.index is not None else torch.cuda.current_device()


def _ensure_buffer(device, nbytes: int) -> torch.Tensor:
    idx = _device_index(device)
    buf = _buffers.get(idx)
    if buf is None or buf.numel() < nbytes:
        if torch.cuda.is_current_stream_capturing():
            # an allocation made now would come from the graph's private pool and then serve eager calls as well
            raise RuntimeError("the shared MoE workspace would have to grow under graph capture: run the layer once "
                               "eagerly at this batch size first, or call reserve_workspace for the largest batch")
        if buf is not None:
            _retired.setdefault(idx, []).append(buf)
            nbytes = max(nbytes, buf.numel() * 3 // 2)
        buf = _buffers[idx] = torch.empty(nbytes, dtype=torch.uint8, device=torch.device("cuda", idx))
        assert buf.data_ptr() % 256 == 0
    return buf


def reserve_workspace(device, T: int, H: int, I: int, E: int, top_k: int, flags: int = 0) -> None:
    """Size the device's shared workspace for calls of up to this shape (an engine: its largest batch), so that
    no later call allocates."""
    _ensure_buffer(device, _lib.workspace_layout(T, H, I, E, top_k, flags & _LAYOUT_FLAGS).total_bytes)


def release_workspaces(device=None) -> None:
    """Drop the shared workspaces (of one device, or of all): only when no captured graph and no pending call
    uses them any more."""
    for idx in ([_device_index(device)] if device is not None else list(_buffers)):
        _buffers.pop(idx, None)
        _retired.pop(idx, None)
        for key in [k for k in _views if k[0] == idx]:
            del _views[key]


_views: Dict[tuple, MoeWorkspace] = {}      # (device, shape, layout flags) -> the view handed out last


def get_workspace(device, T: int, H: int, I: int, E: int, top_k: int, flags: int = 0) -> MoeWorkspace:
    """The layout of a call of this shape in the device's shared workspace.  Calls on one device share that buffer:
    they have to be ordered on one stream (as the layers of a model are); a caller that runs layer calls on several
    streams at once passes each its own ``MoeWorkspace`` through the ``workspace`` argument of the entry points.
    The view of a shape is kept and handed out again while the buffer behind it is still the device's current one
    (a decode step calls this 32 times with one shape)."""
    idx = _device_index(device)
    key = (idx, T, H, I, E, top_k, flags & _LAYOUT_FLAGS)
    ws = _views.get(key)
    if ws is not None and ws.buffer is _buffers.get(idx):
        return ws
    need = _lib.workspace_layout(T, H, I, E, top_k, flags & _LAYOUT_FLAGS).total_bytes
    ws = MoeWorkspace(device, T, H, I, E, top_k, flags, buffer=_ensure_buffer(device, need))
    if len(_views) >= 256:
        _views.clear()
    _views[key] = ws
    return ws


def _w2_flag(w2: torch.Tensor) -> int:
    """w2 may be kept as float16 (converted once from the bfloat16 checkpoint, exactly for every weight of magnitude
    2^-14 .. 65504): the w2 GEMM then needs no conversion of its weight fragments."""
    if w2.dtype == torch.float16:
        return _lib.FLAG_W2_F16
    if w2.dtype != torch.bfloat16:
        raise RuntimeError("the fused MoE path computes in bfloat16: w2 must be bfloat16 (or float16, see _w2_flag)")
    return 0


def fused_experts(hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
                  gating_output: torch.Tensor, topk: int, renormalize: bool = True,
                  inplace: bool = False, activation: str = "silu",
                  out_dtype: Optional[torch.dtype] = None, bf16_act: bool = False, flags: int = 0,
                  workspace: Optional[MoeWorkspace] = None) -> torch.Tensor:
    """The MoE layer body (fused_moe.py:170-293): route, sort, w13 GEMM with
    SiLU*mul, w2 GEMM, weighted top-k combine.

    hidden_states [T, H] bf16; w1 [E, 2I, H] (gate rows then up rows); w2 [E, H, I];
    gating_output [T, E].  With ``inplace`` the result overwrites
    ``hidden_states`` and that tensor is returned, as in the reference.
    ``out_dtype=torch.float32`` returns the un-rounded fp32 result instead
    (not available together with ``inplace``).  Between the two GEMMs the
    SiLU*mul activations are kept as fp16; ``bf16_act=True`` rounds them to
    bf16 as the reference's ``cache2`` does (its range, its rounding error).  A float16
    ``w2`` saves the conversion of the weight fragments inside the w2 kernel.
    """
    if activation != "silu":
        raise NotImplementedError(f"Activation {activation} not supported.")
    _lib.require_device(hidden_states, w1, w2, gating_output)
    T, H = hidden_states.shape
    E, two_i, Hw = w1.shape
    I = two_i // 2
    if Hw != H or tuple(w2.shape) != (E, H, I) or two_i != 2 * I:
        raise RuntimeError("weight shapes do not match hidden_states")
    if gating_output.shape[0] != T or gating_output.shape[1] != E:
        raise RuntimeError("gating_output must be [num_tokens, num_experts]")
    if not (hidden_states.dtype == w1.dtype == torch.bfloat16):
        raise RuntimeError("the fused MoE path computes in bfloat16: hidden_states, w1 and w2 must be bfloat16")
    flags |= _w2_flag(w2)
    want_f32 = out_dtype == torch.float32
    if bf16_act:
        flags |= _lib.FLAG_BF16_ACT
    if want_f32 and inplace:
        raise RuntimeError("a float32 result cannot be written in place over bfloat16 hidden_states")
    if want_f32:
        output = torch.empty((T, H), dtype=torch.float32, device=hidden_states.device)
        flags |= _lib.FLAG_OUT_F32
    else:
        output = hidden_states if inplace else torch.empty_like(hidden_states)
    if T == 0:
        return output
    ws = workspace or get_workspace(hidden_states.device, T, H, I, E, topk, flags)
    code = _lib.load().em_moe_forward(
        hidden_states.data_ptr(), gating_output.data_ptr(), _lib.dtype_code(gating_output.dtype),
        w1.data_ptr(), w2.data_ptr(), output.data_ptr(), T, H, I, E, topk, 1 if renormalize else 0,
        ws.buffer.data_ptr(), ctypes.c_size_t(ws.buffer.numel()), flags,
        _lib.current_stream(hidden_states.device))
    _lib.check(code, "fused_experts")
    return output


def gate_topk(hidden_states: torch.Tensor, gate_weight: torch.Tensor, topk: int, renormalize: bool = True,
              bf16_logits: bool = True, return_logits: bool = False):
    """Router gate and router in one launch: ``fused_topk(hidden_states, F.linear(hidden_states, gate_weight), ...)``
    (models/mixtral.py:59 followed by fused_moe.py:130-164).

    hidden_states [T, H] bf16, gate_weight [E, H] bf16 (``nn.Linear`` layout).  With ``bf16_logits`` the fp32 dot
    products are rounded to bf16 before the selection, as the reference's bf16 linear layer returns them.
    Returns (topk_weights [T, topk] fp32, topk_ids [T, topk] int32[, logits [T, E]]).
    """
    _lib.require_device(hidden_states, gate_weight)
    T, H = hidden_states.shape
    E = gate_weight.shape[0]
    if gate_weight.shape[1] != H:
        raise RuntimeError("gate_weight must be [num_experts, hidden_size]")
    if not (hidden_states.dtype == gate_weight.dtype == torch.bfloat16):
        raise RuntimeError("the router gate computes in bfloat16: hidden_states and gate_weight must be bfloat16")
    dev = hidden_states.device
    topk_weights = torch.empty(T, topk, dtype=torch.float32, device=dev)
    topk_ids = torch.empty(T, topk, dtype=torch.int32, device=dev)
    logits = torch.empty(T, E, dtype=torch.bfloat16 if bf16_logits else torch.float32, device=dev) if return_logits else None
    code = _lib.load().em_gate_topk_softmax(
        hidden_states.data_ptr(), gate_weight.data_ptr(), T, H, E, topk, 1 if renormalize else 0,
        1 if bf16_logits else 0, logits.data_ptr() if logits is not None else None,
        topk_weights.data_ptr(), topk_ids.data_ptr(), _lib.current_stream(dev))
    _lib.check(code, "gate_topk")
    return (topk_weights, topk_ids, logits) if return_logits else (topk_weights, topk_ids)


def fused_experts_gated(hidden_states: torch.Tensor, gate_weight: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
                        topk: int, renormalize: bool = True, inplace: bool = False,
                        out_dtype: Optional[torch.dtype] = None, bf16_act: bool = False, bf16_logits: bool = True,
                        flags: int = 0, workspace: Optional[MoeWorkspace] = None) -> torch.Tensor:
    """``fused_experts(x, w1, w2, F.linear(x, gate_weight), ...)`` in one call: the whole MoE block of the model
    (models/mixtral.py:53-63) with the router gate computed inside the router's launch."""
    _lib.require_device(hidden_states, gate_weight, w1, w2)
    T, H = hidden_states.shape
    E, two_i, Hw = w1.shape
    I = two_i // 2
    if Hw != H or tuple(w2.shape) != (E, H, I) or two_i != 2 * I:
        raise RuntimeError("weight shapes do not match hidden_states")
    if tuple(gate_weight.shape) != (E, H):
        raise RuntimeError("gate_weight must be [num_experts, hidden_size]")
    if not (hidden_states.dtype == gate_weight.dtype == w1.dtype == torch.bfloat16):
        raise RuntimeError("the fused MoE path computes in bfloat16: hidden_states, gate_weight, w1 and w2 must be bfloat16")
    flags |= _w2_flag(w2)
    want_f32 = out_dtype == torch.float32
    if bf16_act:
        flags |= _lib.FLAG_BF16_ACT
    if not bf16_logits:
        flags |= _lib.FLAG_GATE_F32_LOGITS
    if want_f32 and inplace:
        raise RuntimeError("a float32 result cannot be written in place over bfloat16 hidden_states")
    if want_f32:
        output = torch.empty((T, H), dtype=torch.float32, device=hidden_states.device)
        flags |= _lib.FLAG_OUT_F32
    else:
        output = hidden_states if inplace else torch.empty_like(hidden_states)
    if T == 0:
        return output
    ws = workspace or get_workspace(hidden_states.device, T, H, I, E, topk, flags)
    code = _lib.load().em_moe_forward_gated(
        hidden_states.data_ptr(), gate_weight.data_ptr(), w1.data_ptr(), w2.data_ptr(), output.data_ptr(),
        T, H, I, E, topk, 1 if renormalize else 0, ws.buffer.data_ptr(), ctypes.c_size_t(ws.buffer.numel()), flags,
        _lib.current_stream(hidden_states.device))
    _lib.check(code, "fused_experts_gated")
    return output


def _norm_front_args(hidden_states, residual, norm_weight, gate_weight):
    _lib.require_device(hidden_states, norm_weight, gate_weight)
    T, H = hidden_states.shape
    if residual is not None:
        _lib.require_device(residual)
        if residual.shape != hidden_states.shape or residual.dtype != hidden_states.dtype:
            raise RuntimeError("residual must match hidden_states")
    if norm_weight.numel() != H or norm_weight.dtype not in (torch.bfloat16, torch.float32):
        raise RuntimeError("norm_weight must be [hidden_size], bfloat16 or float32")
    if gate_weight.shape[1] != H:
        raise RuntimeError("gate_weight must be [num_experts, hidden_size]")
    if not (hidden_states.dtype == gate_weight.dtype == torch.bfloat16):
        raise RuntimeError("the fused norm + gate computes in bfloat16: hidden_states and gate_weight must be bfloat16")
    return T, H


def norm_gate_topk(hidden_states: torch.Tensor, residual: Optional[torch.Tensor], norm_weight: torch.Tensor,
                   eps: float, gate_weight: torch.Tensor, topk: int, renormalize: bool = True,
                   bf16_logits: bool = True, return_logits: bool = False, op_rounding: bool = False):
    """RMSNorm (behind the residual add when ``residual`` is given), router gate and router in one launch:
    the reference's ``post_attention_layernorm`` followed by the gate and ``fused_topk``
    (models/mixtral.py:194-197,59; layers/layernorm.py:17-41; fused_moe.py:130-164).

    Returns (normed [T, H] bf16, residual_out or None, topk_weights [T, topk] fp32, topk_ids [T, topk] int32
    [, logits [T, E]]).  ``op_rounding`` selects the native add_rms_norm op's rounding points instead of the
    module's.
    """
    T, H = _norm_front_args(hidden_states, residual, norm_weight, gate_weight)
    E = gate_weight.shape[0]
    dev = hidden_states.device
    normed = torch.empty_like(hidden_states)
    res_out = torch.empty_like(hidden_states) if residual is not None else None
    topk_weights = torch.empty(T, topk, dtype=torch.float32, device=dev)
    topk_ids = torch.empty(T, topk, dtype=torch.int32, device=dev)
    logits = torch.empty(T, E, dtype=torch.bfloat16 if bf16_logits else torch.float32, device=dev) if return_logits else None
    code = _lib.load().em_norm_gate_topk_softmax(
        hidden_states.data_ptr(), residual.data_ptr() if residual is not None else None, norm_weight.data_ptr(),
        _lib.dtype_code(norm_weight.dtype), float(eps), _lib.NORM_OP if op_rounding else _lib.NORM_LAYER,
        normed.data_ptr(), res_out.data_ptr() if res_out is not None else None, gate_weight.data_ptr(), T, H, E, topk,
        1 if renormalize else 0, 1 if bf16_logits else 0, logits.data_ptr() if logits is not None else None,
        topk_weights.data_ptr(), topk_ids.data_ptr(), _lib.current_stream(dev))
    _lib.check(code, "norm_gate_topk")
    out = (normed, res_out, topk_weights, topk_ids)
    return out + (logits,) if return_logits else out


def fused_experts_normed(hidden_states: torch.Tensor, residual: Optional[torch.Tensor], norm_weight: torch.Tensor,
                         eps: float, gate_weight: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, topk: int,
                         renormalize: bool = True, out_dtype: Optional[torch.dtype] = None, bf16_act: bool = False,
                         bf16_logits: bool = True, op_rounding: bool = False, flags: int = 0,
                         workspace: Optional[MoeWorkspace] = None):
    """The tail of the reference's decoder layer in one call (models/mixtral.py:194-197):
    ``h, residual = post_attention_layernorm(hidden_states, residual); out = block_sparse_moe(h)``.
    Returns (out [T, H], residual_out or None)."""
    T, H = _norm_front_args(hidden_states, residual, norm_weight, gate_weight)
    _lib.require_device(w1, w2)
    E, two_i, Hw = w1.shape
    I = two_i // 2
    if Hw != H or tuple(w2.shape) != (E, H, I) or two_i != 2 * I or tuple(gate_weight.shape) != (E, H):
        raise RuntimeError("weight shapes do not match hidden_states")
    if w1.dtype != torch.bfloat16:
        raise RuntimeError("the fused MoE path computes in bfloat16: w1 and w2 must be bfloat16")
    flags |= _w2_flag(w2)
    if bf16_act:
        flags |= _lib.FLAG_BF16_ACT
    if not bf16_logits:
        flags |= _lib.FLAG_GATE_F32_LOGITS
    dev = hidden_states.device
    h_buf = torch.empty_like(hidden_states)
    res_out = torch.empty_like(hidden_states) if residual is not None else None
    if out_dtype == torch.float32:
        output = torch.empty((T, H), dtype=torch.float32, device=dev)
        flags |= _lib.FLAG_OUT_F32
    else:
        output = h_buf          # the experts' result overwrites the normalised rows, as the reference's in-place layer does
    if T == 0:
        return output, res_out
    ws = workspace or get_workspace(dev, T, H, I, E, topk, flags)
    code = _lib.load().em_moe_forward_normed(
        hidden_states.data_ptr(), residual.data_ptr() if residual is not None else None, norm_weight.data_ptr(),
        _lib.dtype_code(norm_weight.dtype), float(eps), _lib.NORM_OP if op_rounding else _lib.NORM_LAYER,
        h_buf.data_ptr(), res_out.data_ptr() if res_out is not None else None, gate_weight.data_ptr(), w1.data_ptr(),
        w2.data_ptr(), output.data_ptr(), T, H, I, E, topk, 1 if renormalize else 0, ws.buffer.data_ptr(),
        ctypes.c_size_t(ws.buffer.numel()), flags, _lib.current_stream(dev))
    _lib.check(code, "fused_experts_normed")
    return output, res_out
