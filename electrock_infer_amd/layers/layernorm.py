"""RMSNorm module with the reference's constructor, parameter and call
(layers/layernorm.py:5-55): ``forward(x)`` returns the normalised tensor,
``forward(x, residual)`` returns ``(normalised, x + residual)``; the inputs are left as they are.

The reference runs this as a chain of torch element-wise ops; here one HIP kernel reads
every row once and writes it once, with the same rounding points (float32 sum and variance,
one rounding before and one after the multiplication by the weight).
"""
from typing import Optional, Tuple, Union

import torch
from torch import nn

from .. import _lib


class RMSNorm(nn.Module):

    def __init__(self, hidden_size: int, eps: float = 1e-5) -> None:
        super().__init__()
        self.hidden_size = hidden_size
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.is_custom_ops = True

    def _check(self, x: torch.Tensor) -> int:
        _lib.require_device(x, self.weight)
        if x.size(-1) != self.hidden_size:
            raise RuntimeError("last dimension must be hidden_size")
        return x.numel() // self.hidden_size

    def rms_forward(self, x: torch.Tensor) -> torch.Tensor:
        rows = self._check(x)
        out = torch.empty_like(x)
        code = _lib.load().em_rms_norm(x.data_ptr(), out.data_ptr(), self.weight.data_ptr(), rows, self.hidden_size,
                                       float(self.eps), _lib.dtype_code(x.dtype), _lib.dtype_code(self.weight.dtype),
                                       _lib.NORM_LAYER, _lib.current_stream(x.device))
        _lib.check(code, "RMSNorm")
        return out

    def add_rms_forward(self, x: torch.Tensor, residual: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        rows = self._check(x)
        _lib.require_device(residual)
        if residual.shape != x.shape or residual.dtype != x.dtype:
            raise RuntimeError("residual must match x")
        out = torch.empty_like(x)
        res_out = torch.empty_like(x)
        code = _lib.load().em_add_rms_norm(x.data_ptr(), residual.data_ptr(), out.data_ptr(), res_out.data_ptr(),
                                           self.weight.data_ptr(), rows, self.hidden_size, float(self.eps),
                                           _lib.dtype_code(x.dtype), _lib.dtype_code(self.weight.dtype),
                                           _lib.NORM_LAYER, _lib.current_stream(x.device))
        _lib.check(code, "RMSNorm")
        return out, res_out

    def forward(self, x: torch.Tensor, residual: Optional[torch.Tensor] = None
                ) -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
        if residual is None:
            return self.rms_forward(x)
        return self.add_rms_forward(x, residual)
