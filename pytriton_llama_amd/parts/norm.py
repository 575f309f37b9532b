"""RMSNorm with the residual sum fused in front of it."""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from .base import ParamSource, Part, PendingProduct, PendingScale, as_tensor, place, register_part


@register_part("norm", "rmsnorm")
class RMSNorm(Part):
    """y = (x + residual) * rsqrt(mean((x + residual)^2) + eps) * weight, with the
    sum returned as the new residual (lite_llama/kernels/skip_rmsnorm.py:94-181;
    call sites lite_llama/models/llama.py:149,160,219). Without a residual the
    input itself is the residual (:181). ``offset``: what is added to the checkpoint's vector
    to give the weight (1.0 for a design that stores its norm weights around zero)."""
    kernel_libraries = ("norm", "gemm", "gemm_rows", "stream")
    takes_pending_product = True

    def __init__(self, size: int, eps: float, weight_name: str = "weight", streams: int = 1,
                 offset: float = 0.0):
        self.size = int(size)
        self.eps = float(eps)
        self.offset = float(offset)
        self.streams = int(streams)         # > 1: the rows hold that many float32 streams side by
                                            # side, and their sum is what is normed
        self.weight_name = weight_name
        self.weight: Optional[torch.Tensor] = None
        self.dtype: Optional[torch.dtype] = None

    def param_sources(self) -> List[ParamSource]:
        init = ("normal", 0.0, 0.1) if self.offset else None      # (random weights: around 1 - offset)
        return [ParamSource(self.weight_name, (self.size,), "vector", init=init)]

    def load(self, tensors, dtype, device) -> None:
        self.weight = place(tensors[self.weight_name], "vector", dtype, device)
        if self.offset:
            self.weight = self.weight + self.offset
        self.dtype = dtype

    def forward(self, x, residual: Optional[torch.Tensor], scale_ok: bool = False):
        if isinstance(x, PendingProduct):
            # some tens of rows (from ops.ROWS_MIN on): the product as partial sums over slices of
            # K, then one kernel that adds them up, adds the residual and normalises
            if (residual is not None and x.blocked is not None
                    and ops.gemm_rows_add_rmsnorm_fits(x.x, x.w, x.blocked, residual, self.weight)):
                y = ops.gemm_rows_add_rmsnorm(x.x, x.w, x.blocked, residual, self.weight, self.eps)
                return y, residual
            # the few rows of a decode step: the product, the residual sum and the weight in one
            # kernel; the rsqrt factor is left to the part that takes the result
            if (scale_ok and residual is not None
                    and ops.gemm_skinny_add_norm_fits(x.x, x.w, residual, self.weight)):
                y, scale = ops.gemm_skinny_add_norm(x.x, x.w, residual, self.weight, self.eps,
                                                    blocked=x.blocked)
                return PendingScale(y, scale), residual
        x = as_tensor(x)
        if self.streams > 1:
            if residual is not None:
                raise ValueError("a norm over the sum of several streams takes no residual")
            return ops.hyper_mix(x, self.streams, None, None, None, None, self.weight, self.eps, self.dtype), x
        if residual is None and x.dtype == torch.float32 and self.dtype not in (None, torch.float32):
            # rows of a residual stream that is kept in float32: the result in the engine's dtype
            return ops.stream_rmsnorm(x, self.weight, self.eps, self.dtype), x
        y = ops.add_rmsnorm(x, residual, self.weight, self.eps)
        return y, (x if residual is None else residual)


@register_part("norm", "dynamic_tanh")
class DynamicTanh(Part):
    """y = tanh(alpha * x) * weight + bias, elementwise: a norm that takes no statistics of its row
    (Zhu, Chen, He, LeCun, Liu: "Transformers without Normalization"). ``alpha`` is a scalar
    of the checkpoint. The arithmetic is float32; the result is in the engine's dtype.

    With a residual: the sum is made in a float32 residual stream (``residual`` must be one;
    it is updated in place), as the blocks that keep such a stream do in one kernel with the
    norms around it (``params()`` hands them what they need)."""
    kernel_libraries = ("stream",)

    def __init__(self, size: int, weight_name: str = "weight", bias_name: str = "bias",
                 alpha_name: str = "alpha"):
        self.size = int(size)
        self.names = (weight_name, bias_name, alpha_name)
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None
        self.alpha = 1.0
        self.dtype: Optional[torch.dtype] = None

    def param_sources(self) -> List[ParamSource]:
        w, b, a = self.names
        return [ParamSource(w, (self.size,), "vector"),
                ParamSource(b, (self.size,), "vector", init=("normal", 0.0, 0.1)),
                ParamSource(a, (), "vector", init=("uniform", 0.4, 1.2))]

    def load(self, tensors, dtype, device) -> None:
        w, b, a = self.names
        self.weight = place(tensors[w], "vector", dtype, device)
        self.bias = place(tensors[b], "vector", dtype, device)
        self.alpha = float(tensors[a].float().item())        # (a host tensor of the checkpoint)
        self.dtype = dtype

    def params(self):
        return (self.weight, self.bias, self.alpha)

    def forward(self, x, residual: Optional[torch.Tensor]):
        x = as_tensor(x)
        if residual is None:
            return ops.dyt(x, self.weight, self.bias, self.alpha, self.dtype), x
        y, _ = ops.stream_add_dyt(residual, x, None, self.params(), self.dtype)
        return y, residual
