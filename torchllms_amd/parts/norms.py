"""Normalisations."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import NORMS, Norm, ParamSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    """``y = cast(x32 * rsqrt(mean(x32^2) + eps)) * weight``: statistics and scaling in 32-bit,
    the weight multiply after the cast back (reference: torchllms/models/networks.py:186-200)."""

    graph_safe = True
    takes_split_sums = True  # ops.rmsnorm adds the slices of a split product while it reads them

    def __init__(self, size: int, eps: float):
        self.size = size
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {"weight": ParamSpec((self.size,), kind="vector", init="ones")}

    def check_sizes(self, dtype: torch.dtype) -> None:
        if not 0 < self.size <= ops.rmsnorm_max_hidden():
            raise ValueError(f"rmsnorm: rows of {self.size} elements; the kernel takes 1 to {ops.rmsnorm_max_hidden()}")

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors["weight"].contiguous()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(x, self.weight, self.eps)

    def forward_add(self, h: torch.Tensor, delta: Optional[torch.Tensor]):
        if delta is None:
            return h, ops.rmsnorm(h, self.weight, self.eps)
        return ops.rmsnorm(h, self.weight, self.eps, delta=delta, return_sum=True)

    def forward_add_for(self, reader, h: torch.Tensor, delta):
        if (isinstance(delta, ops.PendingProduct) and getattr(reader, "takes_normed_rows", False)
                and self.weight.dtype == torch.bfloat16 and self.size <= ops.NORMED_ROWS_MAX_WIDTH):
            # the product's own kernel adds it to h and leaves the rows' statistics, which the reader's kernel applies
            return delta.added_to(h, self.weight, self.eps)
        return self.forward_add(h, delta)

    def forward_rows(self, h: torch.Tensor, delta: Optional[torch.Tensor], rows: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(h, self.weight, self.eps, delta=delta, rows=rows)


@NORMS.register("layernorm")
class LayerNorm(Norm):
    """``y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * weight + bias``, statistics in 32-bit.  The
    residual stream it reads may be 32-bit in a bfloat16 model; what it hands on has the model's dtype.
    Its kernel adds a ``ScaledSum`` (a factor times the sum of a layer's branches) to the stream on the way."""

    graph_safe = True

    def __init__(self, size: int, eps: float):
        self.size = size
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None
        self.out_dtype: Optional[torch.dtype] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        # (kind "matrix": the vectors follow the model's dtype, which is the dtype of the normed rows)
        return {"weight": ParamSpec((self.size,), kind="matrix", init="ones"), "bias": ParamSpec((self.size,), kind="matrix", init="zeros")}

    def check_sizes(self, dtype: torch.dtype) -> None:
        if not 0 < self.size <= ops.rmsnorm_max_hidden():
            raise ValueError(f"layernorm: rows of {self.size} elements; the kernel takes 1 to {ops.rmsnorm_max_hidden()}")

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.out_dtype = tensors["weight"].dtype
        self.weight = tensors["weight"].float().contiguous()
        self.bias = tensors["bias"].float().contiguous()

    def delta(self, delta):
        if delta is None or isinstance(delta, ops.ScaledSum):
            return delta
        return ops.ScaledSum([ops.resolved(delta)], 1.0)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.layernorm(x, self.weight, self.bias, self.eps, self.out_dtype)

    def forward_add(self, h: torch.Tensor, delta):
        delta = self.delta(delta)
        if delta is None:
            return h, ops.layernorm(h, self.weight, self.bias, self.eps, self.out_dtype)
        return ops.layernorm(h, self.weight, self.bias, self.eps, self.out_dtype, delta=delta, return_sum=True)

    def forward_rows(self, h: torch.Tensor, delta, rows: torch.Tensor) -> torch.Tensor:
        return ops.layernorm(h, self.weight, self.bias, self.eps, self.out_dtype, delta=self.delta(delta), rows=rows)
