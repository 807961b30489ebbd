"""Norms.  RMSNorm: ``out = (x * rsqrt(mean(x^2) + eps)) * weight`` with the sum in 32-bit; Dynamic Tanh below.
With ``one_plus`` the stored weight lies around zero and the gain is ``1 + weight`` (added once, in 32-bit, when the
weight is loaded).  ``add_into`` is the norm behind a sublayer: the normed rows are added to the 32-bit residual.

Reference: crates/vipera-backend-cpu/src/model.rs:4282-4288 (eps inside the square root, added to
the mean; multiply order ``(x * inv) * w``).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..config.base import PartSpec
from ..ops import kernels
from ..weights.checkpoint import VECTOR, TensorSpec
from .base import Norm, NormHandoff, register_norm


class RMSNorm(Norm):
    """``params``: ``width``, ``eps``, ``name`` (the tensor is ``<name>.weight``, or ``params["tensor"]`` outright),
    ``one_plus`` (the gain is 1 + the stored weight)."""

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        self.width = int(spec.params["width"])
        self.eps = float(spec.params["eps"])
        self.one_plus = bool(spec.params.get("one_plus"))
        self.weight: Optional[torch.Tensor] = None

    @staticmethod
    def _tensor(spec: PartSpec, prefix: str) -> str:
        return f"{prefix}{spec.params['tensor']}" if spec.params.get("tensor") else f"{prefix}{spec.params['name']}.weight"

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        return [TensorSpec(cls._tensor(spec, prefix), (int(spec.params["width"]),), VECTOR,
                           "normal" if spec.params.get("one_plus") else "one_plus_normal",
                           optional=bool(spec.params.get("optional")))]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        weight = tensors.get(self._tensor(self.spec, self.prefix))
        if weight is not None and self.one_plus:
            weight = (weight.float() + 1.0).contiguous()
        self.weight = weight

    def add_into(self, y: torch.Tensor, residual: torch.Tensor, follow=None, as_input: bool = False):
        """``residual += y / rms(y) * gain``, all in 32-bit (the norm behind a sublayer).  ``follow``: the norm in front
        of the next sublayer; if it is of this kind the same launch applies it to the new rows and its output is
        returned.  ``as_input``: the new rows are returned in the run's dtype, for a part that reads the stream itself."""
        if isinstance(follow, RMSNorm) and follow.weight is not None:
            out = self.runtime.empty(tuple(residual.shape))
            kernels.rmsnorm_add(y, self.weight, self.eps, residual, out, follow.weight, follow.eps)
            return out
        if as_input and follow is None:
            if self.runtime.dtype == torch.float32:
                kernels.rmsnorm_add(y, self.weight, self.eps, residual)
                return residual
            out = self.runtime.empty(tuple(residual.shape))
            kernels.rmsnorm_add(y, self.weight, self.eps, residual, out)
            return out
        kernels.rmsnorm_add(y, self.weight, self.eps, residual)
        return follow.forward(residual) if follow is not None else None

    def handoff(self, tokens: int) -> Optional[NormHandoff]:
        if self.runtime.dtype != torch.bfloat16 or self.weight is None or self.weight.dtype != torch.float32:
            return None
        return NormHandoff(self.weight, self.eps, self.runtime.empty((tokens, self.width)),
                           torch.empty(kernels.follow_sumsq_floats(self.width, tokens), dtype=torch.float32,
                                       device=self.weight.device))

    def forward(self, x, out=None, rows=None):
        count = x.shape[0] if rows is None else rows.numel()
        if out is None:
            out = self.runtime.empty((count, self.width))
        kernels.rmsnorm(x, self.weight, self.eps, out, rows)
        return out


class DynamicTanh(Norm):
    """Dynamic Tanh: ``out = tanh(alpha * x) * weight + bias`` per element, with one learned number ``alpha``; no
    mean and no variance is computed (Zhu, Chen, He, LeCun, Liu: "Transformers without Normalization").  Tensors:
    ``<name>`` (the weight), ``<name>.alpha`` and ``<name>.b``; ``params["name"]`` is the weight's name after the
    part's prefix."""

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        self.width = int(spec.params["width"])
        self.weight = self.bias = self.alpha = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        name, width = f"{prefix}{spec.params['name']}", int(spec.params["width"])
        return [TensorSpec(name, (width,), VECTOR, "one_plus_normal"),
                TensorSpec(name + ".b", (width,), VECTOR, "normal"),
                TensorSpec(name + ".alpha", (), VECTOR, "one_plus_normal")]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        name = f"{self.prefix}{self.spec.params['name']}"
        self.weight, self.bias = tensors[name], tensors[name + ".b"]
        self.alpha = tensors[name + ".alpha"].reshape(1)

    def forward(self, x, out=None, rows=None):
        count = x.shape[0] if rows is None else rows.numel()
        if out is None:
            out = self.runtime.empty((count, self.width))
        kernels.dyt(x, self.alpha, self.weight, self.bias, out, rows)
        return out

    def forward_with(self, other: "DynamicTanh", x):
        """This norm's and ``other``'s output of the same rows, in one launch."""
        first, second = self.runtime.empty(tuple(x.shape)), self.runtime.empty(tuple(x.shape))
        kernels.dyt_pair(x, (self.alpha, self.weight, self.bias), (other.alpha, other.weight, other.bias), first, second)
        return first, second


register_norm("rmsnorm", RMSNorm)
register_norm("dyt", DynamicTanh)
