"""Gated feed-forward (SwiGLU): ``x += (up(h) * silu(gate(h))) Wd^T``.

Reference: crates/vipera-backend-cpu/src/model.rs:672-680, 1159-1198; ``silu(z) = z / (1 + exp(-z))``
(model.rs:4368-4370).  Gate and up run as one product over a fused weight; with bfloat16 weights its
rows are interleaved in groups of 16 so that the product's epilogue can apply the gate.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from ..config.base import PartSpec
from ..errors import UnsupportedError
from ..ops import kernels
from ..ops.linear import gated_plan, interleave_gate_up, linear, linear_follow, linear_gated
from ..weights.checkpoint import MATRIX, TensorSpec
from .attention import _cat
from .base import FeedForward, register_ffn


class GatedMLP(FeedForward):
    """``params``: ``hidden``, ``intermediate``, ``name``; tensors ``<name>.gate_proj.weight | up_proj.weight |
    down_proj.weight``, or as ``params["tensors"]`` names them (keys ``gate``, ``up``, ``down``)."""

    @staticmethod
    def _names(spec: PartSpec, prefix: str):
        names = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}
        names.update(spec.params.get("tensors") or {})
        base = f"{prefix}{spec.params['name']}."
        return base + names["gate"], base + names["up"], base + names["down"]

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        self.hidden = int(spec.params["hidden"])
        self.inter = int(spec.params["intermediate"])
        self.activation = spec.params.get("activation", "silu")
        if self.activation not in ("silu", "gelu_tanh"):
            raise UnsupportedError(f"activation {self.activation!r} is not implemented; \"silu\" or \"gelu_tanh\"")
        self.w_gate_up = self.w_down = None
        self.interleaved = False

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        gate, up, down = cls._names(spec, prefix)
        hidden, inter = int(spec.params["hidden"]), int(spec.params["intermediate"])
        return [
            TensorSpec(gate, (inter, hidden), MATRIX),
            TensorSpec(up, (inter, hidden), MATRIX),
            TensorSpec(down, (hidden, inter), MATRIX),
        ]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        gate_name, up_name, down_name = self._names(self.spec, self.prefix)
        gate, up = tensors[gate_name], tensors[up_name]
        # all-bfloat16 weights of a width the kernels can pair are interleaved, so that the product's
        # epilogue can apply the gate; anything else stays [gate; up]
        self.interleaved = gate.dtype == torch.bfloat16 and up.dtype == torch.bfloat16 and self.inter % 16 == 0
        if self.activation != "silu" and self.hidden % 8:
            self.interleaved = False     # only the matrix-core product applies this gate to interleaved rows
        self.w_gate_up = interleave_gate_up(gate, up) if self.interleaved else _cat([gate, up])
        self.w_down = tensors[down_name]

    def _dividing_plan(self, tokens: int):
        """0 or 3 where the gate/up product of ``tokens`` rows runs on a kernel that can divide by the norm in front
        of it (the kernel with resident activations, the tiled kernel), else None."""
        if not (self.interleaved and self.w_gate_up.dtype == torch.bfloat16 and self.runtime.dtype == torch.bfloat16):
            return None
        if tokens > 64:  # no product before the norm leaves its first half for more than 64 tokens
            return None
        plan = gated_plan(tokens, *self.w_gate_up.shape, kernels.compute_units(self.w_gate_up.device))
        return plan if plan in (0, 3) and (plan == 3 or tokens <= 16) else None

    def accepts_handoff(self, tokens: int) -> bool:
        return self._dividing_plan(tokens) is not None

    fills_handoff = True

    can_overwrite = True

    def forward(self, h, batch, residual, handoff=None, outgoing=None, accumulate: bool = True) -> None:
        tokens = residual.shape[0]
        act = self.runtime.empty((tokens, self.inter))
        if self.activation != "silu" and self.interleaved and h.dtype == torch.bfloat16 and kernels.gemm_bf16_supported(
                h, self.w_gate_up, act):
            kernels.gemm_bf16_gated_act(h, self.w_gate_up, act, self.activation)   # the tiled product's epilogue
        elif self.activation != "silu":
            # the product's 32-bit sums, then act(gate) * up in one pass
            if self.interleaved:
                raise UnsupportedError("gated_mlp: this step's operands leave the matrix-core product, which alone applies "
                                       f"{self.activation} to interleaved gate and up rows")
            both = torch.empty((tokens, 2 * self.inter), dtype=torch.float32, device=residual.device)
            linear(h, self.w_gate_up, None, both)
            kernels.activation(both[:, :self.inter], self.activation, act, mul=both[:, self.inter:])
        elif handoff is not None and self._dividing_plan(tokens) == 0:
            kernels.gemm_bf16_gated_scaled(handoff.scaled, self.w_gate_up, act, handoff.sumsq, handoff.groups, handoff.eps)
        elif handoff is not None:
            kernels.gemm_bf16_gated_tile_scaled(handoff.scaled, self.w_gate_up, act, handoff.sumsq, handoff.groups,
                                                handoff.eps)
        else:
            linear_gated(h, self.w_gate_up, act, self.interleaved)
        if outgoing is not None:
            # the down product also prepares the next layer's first norm where its kernel can
            outgoing.groups = linear_follow(act, self.w_down, None, residual, outgoing.gain, outgoing.scaled, outgoing.sumsq)
        else:
            linear(act, self.w_down, None, residual, accumulate=accumulate)


class NoFeedForward(FeedForward):
    """A layer without a feed-forward: adds nothing."""

    def forward(self, h, batch, residual, **_unused) -> None:
        return None


class PlainMLP(FeedForward):
    """``x += Wdown act(Wup h)`` without a gate.  ``params``: ``hidden``, ``intermediate``, ``activation`` ("relu2":
    the square of relu; "silu"; "gelu_tanh"), ``name``; tensors ``<name>.up`` and ``<name>.down`` (or as
    ``params["tensors"]`` names them)."""

    can_overwrite = True

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        self.hidden, self.inter = int(spec.params["hidden"]), int(spec.params["intermediate"])
        self.activation = spec.params.get("activation", "relu2")
        self.w_up = self.w_down = None

    @staticmethod
    def _names(spec: PartSpec, prefix: str):
        names = {"up": "up", "down": "down"}
        names.update(spec.params.get("tensors") or {})
        base = f"{prefix}{spec.params['name']}."
        return base + names["up"], base + names["down"]

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        up, down = cls._names(spec, prefix)
        hidden, inter = int(spec.params["hidden"]), int(spec.params["intermediate"])
        return [TensorSpec(up, (inter, hidden), MATRIX), TensorSpec(down, (hidden, inter), MATRIX)]

    @classmethod
    def check_supported(cls, spec: PartSpec, dtype) -> None:
        kind = spec.params.get("activation", "relu2")
        if kind not in ("relu2", "silu", "gelu_tanh"):
            raise UnsupportedError(f"mlp: activation {kind!r} is not implemented; relu2, silu or gelu_tanh")

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        up, down = self._names(self.spec, self.prefix)
        self.w_up, self.w_down = tensors[up], tensors[down]

    def forward(self, h, batch, residual, accumulate: bool = True, **_unused) -> None:
        tokens = residual.shape[0]
        up = self.runtime.empty((tokens, self.inter))
        linear(h, self.w_up, None, up)
        act = self.runtime.empty((tokens, self.inter))
        kernels.activation(up, self.activation, act)
        linear(act, self.w_down, None, residual, accumulate=accumulate)


register_ffn("mlp", PlainMLP)
register_ffn("gated_mlp", GatedMLP)
register_ffn("none", NoFeedForward)
