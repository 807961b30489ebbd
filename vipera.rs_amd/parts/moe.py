"""Mixture of experts: each token runs ``top`` of ``experts`` small gated feed-forwards.

Router logits ``z = W_router h`` in 32-bit; the ``top`` largest are chosen (the lowest id among equals) and weighted
by the softmax over the chosen logits only.  An expert computes ``g = min(W_gate h, limit)``,
``u = clamp(W_up h, -limit, limit)``, ``y = g * sigmoid(alpha * g) * (u + 1)`` and returns ``W_down y``; the layer
adds the weighted sum of the chosen experts' outputs to the residual.  ``limit`` and ``alpha`` are parameters; without
a ``limit`` nothing is clamped and ``y = g * sigmoid(alpha * g) * u`` (``alpha`` 1: ``silu(g) * u``).  ``groups`` and
``keep``: the experts form that many equal groups of neighbours, a group's score is its largest logit, and only experts
of the ``keep`` best groups can be chosen.  ``scores: "all"``: the weights are the chosen experts' shares of the softmax
over all experts, not renormalized; ``scores: "sigmoid"``: a chosen expert's weight is the sigmoid of its own logit, not
renormalized; ``scores: "steered"``: the experts are chosen by ``sigmoid(z) + correction`` (a learned number per
expert, tensor ``<name>.correction``, that steers the choice and nothing else) and a chosen expert's weight is
``weight_scale * sigmoid(z)``, not renormalized.  ``weigh: "input"``: the weight multiplies what the expert reads instead of what it returns, so the layer
adds the sum of ``expert(w h)``.  ``shared``: a gated feed-forward of that width (``silu(Wg h) * (Wu h)`` through
``Wd``, tensors ``<name>.shared.gate | up | down``) that every token runs beside its experts; with ``shared_gate``
("sigmoid") its output is multiplied by ``sigmoid(Wsg h)``, one number per token (tensor ``<name>.shared.sg``).

The step's (token, choice) pairs are grouped by expert on the device, so nothing about the routing reaches the
host and a step of single tokens can be captured; see ``csrc/kernels/moe.hip``.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from ..config.base import PartSpec
from ..errors import InvalidArgumentError, UnsupportedError
from ..ops import kernels
from ..ops.linear import linear
from ..weights.checkpoint import MATRIX, VECTOR, TensorSpec
from .base import FeedForward, register_ffn


class MixtureOfExperts(FeedForward):
    """``params``: ``hidden``, ``intermediate`` (an expert's width), ``experts``, ``top``, ``limit`` (None: no clamp),
    ``alpha`` (1.702 unless given), ``groups`` and ``keep`` (1 and 1 unless given), ``scores`` ("chosen", "all" or
    "sigmoid"), ``weigh`` ("output" or "input"), ``shared`` (the shared expert's width, or None), ``name``; tensors
    ``<name>.router``, ``<name>.e<i>.gate | up | down`` and ``<name>.shared.gate | up | down``."""

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        p = spec.params
        self.hidden, self.inter = int(p["hidden"]), int(p["intermediate"])
        self.experts, self.top = int(p["experts"]), int(p["top"])
        self.limit = float(p["limit"]) if p.get("limit") is not None else float("inf")
        self.alpha = float(p.get("alpha", 1.702))
        self.groups, self.keep = int(p.get("groups") or 1), int(p.get("keep") or p.get("groups") or 1)
        self.all_scores = {"chosen": False, "all": True, "sigmoid": "sigmoid", "steered": "steered"}[p.get("scores", "chosen")]
        self.weight_scale = float(p.get("weight_scale", 1.0))
        self.shared_gate = p.get("shared_gate")
        self.correction = self.w_shared_gate = None
        self.weigh_input = p.get("weigh", "output") == "input"
        self.shared = None
        if p.get("shared"):
            from .mlp import GatedMLP
            self.shared = GatedMLP(self._shared_spec(p), prefix, runtime)
        if not 1 <= self.top <= self.experts:
            raise InvalidArgumentError(f"a token cannot use {self.top} of {self.experts} experts")
        self.w_router = self.w_gate = self.w_up = self.w_down = None

    @staticmethod
    def _shared_spec(p) -> PartSpec:
        return PartSpec("gated_mlp", {"hidden": int(p["hidden"]), "intermediate": int(p["shared"]),
                                      "name": f"{p['name']}.shared",
                                      "tensors": {"gate": "gate", "up": "up", "down": "down"}})

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        p = spec.params
        base = f"{prefix}{p['name']}."
        hidden, inter = int(p["hidden"]), int(p["intermediate"])
        specs = []
        for e in range(int(p["experts"])):
            specs += [TensorSpec(f"{base}e{e}.gate", (inter, hidden), MATRIX),
                      TensorSpec(f"{base}e{e}.up", (inter, hidden), MATRIX),
                      TensorSpec(f"{base}e{e}.down", (hidden, inter), MATRIX)]
        specs.append(TensorSpec(base + "router", (int(p["experts"]), hidden), MATRIX))
        if p.get("scores") == "steered":
            specs.append(TensorSpec(base + "correction", (int(p["experts"]),), VECTOR, std=0.1))
        if p.get("shared"):
            from .mlp import GatedMLP
            specs += GatedMLP.declare(cls._shared_spec(p), prefix)
            if p.get("shared_gate"):
                specs.append(TensorSpec(base + "shared.sg", (1, hidden), MATRIX))
        return specs

    @classmethod
    def check_supported(cls, spec: PartSpec, dtype: torch.dtype) -> None:
        experts, top = int(spec.params["experts"]), int(spec.params["top"])
        if top > 64 or experts > 4096:
            raise UnsupportedError(f"mixture of experts: top {top} of {experts} experts is above the routing kernel's "
                                   "limits of 64 of 4,096")
        groups = int(spec.params.get("groups") or 1)
        keep = int(spec.params.get("keep") or groups)
        if groups > 64:
            raise UnsupportedError(f"mixture of experts: {groups} groups are above the routing kernel's limit of 64")
        if groups < 1 or experts % groups or not 1 <= keep <= groups or (keep < groups and keep * (experts // groups) < top):
            raise InvalidArgumentError(f"mixture of experts: {keep} of {groups} groups of {experts} experts cannot "
                                       f"give a token its {top}")
        if spec.params.get("scores", "chosen") not in ("chosen", "all", "sigmoid", "steered"):
            raise UnsupportedError(f"mixture of experts: scores {spec.params.get('scores')!r}; \"chosen\", \"all\", "
                                   "\"sigmoid\" or \"steered\"")
        if spec.params.get("shared_gate") not in (None, "sigmoid"):
            raise UnsupportedError(f"mixture of experts: shared_gate {spec.params.get('shared_gate')!r}; \"sigmoid\" or none")
        if spec.params.get("weigh", "output") not in ("output", "input"):
            raise UnsupportedError(f"mixture of experts: weigh {spec.params.get('weigh')!r}; \"output\" or \"input\"")

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        base = f"{self.prefix}{self.spec.params['name']}."
        dtype = self.runtime.dtype
        stack = lambda kind: torch.stack([tensors[f"{base}e{e}.{kind}"].to(dtype) for e in range(self.experts)]).contiguous()
        self.w_gate, self.w_up, self.w_down = stack("gate"), stack("up"), stack("down")
        self.w_router = tensors[base + "router"]
        if self.all_scores == "steered":
            self.correction = tensors[base + "correction"]
        if self.shared is not None:
            self.shared.load(tensors)
            if self.shared_gate:
                # the gate's row rides behind the router's rows: one product for all that is one number per token
                self.w_shared_gate = tensors[base + "shared.sg"]
                self.w_router = torch.cat([self.w_router.to(self.w_shared_gate.dtype), self.w_shared_gate]).contiguous()

    can_overwrite = True

    def forward(self, h, batch, residual, accumulate: bool = True, **_unused) -> None:
        tokens = residual.shape[0]
        device = residual.device
        pairs = tokens * self.top
        rows = torch.empty((tokens, self.w_router.shape[0]), dtype=torch.float32, device=device)
        linear(h, self.w_router, None, rows)
        logits = rows[:, :self.experts]
        tile_rows = kernels.moe_tile_rows(h, self.hidden, self.inter)
        ints = torch.empty(2 * pairs + self.experts + 2 + 2 * kernels.moe_max_tiles(pairs, self.experts, tile_rows),
                           dtype=torch.int32, device=device)
        ids, order = ints[:pairs], ints[pairs:2 * pairs]
        offsets = ints[2 * pairs:2 * pairs + self.experts + 1]
        num_tiles = ints[2 * pairs + self.experts + 1:2 * pairs + self.experts + 2]
        tiles = ints[2 * pairs + self.experts + 2:]
        weights = torch.empty(pairs, dtype=torch.float32, device=device)
        kernels.moe_route(logits, self.top, ids, weights, offsets, order, tiles, num_tiles, tile_rows,
                          groups=self.groups, keep=self.keep, all_scores=self.all_scores, correction=self.correction,
                          weight_scale=self.weight_scale)
        act = self.runtime.empty((pairs, self.inter))
        pair_out = torch.empty((pairs, self.hidden), dtype=torch.float32, device=device)
        kernels.moe_experts(h, self.w_gate, self.w_up, self.w_down, offsets, order, tiles, num_tiles, weights,
                            self.top, self.limit, self.alpha, act, pair_out, residual, accumulate, self.weigh_input)
        if self.shared is not None and self.w_shared_gate is None:
            self.shared.forward(h, batch, residual)
        elif self.shared is not None:
            # the shared expert into a buffer of its own, which joins the others' sum times the token's gate
            own = torch.empty_like(residual)
            self.shared.forward(h, batch, own, accumulate=False)
            kernels.row_gate_add(own, rows[:, self.experts:], self.shared_gate, residual)


register_ffn("moe", MixtureOfExperts)
