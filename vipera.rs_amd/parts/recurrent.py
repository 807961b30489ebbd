"""Recurrent mixers: layers that keep a matrix of state per head instead of a cache of keys and values.

``gated_delta``: the gated delta rule.  ``q = Wq h``, ``k = Wk h`` (``kv_heads x dim``), ``v = Wv h``
(``heads x vdim``); each passes a short causal convolution over time per channel and silu; q and k become unit
vectors per head (q also times ``dim^-1/2``); ``beta = sigmoid(Wb h)``, ``g = exp(-exp(A_log) softplus(Wa h +
dt_bias))`` per head; then per head ``S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``; the read-out is
``o / rms(o) * norm * silu(Wg h)`` and goes through ``Wo``.  Options: ``decay: "channel"`` (one decay per head and key
channel, ``g[h, d]``, which scales row ``d`` of ``S``; ``dt_bias`` is then ``[heads * dim]``), ``decay_rank`` and
``gate_rank`` (the decay's and the gate's projections in two steps, ``Wa2 (Wa1 h)`` and ``Wg2 (Wg1 h)``, through that
many numbers), ``gate: "sigmoid"``.

``matrix_memory``: the matrix memory with exponential gates (mLSTM; Beck et al., "xLSTM: Extended Long Short-Term
Memory").  ``q = Wq h * dim^-1/2``, ``k = Wk h`` (``heads x dim``), ``v = Wv h`` (``heads x vdim``); per head the
logarithms of an input gate ``li = cap tanh((Wi h + bi) / cap)`` and of a forget gate
``lf = logsigmoid(cap tanh((Wf h + bf) / cap))``; with a running maximum ``m`` that starts at 0:
``m' = max(lf + m, li); S <- exp(lf + m - m') S + exp(li - m') k v^T``, ``n`` likewise with ``k`` alone,
``o = S^T q / (max(|n . q|, exp(-m')) + 1e-6)``; the read-out is ``o / rms(o)`` per head ``* norm * sigmoid(Wg h)`` and
goes through ``Wo``.

``wkv``: RWKV-style time mixing.  Each of r, k, v, g, w reads its own mix ``h + (h_prev - h) * mu``; the decay is
``w = exp(-exp(W2 tanh(W1 mix_w) + w0))`` per key channel; per head ``o = (S + diag(u) k v^T)^T r`` and then
``S <- diag(w) S + k v^T``; the read-out is ``o / rms(o) * norm * silu(Wg mix_g)`` and goes through ``Wo``.

``decay_attention``: linear attention whose heads forget at a fixed rate each.  ``q = act(Wq h)``, ``k = act(Wk h)``
(``heads x dim``), ``v = act(Wv h)`` (``heads x vdim``); per head ``S <- decay_h S + k v^T; o = S^T q``; the heads'
outputs are normed together (one RMS norm over ``heads * vdim`` numbers), gated by ``sigmoid(Wg h)`` and go through
``Wo``.  Options: ``rotary`` (q and k rotated by position before they enter the recurrence, as an attention layer's
are), ``k_scale`` (k multiplied by it behind the rotation), ``norm: "head"`` (every head's output divided by its own
root mean square, no weight: retention).

``selective_scan``: Mamba.  ``W_in h = [x | z]``; x passes a short causal convolution per channel with a bias, and
silu; ``W_x x = [dt | B | C]``; ``step = softplus(W_dt dt + dt_bias)``; per channel c and state n
``S[c, n] <- exp(step_c A[c, n]) S[c, n] + step_c x_c B_n`` with ``A = -exp(A_log)``; ``y_c = S[c, :] . C + D_c x_c``;
``y * silu(z)`` goes through ``Wo``.

All keep their state in 32-bit in the request's slot: the matrices, and what the next token needs of this one (the
convolution's last inputs; the last ``h``).  An entry that starts at position 0 starts from zeros.  Everything the
kernels look at lies on the device, so a step of single tokens can be captured.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from ..config.base import PartSpec
from ..errors import InvalidArgumentError, UnsupportedError
from ..ops import kernels
from ..ops.linear import linear
from ..weights.checkpoint import MATRIX, VECTOR, TensorSpec
from .attention import _cat
from .base import Mixer, StateSpec, register_mixer

UNIT_EPS = 1e-6   # q and k of the delta rule: x / sqrt(sum(x^2) + UNIT_EPS)


class GatedDelta(Mixer):
    """``params``: ``hidden``, ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``conv`` (taps), ``eps`` (of the read-out's
    norm), ``name``; optional ``decay`` ("head": one per head, tensors ``a`` ``[heads, hidden]`` and ``dt_bias``
    ``[heads]``; "channel": one per head and key channel, ``heads * dim`` of each), ``decay_rank`` and ``gate_rank``
    (0: one projection ``a`` / ``g``; a number: two, ``a1`` ``[rank, hidden]`` and ``a2`` ``[., rank]``, ``g1`` and
    ``g2``; -1: as many as the folder's tensor has), ``gate`` ("silu" or "sigmoid")."""

    can_overwrite = True

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        p = spec.params
        self.hidden, self.heads, self.kv_heads = int(p["hidden"]), int(p["heads"]), int(p["kv_heads"])
        self.dim, self.vdim, self.taps = int(p["dim"]), int(p["vdim"]), int(p["conv"])
        self.eps = float(p["eps"])
        if self.heads % self.kv_heads:
            raise InvalidArgumentError(f"heads {self.heads} is not a multiple of kv_heads {self.kv_heads}")
        self.qk, self.vw = self.kv_heads * self.dim, self.heads * self.vdim
        self.channels = 2 * self.qk + self.vw
        self.per_channel = p.get("decay", "head") == "channel"
        self.decays = self.heads * self.dim if self.per_channel else self.heads
        self.decay_rank, self.gate_rank = int(p.get("decay_rank") or 0), int(p.get("gate_rank") or 0)
        self.gate_kind = p.get("gate", "silu")
        self.w_in = self.w_o = self.conv = self.a_log = self.dt_bias = self.norm = self.w_a2 = self.w_g2 = None

    @classmethod
    def _sizes(cls, p):
        qk, vw = int(p["kv_heads"]) * int(p["dim"]), int(p["heads"]) * int(p["vdim"])
        return qk, vw, 2 * qk + vw

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        p = spec.params
        base = f"{prefix}{p['name']}."
        hidden, heads, taps = int(p["hidden"]), int(p["heads"]), int(p["conv"])
        qk, vw, _ = cls._sizes(p)
        decays = heads * int(p["dim"]) if p.get("decay", "head") == "channel" else heads
        specs = []
        for name, rows in (("q", qk), ("k", qk), ("v", vw)):
            specs.append(TensorSpec(base + name, (rows, hidden), MATRIX))
            specs.append(TensorSpec(f"{base}{name}.conv", (rows, taps), VECTOR, std=0.5))
        specs += [TensorSpec(base + "b", (heads, hidden), MATRIX), TensorSpec(base + "A_log", (heads,), VECTOR),
                  TensorSpec(base + "norm", (int(p["vdim"]),), VECTOR, "one_plus_normal"),
                  TensorSpec(base + "dt_bias", (decays,), VECTOR), TensorSpec(base + "o", (hidden, vw), MATRIX)]
        for letter, rows, rank in (("a", decays, int(p.get("decay_rank") or 0)), ("g", vw, int(p.get("gate_rank") or 0))):
            if rank:
                specs += [TensorSpec(f"{base}{letter}1", (rank, hidden), MATRIX),
                          TensorSpec(f"{base}{letter}2", (rows, rank), MATRIX, std=0.2)]
            else:
                specs.append(TensorSpec(base + letter, (rows, hidden), MATRIX))
        return specs

    @classmethod
    def declare_cache(cls, spec: PartSpec):
        p = spec.params
        _, _, channels = cls._sizes(p)
        floats = int(p["heads"]) * kernels.recurrent_head_floats(int(p["dim"]), int(p["vdim"])) + (int(p["conv"]) - 1) * channels
        return None, StateSpec((floats,), torch.float32)

    @classmethod
    def check_supported(cls, spec: PartSpec, dtype: torch.dtype) -> None:
        p = spec.params
        if int(p["dim"]) > kernels.RECURRENT_MAX_KEY_DIM:
            raise UnsupportedError(f"gated_delta: a key width of {p['dim']} is above the kernel's limit of "
                                   f"{kernels.RECURRENT_MAX_KEY_DIM}")
        if int(p["conv"]) < 1:
            raise UnsupportedError(f"gated_delta: the convolution needs at least one tap, got {p['conv']}")
        if cls._sizes(p)[2] > 16_384:
            raise UnsupportedError("gated_delta: more than 16,384 convolved channels do not fit the kernel's LDS row")
        if p.get("decay", "head") not in ("head", "channel") or p.get("gate", "silu") not in ("silu", "sigmoid"):
            raise UnsupportedError(f"gated_delta: decay {p.get('decay')!r} with gate {p.get('gate')!r} is not implemented")

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        base = f"{self.prefix}{self.spec.params['name']}."
        # one product for everything that reads h: [q | k | v | g or g1 | b | a or a1] rows
        gate, decay = ("g1" if self.gate_rank else "g"), ("a1" if self.decay_rank else "a")
        self.w_in = _cat([tensors[base + n] for n in ("q", "k", "v", gate, "b", decay)])
        self.gate_rows, self.decay_rows = int(tensors[base + gate].shape[0]), int(tensors[base + decay].shape[0])
        if self.gate_rank:
            self.w_g2 = tensors[base + "g2"]
        if self.decay_rank:
            self.w_a2 = tensors[base + "a2"]
        for name, second, first_rows in (("g", self.w_g2, self.gate_rows), ("a", self.w_a2, self.decay_rows)):
            if second is not None and second.shape[1] != first_rows:
                raise InvalidArgumentError(f"{base}{name}2 has {second.shape[1]} columns for the {first_rows} rows of "
                                           f"{base}{name}1")
        self.conv = torch.cat([tensors[f"{base}{n}.conv"] for n in ("q", "k", "v")]).contiguous()
        self.a_log, self.dt_bias, self.norm = tensors[base + "A_log"], tensors[base + "dt_bias"], tensors[base + "norm"]
        self.w_o = tensors[base + "o"]

    def _second_step(self, low: torch.Tensor, weight: torch.Tensor, out_dtype) -> torch.Tensor:
        """``weight`` applied to the 32-bit columns ``low`` of the first product: in the run's dtype, as every product."""
        tokens = low.shape[0]
        rows = self.runtime.empty((tokens, low.shape[1]))
        kernels.activation(low, "none", rows)
        out = torch.empty((tokens, weight.shape[0]), dtype=out_dtype, device=low.device)
        linear(rows, weight, None, out)
        return out

    def forward(self, h, batch, cache, state, position, residual, reads_only: bool = False, accumulate: bool = True) -> None:
        tokens, entries = residual.shape[0], batch.num_entries
        device = residual.device
        f32 = dict(dtype=torch.float32, device=device)
        # what enters the recurrence stays 32-bit from the product's sums on
        proj = torch.empty((tokens, self.w_in.shape[0]), **f32)
        linear(h, self.w_in, None, proj)
        g_col = self.channels
        b_col = g_col + self.gate_rows
        a_col = b_col + self.heads
        plain = not self.per_channel and not self.decay_rank       # the decay per head straight from the first product
        # q, k, v and, behind them, the decays per key channel where the layer has those
        rows = torch.empty((tokens, self.channels + (self.decays if self.per_channel else 0)), **f32)
        qkv = rows[:, :self.channels]
        beta = torch.empty((tokens, self.heads), **f32)
        decay = None if self.per_channel else torch.empty((tokens, self.heads), **f32)
        matrices = self.heads * kernels.recurrent_head_floats(self.dim, self.vdim)
        kernels.delta_prepare(proj, self.conv, state, matrices, batch.entry_of_token, batch.entry_start,
                              batch.entry_first_pos, batch.slots, self.a_log if plain else None,
                              self.dt_bias if plain else None, self.kv_heads, self.dim, self.heads, self.vdim, b_col,
                              a_col if plain else -1, UNIT_EPS, qkv, beta, decay if plain else None, entries)
        if not plain:
            raw = proj[:, a_col:a_col + self.decay_rows]
            if self.decay_rank:
                raw = self._second_step(raw, self.w_a2, torch.float32)
            kernels.channel_decay(raw, self.a_log, self.dt_bias, self.heads, self.dim if self.per_channel else 1,
                                  rows[:, self.channels:] if self.per_channel else decay)
        o = torch.empty((tokens, self.vw), **f32)
        kernels.delta_rule(qkv, beta, decay, state, batch.entry_start, batch.entry_first_pos, batch.slots,
                           self.kv_heads, self.dim, self.heads, self.vdim, o, entries, short_entries=batch.all_single,
                           channel_decay_col=self.channels if self.per_channel else -1)
        gate = proj[:, g_col:g_col + self.gate_rows]
        if self.gate_rank:
            gate = self._second_step(gate, self.w_g2, self.runtime.dtype)
        gated = self.runtime.empty((tokens, self.vw))
        kernels.head_norm_gate(o, self.norm, gate, self.gate_kind, self.eps, self.heads, self.vdim, gated)
        linear(gated, self.w_o, None, residual, accumulate=accumulate)


class MatrixMemory(Mixer):
    """``params``: ``hidden``, ``heads``, ``dim``, ``vdim``, ``gate_cap``, ``eps`` (of the read-out's norm), ``name``;
    tensors ``<name>.q | k | v | g | o | norm | i | i.b | f | f.b``."""

    can_overwrite = True

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        p = spec.params
        self.hidden, self.heads, self.dim, self.vdim = int(p["hidden"]), int(p["heads"]), int(p["dim"]), int(p["vdim"])
        self.cap, self.eps = float(p["gate_cap"]), float(p["eps"])
        self.qk, self.vw = self.heads * self.dim, self.heads * self.vdim
        self.w_in = self.b_in = self.w_o = self.norm = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        p = spec.params
        base = f"{prefix}{p['name']}."
        hidden, heads = int(p["hidden"]), int(p["heads"])
        qk, vw = heads * int(p["dim"]), heads * int(p["vdim"])
        return [TensorSpec(base + "q", (qk, hidden), MATRIX), TensorSpec(base + "k", (qk, hidden), MATRIX),
                TensorSpec(base + "v", (vw, hidden), MATRIX), TensorSpec(base + "g", (vw, hidden), MATRIX),
                TensorSpec(base + "o", (hidden, vw), MATRIX), TensorSpec(base + "norm", (vw,), VECTOR, "one_plus_normal"),
                TensorSpec(base + "i", (heads, hidden), MATRIX), TensorSpec(base + "i.b", (heads,), VECTOR, std=0.5),
                TensorSpec(base + "f", (heads, hidden), MATRIX), TensorSpec(base + "f.b", (heads,), VECTOR, std=0.5)]

    @classmethod
    def declare_cache(cls, spec: PartSpec):
        p = spec.params
        return None, StateSpec((kernels.memory_state_floats(int(p["heads"]), int(p["dim"]), int(p["vdim"])),), torch.float32)

    @classmethod
    def check_supported(cls, spec: PartSpec, dtype: torch.dtype) -> None:
        p = spec.params
        if int(p["dim"]) > kernels.RECURRENT_MAX_KEY_DIM:
            raise UnsupportedError(f"matrix_memory: a key width of {p['dim']} is above the kernel's limit of "
                                   f"{kernels.RECURRENT_MAX_KEY_DIM}")
        if not float(p["gate_cap"]) > 0.0:
            raise InvalidArgumentError(f"matrix_memory: gate_cap is {p['gate_cap']!r}; it must be above 0")

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        base = f"{self.prefix}{self.spec.params['name']}."
        self.w_in = _cat([tensors[base + n] for n in ("q", "k", "v", "g", "i", "f")])   # one product for all that reads h
        bias = torch.zeros(self.w_in.shape[0], dtype=torch.float32, device=self.w_in.device)
        bias[-2 * self.heads:-self.heads] = tensors[base + "i.b"].float()
        bias[-self.heads:] = tensors[base + "f.b"].float()
        self.b_in = bias
        self.w_o, self.norm = tensors[base + "o"], tensors[base + "norm"]

    def forward(self, h, batch, cache, state, position, residual, reads_only: bool = False, accumulate: bool = True) -> None:
        tokens, entries = residual.shape[0], batch.num_entries
        proj = torch.empty((tokens, self.w_in.shape[0]), dtype=torch.float32, device=residual.device)
        linear(h, self.w_in, self.b_in, proj)              # 32-bit from the product's sums on
        k_col, v_col = self.qk, 2 * self.qk
        g_col = v_col + self.vw
        i_col = g_col + self.vw
        o = torch.empty((tokens, self.vw), dtype=torch.float32, device=residual.device)
        kernels.memory_rule(proj, 0, k_col, v_col, i_col, i_col + self.heads, self.dim ** -0.5, self.cap, state,
                            batch.entry_start, batch.entry_first_pos, batch.slots, self.dim, self.heads, self.vdim, o,
                            entries, short_entries=batch.all_single)
        gated = self.runtime.empty((tokens, self.vw))
        kernels.head_norm_gate(o, self.norm, proj[:, g_col:g_col + self.vw], "sigmoid", self.eps, self.heads, self.vdim, gated)
        linear(gated, self.w_o, None, residual, accumulate=accumulate)


class Wkv(Mixer):
    """``params``: ``hidden``, ``heads``, ``dim``, ``eps``, ``name``, and ``decay_rank`` (rows of W1; 0 or absent: as many
    as the folder's tensor has)."""

    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        p = spec.params
        self.hidden, self.heads, self.dim = int(p["hidden"]), int(p["heads"]), int(p["dim"])
        self.rank, self.eps = int(p.get("decay_rank") or 0), float(p["eps"])
        self.width = self.heads * self.dim
        self.mu = self.w = self.w1 = self.w2 = self.w0 = self.bonus = self.norm = self.w_o = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        p = spec.params
        base = f"{prefix}{p['name']}."
        hidden, heads, dim, rank = int(p["hidden"]), int(p["heads"]), int(p["dim"]), int(p.get("decay_rank") or 0) or -1
        width = heads * dim
        specs = [TensorSpec(f"{base}mu.{s}", (hidden,), VECTOR, std=0.3) for s in cls.MIXES]
        specs += [TensorSpec(base + "k", (width, hidden), MATRIX), TensorSpec(base + "v", (width, hidden), MATRIX),
                  TensorSpec(base + "g", (width, hidden), MATRIX), TensorSpec(base + "w1", (rank, hidden), MATRIX),
                  TensorSpec(base + "w2", (width, rank), MATRIX), TensorSpec(base + "w0", (width,), VECTOR),
                  TensorSpec(base + "u", (heads, dim), VECTOR), TensorSpec(base + "norm", (width,), VECTOR, "one_plus_normal"),
                  TensorSpec(base + "o", (hidden, width), MATRIX), TensorSpec(base + "r", (width, hidden), MATRIX)]
        return specs

    @classmethod
    def declare_cache(cls, spec: PartSpec):
        p = spec.params
        matrices = int(p["heads"]) * kernels.recurrent_head_floats(int(p["dim"]), int(p["dim"]))
        return None, StateSpec((matrices + int(p["hidden"]),), torch.float32)

    @classmethod
    def check_supported(cls, spec: PartSpec, dtype: torch.dtype) -> None:
        if int(spec.params["dim"]) > kernels.RECURRENT_MAX_KEY_DIM:
            raise UnsupportedError(f"wkv: a head width of {spec.params['dim']} is above the kernel's limit of "
                                   f"{kernels.RECURRENT_MAX_KEY_DIM}")

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        base = f"{self.prefix}{self.spec.params['name']}."
        self.mu = torch.stack([tensors[f"{base}mu.{s}"] for s in self.MIXES]).contiguous()
        self.w = {s: tensors[base + s] for s in ("r", "k", "v", "g")}
        self.w1, self.w2 = tensors[base + "w1"], tensors[base + "w2"]
        self.rank = int(self.w1.shape[0])
        if self.w2.shape[1] != self.rank:
            raise InvalidArgumentError(f"{base}w2 has {self.w2.shape[1]} columns for the {self.rank} rows of {base}w1")
        self.w0, self.bonus = tensors[base + "w0"], tensors[base + "u"].reshape(-1).contiguous()
        self.norm, self.w_o = tensors[base + "norm"], tensors[base + "o"]

    def forward(self, h, batch, cache, state, position, residual, reads_only: bool = False) -> None:
        tokens, entries = residual.shape[0], batch.num_entries
        device = residual.device
        f32 = dict(dtype=torch.float32, device=device)
        matrices = self.heads * kernels.recurrent_head_floats(self.dim, self.dim)
        mixes = self.runtime.empty((len(self.MIXES), tokens, self.hidden))
        kernels.token_shift(h, self.mu, state, matrices, batch.entry_of_token, batch.entry_start,
                            batch.entry_first_pos, batch.slots, mixes, entries)
        # r, k, v and the decay enter the recurrence: 32-bit from their products' sums on
        rkv = torch.empty((3, tokens, self.width), **f32)
        for index, name in enumerate(("r", "k", "v")):
            linear(mixes[index], self.w[name], None, rkv[index])
        gate = self.runtime.empty((tokens, self.width))
        linear(mixes[3], self.w["g"], None, gate)
        low = torch.empty((tokens, self.rank), **f32)
        linear(mixes[4], self.w1, None, low)
        squashed = torch.empty((tokens, self.rank), **f32)
        kernels.tanh(low, squashed)
        wraw = torch.empty((tokens, self.width), **f32)
        linear(squashed, self.w2, None, wraw)
        o = torch.empty((tokens, self.width), **f32)
        # a prompt's recurrence reads a token's decay once per workgroup of value channels: the two exponentials are
        # taken once, ahead of it; a step of single tokens takes them inside the recurrence (one launch less)
        ahead = not batch.all_single
        if ahead:
            kernels.decay_(wraw, self.w0)
        kernels.wkv_rule(rkv[0], rkv[1], rkv[2], wraw, self.w0, self.bonus, state, batch.entry_start,
                         batch.entry_first_pos, batch.slots, self.dim, self.heads, o, entries,
                         short_entries=batch.all_single, decayed=ahead)
        gated = self.runtime.empty((tokens, self.width))
        kernels.head_norm_gate(o, self.norm, gate, True, self.eps, self.heads, self.dim, gated)
        linear(gated, self.w_o, None, residual, accumulate=True)


class DecayAttention(Mixer):
    """``params``: ``hidden``, ``heads``, ``dim``, ``vdim``, ``decay`` (one number per head), ``eps`` (of the read-out's
    norm), ``activation`` ("silu" or "none", of q, k and v), ``gate`` ("sigmoid", "silu" or "none"), ``name``; tensors
    ``<name>.q | k | v | g | o | norm``.  Optional: ``rotary`` (``{"dims", "base"}``: the first ``dims`` numbers of every
    q and k head rotate by position in half-split pairs, in 32-bit), ``k_scale`` (1 unless given), ``norm`` ("whole":
    one norm over all heads with the weight ``norm``; "head": each head over its own root mean square, no tensor)."""

    can_overwrite = True

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        p = spec.params
        self.hidden, self.heads, self.dim, self.vdim = int(p["hidden"]), int(p["heads"]), int(p["dim"]), int(p["vdim"])
        self.eps = float(p["eps"])
        self.activation, self.gate = p.get("activation", "silu"), p.get("gate", "sigmoid")
        rates = [float(r) for r in p["decay"]]
        if len(rates) != self.heads:
            raise InvalidArgumentError(f"decay_attention: {len(rates)} decays for {self.heads} heads")
        if self.activation not in ("silu", "none") or self.gate not in ("sigmoid", "silu", "none"):
            raise UnsupportedError(f"decay_attention: activation {self.activation!r} with gate {self.gate!r} is not implemented")
        self.decay = torch.tensor(rates, dtype=torch.float32, device=runtime.device)
        self.qk, self.vw = self.heads * self.dim, self.heads * self.vdim
        self.w_in = self.w_o = self.norm = None
        self.k_scale = float(p.get("k_scale") or 1.0)
        self.norm_kind = p.get("norm", "whole")
        rotary = p.get("rotary") or {}
        self.rot_dims = int(rotary.get("dims") or 0)
        self.inv_freq = None
        if self.rot_dims:
            from .rotary import neox_inverse_frequencies
            if self.rot_dims % 2 or self.rot_dims > self.dim:
                raise InvalidArgumentError(f"decay_attention: {self.rot_dims} rotated numbers of a head of {self.dim}")
            self.inv_freq = torch.from_numpy(neox_inverse_frequencies(self.rot_dims, float(rotary["base"]))).to(runtime.device)
        if self.norm_kind == "head":
            self.norm = torch.ones(self.vdim, dtype=torch.float32, device=runtime.device)

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        p = spec.params
        base = f"{prefix}{p['name']}."
        hidden, qk, vw = int(p["hidden"]), int(p["heads"]) * int(p["dim"]), int(p["heads"]) * int(p["vdim"])
        specs = [TensorSpec(base + "q", (qk, hidden), MATRIX), TensorSpec(base + "k", (qk, hidden), MATRIX),
                 TensorSpec(base + "v", (vw, hidden), MATRIX), TensorSpec(base + "g", (vw, hidden), MATRIX),
                 TensorSpec(base + "o", (hidden, vw), MATRIX)]
        if p.get("norm", "whole") == "whole":
            specs.append(TensorSpec(base + "norm", (vw,), VECTOR, "one_plus_normal"))
        return specs

    @classmethod
    def declare_cache(cls, spec: PartSpec):
        p = spec.params
        return None, StateSpec((int(p["heads"]) * kernels.decay_rule_head_floats(int(p["dim"]), int(p["vdim"])),), torch.float32)

    @classmethod
    def check_supported(cls, spec: PartSpec, dtype: torch.dtype) -> None:
        if int(spec.params["dim"]) > kernels.DECAY_RULE_MAX_KEY_DIM:
            raise UnsupportedError(f"decay_attention: a key width of {spec.params['dim']} is above the kernel's limit of "
                                   f"{kernels.DECAY_RULE_MAX_KEY_DIM}")
        if spec.params.get("norm", "whole") not in ("whole", "head"):
            raise UnsupportedError(f"decay_attention: norm {spec.params.get('norm')!r}; \"whole\" or \"head\"")

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        base = f"{self.prefix}{self.spec.params['name']}."
        self.w_in = _cat([tensors[base + n] for n in ("q", "k", "v", "g")])     # one product for all that reads h
        self.w_o = tensors[base + "o"]
        if self.norm_kind == "whole":
            self.norm = tensors[base + "norm"]

    def forward(self, h, batch, cache, state, position, residual, reads_only: bool = False, accumulate: bool = True) -> None:
        tokens, entries = residual.shape[0], batch.num_entries
        f32 = dict(dtype=torch.float32, device=residual.device)
        proj = torch.empty((tokens, self.w_in.shape[0]), **f32)        # 32-bit from the product's sums on
        linear(h, self.w_in, None, proj)
        q, k = proj[:, :self.qk], proj[:, self.qk:2 * self.qk]
        v, g = proj[:, 2 * self.qk:2 * self.qk + self.vw], proj[:, 2 * self.qk + self.vw:]
        o = torch.empty((tokens, self.vw), **f32)
        inside = self.activation == "silu"
        if self.rot_dims or self.k_scale != 1.0:
            if inside:
                raise UnsupportedError("decay_attention: a rotation behind an activation of q and k is not implemented")
            if self.rot_dims:
                kernels.rotate_scale(q, batch.positions, self.inv_freq, self.rot_dims, self.heads, self.dim)
            kernels.rotate_scale(k, batch.positions, self.inv_freq, self.rot_dims, self.heads, self.dim, self.k_scale)
        if inside and not batch.all_single:
            # every workgroup of value channels would take the activation of a token's q and k again, token behind
            # token: a prompt's portion takes it once, ahead of the recurrence; a step of single tokens saves the launch
            width = 2 * self.qk + self.vw
            ready = torch.empty((tokens, width), **f32)
            kernels.activation(proj[:, :width], "silu", ready)
            q, k, v = ready[:, :self.qk], ready[:, self.qk:2 * self.qk], ready[:, 2 * self.qk:]
            inside = False
        kernels.decay_rule(q, k, v, inside, self.decay, state, batch.entry_start,
                           batch.entry_first_pos, batch.slots, self.heads, self.dim, self.vdim, o, entries)
        gated = self.runtime.empty((tokens, self.vw))
        if self.norm_kind == "head":
            if self.gate == "none":
                raise UnsupportedError("decay_attention: a norm per head without a gate is not implemented")
            kernels.head_norm_gate(o, self.norm, g, self.gate, self.eps, self.heads, self.vdim, gated)
        else:
            kernels.gated_norm(o, self.norm, g, self.gate, self.eps, gated)
        linear(gated, self.w_o, None, residual, accumulate=accumulate)


class SelectiveScan(Mixer):
    """``params``: ``hidden``, ``inner`` (channels), ``state`` (numbers per channel), ``dt_rank``, ``conv`` (taps),
    ``name``; tensors ``<name>.in | conv | conv.b | x | dt | dt.b | A_log | D | o``."""

    can_overwrite = True

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        p = spec.params
        self.hidden, self.inner, self.states = int(p["hidden"]), int(p["inner"]), int(p["state"])
        self.rank, self.taps = int(p["dt_rank"]), int(p["conv"])
        self.w_in = self.conv = self.conv_b = self.w_x = self.w_dt = self.dt_b = self.a_log = self.skip = self.w_o = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        p = spec.params
        base = f"{prefix}{p['name']}."
        hidden, inner, states, rank, taps = (int(p[k]) for k in ("hidden", "inner", "state", "dt_rank", "conv"))
        return [TensorSpec(base + "in", (2 * inner, hidden), MATRIX),
                TensorSpec(base + "conv", (inner, taps), VECTOR, std=0.5), TensorSpec(base + "conv.b", (inner,), VECTOR),
                TensorSpec(base + "x", (rank + 2 * states, inner), MATRIX),
                TensorSpec(base + "dt", (inner, rank), MATRIX, std=0.2), TensorSpec(base + "dt.b", (inner,), VECTOR, std=0.5),
                TensorSpec(base + "A_log", (inner, states), VECTOR, std=0.5), TensorSpec(base + "D", (inner,), VECTOR, std=0.5),
                TensorSpec(base + "o", (hidden, inner), MATRIX)]

    @classmethod
    def state_floats(cls, p) -> int:
        return int(p["inner"]) * kernels.selective_scan_channel_floats(int(p["state"])) + (int(p["conv"]) - 1) * int(p["inner"])

    @classmethod
    def declare_cache(cls, spec: PartSpec):
        return None, StateSpec((cls.state_floats(spec.params),), torch.float32)

    @classmethod
    def check_supported(cls, spec: PartSpec, dtype: torch.dtype) -> None:
        p = spec.params
        if int(p["state"]) > kernels.SELECTIVE_SCAN_MAX_STATES:
            raise UnsupportedError(f"selective_scan: {p['state']} states a channel are above the kernel's limit of "
                                   f"{kernels.SELECTIVE_SCAN_MAX_STATES}")
        if int(p["conv"]) < 1 or int(p["dt_rank"]) < 1:
            raise UnsupportedError("selective_scan: the convolution needs at least one tap and dt at least one row")

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        base = f"{self.prefix}{self.spec.params['name']}."
        self.w_in, self.w_x, self.w_dt, self.w_o = (tensors[base + n] for n in ("in", "x", "dt", "o"))
        self.conv, self.conv_b, self.dt_b = tensors[base + "conv"], tensors[base + "conv.b"], tensors[base + "dt.b"]
        self.a_log, self.skip = tensors[base + "A_log"], tensors[base + "D"]

    def forward(self, h, batch, cache, state, position, residual, reads_only: bool = False, accumulate: bool = True) -> None:
        tokens, entries = residual.shape[0], batch.num_entries
        f32 = dict(dtype=torch.float32, device=residual.device)
        xz = torch.empty((tokens, 2 * self.inner), **f32)
        linear(h, self.w_in, None, xz)
        matrices = self.inner * kernels.selective_scan_channel_floats(self.states)
        # the convolved x enters the recurrence in 32-bit; the product behind it reads it in the run's dtype
        x32 = torch.empty((tokens, self.inner), **f32)
        x_run = None if self.runtime.dtype == torch.float32 else self.runtime.empty((tokens, self.inner))
        kernels.causal_conv(xz[:, :self.inner], self.conv, self.conv_b, state, matrices, batch.entry_of_token,
                            batch.entry_start, batch.entry_first_pos, batch.slots, x32, x_run, entries)
        low = torch.empty((tokens, self.rank + 2 * self.states), **f32)
        linear(x32 if x_run is None else x_run, self.w_x, None, low)
        dt = torch.empty((tokens, self.inner), **f32)
        steps = low[:, :self.rank]
        if self.runtime.dtype != torch.float32 and self.w_dt.dtype == self.runtime.dtype and self.rank % 8 == 0:
            # in the run's dtype the product runs on the matrix cores (a 32-bit input beside 16-bit weights would not)
            steps = self.runtime.empty((tokens, self.rank))
            kernels.activation(low[:, :self.rank], "none", steps)
        linear(steps, self.w_dt, None, dt)
        y = self.runtime.empty((tokens, self.inner))
        z = xz[:, self.inner:]
        ahead = not batch.all_single
        if ahead:   # a prompt's portion: the step sizes' softplus and the gate's silu once, ahead of the recurrence
            gate = torch.empty((tokens, self.inner), **f32)
            kernels.scan_prepare(dt, self.dt_b, z, gate)
            z = gate
        kernels.selective_scan(x32, dt, self.dt_b, low[:, self.rank:self.rank + self.states],
                               low[:, self.rank + self.states:], self.a_log, self.skip, z, state,
                               batch.entry_start, batch.entry_first_pos, batch.slots, y, entries, prepared=ahead)
        linear(y, self.w_o, None, residual, accumulate=accumulate)


register_mixer("gated_delta", GatedDelta)
register_mixer("matrix_memory", MatrixMemory)
register_mixer("decay_attention", DecayAttention)
register_mixer("selective_scan", SelectiveScan)
register_mixer("wkv", Wkv)
