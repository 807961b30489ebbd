"""Grouped-query attention over the paged cache.

Order of work as in the reference's batched pass (crates/vipera-backend-cpu/src/model.rs:1005-1126):
``q, k, v = h W^T + b``; rotate q and k; write K (rotated) and V of every token of the step into the
cache; attend causally by count (a token at position p reads positions ``<= p`` of its own request,
or the last ``window`` of them); ``x += attn Wo^T``.  The three projections run as one product over
the concatenated weight ``[Wq; Wk; Wv]``, whose rows equal the separate products' rows.

Options, each a parameter that any architecture may set: ``softcap`` (a score becomes ``softcap * tanh(score /
softcap)``); ``chunk`` (a token sees the earlier tokens of its own block of that many positions, blocks counted from
position 0, instead of a window); ``value_dim`` (values narrower or wider than keys); ``qk_norm: "whole"`` (q and k
each RMS-normed over the whole projection, all heads at once, with a weight per number, before the rotation) or
``qk_norm: "head"`` (every q head and every k head RMS-normed by itself, with one weight of ``head_dim`` numbers for
all q heads and one for all k heads); ``gate: "sigmoid"`` (the heads' outputs times ``sigmoid(Wg h)`` before the output
projection); ``value_mix`` (``"source"``: the layer's values of the step's tokens are kept for later layers;
``"blend"``: its values become ``(1 - l) v + l v_source`` with the learned number ``l`` and the source layer's values
of the same token, and the blended values are what is cached; a ``"source"`` layer declares the number too and does not
read it); ``qk_norm: "unit"`` (every q and k head divided by its root mean square *behind* the rotation, no weight);
``gate: "head_sigmoid"`` (one number per head, ``sigmoid(Wg h)_h``); ``sink`` (a learned logit per head that joins the
softmax's denominator and nothing else); ``keep_first`` (with a window: the first that many positions of a sequence stay
visible; the layer then keeps all its pages); ``rel_bias`` (``{"rows", "far"}``: a learned table ``[rows, heads]`` added
to the scaled score by the distance between query and key: one row per distance below ``rows / 2``, logarithmic steps
from there to ``far``, the last row from ``far`` on); ``maps: 2`` with ``diff`` (differential attention: q and k hold two
maps per head, each an attention of its own over the same values; the head's output is ``a_1 - lambda a_2`` with
``lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff``, divided by its root mean square and multiplied by ``1 - diff``);
``tensors`` (the tensors' names after the part's name).  With any of these but the first three the step runs
as one product ``[q | k | v | g]`` with 32-bit sums (biases added there), a kernel that norms and lays the heads out at
one padded width, the rotation with the cache write, the paged attention kernels at that width, and a kernel that
unpacks and gates.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from ..config.base import PartSpec
from ..errors import InvalidArgumentError, UnsupportedError
from ..ops import kernels
from ..ops.attention import AttentionExtras, paged_attention
from ..ops.linear import linear, linear_follow, split_qkv_plan, streams_in_wave_order
from ..weights.checkpoint import MATRIX, VECTOR, TensorSpec
from .base import KVCacheSpec, Mixer, register_mixer


def _cat(tensors: List[torch.Tensor]) -> torch.Tensor:
    dtypes = {t.dtype for t in tensors}
    if len(dtypes) > 1:  # a matrix kept in 32-bit pulls its companions up with it
        tensors = [t.float() for t in tensors]
    return torch.cat(tensors, dim=0).contiguous()


_DEFAULT_NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
                  "g": "g_proj.weight", "q_norm": "q_norm.weight", "k_norm": "k_norm.weight",
                  "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias", "o_bias": "o_proj.bias",
                  "value_mix": "value_mix", "sink": "sink", "rel": "rel", "lq1": "lq1", "lk1": "lk1", "lq2": "lq2",
                  "lk2": "lk2"}

VALUE_MIX_KEY = "attention.value_mix.source"    # where a step keeps the source layer's values (``batch.shared``)


def _tensor_names(p) -> Dict[str, str]:
    names = dict(_DEFAULT_NAMES)
    names.update(p.get("tensors") or {})
    return names


def _is_general(p) -> bool:
    """Whether the layer needs the path that norms, pads and gates (see the module's text)."""
    return bool(p.get("qk_norm") or p.get("gate") or p.get("value_mix") or int(p.get("maps") or 1) > 1
                or int(p.get("value_dim") or p["head_dim"]) != int(p["head_dim"]))


def _padded_width(p) -> int:
    """The one width that keys and values have in the cache and in the attention kernels: the head width, or with
    values of another width the larger of the two, rounded up to a multiple of 16."""
    head_dim = int(p["head_dim"])
    if not _is_general(p):
        return head_dim
    # a key head holds its maps side by side
    return (max(head_dim * int(p.get("maps") or 1), int(p.get("value_dim") or head_dim)) + 15) // 16 * 16


def distance_rows(rows: int, far: float, upto: int) -> List[int]:
    """The table row of every distance 0 .. ``upto``: its own row below ``rows / 2``, then logarithmic steps up to the
    distance ``far``, at and beyond which it is the last row."""
    half = rows // 2
    out = []
    for n in range(upto + 1):
        if n < half:
            out.append(n)
        else:
            out.append(min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half)))))
    return out


class Attention(Mixer):
    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        p = spec.params
        self.hidden = int(p["hidden"])
        self.heads = int(p["heads"])
        self.kv_heads = int(p["kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.window = int(p.get("window") or 0)
        self.qkv_bias = bool(p.get("qkv_bias", False))
        self.out_bias = bool(p.get("out_bias", False))
        self.softcap = float(p.get("softcap") or 0.0)
        self.chunk = int(p.get("chunk") or 0)
        if self.chunk and self.window:
            raise InvalidArgumentError("attention: a window and blocks of positions exclude each other")
        self.mask = -self.chunk if self.chunk else self.window      # what the kernels take as `window`
        self.value_dim = int(p.get("value_dim") or self.head_dim)
        self.qk_norm, self.gate, self.value_mix = p.get("qk_norm"), p.get("gate"), p.get("value_mix")
        self.general = _is_general(p)
        self.padded = _padded_width(p)
        self.maps = int(p.get("maps") or 1)
        self.diff = float(p.get("diff") or 0.0)
        self.keep_first = int(p.get("keep_first") or 0)
        self.has_sink, self.rel_bias = bool(p.get("sink")), p.get("rel_bias")
        if self.keep_first and not self.window:
            raise InvalidArgumentError("attention: kept first positions need a window")
        # the kernel that rotates and norms in one pass, in 32-bit from the product's sums
        if (self.qk_norm == "unit" or self.maps > 1) and self.value_mix:
            raise UnsupportedError("attention: value_mix beside qk_norm \"unit\" or several maps is not implemented")
        self.prepares = (self.qk_norm in ("unit", "head") or self.maps > 1) and not self.value_mix
        self.extras = AttentionExtras(keep_first=self.keep_first)
        self.subtract = 0.0
        scale = p.get("scale")
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        if self.heads % self.kv_heads:
            raise InvalidArgumentError(f"heads {self.heads} is not a multiple of kv_heads {self.kv_heads}")
        self.q_width = self.heads * self.maps * self.head_dim
        self.kv_width = self.kv_heads * self.maps * self.head_dim
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = self.q_norm = self.k_norm = self.mix = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        p = spec.params
        base = f"{prefix}{p['name']}."
        names = _tensor_names(p)
        hidden, hd = int(p["hidden"]), int(p["head_dim"])
        vd = int(p.get("value_dim") or hd)
        maps = int(p.get("maps") or 1)
        q, kv = int(p["heads"]) * maps * hd, int(p["kv_heads"]) * maps * hd
        specs: List[TensorSpec] = []
        for name, rows in (("q", q), ("k", kv), ("v", int(p["kv_heads"]) * vd)):
            specs.append(TensorSpec(base + names[name], (rows, hidden), MATRIX))
            if p.get("qkv_bias"):
                specs.append(TensorSpec(base + names[name + "_bias"], (rows,), VECTOR))
        specs.append(TensorSpec(base + names["o"], (hidden, int(p["heads"]) * vd), MATRIX))
        if p.get("out_bias"):
            specs.append(TensorSpec(base + names["o_bias"], (hidden,), VECTOR))
        if p.get("qk_norm"):
            per_head = p.get("qk_norm") == "head"
        if p.get("qk_norm") in ("whole", "head"):
            specs += [TensorSpec(base + names["q_norm"], (hd if per_head else q,), VECTOR, "one_plus_normal"),
                      TensorSpec(base + names["k_norm"], (hd if per_head else kv,), VECTOR, "one_plus_normal")]
        if p.get("value_mix"):
            specs.append(TensorSpec(base + names["value_mix"], (), VECTOR, std=0.3))
        elif "value_mix" in (p.get("tensors") or {}):
            # a layer of a design that has the number but does not blend here: a folder may hold it all the same
            specs.append(TensorSpec(base + names["value_mix"], (), VECTOR, std=0.3, optional=True))
        if p.get("gate"):
            rows = int(p["heads"]) if p.get("gate") == "head_sigmoid" else int(p["heads"]) * vd
            specs.append(TensorSpec(base + names["g"], (rows, hidden), MATRIX))
        if p.get("sink"):
            specs.append(TensorSpec(base + names["sink"], (int(p["heads"]),), VECTOR, std=1.0))
        if p.get("rel_bias"):
            specs.append(TensorSpec(base + names["rel"], (int(p["rel_bias"]["rows"]), int(p["heads"])), VECTOR, std=0.5))
        if maps > 1:
            specs += [TensorSpec(base + names[n], (hd,), VECTOR, std=0.3) for n in ("lq1", "lk1", "lq2", "lk2")]
        return specs

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        base = f"{self.prefix}{self.spec.params['name']}."
        names = _tensor_names(self.spec.params)
        parts = [tensors[base + names[n]] for n in "qkv"]
        if self.gate:
            parts.append(tensors[base + names["g"]])
        self.w_qkv = _cat(parts)
        if self.qkv_bias:
            biases = [tensors[base + names[n + "_bias"]] for n in "qkv"]
            if self.gate:   # the gate's rows of the one product have no bias
                biases.append(torch.zeros(parts[-1].shape[0], dtype=biases[0].dtype, device=biases[0].device))
            self.b_qkv = torch.cat(biases).contiguous()
        self.w_o = tensors[base + names["o"]]
        if self.out_bias:
            self.b_o = tensors[base + names["o_bias"]]
        if self.qk_norm in ("whole", "head"):
            self.q_norm, self.k_norm = tensors[base + names["q_norm"]], tensors[base + names["k_norm"]]
        if self.has_sink:
            self.extras.sink = tensors[base + names["sink"]].float().contiguous()
        if self.rel_bias:
            # by distance instead of by row: the kernels then need no logarithm
            table = tensors[base + names["rel"]].float()
            far = int(math.ceil(float(self.rel_bias["far"])))
            rows = torch.tensor(distance_rows(table.shape[0], float(self.rel_bias["far"]), far), device=table.device)
            self.extras.rel = table[rows].t().contiguous()
        if self.maps > 1:
            dot = lambda a, b: float((tensors[base + names[a]].double() * tensors[base + names[b]].double()).sum())
            self.subtract = math.exp(dot("lq1", "lk1")) - math.exp(dot("lq2", "lk2")) + self.diff
        if self.value_mix:
            self.mix = tensors[base + names["value_mix"]].reshape(1)

    @classmethod
    def declare_cache(cls, spec: PartSpec):
        p = spec.params
        # blocks of positions keep everything: a page is only ever passed by all tokens at a block's edge, and the
        # pool is sized for whole requests
        # kept first positions lie outside the window that the pool's bookkeeping knows: such a layer keeps everything
        window = 0 if p.get("keep_first") else int(p.get("window") or 0)
        return KVCacheSpec(int(p["kv_heads"]), _padded_width(p), window), None

    @classmethod
    def check_supported(cls, spec: PartSpec, dtype: torch.dtype) -> None:
        p = spec.params
        heads, kv_heads, head_dim = int(p["heads"]) * int(p.get("maps") or 1), int(p["kv_heads"]), _padded_width(p)
        if p.get("qk_norm") not in (None, "whole", "head", "unit"):
            raise UnsupportedError(f"attention: qk_norm {p.get('qk_norm')!r} is not implemented; \"whole\", \"head\", "
                                   "\"unit\" or none")
        if int(p.get("maps") or 1) not in (1, 2):
            raise UnsupportedError(f"attention: {p.get('maps')} maps per head are not implemented; 1 or 2")
        if int(p.get("maps") or 1) > 1 and p.get("qk_norm") == "whole":
            raise UnsupportedError("attention: several maps beside qk_norm \"whole\" are not implemented")
        if p.get("rel_bias") and int(p["rel_bias"]["rows"]) != -1 and not (
                int(p["rel_bias"]["rows"]) >= 2 and float(p["rel_bias"]["far"]) > int(p["rel_bias"]["rows"]) // 2):
            raise InvalidArgumentError(f"attention: a bias by distance of {p['rel_bias']} needs at least two rows and a "
                                       "far distance beyond half of them")
        if p.get("value_mix") not in (None, "source", "blend"):
            raise UnsupportedError(f"attention: value_mix {p.get('value_mix')!r} is not implemented; \"source\", "
                                   "\"blend\" or none")
        if p.get("gate") not in (None, "sigmoid", "silu", "head_sigmoid"):
            raise UnsupportedError(f"attention: gate {p.get('gate')!r} is not implemented; \"sigmoid\", \"silu\", "
                                   "\"head_sigmoid\" or none")
        if head_dim > kernels.ATTENTION_MAX_HEAD_DIM:
            raise UnsupportedError(f"attention: head_dim {head_dim} is above the kernels' limit of "
                                   f"{kernels.ATTENTION_MAX_HEAD_DIM}")
        if heads + 2 * kv_heads > kernels.ATTENTION_MAX_HEADS:
            raise UnsupportedError(f"attention: {heads} query heads with {kv_heads} key/value heads are above the "
                                   f"kernels' limit of {kernels.ATTENTION_MAX_HEADS} heads in all")

    fills_handoff = True
    can_overwrite = True

    def _fused(self, tokens: int, position, batch) -> Optional[str]:
        """How product, rotation and cache write of a step of ``tokens`` run as one launch sequence without a
        rotation kernel, if they do: "stream" (up to 16 tokens, one kernel) or "split" (up to 64 tokens, K split
        over workgroups and the kernel that adds the ranges rotates).  All bfloat16, a full rotation computed in the
        kernel (no table of the step's angles)."""
        fused = position.fused_rotary()
        n, k = self.w_qkv.shape
        if self.general:
            return None
        if not (fused is not None and fused[1] == self.head_dim and self.runtime.dtype == torch.bfloat16
                and self.w_qkv.dtype == torch.bfloat16 and self.head_dim % 2 == 0 and k % 8 == 0
                and position.step_angles(batch) is None):
            return None
        if tokens <= 16 and streams_in_wave_order(tokens, n, k, rotates=True) and n * k * 2 < 2 ** 31:
            return "stream"
        if self.head_dim % 8 == 0 and split_qkv_plan(tokens, n, k) is not None:
            return "split"
        return None

    def accepts_handoff(self, tokens: int, position, batch) -> bool:
        # the fused products can divide by the norm themselves
        return self._fused(tokens, position, batch) is not None

    def _forward_general(self, h, batch, cache, position, residual, reads_only: bool, accumulate: bool) -> None:
        """q and k normed over the whole projection, values of another width, a gate on the output: see the module's
        text.  Heads are ``padded`` wide in the buffers that the rotation and the attention kernels see."""
        tokens = residual.shape[0]
        width = self.padded
        proj = torch.empty((tokens, self.w_qkv.shape[0]), dtype=torch.float32, device=residual.device)
        linear(h, self.w_qkv, self.b_qkv, proj)
        heads = self.heads * self.maps            # query heads as the attention kernels count them
        qkv = self.runtime.empty((tokens, (heads + 2 * self.kv_heads) * width))
        eps = float(self.spec.params.get("eps") or 0.0)
        first = None
        if self.value_mix:
            # the source layer's values of the step's tokens, as its product left them, are kept for the step
            v_col = (self.heads + self.kv_heads) * self.head_dim
            mine = proj[:, v_col:v_col + self.kv_heads * self.value_dim]
            if self.value_mix == "source":
                batch.shared[VALUE_MIX_KEY] = mine
            else:
                first = batch.shared.get(VALUE_MIX_KEY)
                if first is None or first.shape != mine.shape:
                    raise InvalidArgumentError("attention: a layer blends its values with a source layer's, but no layer "
                                               "before it in the run order keeps values of this shape")
        fused = position.fused_rotary()
        inv_freq, rotary_dim = fused if fused is not None else (None, 0)
        if self.prepares:
            if fused is None:
                raise UnsupportedError("attention: qk_norm \"unit\" and several maps need a rotation the kernels know, or none")
            # rotation, norm, layout and the cache write in one pass
            written = () if reads_only else (cache.k, cache.v, batch.entry_of_token, batch.block_tables[cache.group])
            kernels.head_prepare(proj, self.q_norm, self.k_norm, bool(self.qk_norm), self.qk_norm != "unit", eps,
                                 batch.positions, inv_freq, rotary_dim, self.heads, self.kv_heads, self.maps,
                                 self.head_dim, self.value_dim, width, qkv, *written)
        elif self.qk_norm == "whole" and first is None:
            kernels.whole_norm_pack(proj, self.q_norm, self.k_norm, eps, self.heads, self.kv_heads, self.head_dim,
                                    self.value_dim, width, qkv)
        elif self.qk_norm == "whole":
            raise UnsupportedError("attention: value_mix beside qk_norm \"whole\" is not implemented")
        else:
            kernels.head_norm_pack(proj, self.q_norm, self.k_norm, eps, self.heads, self.kv_heads, self.head_dim,
                                   self.value_dim, width, qkv, first, self.mix if first is not None else None)
        table = batch.block_tables[cache.group]
        if fused is None:
            position.apply(qkv, batch, heads, self.kv_heads, width)
        angles = position.step_angles(batch) if rotary_dim and not self.prepares else None
        if self.prepares:
            pass
        elif not reads_only:
            kernels.rope_kvwrite(qkv, batch.positions, inv_freq, rotary_dim, cache.k, cache.v, batch.entry_of_token,
                                 table, heads, self.kv_heads, width, angles)
        elif rotary_dim:
            kernels.rope_kvwrite(qkv, batch.positions, inv_freq, rotary_dim, None, None, batch.entry_of_token, None,
                                 heads, self.kv_heads, width, angles)
        attn = self.runtime.empty((tokens, heads * width))
        paged_attention(qkv, cache.k, cache.v, attn, batch, table, heads, self.kv_heads, width, self.scale,
                        self.mask, self.softcap, self.extras)
        values = self.runtime.empty((tokens, self.heads * self.value_dim))
        gate = proj[:, self.q_width + self.kv_width + self.kv_heads * self.value_dim:] if self.gate else None
        if self.maps > 1 or self.gate == "head_sigmoid":
            kernels.head_finish(attn, values, self.heads, self.value_dim, width, self.maps, self.subtract,
                                unit_norm=self.maps > 1, eps=eps, factor=1.0 - self.diff if self.maps > 1 else 1.0,
                                gate=gate, gate_kind="sigmoid" if self.gate else "none", gate_per_head=True)
        else:
            kernels.head_unpack_gate(attn, gate, self.gate or "none", self.heads, self.value_dim, width, values)
        linear(values, self.w_o, self.b_o, residual, accumulate=accumulate)

    def forward(self, h, batch, cache, state, position, residual, reads_only: bool = False, handoff=None,
                incoming=None, accumulate: bool = True) -> None:
        tokens = residual.shape[0]
        if self.general:
            return self._forward_general(h, batch, cache, position, residual, reads_only, accumulate)
        how = self._fused(tokens, position, batch)
        if incoming is not None and how is None:
            raise UnsupportedError("attention was handed a split norm for a step whose product cannot divide by it")
        scaled = {} if incoming is None else {"sumsq": incoming.sumsq, "groups": incoming.groups, "eps": incoming.eps}
        if incoming is not None:
            h = incoming.scaled
        qkv = self.runtime.empty((tokens, self.q_width + 2 * self.kv_width))
        table = batch.block_tables[cache.group]
        fused = position.fused_rotary()
        inv_freq, rotary_dim = fused if fused is not None else (None, 0)
        angles = position.step_angles(batch) if rotary_dim else None
        caches = (None, None, batch.entry_of_token, None) if reads_only else (cache.k, cache.v, batch.entry_of_token, table)
        if how == "stream" and kernels.gemm_bf16_qkv_rope_supported(h, self.w_qkv, qkv, self.head_dim):
            kernels.gemm_bf16_qkv_rope(h, self.w_qkv, self.b_qkv, qkv, batch.positions, inv_freq, *caches, self.heads,
                                       self.kv_heads, self.head_dim, **scaled)
        elif how == "split" and kernels.gemm_bf16_supported(h, self.w_qkv, qkv):
            ranges, rows_per_wave = split_qkv_plan(tokens, *self.w_qkv.shape)
            kernels.gemm_bf16_mid_qkv_rope(h, self.w_qkv, self.b_qkv, qkv, ranges, rows_per_wave, batch.positions, inv_freq,
                                           *caches, self.heads, self.kv_heads, self.head_dim, **scaled)
        else:
            if incoming is not None:
                raise UnsupportedError("attention was handed a split norm for operands its fused product does not take")
            linear(h, self.w_qkv, self.b_qkv, qkv)
            if fused is None:
                position.apply(qkv, batch, self.heads, self.kv_heads, self.head_dim)
            if not reads_only:
                kernels.rope_kvwrite(qkv, batch.positions, inv_freq, rotary_dim, cache.k, cache.v, batch.entry_of_token,
                                     table, self.heads, self.kv_heads, self.head_dim, angles)
            elif rotary_dim:
                kernels.rope_kvwrite(qkv, batch.positions, inv_freq, rotary_dim, None, None, batch.entry_of_token,
                                     None, self.heads, self.kv_heads, self.head_dim, angles)
        attn = self.runtime.empty((tokens, self.q_width))
        paged_attention(qkv, cache.k, cache.v, attn, batch, table, self.heads, self.kv_heads, self.head_dim,
                        self.scale, self.mask, self.softcap, self.extras)
        if handoff is not None:
            # the output product also prepares the norm that follows (its gained copy of the residual, its squares)
            # where its kernel can; 0 groups say that it could not
            handoff.groups = linear_follow(attn, self.w_o, self.b_o, residual, handoff.gain, handoff.scaled, handoff.sumsq)
        else:
            linear(attn, self.w_o, self.b_o, residual, accumulate=accumulate)


register_mixer("attention", Attention)
