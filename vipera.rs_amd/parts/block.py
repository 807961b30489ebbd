"""Arrangements of a layer's parts.

``prenorm``: ``x += mixer(norm_1(x)); x += ffn(norm_2(x))``, the pre-norm residual block of the
reference (crates/vipera-backend-cpu/src/model.rs:3-4, 975-1198).
``parallel``: ``h = norm(x); x += mixer(h) + ffn(h)``; with a second norm of its own for the feed-forward,
``x += m * (mixer(norm_1(x)) + ffn(norm_2(x)))``, both norms of the same ``x``, ``m`` = ``params["residual_mult"]``.
``sandwich_norm``: a norm before and behind each sublayer, ``x += norm_1b(mixer(norm_1(x))); x += norm_2b(ffn(norm_2(x)))``,
and optionally a part that adds to the stream after both (``extras["after"]``, of the feed-forward family; it reads the
32-bit stream itself).  The norms behind the sublayers are ``extras["mixer_post_norm"]`` and ``extras["ffn_post_norm"]``.
``postnorm``: a norm behind each sublayer only, ``x += norm_1(mixer(x)); x += norm_2(ffn(x))``; the sublayers read the
stream itself (``LayerSpec.mixer_norm`` and ``ffn_norm`` are the two norms behind).
"""
from __future__ import annotations

from typing import List

from ..config.base import LayerSpec
from ..weights.checkpoint import TensorSpec
from .base import Block, part_class, register_block


class PreNormBlock(Block):
    def __init__(self, spec: LayerSpec, runtime):
        super().__init__(spec, runtime)
        self.mixer_norm = part_class("norm", spec.mixer_norm.kind)(spec.mixer_norm, spec.prefix, runtime)
        self.mixer = part_class("mixer", spec.mixer.kind)(spec.mixer, spec.prefix, runtime)
        self.ffn_norm = part_class("norm", spec.ffn_norm.kind)(spec.ffn_norm, spec.prefix, runtime)
        self.ffn = part_class("ffn", spec.ffn.kind)(spec.ffn, spec.prefix, runtime)
        self.position = part_class("position", spec.position.kind)(spec.position, spec.prefix, runtime)

    @classmethod
    def declare(cls, spec: LayerSpec) -> List[TensorSpec]:
        out: List[TensorSpec] = []
        out += part_class("norm", spec.mixer_norm.kind).declare(spec.mixer_norm, spec.prefix)
        out += part_class("mixer", spec.mixer.kind).declare(spec.mixer, spec.prefix)
        out += part_class("norm", spec.ffn_norm.kind).declare(spec.ffn_norm, spec.prefix)
        out += part_class("ffn", spec.ffn.kind).declare(spec.ffn, spec.prefix)
        out += part_class("position", spec.position.kind).declare(spec.position, spec.prefix)
        return out

    def load(self, tensors) -> None:
        for part in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn, self.position):
            part.load(tensors)

    hands_off = True

    def accepts_incoming(self, tokens: int, batch):
        """A :class:`NormHandoff` of this block's first norm for the layer before to fill, or None."""
        if not self.mixer.accepts_handoff(tokens, self.position, batch):
            return None
        return self.mixer_norm.handoff(tokens)

    def fills_outgoing(self) -> bool:
        return self.ffn.fills_handoff

    def forward(self, x, batch, cache, state, reads_only: bool = False, incoming=None, outgoing=None) -> None:
        """With a few tokens a norm may be split between the product before it and the product after it, if all
        three can (see NormHandoff); otherwise it is a kernel of its own. ``incoming``: this block's first norm,
        filled by the layer before (``groups`` > 0) or not; ``outgoing``: the next layer's first norm, for this
        block's feed-forward to fill."""
        if incoming is not None and incoming.groups:
            h = None
            mixer_kwargs = {"incoming": incoming}
        else:
            h = self.mixer_norm.forward(x)
            mixer_kwargs = {}
        between = None
        if self.mixer.fills_handoff and self.ffn.accepts_handoff(x.shape[0]):
            between = self.ffn_norm.handoff(x.shape[0])
            if between is not None:
                mixer_kwargs["handoff"] = between
        self.mixer.forward(h, batch, cache, state, self.position, x, reads_only, **mixer_kwargs)
        ffn_kwargs = {"outgoing": outgoing} if outgoing is not None and self.ffn.fills_handoff else {}
        if between is not None and between.groups:
            self.ffn.forward(None, batch, x, handoff=between, **ffn_kwargs)
        else:
            h = self.ffn_norm.forward(x)
            self.ffn.forward(h, batch, x, **ffn_kwargs)


class ParallelBlock(Block):
    """``h = norm(x); x += mixer(h) + ffn(h)``: one norm, and both sublayers read its output.  The layer's norm is
    ``LayerSpec.mixer_norm``.  Where ``ffn_norm`` is another norm than ``mixer_norm`` (another tensor name) the
    feed-forward reads that one, of the same ``x``.  ``LayerSpec.params["residual_mult"]`` (1 unless given) multiplies the
    sublayers' sum: they then add into a 32-bit buffer of their own, which joins the stream in one step."""

    def __init__(self, spec: LayerSpec, runtime):
        super().__init__(spec, runtime)
        self.norm = part_class("norm", spec.mixer_norm.kind)(spec.mixer_norm, spec.prefix, runtime)
        self.mixer = part_class("mixer", spec.mixer.kind)(spec.mixer, spec.prefix, runtime)
        self.ffn = part_class("ffn", spec.ffn.kind)(spec.ffn, spec.prefix, runtime)
        self.position = part_class("position", spec.position.kind)(spec.position, spec.prefix, runtime)
        self.has_ffn = spec.ffn.kind != "none"
        self.ffn_norm = None
        if self._two_norms(spec):
            self.ffn_norm = part_class("norm", spec.ffn_norm.kind)(spec.ffn_norm, spec.prefix, runtime)
        self.mult = float(spec.params.get("residual_mult", 1.0))

    @staticmethod
    def _two_norms(spec: LayerSpec) -> bool:
        return spec.ffn.kind != "none" and spec.ffn_norm != spec.mixer_norm

    @classmethod
    def _families(cls, spec: LayerSpec):
        parts = [("norm", spec.mixer_norm), ("mixer", spec.mixer), ("ffn", spec.ffn), ("position", spec.position)]
        if cls._two_norms(spec):
            parts.append(("norm", spec.ffn_norm))
        return parts

    @classmethod
    def declare(cls, spec: LayerSpec) -> List[TensorSpec]:
        out: List[TensorSpec] = []
        for family, part in cls._families(spec):
            out += part_class(family, part.kind).declare(part, spec.prefix)
        if spec.ffn.kind == "none" and spec.ffn_norm != spec.mixer_norm:
            # a layer without a feed-forward does not read the norm in front of it; a folder that stores it all the
            # same is not refused for it
            out += [TensorSpec(t.name, t.shape, t.role, t.init, t.std, True)
                    for t in part_class("norm", spec.ffn_norm.kind).declare(spec.ffn_norm, spec.prefix)]
        return out

    @classmethod
    def check_supported(cls, spec: LayerSpec, dtype) -> None:
        for family, part in cls._families(spec):
            part_class(family, part.kind).check_supported(part, dtype)

    def load(self, tensors) -> None:
        for part in (self.norm, self.mixer, self.ffn, self.position, self.ffn_norm):
            if part is not None:
                part.load(tensors)

    def forward(self, x, batch, cache, state, reads_only: bool = False) -> None:
        if self.ffn_norm is not None and type(self.ffn_norm) is type(self.norm):
            h, h_ffn = self.norm.forward_with(self.ffn_norm, x)       # both norms of the same rows: one launch
        else:
            h = self.norm.forward(x)
            h_ffn = self.ffn_norm.forward(x) if self.ffn_norm is not None else h
        if self.mult == 1.0:
            # both sublayers add into the 32-bit residual; neither reads it after the norms, so their order does not matter
            self.mixer.forward(h, batch, cache, state, self.position, x, reads_only)
            self.ffn.forward(h_ffn, batch, x)
            return
        import torch
        from ..ops import kernels
        if self.mixer.can_overwrite:
            y = torch.empty_like(x)
            self.mixer.forward(h, batch, cache, state, self.position, y, reads_only, accumulate=False)
        else:
            y = torch.zeros_like(x)
            self.mixer.forward(h, batch, cache, state, self.position, y, reads_only)
        self.ffn.forward(h_ffn, batch, y)
        kernels.axpby(y, self.mult, y, 0.0, x, accumulate=True)      # x += m * y


class SandwichBlock(Block):
    """See the module's text.  A sublayer's output goes into a 32-bit buffer of its own (written, where the part can,
    instead of cleared and added to), is normed there and added to the stream by one kernel."""

    def __init__(self, spec: LayerSpec, runtime):
        super().__init__(spec, runtime)
        self.parts = {}
        for role, family, part in self._roles(spec):
            self.parts[role] = part_class(family, part.kind)(part, spec.prefix, runtime)
        self.mixer = self.parts["mixer"]
        self.has_ffn = spec.ffn.kind != "none"

    @classmethod
    def _roles(cls, spec: LayerSpec):
        roles = [("mixer_norm", "norm", spec.mixer_norm), ("mixer", "mixer", spec.mixer),
                 ("mixer_post_norm", "norm", spec.extras["mixer_post_norm"]), ("position", "position", spec.position)]
        if spec.ffn.kind != "none":
            roles += [("ffn_norm", "norm", spec.ffn_norm), ("ffn", "ffn", spec.ffn),
                      ("ffn_post_norm", "norm", spec.extras["ffn_post_norm"])]
        if "after" in spec.extras:
            roles.append(("after", "ffn", spec.extras["after"]))
        return roles

    @classmethod
    def declare(cls, spec: LayerSpec) -> List[TensorSpec]:
        out: List[TensorSpec] = []
        for _, family, part in cls._roles(spec):
            out += part_class(family, part.kind).declare(part, spec.prefix)
        if spec.ffn.kind == "none":
            # a layer without a feed-forward does not read the norms around it; a folder that stores them all the
            # same is not refused for it
            for norm in (spec.ffn_norm, spec.extras.get("ffn_post_norm")):
                if norm is not None:
                    out += [TensorSpec(t.name, t.shape, t.role, t.init, t.std, True)
                            for t in part_class("norm", norm.kind).declare(norm, spec.prefix)]
        return out

    @classmethod
    def check_supported(cls, spec: LayerSpec, dtype) -> None:
        for _, family, part in cls._roles(spec):
            part_class(family, part.kind).check_supported(part, dtype)

    def load(self, tensors) -> None:
        for part in self.parts.values():
            part.load(tensors)

    def forward(self, x, batch, cache, state, reads_only: bool = False) -> None:
        import torch
        parts = self.parts
        h = parts["mixer_norm"].forward(x)
        if parts["mixer"].can_overwrite:
            y = torch.empty_like(x)
            parts["mixer"].forward(h, batch, cache, state, parts["position"], y, reads_only, accumulate=False)
        else:
            y = torch.zeros_like(x)
            parts["mixer"].forward(h, batch, cache, state, parts["position"], y, reads_only)
        after = parts.get("after")
        feeds_after = after is not None and getattr(after, "reads_stream_input", False)
        if not self.has_ffn:
            stream = parts["mixer_post_norm"].add_into(y, x, as_input=feeds_after)
        else:
            # the norm behind the mixer and the one in front of the feed-forward: one launch where both are of a kind
            h = parts["mixer_post_norm"].add_into(y, x, follow=parts["ffn_norm"])
            if parts["ffn"].can_overwrite:
                parts["ffn"].forward(h, batch, y, accumulate=False)
            else:
                y.zero_()
                parts["ffn"].forward(h, batch, y)
            stream = parts["ffn_post_norm"].add_into(y, x, as_input=feeds_after)
        if after is not None:
            after.forward(stream if feeds_after else None, batch, x)


class PostNormBlock(Block):
    """``x += norm_1(mixer(x)); x += norm_2(ffn(x))``: nothing stands in front of a sublayer, which reads the 32-bit
    stream in the run's dtype; its output goes into a 32-bit buffer of its own and is normed there and added to the
    stream by one kernel, which also hands the new stream on in the run's dtype for the sublayer that follows (this
    layer's feed-forward, or the next layer's mixer through ``batch.shared``)."""

    STREAM_KEY = "postnorm.stream"     # (the stream tensor, its rows in the run's dtype) as the layer before left them

    def __init__(self, spec: LayerSpec, runtime):
        super().__init__(spec, runtime)
        self.mixer_post = part_class("norm", spec.mixer_norm.kind)(spec.mixer_norm, spec.prefix, runtime)
        self.mixer = part_class("mixer", spec.mixer.kind)(spec.mixer, spec.prefix, runtime)
        self.position = part_class("position", spec.position.kind)(spec.position, spec.prefix, runtime)
        self.has_ffn = spec.ffn.kind != "none"
        self.ffn = self.ffn_post = None
        if self.has_ffn:
            self.ffn = part_class("ffn", spec.ffn.kind)(spec.ffn, spec.prefix, runtime)
            self.ffn_post = part_class("norm", spec.ffn_norm.kind)(spec.ffn_norm, spec.prefix, runtime)

    @classmethod
    def _families(cls, spec: LayerSpec):
        parts = [("norm", spec.mixer_norm), ("mixer", spec.mixer), ("position", spec.position)]
        if spec.ffn.kind != "none":
            parts += [("ffn", spec.ffn), ("norm", spec.ffn_norm)]
        return parts

    @classmethod
    def declare(cls, spec: LayerSpec) -> List[TensorSpec]:
        out: List[TensorSpec] = []
        for family, part in cls._families(spec):
            out += part_class(family, part.kind).declare(part, spec.prefix)
        if spec.ffn.kind == "none":
            # a layer without a feed-forward does not read the norm behind it; a folder may hold it all the same
            out += [TensorSpec(t.name, t.shape, t.role, t.init, t.std, True)
                    for t in part_class("norm", spec.ffn_norm.kind).declare(spec.ffn_norm, spec.prefix)]
        return out

    @classmethod
    def check_supported(cls, spec: LayerSpec, dtype) -> None:
        for family, part in cls._families(spec):
            part_class(family, part.kind).check_supported(part, dtype)

    def load(self, tensors) -> None:
        for part in (self.mixer_post, self.mixer, self.position, self.ffn, self.ffn_post):
            if part is not None:
                part.load(tensors)

    def _as_input(self, x, batch):
        import torch
        from ..ops import kernels
        left = batch.shared.pop(self.STREAM_KEY, None)
        if left is not None and left[0] is x:
            return left[1]
        if self.runtime.dtype == torch.float32:
            return x
        h = self.runtime.empty(tuple(x.shape))
        kernels.activation(x, "none", h)            # a change of type
        return h

    def _sublayer(self, run, part, x):
        import torch
        if part.can_overwrite:
            y = torch.empty_like(x)
            run(y, {"accumulate": False})
        else:
            y = torch.zeros_like(x)
            run(y, {})
        return y

    def forward(self, x, batch, cache, state, reads_only: bool = False) -> None:
        h = self._as_input(x, batch)
        y = self._sublayer(lambda out, kw: self.mixer.forward(h, batch, cache, state, self.position, out, reads_only, **kw),
                           self.mixer, x)
        h = self.mixer_post.add_into(y, x, as_input=True)
        if self.has_ffn:
            y = self._sublayer(lambda out, kw: self.ffn.forward(h, batch, out, **kw), self.ffn, x)
            h = self.ffn_post.add_into(y, x, as_input=True)
        batch.shared[self.STREAM_KEY] = (x, h)


register_block("prenorm", PreNormBlock)
register_block("postnorm", PostNormBlock)
register_block("sandwich_norm", SandwichBlock)
register_block("parallel", ParallelBlock)
