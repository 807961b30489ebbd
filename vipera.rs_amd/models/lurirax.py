"""Lurirax: a decoder whose layers are listed one by one in its configuration (softmax attention in a sliding window
with a sink; differential attention; attention within chunks, biased by distance, beside retention; a dense gated
feed-forward or a mixture of experts steered by a correction, with a gated shared expert; a norm behind every
sublayer).

Everything specific to the architecture is in :class:`~vipera_rs_amd.config.LuriraxConfig`, which describes the
layers as data; the model itself is the generic decoder.
"""
from __future__ import annotations

from ..config.lurirax import LuriraxConfig
from ..config.registry import register_architecture
from .decoder import DecoderModel


def build_lurirax(config: LuriraxConfig, runtime) -> DecoderModel:
    return DecoderModel(config, runtime)


register_architecture("Lurirax", LuriraxConfig, build_lurirax)
