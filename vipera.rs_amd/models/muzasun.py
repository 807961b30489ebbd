"""Muzasun: a decoder whose layers are listed one by one in its configuration (softmax attention with a norm per head
and values blended across layers, the matrix memory with exponential gates, the gated delta rule with a decay per key
channel; a dense or mixed feed-forward beside each, behind a Dynamic Tanh norm of its own).

Everything specific to the architecture is in :class:`~vipera_rs_amd.config.MuzasunConfig`, which describes the
layers as data; the model itself is the generic decoder.
"""
from __future__ import annotations

from ..config.muzasun import MuzasunConfig
from ..config.registry import register_architecture
from .decoder import DecoderModel


def build_muzasun(config: MuzasunConfig, runtime) -> DecoderModel:
    return DecoderModel(config, runtime)


register_architecture("Muzasun", MuzasunConfig, build_muzasun)
