"""Gilidra: a decoder whose layers are listed one by one in its configuration (latent attention with a window,
the gated delta rule, RWKV-style time mixing; a mixture of experts beside each; Dynamic Tanh norms).

Everything specific to the architecture is in :class:`~vipera_rs_amd.config.GilidraConfig`, which describes the
layers as data; the model itself is the generic decoder.
"""
from __future__ import annotations

from ..config.gilidra import GilidraConfig
from ..config.registry import register_architecture
from .decoder import DecoderModel


def build_gilidra(config: GilidraConfig, runtime) -> DecoderModel:
    return DecoderModel(config, runtime)


register_architecture("Gilidra", GilidraConfig, build_gilidra)
