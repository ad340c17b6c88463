"""Zulesun: a decoder whose layers are listed one by one in its configuration (linear attention with a decay per head,
or softmax attention over blocks of positions beside a selective scan; a dense feed-forward or a mixture of experts
chosen within groups; a norm before and behind every sublayer; a per-token side table that every layer reads).

Everything specific to the architecture is in :class:`~vipera_rs_amd.config.ZulesunConfig`, which describes the
layers as data; the model itself is the generic decoder.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.zulesun import ZulesunConfig
from .decoder import DecoderModel


def build_zulesun(config: ZulesunConfig, runtime) -> DecoderModel:
    return DecoderModel(config, runtime)


register_architecture("Zulesun", ZulesunConfig, build_zulesun)
