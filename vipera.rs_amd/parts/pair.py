"""Two mixers side by side: both read the same input, and the layer's output is a weighted sum of theirs.

``params``: ``left`` and ``right`` (the two mixers' ``PartSpec``), ``left_scale`` and ``right_scale``.  What the two
keep per request is kept side by side: pages of keys and values from the one that has them (at most one of the two
may), fixed-size state from either or both (one row per request, the left one's numbers first).  The two outputs are
computed into 32-bit buffers of their own and added with their scales by one kernel, so neither product's rounding
depends on the other's.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from ..config.base import PartSpec
from ..errors import UnsupportedError
from ..ops import kernels
from ..weights.checkpoint import TensorSpec
from .base import Mixer, StateSpec, part_class, register_mixer


class MixerPair(Mixer):
    can_overwrite = True

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        p = spec.params
        self.left = part_class("mixer", p["left"].kind)(p["left"], prefix, runtime)
        self.right = part_class("mixer", p["right"].kind)(p["right"], prefix, runtime)
        self.left_scale, self.right_scale = float(p.get("left_scale", 1.0)), float(p.get("right_scale", 1.0))
        left_state = self.left.state_spec()
        self.left_floats = int(left_state.shape[0]) if left_state is not None else 0

    @classmethod
    def _halves(cls, spec: PartSpec):
        return [(side, part_class("mixer", side.kind)) for side in (spec.params["left"], spec.params["right"])]

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        return [t for side, kind in cls._halves(spec) for t in kind.declare(side, prefix)]

    @classmethod
    def declare_cache(cls, spec: PartSpec):
        kv, floats = None, 0
        for side, kind in cls._halves(spec):
            side_kv, side_state = kind.declare_cache(side)
            if side_kv is not None:
                if kv is not None:
                    raise UnsupportedError("mixer_pair: both mixers keep pages of keys and values; one of them may")
                kv = side_kv
            if side_state is not None:
                if len(side_state.shape) != 1 or side_state.dtype != torch.float32:
                    raise UnsupportedError("mixer_pair: a mixer's state must be one row of 32-bit numbers")
                floats += int(side_state.shape[0])
        return kv, (StateSpec((floats,), torch.float32) if floats else None)

    @classmethod
    def check_supported(cls, spec: PartSpec, dtype: torch.dtype) -> None:
        for side, kind in cls._halves(spec):
            kind.check_supported(side, dtype)
        cls.declare_cache(spec)

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.left.load(tensors)
        self.right.load(tensors)

    def forward(self, h, batch, cache, state, position, residual, reads_only: bool = False, accumulate: bool = True) -> None:
        outs = []
        for mixer, first in ((self.left, 0), (self.right, self.left_floats)):
            own = mixer.state_spec()
            view = state[:, first:first + int(own.shape[0])] if own is not None else None
            if mixer.can_overwrite:
                out = torch.empty_like(residual)
                mixer.forward(h, batch, cache, view, position, out, reads_only, accumulate=False)
            else:
                out = torch.zeros_like(residual)
                mixer.forward(h, batch, cache, view, position, out, reads_only)
            outs.append(out)
        kernels.axpby(outs[0], self.left_scale, outs[1], self.right_scale, residual, accumulate)


register_mixer("mixer_pair", MixerPair)
