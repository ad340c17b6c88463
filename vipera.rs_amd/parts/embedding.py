"""Token embedding and the output projection.

Reference: the embedding is a row read with no scaling (crates/vipera-backend-cpu/src/model.rs:607-616);
the head is ``logits = Wout h`` on the normed rows that are wanted, and when the model has no output
matrix the embedding table serves as one (model.rs:425, 1201-1237).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..config.base import PartSpec
from ..ops import kernels
from ..ops.linear import linear
from ..errors import InvalidArgumentError
from ..weights.checkpoint import MATRIX, VECTOR, TensorSpec
from .base import FeedForward, Part, part_class, register_embedding, register_ffn, register_head


def _tensor_name(spec: PartSpec, prefix: str) -> str:
    """``params["tensor"]`` names the matrix outright; otherwise it is ``<name>.weight``."""
    return f"{prefix}{spec.params['tensor']}" if spec.params.get("tensor") else f"{prefix}{spec.params['name']}.weight"


SIDE_ROWS = "token_side_rows"   # key in ``batch.shared``: the step's rows of the per-token side table, 32-bit


class Embedding(Part):
    """``params``: ``vocab``, ``width``, ``name`` / ``tensor``, ``norm`` (a norm right after the table), ``scale`` (the
    rows are multiplied by it), ``side`` (``{"tensor": name, "width": columns}``: a second table with a row per token id,
    whose rows for the step's tokens are gathered once a step and left in ``batch.shared`` for the layers that read
    their own columns of it, see :class:`TokenSide`)."""

    reads_device_tokens = True  # forward() takes (source, sampled): ids may be read from the device

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        self.vocab = int(spec.params["vocab"])
        self.width = int(spec.params["width"])
        self.table: Optional[torch.Tensor] = None
        # a norm right after the table (``params["norm"]``, a PartSpec of a registered norm): the residual starts
        # as its 32-bit output
        norm = spec.params.get("norm")
        self.norm = part_class("norm", norm.kind)(norm, prefix, runtime) if norm is not None else None
        scale = spec.params.get("scale")
        self.scale = float(scale) if scale is not None else 1.0
        self.side = spec.params.get("side")
        self.side_table: Optional[torch.Tensor] = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        specs = [TensorSpec(_tensor_name(spec, prefix), (int(spec.params["vocab"]), int(spec.params["width"])), MATRIX)]
        side = spec.params.get("side")
        if side is not None:
            specs.append(TensorSpec(f"{prefix}{side['tensor']}", (int(spec.params["vocab"]), int(side["width"])), MATRIX))
        norm = spec.params.get("norm")
        if norm is not None:
            specs += part_class("norm", norm.kind).declare(norm, prefix)
        return specs

    @classmethod
    def check_supported(cls, spec: PartSpec, dtype) -> None:
        norm = spec.params.get("norm")
        if norm is not None:
            part_class("norm", norm.kind).check_supported(norm, dtype)

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.table = tensors[_tensor_name(self.spec, self.prefix)]
        if self.side is not None:
            self.side_table = tensors[f"{self.prefix}{self.side['tensor']}"]
        if self.norm is not None:
            self.norm.load(tensors)

    def embed(self, batch) -> torch.Tensor:
        """The 32-bit residual ``[tokens, width]`` a step starts from.  An embedding sees the whole batch, so one
        that adds something by position (``batch.positions``) needs nothing else."""
        device_ids = (batch.token_source, batch.sampled_tokens) \
            if batch.sampled_tokens is not None and batch.token_source is not None else ()  # ids the sampler left on the device
        if self.side_table is not None:
            rows = self.runtime.empty((batch.num_tokens, self.side_table.shape[1]), torch.float32)
            kernels.embed_gather(self.side_table, batch.tokens, rows, *device_ids)
            batch.shared[SIDE_ROWS] = rows
        return self.forward(batch.tokens, batch.num_tokens, *device_ids)

    def forward(self, tokens: torch.Tensor, count: int, source: Optional[torch.Tensor] = None,
                sampled: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Rows of the table for ``tokens``; where ``source`` is not negative the id is read from
        ``sampled`` on the device instead (see ``kernels.embed_gather``)."""
        out = self.runtime.empty((count, self.width), torch.float32)
        kernels.embed_gather(self.table, tokens, out, source, sampled)
        if self.scale != 1.0:
            kernels.scale_(out, self.scale)
        if self.norm is not None:
            out = self.norm.forward(out, out=self.runtime.empty((count, self.width), torch.float32))
        return out


class TokenSide(FeedForward):
    """What a layer adds to the stream from its own columns of the per-token side table (see :class:`Embedding`):
    ``e = side[token][index * dim : (index + 1) * dim]``, ``g = gelu_tanh(Wgate x) * e``, ``y = Wproj g``,
    ``x += y / rms(y) * norm``.  It reads the stream ``x`` itself: ``h`` is the stream in the run's dtype if the block
    has it at hand (``reads_stream_input``), else it is made here.  ``params``: ``hidden``,
    ``dim``, ``index``, ``eps``, ``activation`` ("gelu_tanh" unless given), ``name``; tensors ``<name>.gate | proj | norm``."""

    reads_stream_input = True     # forward's ``h`` may be the residual itself in the run's dtype

    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        p = spec.params
        self.hidden, self.dim, self.index, self.eps = int(p["hidden"]), int(p["dim"]), int(p["index"]), float(p["eps"])
        self.activation = p.get("activation", "gelu_tanh")
        self.w_gate = self.w_proj = self.norm = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        p = spec.params
        base = f"{prefix}{p['name']}."
        hidden, dim = int(p["hidden"]), int(p["dim"])
        return [TensorSpec(base + "gate", (dim, hidden), MATRIX), TensorSpec(base + "proj", (hidden, dim), MATRIX),
                TensorSpec(base + "norm", (hidden,), VECTOR, "one_plus_normal")]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        base = f"{self.prefix}{self.spec.params['name']}."
        self.w_gate, self.w_proj, self.norm = tensors[base + "gate"], tensors[base + "proj"], tensors[base + "norm"]

    def forward(self, h, batch, residual, **_unused) -> None:
        tokens = residual.shape[0]
        rows = batch.shared.get(SIDE_ROWS)
        if rows is None or rows.shape[1] < (self.index + 1) * self.dim:
            raise InvalidArgumentError("token_side: the embedding has left no side rows for this layer in the step")
        x = h if h is not None else residual
        if h is None and self.runtime.dtype != torch.float32:
            x = self.runtime.empty((tokens, self.hidden))
            kernels.activation(residual, "none", x)
        gate = torch.empty((tokens, self.dim), dtype=torch.float32, device=residual.device)
        linear(x, self.w_gate, None, gate)
        gated = self.runtime.empty((tokens, self.dim))
        kernels.activation(gate, self.activation, gated, mul=rows[:, self.index * self.dim:(self.index + 1) * self.dim])
        y = torch.empty((tokens, self.hidden), dtype=torch.float32, device=residual.device)
        linear(gated, self.w_proj, None, y)
        kernels.rmsnorm_add(y, self.norm, self.eps, residual)


class LMHead(Part):
    def __init__(self, spec: PartSpec, prefix: str, runtime):
        super().__init__(spec, prefix, runtime)
        self.vocab = int(spec.params["vocab"])
        self.width = int(spec.params["width"])
        self.tied_to = spec.params.get("tied_to")
        scale = spec.params.get("scale")
        self.scale = float(scale) if scale is not None else 1.0     # logits = (W h) * scale
        self.weight: Optional[torch.Tensor] = None

    @classmethod
    def declare(cls, spec: PartSpec, prefix: str) -> List[TensorSpec]:
        # With tied embeddings the output matrix is optional: a folder that holds one has it used, as the reference
        # uses `output.weight` whenever the file has it and the embedding table only otherwise (model.rs:424-425).
        return [TensorSpec(_tensor_name(spec, prefix),
                           (int(spec.params["vocab"]), int(spec.params["width"])), MATRIX,
                           optional=bool(spec.params.get("tied_to")))]

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        own = _tensor_name(self.spec, self.prefix)
        if self.tied_to and own not in tensors:
            self.weight = tensors[f"{self.tied_to}.weight"]  # tied: the same buffer, no copy
        else:
            self.weight = tensors[own]

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        logits = self.runtime.empty((h.shape[0], self.vocab), torch.float32)
        linear(h, self.weight, None, logits)
        if self.scale != 1.0:
            kernels.scale_(logits, self.scale)
        return logits


register_embedding("embedding", Embedding)
register_ffn("token_side", TokenSide)
register_head("lm_head", LMHead)
