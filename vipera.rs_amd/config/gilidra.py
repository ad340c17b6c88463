"""Configuration of the Gilidra decoder, read from its own ``config.json``.

The file lists the layers one by one: ``layers[i]`` has ``type`` (which mixer: ``latent_attention``, ``delta`` or
``wkv``), ``mixer`` (its sizes and constants) and ``mlp`` (a mixture of experts, or null for none).  Beside the list
stand ``vocab``, ``width``, ``norm.eps`` and ``logit_scale``.  Every layer is a parallel block behind one Dynamic Tanh
norm; the embedding is followed by such a norm, and so is the last layer.  A latent-attention layer with ``kv_from: j``
keeps no cache of its own and reads layer ``j``'s.  Tensor names: ``embed``, ``embed.norm``, ``l<i>.norm1``,
``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple

from ..errors import InvalidArgumentError, UnsupportedError
from .base import KeyReader, LayerSpec, ModelConfig, PartSpec, ScheduleEntry

MIXER_TYPES = ("latent_attention", "delta", "wkv")


def _sub(data: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    value = data.get(key)
    if not isinstance(value, dict):
        raise InvalidArgumentError(f"{where}: key \"{key}\" is {value!r}, expected an object")
    return value


@dataclass
class GilidraConfig(ModelConfig):
    vocab: int
    width: int
    eps: float
    logit_scale: float
    layers: List[Dict[str, Any]] = field(default_factory=list)
    max_positions: int = 1 << 20       # no learned or tabled positions bound the context; a file may give "max_positions"
    eos_token_ids: Tuple[int, ...] = ()

    architecture = "Gilidra"

    # --- reading ----------------------------------------------------------------------
    @classmethod
    def from_dict(cls, data: Dict[str, Any]) -> "GilidraConfig":
        r = KeyReader(data)
        layers = data.get("layers")
        if not isinstance(layers, list) or not all(isinstance(layer, dict) for layer in layers):
            raise InvalidArgumentError("config.json: key \"layers\" must be a list of objects, one per layer")
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else (eos,) if isinstance(eos, int) else tuple(eos)
        config = cls(vocab=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
                     eps=KeyReader(_sub(data, "norm", "config.json"), "config.json: norm").number("eps"),
                     logit_scale=r.number("logit_scale", default=1.0), layers=copy.deepcopy(layers),
                     max_positions=r.integer("max_positions", default=1 << 20, minimum=1), eos_token_ids=eos_ids)
        config.validate()
        return config

    def validate(self) -> None:
        if not self.eps >= 0.0:
            raise InvalidArgumentError(f"config.json: norm: key \"eps\" is {self.eps!r}, expected a number at or above 0")
        for index, layer in enumerate(self.layers):
            where = f"config.json: layers[{index}]"
            kind = layer.get("type")
            if kind not in MIXER_TYPES:
                raise UnsupportedError(f"{where}: type {kind!r} is not implemented; known: {', '.join(MIXER_TYPES)}")
            mixer = KeyReader(_sub(layer, "mixer", where), where + ".mixer")
            if kind == "latent_attention":
                for key in ("heads", "dim", "vdim", "q_rank", "kv_rank"):
                    mixer.integer(key, minimum=1)
                rot = mixer.integer("rot_dim", minimum=0)
                mixer.number("scale")
                if rot:
                    rotation = KeyReader(_sub(mixer.data, "rot", where + ".mixer"), where + ".mixer.rot")
                    dims = rotation.integer("dims", minimum=0)
                    if dims % 2 or dims > rot:
                        raise InvalidArgumentError(f"{where}.mixer.rot: \"dims\" is {dims}; it must be even and at most "
                                                   f"\"rot_dim\" {rot}")
                    if not rotation.number("base") > 0:
                        raise InvalidArgumentError(f"{where}.mixer.rot: \"base\" must be above 0")
                if mixer.has("kv_from"):
                    source = mixer.integer("kv_from")
                    owner = self.layers[source] if source < index else None
                    if owner is None or owner.get("type") != "latent_attention" or owner["mixer"].get("kv_from") is not None:
                        raise InvalidArgumentError(f"{where}.mixer: \"kv_from\" is {source}; it must name an earlier "
                                                   "latent-attention layer that has a cache of its own")
                    for key in ("kv_rank", "rot_dim"):
                        if owner["mixer"].get(key) != mixer.data.get(key):
                            raise InvalidArgumentError(f"{where}.mixer: \"{key}\" differs from layer {source}'s, whose "
                                                       "cache this layer reads")
            elif kind == "delta":
                heads, kv_heads = mixer.integer("heads", minimum=1), mixer.integer("kv_heads", minimum=1)
                if heads % kv_heads:
                    raise InvalidArgumentError(f"{where}.mixer: \"heads\" {heads} is not a multiple of \"kv_heads\" {kv_heads}")
                for key in ("dim", "vdim", "conv"):
                    mixer.integer(key, minimum=1)
            else:
                mixer.integer("heads", minimum=1)
                mixer.integer("dim", minimum=1)
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind", "moe") != "moe":
                    raise UnsupportedError(f"{where}: mlp {mlp!r} is not implemented; a mixture of experts (\"kind\": "
                                           "\"moe\") or null")
                expert = KeyReader(_sub(mlp, "expert", where + ".mlp"), where + ".mlp.expert")
                router = KeyReader(_sub(mlp, "router", where + ".mlp"), where + ".mlp.router")
                expert.integer("ff", minimum=1)
                expert.number("limit")
                experts, top = router.integer("experts", minimum=1), router.integer("top", minimum=1)
                if top > experts:
                    raise InvalidArgumentError(f"{where}.mlp.router: \"top\" {top} is above \"experts\" {experts}")

    def to_dict(self) -> Dict[str, Any]:
        data: Dict[str, Any] = {"architecture": self.architecture, "layers": copy.deepcopy(self.layers),
                                "logit_scale": self.logit_scale, "norm": {"eps": self.eps}, "vocab": self.vocab,
                                "width": self.width}
        if self.max_positions != 1 << 20:
            data["max_positions"] = self.max_positions
        if self.eos_token_ids:
            data["eos_token_id"] = list(self.eos_token_ids)
        return data

    @property
    def context_limit(self) -> int:
        return int(self.max_positions)

    # --- for callers that ask a configuration for its sizes by the common names ---------------------
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    # --- the description the generic decoder consumes ---------------------------------------
    @staticmethod
    def _window(mixer: Dict[str, Any]) -> int:
        mask = mixer.get("mask")
        return int(mask.get("size") or 0) if isinstance(mask, dict) else 0

    def _retained(self, owner: int) -> int:
        """Positions that layer ``owner``'s cache must keep: the widest window among the layers that read it (0: all)."""
        windows = [self._window(layer["mixer"]) for index, layer in enumerate(self.layers)
                   if layer["type"] == "latent_attention" and (index == owner or layer["mixer"].get("kv_from") == owner)]
        return 0 if min(windows) == 0 else max(windows)

    def _norm(self, name: str) -> PartSpec:
        return PartSpec("dyt", {"width": self.width, "eps": self.eps, "name": name})

    def layer_specs(self) -> List[LayerSpec]:
        specs = []
        for index, layer in enumerate(self.layers):
            kind, m = layer["type"], layer["mixer"]
            position = PartSpec("none", {})
            if kind == "latent_attention":
                source = m.get("kv_from")
                rot = int(m["rot_dim"])
                mixer = PartSpec("latent_attention", {
                    "hidden": self.width, "heads": int(m["heads"]), "dim": int(m["dim"]), "rot_dim": rot,
                    "vdim": int(m["vdim"]), "q_rank": int(m["q_rank"]), "kv_rank": int(m["kv_rank"]),
                    "scale": float(m["scale"]), "window": self._window(m),
                    "retain": self._retained(index if source is None else int(source)), "eps": self.eps,
                    "shares_cache": source is not None, "name": "mix"})
                if rot and int(m["rot"]["dims"]):
                    position = PartSpec("rotary_neox", {"head_dim": rot, "rotary_dim": int(m["rot"]["dims"]),
                                                        "base": float(m["rot"]["base"])})
            elif kind == "delta":
                mixer = PartSpec("gated_delta", {
                    "hidden": self.width, "heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]), "dim": int(m["dim"]),
                    "vdim": int(m["vdim"]), "conv": int(m["conv"]), "eps": self.eps, "name": "mix"})
            else:
                mixer = PartSpec("wkv", {"hidden": self.width, "heads": int(m["heads"]), "dim": int(m["dim"]),
                                         "decay_rank": int(m.get("decay_rank") or 0), "eps": self.eps, "name": "mix"})
            mlp = layer.get("mlp")
            if mlp is None:
                ffn = PartSpec("none", {})
            else:
                ffn = PartSpec("moe", {"hidden": self.width, "intermediate": int(mlp["expert"]["ff"]),
                                       "experts": int(mlp["router"]["experts"]), "top": int(mlp["router"]["top"]),
                                       "limit": float(mlp["expert"]["limit"]), "alpha": 1.702, "name": "mlp"})
            norm = self._norm("norm1")
            specs.append(LayerSpec("parallel", mixer, ffn, norm, norm, position, f"l{index}."))
        return specs

    def schedule(self) -> List[ScheduleEntry]:
        return [ScheduleEntry(index, layer["mixer"].get("kv_from") if layer["type"] == "latent_attention" else None)
                for index, layer in enumerate(self.layers)]

    def embedding_spec(self) -> PartSpec:
        return PartSpec("embedding", {"vocab": self.vocab, "width": self.width, "name": "embed", "tensor": "embed",
                                      "norm": self._norm("embed.norm")})

    def final_norm_spec(self) -> PartSpec:
        return self._norm("final.norm")

    def head_spec(self) -> PartSpec:
        return PartSpec("lm_head", {"vocab": self.vocab, "width": self.width, "name": "head", "tensor": "head",
                                    "tied_to": None, "scale": self.logit_scale})
