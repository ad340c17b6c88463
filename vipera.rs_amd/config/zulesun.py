"""Configuration of the Zulesun decoder, read from its own ``config.json``.

The file lists the layers one by one: ``layers[i]`` has ``type`` (``lightning``: linear attention with a decay per head;
``parallel``: softmax attention over blocks of positions beside a selective scan), ``mixer`` (its sizes and constants)
and ``mlp`` (``{"kind": "dense", "ff"}``, ``{"kind": "moe", "expert": {"ff"}, "router": {"experts", "top", "groups":
{"count", "keep"}}}``, or null).  Beside the list stand ``vocab``, ``width``, ``norm.eps``, ``embedding.scale`` and
``token_side.dim`` (columns per layer of the per-token side table).  Every layer has an RMS norm (gain ``1 + w``) before
and behind each sublayer, and then adds its share of the side table.  Tensor names: ``embed``, ``side.embed``,
``l<i>.norm1 | norm1b | norm2 | norm2b``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``l<i>.side.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple

from ..errors import InvalidArgumentError, UnsupportedError
from .base import KeyReader, LayerSpec, ModelConfig, PartSpec

MIXER_TYPES = ("lightning", "parallel")
MLP_KINDS = ("dense", "moe")


def _sub(data: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    value = data.get(key)
    if not isinstance(value, dict):
        raise InvalidArgumentError(f"{where}: key \"{key}\" is {value!r}, expected an object")
    return value


def _optional(data: Dict[str, Any], key: str, where: str) -> Optional[Dict[str, Any]]:
    return _sub(data, key, where) if data.get(key) is not None else None


@dataclass
class ZulesunConfig(ModelConfig):
    vocab: int
    width: int
    eps: float
    embedding_scale: float
    side_dim: int                      # 0: the model has no per-token side table
    layers: List[Dict[str, Any]] = field(default_factory=list)
    max_positions: int = 1 << 20       # nothing learned or tabled bounds the context; a file may give "max_positions"
    eos_token_ids: Tuple[int, ...] = ()

    architecture = "Zulesun"

    # --- reading ----------------------------------------------------------------------
    @classmethod
    def from_dict(cls, data: Dict[str, Any]) -> "ZulesunConfig":
        r = KeyReader(data)
        layers = data.get("layers")
        if not isinstance(layers, list) or not all(isinstance(layer, dict) for layer in layers):
            raise InvalidArgumentError("config.json: key \"layers\" must be a list of objects, one per layer")
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else (eos,) if isinstance(eos, int) else tuple(eos)
        embedding = _optional(data, "embedding", "config.json")
        side = _optional(data, "token_side", "config.json")
        config = cls(
            vocab=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
            eps=KeyReader(_sub(data, "norm", "config.json"), "config.json: norm").number("eps"),
            embedding_scale=KeyReader(embedding, "config.json: embedding").number("scale", default=1.0) if embedding else 1.0,
            side_dim=KeyReader(side, "config.json: token_side").integer("dim", minimum=1) if side else 0,
            layers=copy.deepcopy(layers), max_positions=r.integer("max_positions", default=1 << 20, minimum=1),
            eos_token_ids=eos_ids)
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
            mixer = _sub(layer, "mixer", where)
            if kind == "lightning":
                self._check_lightning(mixer, where + ".mixer")
            else:
                self._check_attention(_sub(mixer, "left", where + ".mixer"), where + ".mixer.left")
                self._check_scan(_sub(mixer, "right", where + ".mixer"), where + ".mixer.right")
                scales = KeyReader(mixer, where + ".mixer")
                scales.number("left_scale", default=1.0)
                scales.number("right_scale", default=1.0)
            self._check_mlp(layer.get("mlp"), where)

    @staticmethod
    def _check_lightning(mixer: Dict[str, Any], where: str) -> None:
        r = KeyReader(mixer, where)
        heads = r.integer("heads", minimum=1)
        r.integer("dim", minimum=1)
        r.integer("vdim", minimum=1)
        decay = mixer.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or not all(
                isinstance(d, (int, float)) and not isinstance(d, bool) for d in decay):
            raise InvalidArgumentError(f"{where}: key \"decay\" is {decay!r}, expected one number per head ({heads})")

    @staticmethod
    def _check_attention(left: Dict[str, Any], where: str) -> None:
        r = KeyReader(left, where)
        heads, kv_heads = r.integer("heads", minimum=1), r.integer("kv_heads", minimum=1)
        if heads % kv_heads:
            raise InvalidArgumentError(f"{where}: \"heads\" {heads} is not a multiple of \"kv_heads\" {kv_heads}")
        dim = r.integer("dim", minimum=1)
        r.integer("vdim", minimum=1)
        r.number("scale")
        if r.has("softcap") and not r.number("softcap") >= 0:
            raise InvalidArgumentError(f"{where}: \"softcap\" must not be negative")
        mask = _optional(left, "mask", where)
        if mask is not None:
            KeyReader(mask, where + ".mask").integer("size", minimum=1)
        rot = _optional(left, "rot", where)
        if rot is not None:
            rr = KeyReader(rot, where + ".rot")
            dims = rr.integer("dims", minimum=0)
            if dims % 2 or dims > dim:
                raise InvalidArgumentError(f"{where}.rot: \"dims\" is {dims}; it must be even and at most \"dim\" {dim}")
            if dims and not rr.number("base") > 0:
                raise InvalidArgumentError(f"{where}.rot: \"base\" must be above 0")
            scaling = _optional(rot, "scaling", where + ".rot")
            if scaling is not None and not KeyReader(scaling, where + ".rot.scaling").number("factor", default=1.0) > 0:
                raise InvalidArgumentError(f"{where}.rot.scaling: \"factor\" must be above 0")

    @staticmethod
    def _check_scan(right: Dict[str, Any], where: str) -> None:
        r = KeyReader(right, where)
        for key in ("inner", "state", "dt_rank", "conv"):
            r.integer(key, minimum=1)

    @staticmethod
    def _check_mlp(mlp: Any, where: str) -> None:
        if mlp is None:
            return
        if not isinstance(mlp, dict) or mlp.get("kind") not in MLP_KINDS:
            raise UnsupportedError(f"{where}: mlp {mlp!r} is not implemented; \"kind\" {' or '.join(MLP_KINDS)}, or null")
        if mlp["kind"] == "dense":
            KeyReader(mlp, where + ".mlp").integer("ff", minimum=1)
            return
        KeyReader(_sub(mlp, "expert", where + ".mlp"), where + ".mlp.expert").integer("ff", minimum=1)
        router = KeyReader(_sub(mlp, "router", where + ".mlp"), where + ".mlp.router")
        experts, top = router.integer("experts", minimum=1), router.integer("top", minimum=1)
        if top > experts:
            raise InvalidArgumentError(f"{where}.mlp.router: \"top\" {top} is above \"experts\" {experts}")
        groups = _optional(router.data, "groups", where + ".mlp.router")
        if groups is not None:
            g = KeyReader(groups, where + ".mlp.router.groups")
            count = g.integer("count", minimum=1)
            keep = g.integer("keep", default=count, minimum=1)
            if experts % count or keep > count or keep * (experts // count) < top:
                raise InvalidArgumentError(f"{where}.mlp.router.groups: {keep} of {count} groups of {experts} experts "
                                           f"cannot give a token its {top}")

    def to_dict(self) -> Dict[str, Any]:
        data: Dict[str, Any] = {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
                                "layers": copy.deepcopy(self.layers), "norm": {"eps": self.eps}, "vocab": self.vocab,
                                "width": self.width}
        if self.side_dim:
            data["token_side"] = {"dim": self.side_dim}
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
    def _norm(self, name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"width": self.width, "eps": self.eps, "name": name, "tensor": name, "one_plus": True})

    def _lightning(self, m: Dict[str, Any], name: str) -> PartSpec:
        return PartSpec("decay_attention", {
            "hidden": self.width, "heads": int(m["heads"]), "dim": int(m["dim"]), "vdim": int(m["vdim"]),
            "decay": [float(d) for d in m["decay"]], "eps": self.eps, "activation": "silu", "gate": "sigmoid",
            "name": name})

    def _attention(self, m: Dict[str, Any], name: str) -> Tuple[PartSpec, PartSpec]:
        rot = m.get("rot") or {}
        dims = int(rot.get("dims") or 0)
        mixer = PartSpec("attention", {
            "hidden": self.width, "heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]), "head_dim": int(m["dim"]),
            "value_dim": int(m["vdim"]), "scale": float(m["scale"]), "softcap": float(m.get("softcap") or 0.0),
            "chunk": int((m.get("mask") or {}).get("size") or 0), "qk_norm": "whole", "gate": "sigmoid", "eps": self.eps,
            "tensors": {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g", "q_norm": "q.norm", "k_norm": "k.norm"},
            "name": name})
        position = PartSpec("none", {})
        if dims:
            position = PartSpec("rotary_neox", {
                "head_dim": int(m["dim"]), "rotary_dim": dims, "base": float(rot["base"]),
                "scaling_factor": float((rot.get("scaling") or {}).get("factor") or 1.0)})
        return mixer, position

    def _scan(self, m: Dict[str, Any], name: str) -> PartSpec:
        return PartSpec("selective_scan", {"hidden": self.width, "inner": int(m["inner"]), "state": int(m["state"]),
                                           "dt_rank": int(m["dt_rank"]), "conv": int(m["conv"]), "name": name})

    def _ffn(self, mlp: Optional[Dict[str, Any]]) -> PartSpec:
        if mlp is None:
            return PartSpec("none", {})
        if mlp["kind"] == "dense":
            return PartSpec("mlp", {"hidden": self.width, "intermediate": int(mlp["ff"]), "activation": "relu2",
                                    "name": "mlp"})
        router = mlp["router"]
        groups = router.get("groups") or {}
        count = int(groups.get("count") or 1)
        return PartSpec("moe", {"hidden": self.width, "intermediate": int(mlp["expert"]["ff"]),
                                "experts": int(router["experts"]), "top": int(router["top"]), "limit": None, "alpha": 1.0,
                                "groups": count, "keep": int(groups.get("keep") or count), "scores": "all", "name": "mlp"})

    def layer_specs(self) -> List[LayerSpec]:
        specs = []
        for index, layer in enumerate(self.layers):
            m = layer["mixer"]
            position = PartSpec("none", {})
            if layer["type"] == "lightning":
                mixer = self._lightning(m, "mix")
            else:
                left, position = self._attention(m["left"], "mix.left")
                mixer = PartSpec("mixer_pair", {"left": left, "right": self._scan(m["right"], "mix.right"),
                                                "left_scale": float(m.get("left_scale", 1.0)),
                                                "right_scale": float(m.get("right_scale", 1.0))})
            extras = {"mixer_post_norm": self._norm("norm1b"), "ffn_post_norm": self._norm("norm2b")}
            if self.side_dim:
                extras["after"] = PartSpec("token_side", {"hidden": self.width, "dim": self.side_dim, "index": index,
                                                          "eps": self.eps, "activation": "gelu_tanh", "name": "side"})
            specs.append(LayerSpec("sandwich_norm", mixer, self._ffn(layer.get("mlp")), self._norm("norm1"),
                                   self._norm("norm2"), position, f"l{index}.", extras))
        return specs

    def embedding_spec(self) -> PartSpec:
        params = {"vocab": self.vocab, "width": self.width, "name": "embed", "tensor": "embed",
                  "scale": self.embedding_scale}
        if self.side_dim:
            params["side"] = {"tensor": "side.embed", "width": self.side_dim * len(self.layers)}
        return PartSpec("embedding", params)

    def final_norm_spec(self) -> PartSpec:
        return self._norm("final.norm")

    def head_spec(self) -> PartSpec:
        return PartSpec("lm_head", {"vocab": self.vocab, "width": self.width, "name": "head", "tensor": "head",
                                    "tied_to": None})
