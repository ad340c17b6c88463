"""Small Gilidra configurations and model folders with the tests' own random weights.

The weights are drawn here with numpy (not by the engine's random-weights mode) at magnitudes that keep every
mechanism alive: decays between 0.5 and 0.97, routers with clear preferences, norms near one.  Every value is
rounded to bfloat16 before it is stored, so a 32-bit run, a bfloat16 run and the plain implementation read the
same numbers.
"""
from __future__ import annotations

import copy
import json
import os
from typing import Dict, List

import numpy as np
import torch


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, window=None, kv_from=None, rot_dims=None, base=10000.0, scale=None):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
             "rot": {"base": base, "dims": rot_dim if rot_dims is None else rot_dims},
             "scale": float(scale if scale is not None else (dim + rot_dim) ** -0.5)}
    if window:
        mixer["mask"] = {"size": window}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mixer}


def delta(heads, kv_heads, dim, vdim, conv):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def wkv(heads, dim, decay_rank):
    # `decay_rank` is for the weight maker only: the engine takes it from the tensor's shape
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim}, "_decay_rank": decay_rank}


def moe(experts, top, ff, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def config(vocab, width, layers, mlps, eps=1e-5, logit_scale=None):
    out = {"architecture": "Gilidra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": []}
    if logit_scale is not None:
        out["logit_scale"] = logit_scale
    for layer, mlp in zip(layers, mlps):
        out["layers"].append(dict(copy.deepcopy(layer), mlp=copy.deepcopy(mlp)))
    return out


# Five layers of all three mixers; the two latent layers share one cache and have different windows; heads, key
# heads, key and value widths all differ; one layer has no feed-forward.
G1 = config(211, 96,
            [latent(3, 16, 8, 24, 40, 56, window=13), wkv(3, 16, 8), delta(4, 2, 16, 24, 4),
             latent(2, 24, 8, 16, 32, 56, window=29, kv_from=0), delta(2, 2, 32, 16, 2)],
            [moe(5, 2, 32, 1.5), moe(5, 2, 32, 1.5), None, moe(6, 3, 16, 0.75), moe(5, 1, 32, 1.5)], logit_scale=0.5)
# Another order; a latent layer that sees everything beside a windowed one that reads its cache; a partial rotation;
# a convolution of one tap; one head; no logit scale.
G2 = config(157, 64,
            [delta(1, 1, 24, 40, 1), latent(4, 8, 16, 8, 24, 40, rot_dims=8, base=500.0), wkv(1, 32, 4),
             latent(4, 8, 16, 8, 24, 40, window=7, kv_from=1, rot_dims=8, base=500.0), wkv(4, 8, 12)],
            [moe(3, 3, 24, 2.0), None, moe(4, 2, 40, 0.5), moe(3, 3, 24, 2.0), None], eps=1e-6)


def single(layer, mlp=None, vocab=97, width=64, **kw):
    """A model of one layer: a mechanism alone."""
    return config(vocab, width, [layer], [mlp], **kw)


def _bf16(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.asarray(a, dtype=np.float32)).to(torch.bfloat16)


def make_weights(cfg: dict, seed: int, sharp: float = 1.0) -> Dict[str, torch.Tensor]:
    """``sharp`` scales the query and key up-projections of latent layers (peaked attention weights)."""
    rng = np.random.default_rng(seed)
    W = cfg["width"]
    out: Dict[str, torch.Tensor] = {}

    def mat(rows, cols, gain=1.0):
        return _bf16(rng.standard_normal((rows, cols)) * gain / np.sqrt(cols))

    def norm(name, width):
        out[name] = _bf16(1.0 + 0.1 * rng.standard_normal(width))
        out[name + ".b"] = _bf16(0.1 * rng.standard_normal(width))
        out[name + ".alpha"] = _bf16(np.array(rng.uniform(0.5, 1.2)))

    out["embed"] = _bf16(rng.standard_normal((cfg["vocab"], W)))
    norm("embed.norm", W)
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}.mix."
        norm(f"l{i}.norm1", W)
        if layer["type"] == "latent_attention":
            H, D, R, V, QR, KR = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            out[p + "dq"] = mat(QR, W)
            out[p + "dq.norm"] = _bf16(1.0 + 0.1 * rng.standard_normal(QR))
            out[p + "uq"] = mat(H * (D + R), QR, sharp)
            if m.get("kv_from") is None:
                out[p + "dkv"] = mat(KR + R, W, 1.5)
                out[p + "dkv.norm"] = _bf16(1.0 + 0.1 * rng.standard_normal(KR))
            out[p + "uk"] = mat(H * D, KR, sharp)
            out[p + "uv"] = mat(H * V, KR)
            out[p + "o"] = mat(W, H * V)
        elif layer["type"] == "delta":
            H, G, D, V, J = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            for name, rows in (("q", G * D), ("k", G * D), ("v", H * V)):
                out[p + name] = mat(rows, W, 1.5)
                out[f"{p}{name}.conv"] = _bf16(rng.standard_normal((rows, J)) * 0.6)
            out[p + "b"] = mat(H, W, 2.0)
            out[p + "a"] = mat(H, W, 1.0)
            out[p + "A_log"] = _bf16(rng.uniform(-3.0, -0.5, H))
            out[p + "dt_bias"] = _bf16(rng.standard_normal(H) * 0.5)
            out[p + "norm"] = _bf16(1.0 + 0.1 * rng.standard_normal(V))
            out[p + "g"] = mat(H * V, W)
            out[p + "o"] = mat(W, H * V)
        else:
            H, D, rank = m["heads"], m["dim"], layer["_decay_rank"]
            for s in "rkvgw":
                out[f"{p}mu.{s}"] = _bf16(rng.uniform(0.0, 1.0, W))
            for s in "rkvg":
                out[p + s] = mat(H * D, W)
            out[p + "w1"] = mat(rank, W)
            out[p + "w2"] = mat(H * D, rank)
            out[p + "w0"] = _bf16(rng.uniform(-3.0, -0.5, H * D))
            out[p + "u"] = _bf16(rng.standard_normal((H, D)) * 0.5)
            out[p + "norm"] = _bf16(1.0 + 0.1 * rng.standard_normal(H * D))
            out[p + "o"] = mat(W, H * D)
        mlp = layer.get("mlp")
        if mlp is not None:
            q = f"l{i}.mlp."
            ff = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                out[f"{q}e{e}.gate"] = mat(ff, W, 1.5)
                out[f"{q}e{e}.up"] = mat(ff, W, 1.5)
                out[f"{q}e{e}.down"] = mat(W, ff)
            out[q + "router"] = mat(mlp["router"]["experts"], W, 2.0)
    norm("final.norm", W)
    out["head"] = mat(cfg["vocab"], W)
    return out


def written_config(cfg: dict) -> dict:
    """The configuration as a file holds it: without the weight maker's own keys."""
    clean = copy.deepcopy(cfg)
    for layer in clean["layers"]:
        layer.pop("_decay_rank", None)
    return clean


def make_folder(path, cfg: dict, seed: int, dtype=torch.float32, sharp: float = 1.0, edit=None) -> str:
    """Write ``config.json`` and ``model.safetensors``; ``edit(tensors)`` may change the weights before."""
    from vipera_rs_amd.weights import write_safetensors

    path = str(path)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as handle:
        json.dump(written_config(cfg), handle)
    tensors = make_weights(cfg, seed, sharp)
    if edit is not None:
        edit(tensors)
    write_safetensors(os.path.join(path, "model.safetensors"), [(name, t.to(dtype)) for name, t in tensors.items()])
    return path


def tokens_of(vocab: int, count: int, seed: int) -> List[int]:
    return [int(t) for t in np.random.default_rng(seed).integers(0, vocab, count)]
