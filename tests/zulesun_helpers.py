"""Small Zulesun configurations and model folders with the tests' own random weights.

The weights are drawn here with numpy (not by the engine's random-weights mode) at magnitudes that keep every
mechanism alive: step sizes and decays that neither freeze nor wipe the state, routers with clear preferences, norm
weights around zero.  Every value is rounded to bfloat16 before it is stored, so a 32-bit run, a bfloat16 run and the
plain implementation read the same numbers.
"""
from __future__ import annotations

import copy
import json
import os
from typing import Dict, List, Optional

import numpy as np
import torch


def lightning(heads, dim, vdim, decay=None):
    decay = list(decay) if decay is not None else [float(d) for d in np.linspace(0.55, 0.995, heads)]
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}}


def left(heads, kv_heads, dim, vdim, mask=None, rot_dims=None, base=10000.0, factor=None, scale=None, softcap=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "scale": float(scale if scale is not None else dim ** -0.5)}
    if mask:
        m["mask"] = {"size": mask}
    if rot_dims is None:
        rot_dims = dim
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
        if factor:
            m["rot"]["scaling"] = {"factor": factor}
    if softcap:
        m["softcap"] = softcap
    return m


def right(inner, state, dt_rank, conv):
    return {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}


def parallel(left_part, right_part, left_scale=1.0, right_scale=1.0):
    return {"type": "parallel", "mixer": {"left": left_part, "right": right_part, "left_scale": left_scale,
                                          "right_scale": right_scale}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, groups=None, keep=None):
    router = {"experts": experts, "top": top}
    if groups:
        router["groups"] = {"count": groups, "keep": keep if keep is not None else groups}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def config(vocab, width, layers, mlps, eps=1e-5, scale=None, side=None):
    out = {"architecture": "Zulesun", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "embedding": {"scale": float(scale if scale is not None else width ** 0.5)}, "layers": []}
    if side:
        out["token_side"] = {"dim": side}
    for layer, mlp in zip(layers, mlps):
        out["layers"].append(dict(copy.deepcopy(layer), mlp=copy.deepcopy(mlp)))
    return out


# Four layers of both kinds.  Values wider than keys in one attention and narrower in the other; blocks of 13 and 29
# positions (neither a multiple of a page); a partial rotation with scaled frequencies beside a full one without; a
# cap on the scores in one; three heads over one key head and four over two; two of three expert groups kept, and a
# mixture in which every expert is chosen; a layer without a feed-forward; unequal scales of the two sides.
Z1 = config(131, 48,
            [parallel(left(4, 2, 16, 24, mask=13, rot_dims=8, base=1000.0, factor=4.0, scale=0.3, softcap=5.0),
                      right(40, 12, 5, 3), 0.7, 1.3),
             lightning(3, 24, 8, [0.5, 0.9, 0.99]),
             parallel(left(3, 1, 24, 16, mask=29), right(24, 16, 4, 4), 1.5, 0.5),
             lightning(1, 40, 20, [0.97])],
            [moe(6, 2, 24, groups=3, keep=2), dense(40), None, moe(4, 4, 16)], side=6)
# Another order and widths that fit no fast path: nothing is a multiple of 8, the model's width not even of 4; no side
# table; an attention that sees everything and does not rotate; a convolution of one tap; as many key heads as heads;
# groups of one expert each.
Z2 = config(83, 50,
            [lightning(2, 10, 14), parallel(left(2, 2, 10, 6, rot_dims=0, scale=0.4), right(18, 5, 3, 1), 1.0, 1.0),
             parallel(left(3, 1, 6, 10, mask=7, rot_dims=4, base=50.0, factor=2.0, softcap=2.0), right(30, 20, 7, 2), 0.4, 2.0)],
            [moe(5, 2, 18, groups=5, keep=3), dense(22), moe(3, 1, 10)], eps=1e-6, scale=3.0)


def single(layer, mlp=None, vocab=97, width=64, **kw):
    """A model of one layer: a mechanism alone."""
    return config(vocab, width, [layer], [mlp], **kw)


def _bf16(a) -> torch.Tensor:
    return torch.from_numpy(np.asarray(a, dtype=np.float32)).to(torch.bfloat16)


def make_weights(cfg: dict, seed: int, sharp: float = 1.0) -> Dict[str, torch.Tensor]:
    """``sharp`` scales the weights of the query and key norms of attention layers (peaked attention weights)."""
    rng = np.random.default_rng(seed)
    W, L = cfg["width"], len(cfg["layers"])
    out: Dict[str, torch.Tensor] = {}

    def mat(rows, cols, gain=1.0):
        return _bf16(rng.standard_normal((rows, cols)) * gain / np.sqrt(cols))

    def around_zero(width):
        return _bf16(0.1 * rng.standard_normal(width))

    out["embed"] = _bf16(rng.standard_normal((cfg["vocab"], W)) / np.sqrt(W))
    side = (cfg.get("token_side") or {}).get("dim")
    if side:
        out["side.embed"] = _bf16(rng.standard_normal((cfg["vocab"], side * L)))
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}.mix."
        out[f"l{i}.norm1"], out[f"l{i}.norm1b"] = around_zero(W), around_zero(W)
        if layer["type"] == "lightning":
            H, D, V = m["heads"], m["dim"], m["vdim"]
            out[p + "q"], out[p + "k"] = mat(H * D, W, 1.5), mat(H * D, W, 1.5)
            out[p + "v"], out[p + "g"] = mat(H * V, W, 1.5), mat(H * V, W, 2.0)
            out[p + "o"] = mat(W, H * V)
            out[p + "norm"] = _bf16(1.0 + 0.1 * rng.standard_normal(H * V))
        else:
            a, q = m["left"], p + "left."
            H, G, D, V = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            out[q + "q"], out[q + "k"], out[q + "v"] = mat(H * D, W), mat(G * D, W), mat(G * V, W, 1.5)
            out[q + "q.norm"] = _bf16(sharp * (1.0 + 0.1 * rng.standard_normal(H * D)))
            out[q + "k.norm"] = _bf16(sharp * (1.0 + 0.1 * rng.standard_normal(G * D)))
            out[q + "g"], out[q + "o"] = mat(H * V, W, 2.0), mat(W, H * V)
            s, q = m["right"], p + "right."
            C, N, R, J = s["inner"], s["state"], s["dt_rank"], s["conv"]
            out[q + "in"] = mat(2 * C, W, 1.5)
            out[q + "conv"] = _bf16(rng.standard_normal((C, J)) * 0.6)
            out[q + "conv.b"] = _bf16(rng.standard_normal(C) * 0.2)
            out[q + "x"] = mat(R + 2 * N, C, 1.5)
            out[q + "dt"] = mat(C, R, 1.5)
            out[q + "dt.b"] = _bf16(rng.uniform(-2.5, 0.0, C))
            out[q + "A_log"] = _bf16(rng.uniform(-1.5, 1.0, (C, N)))
            out[q + "D"] = _bf16(rng.standard_normal(C) * 0.5)
            out[q + "o"] = mat(W, C)
        mlp = layer.get("mlp")
        if mlp is not None:
            out[f"l{i}.norm2"], out[f"l{i}.norm2b"] = around_zero(W), around_zero(W)
            q = f"l{i}.mlp."
            if mlp["kind"] == "dense":
                out[q + "up"], out[q + "down"] = mat(mlp["ff"], W, 1.5), mat(W, mlp["ff"])
            else:
                ff = mlp["expert"]["ff"]
                for e in range(mlp["router"]["experts"]):
                    out[f"{q}e{e}.gate"] = mat(ff, W, 1.5)
                    out[f"{q}e{e}.up"] = mat(ff, W, 1.5)
                    out[f"{q}e{e}.down"] = mat(W, ff)
                out[q + "router"] = mat(mlp["router"]["experts"], W, 2.0)
        if side:
            q = f"l{i}.side."
            out[q + "gate"], out[q + "proj"] = mat(side, W, 1.5), mat(W, side)
            out[q + "norm"] = _bf16(0.5 + 0.1 * rng.standard_normal(W))
    out["final.norm"] = around_zero(W)
    out["head"] = mat(cfg["vocab"], W)
    return out


def make_folder(path, cfg: dict, seed: int, dtype=torch.float32, sharp: float = 1.0, edit=None) -> str:
    """Write ``config.json`` and ``model.safetensors``; ``edit(tensors)`` may change the weights before."""
    from vipera_rs_amd.weights import write_safetensors

    path = str(path)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as handle:
        json.dump(cfg, handle)
    tensors = make_weights(cfg, seed, sharp)
    if edit is not None:
        edit(tensors)
    write_safetensors(os.path.join(path, "model.safetensors"), [(name, t.to(dtype)) for name, t in tensors.items()])
    return path


def load_folder(folder):
    """(configuration dict, tensors as float64 numpy arrays) of a model folder, for the plain implementation."""
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as handle:
        cfg = json.load(handle)
    w = {name: t.to(torch.float64).numpy() for name, t in load_file(os.path.join(folder, "model.safetensors")).items()}
    return cfg, w


def tokens_of(vocab: int, count: int, seed: int) -> List[int]:
    return [int(t) for t in np.random.default_rng(seed).integers(0, vocab, count)]


def clear_tokens(cfg: dict, w: dict, count: int, seed: int, gap: float = 0.2) -> List[int]:
    """Random tokens whose routing is no close call: wherever the plain implementation finds a token's router logits
    within ``gap`` of another choice of experts or groups, the token is drawn again (what comes before it does not
    change, so the sequence settles from the left).  A bfloat16 run then chooses as float64 does, and a difference
    between the two is a difference of the mechanisms.  A model without a mixture of experts gets plain random tokens."""
    from plain import zulesun_plain as P

    tokens = tokens_of(cfg["vocab"], count, seed)
    if not any((layer.get("mlp") or {}).get("kind") == "moe" for layer in cfg["layers"]):
        return tokens
    rng = np.random.default_rng(seed + 1000)
    for _ in range(200):
        gaps: list = []
        P.forward(cfg, w, tokens, gaps=gaps)
        close = np.nonzero(np.min(np.stack(gaps), axis=0) < gap)[0]
        if close.size == 0:
            return tokens
        tokens[int(close[0])] = int(rng.integers(0, cfg["vocab"]))
    raise AssertionError("no sequence with clear routing found")
