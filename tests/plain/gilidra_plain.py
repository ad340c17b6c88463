"""A plain, slow implementation of the Gilidra decoder in float64 numpy: one function per mechanism, whole
sequences only (no cache, no state passing, no batching).  It shares no code with the engine; the tests hold the
engine's kernels, cache, state slots and scheduler to it.

Notation: ``h`` [T, width] is a sublayer's input, ``w`` the dict of a folder's tensors as float64 arrays, ``pre`` a
tensor-name prefix such as ``l3.mix.``, ``m`` the layer's ``mixer`` or ``mlp`` object from the configuration.
"""
import json
import os

import numpy as np


def load_folder(folder):
    """(configuration dict, tensors as float64) of a model folder written by the tests' helpers."""
    import torch

    from vipera_rs_amd.weights import Checkpoint

    with open(os.path.join(folder, "config.json")) as handle:
        cfg = json.load(handle)
    checkpoint = Checkpoint(folder)
    try:
        w = {name: checkpoint.read(name).to(torch.float64).numpy() for name in checkpoint.names()}
    finally:
        checkpoint.close()
    return cfg, w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def dynamic_tanh(x, w, name):
    """tanh(alpha x) * weight + bias, elementwise."""
    return np.tanh(float(w[name + ".alpha"]) * x) * w[name] + w[name + ".b"]


def over_rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / np.sqrt(np.mean(np.square(x), axis=-1, keepdims=True) + eps)


def mixture_of_experts(h, w, pre, m):
    experts, top, limit = m["router"]["experts"], m["router"]["top"], m["expert"]["limit"]
    scores = h @ w[pre + "router"].T
    out = np.zeros((h.shape[0], w[pre + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        chosen = sorted(range(experts), key=lambda e: (-scores[t, e], e))[:top]
        share = np.exp(scores[t, chosen] - scores[t, chosen].max())
        share /= share.sum()
        for e, s in zip(chosen, share):
            g = np.minimum(w[f"{pre}e{e}.gate"] @ h[t], limit)
            u = np.clip(w[f"{pre}e{e}.up"] @ h[t], -limit, limit)
            out[t] += s * (w[f"{pre}e{e}.down"] @ (g * sigmoid(1.702 * g) * (u + 1.0)))
    return out


def short_convolution(x, taps):
    """Causal, per channel: y[t] = sum_j taps[:, j] x[t - (J - 1 - j)], zeros before the start; then silu."""
    count = taps.shape[1]
    y = np.zeros_like(x)
    for t in range(x.shape[0]):
        for j in range(count):
            back = count - 1 - j
            if t - back >= 0:
                y[t] += taps[:, j] * x[t - back]
    return silu(y)


def delta_mixer(h, w, pre, m, eps):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_convolution(h @ w[pre + "q"].T, w[pre + "q.conv"]).reshape(T, G, D)
    k = short_convolution(h @ w[pre + "k"].T, w[pre + "k.conv"]).reshape(T, G, D)
    v = short_convolution(h @ w[pre + "v"].T, w[pre + "v.conv"]).reshape(T, H, V)
    q = q / np.sqrt(np.square(q).sum(-1, keepdims=True) + 1e-6) / np.sqrt(D)
    k = k / np.sqrt(np.square(k).sum(-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ w[pre + "b"].T)
    decay = np.exp(-np.exp(w[pre + "A_log"]) * softplus(h @ w[pre + "a"].T + w[pre + "dt_bias"]))
    out = np.zeros((T, H, V))
    for head in range(H):
        shared = head // (H // G)
        S = np.zeros((D, V))
        for t in range(T):
            S = decay[t, head] * S
            u = beta[t, head] * (v[t, head] - S.T @ k[t, shared])
            S = S + np.outer(k[t, shared], u)
            out[t, head] = S.T @ q[t, shared]
    gate = silu(h @ w[pre + "g"].T).reshape(T, H, V)
    return (over_rms(out, eps) * w[pre + "norm"] * gate).reshape(T, H * V) @ w[pre + "o"].T


def wkv_mixer(h, w, pre, m, eps):
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    before = np.vstack([np.zeros((1, h.shape[1])), h[:-1]])

    def mixed(which):
        return h + (before - h) * w[f"{pre}mu.{which}"]

    r = (mixed("r") @ w[pre + "r"].T).reshape(T, H, D)
    k = (mixed("k") @ w[pre + "k"].T).reshape(T, H, D)
    v = (mixed("v") @ w[pre + "v"].T).reshape(T, H, D)
    gate = silu(mixed("g") @ w[pre + "g"].T)
    decay = np.exp(-np.exp(np.tanh(mixed("w") @ w[pre + "w1"].T) @ w[pre + "w2"].T + w[pre + "w0"])).reshape(T, H, D)
    bonus = w[pre + "u"].reshape(H, D)
    out = np.zeros((T, H, D))
    for head in range(H):
        S = np.zeros((D, D))
        for t in range(T):
            kv = np.outer(k[t, head], v[t, head])
            out[t, head] = (S + bonus[head][:, None] * kv).T @ r[t, head]
            S = decay[t, head][:, None] * S + kv
    return (over_rms(out, eps).reshape(T, H * D) * w[pre + "norm"] * gate) @ w[pre + "o"].T


def rotate_half(x, positions, dims, base):
    """x [T, n]: dimension i < dims/2 is paired with i + dims/2; the rest passes."""
    half = dims // 2
    angle = positions[:, None] * base ** (-2.0 * np.arange(half) / dims) if half else np.zeros((len(positions), 0))
    lo, hi = x[:, :half], x[:, half:dims]
    return np.concatenate([lo * np.cos(angle) - hi * np.sin(angle), hi * np.cos(angle) + lo * np.sin(angle), x[:, dims:]], 1)


def latent_rows(h, w, pre, m, eps):
    """What a latent-attention layer caches per position: (normed latent c, rotated shared key part)."""
    positions = np.arange(h.shape[0], dtype=np.float64)
    down = h @ w[pre + "dkv"].T
    rank = m["kv_rank"]
    c = over_rms(down[:, :rank], eps) * w[pre + "dkv.norm"]
    return c, rotate_half(down[:, rank:], positions, m["rot"]["dims"] if m["rot_dim"] else 0, m["rot"]["base"] if m["rot_dim"] else 1.0)


def latent_attention(h, w, pre, m, eps, rows):
    """``rows``: (c, kr) of the layer whose cache this one reads (its own, or another's)."""
    T = h.shape[0]
    H, D, R, V = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    positions = np.arange(T, dtype=np.float64)
    c, kr = rows
    c_q = over_rms(h @ w[pre + "dq"].T, eps) * w[pre + "dq.norm"]
    q = (c_q @ w[pre + "uq"].T).reshape(T, H, D + R)
    keys = (c @ w[pre + "uk"].T).reshape(T, H, D)
    values = (c @ w[pre + "uv"].T).reshape(T, H, V)
    window = (m.get("mask") or {}).get("size") or 0
    out = np.zeros((T, H, V))
    for head in range(H):
        q_rot = rotate_half(q[:, head, D:], positions, m["rot"]["dims"], m["rot"]["base"]) if R else q[:, head, D:]
        for i in range(T):
            first = max(0, i - window + 1) if window else 0
            score = (keys[first:i + 1, head] @ q[i, head, :D] + kr[first:i + 1] @ q_rot[i]) * m["scale"]
            share = np.exp(score - score.max())
            out[i, head] = (share / share.sum()) @ values[first:i + 1, head]
    return out.reshape(T, H * V) @ w[pre + "o"].T


def forward(cfg, w, tokens, residuals=None):
    """Logits [T, vocab] of one whole sequence; ``residuals`` (a list) receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = dynamic_tanh(w["embed"][np.asarray(tokens)], w, "embed.norm")
    cached = {}
    for index, layer in enumerate(cfg["layers"]):
        pre, m = f"l{index}.mix.", layer["mixer"]
        h = dynamic_tanh(x, w, f"l{index}.norm1")
        if layer["type"] == "delta":
            y = delta_mixer(h, w, pre, m, eps)
        elif layer["type"] == "wkv":
            y = wkv_mixer(h, w, pre, m, eps)
        else:
            source = m.get("kv_from")
            if source is None:
                cached[index] = latent_rows(h, w, pre, m, eps)
                source = index
            y = latent_attention(h, w, pre, m, eps, cached[source])
        if layer.get("mlp") is not None:
            y = y + mixture_of_experts(h, w, f"l{index}.mlp.", layer["mlp"])
        x = x + y
        if residuals is not None:
            residuals.append(x.copy())
    return (dynamic_tanh(x, w, "final.norm") @ w["head"].T) * cfg.get("logit_scale", 1.0)


def greedy_generate(cfg, w, prompt, new_tokens):
    tokens = list(prompt)
    for _ in range(new_tokens):
        tokens.append(int(np.argmax(forward(cfg, w, tokens)[-1])))
    return tokens[len(prompt):]
