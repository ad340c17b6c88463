"""A plain, slow implementation of the Zulesun decoder in float64 numpy: one function per mechanism, whole
sequences only, no cache, no batching.  It is what the engine's kernels are held to; it shares no code with them.

``weights`` maps tensor names to float64 arrays; ``config`` is the parsed ``config.json``.
"""
from __future__ import annotations

import math

import numpy as np


# --- small pieces -------------------------------------------------------------------------------------------
def unit_rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def norm_around_zero(x, w, eps):
    """RMS norm whose stored weight lies around zero: the gain is 1 + w."""
    return unit_rms(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return unit_rms(x, eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# --- mixers -------------------------------------------------------------------------------------------------
def lightning(h, w, p, eps):
    """Linear attention with one decay per head: S <- decay S + k v^T, o = S^T q; all heads normed together."""
    heads, dim, vdim = p["heads"], p["dim"], p["vdim"]
    tokens = h.shape[0]
    q = silu(h @ w["q"].T).reshape(tokens, heads, dim)
    k = silu(h @ w["k"].T).reshape(tokens, heads, dim)
    v = silu(h @ w["v"].T).reshape(tokens, heads, vdim)
    out = np.zeros((tokens, heads, vdim))
    for head in range(heads):
        state = np.zeros((dim, vdim))
        decay = float(p["decay"][head])
        for t in range(tokens):
            state = decay * state + np.outer(k[t, head], v[t, head])
            out[t, head] = state.T @ q[t, head]
    flat = norm_plain(out.reshape(tokens, heads * vdim), w["norm"], eps)
    return (flat * sigmoid(h @ w["g"].T)) @ w["o"].T


def rotate_half(x, positions, dims, base, factor):
    """x: [tokens, heads, dim]; the first ``dims`` of each head turn, dimension i with i + dims / 2."""
    if not dims:
        return x
    half = dims // 2
    freq = base ** (-2.0 * np.arange(half) / dims) / factor
    angle = positions[:, None] * freq[None, :]
    cos, sin = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    out = x.copy()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * cos - v * sin
    out[..., half:dims] = v * cos + u * sin
    return out


def chunked_attention(h, w, p, eps, first_position=0):
    """Grouped-query softmax attention: q and k normed over the whole projection, partly rotated, scores capped by a
    tanh, a token sees the earlier tokens of its own chunk of positions, the output gated by a sigmoid of the input."""
    heads, groups, dim, vdim = p["heads"], p["kv_heads"], p["dim"], p["vdim"]
    tokens = h.shape[0]
    positions = np.arange(tokens, dtype=np.float64) + first_position
    q = norm_plain(h @ w["q"].T, w["q.norm"], eps).reshape(tokens, heads, dim)
    k = norm_plain(h @ w["k"].T, w["k.norm"], eps).reshape(tokens, groups, dim)
    v = (h @ w["v"].T).reshape(tokens, groups, vdim)
    rot = p.get("rot") or {}
    dims = int(rot.get("dims") or 0)
    factor = float((rot.get("scaling") or {}).get("factor", 1.0)) if dims else 1.0
    if dims:
        q = rotate_half(q, positions, dims, float(rot["base"]), factor)
        k = rotate_half(k, positions, dims, float(rot["base"]), factor)
    cap = float(p.get("softcap") or 0.0)
    size = int((p.get("mask") or {}).get("size") or 0)
    out = np.zeros((tokens, heads, vdim))
    per = heads // groups
    for head in range(heads):
        g = head // per
        scores = (q[:, head] @ k[:, g].T) * p["scale"]
        if cap:
            scores = cap * np.tanh(scores / cap)
        for i in range(tokens):
            pi = int(positions[i])
            lo = (pi // size) * size - first_position if size else 0
            lo = max(lo, 0)
            s = scores[i, lo:i + 1]
            e = np.exp(s - s.max())
            out[i, head] = (e / e.sum()) @ v[lo:i + 1, g]
    flat = out.reshape(tokens, heads * vdim) * sigmoid(h @ w["g"].T)
    return flat @ w["o"].T


def selective_scan(h, w, p):
    """Mamba: a short causal convolution, then a diagonal state per channel whose step size depends on the token."""
    inner, n, rank, taps = p["inner"], p["state"], p["dt_rank"], p["conv"]
    tokens = h.shape[0]
    xz = h @ w["in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    padded = np.concatenate([np.zeros((taps - 1, inner)), x])
    conv = np.zeros((tokens, inner))
    for j in range(taps):
        conv += padded[j:j + tokens] * w["conv"][:, j][None, :]
    x = silu(conv + w["conv.b"])
    low = x @ w["x"].T
    dt = softplus(low[:, :rank] @ w["dt"].T + w["dt.b"])
    b, c = low[:, rank:rank + n], low[:, rank + n:rank + 2 * n]
    a = -np.exp(w["A_log"])
    state = np.zeros((inner, n))
    y = np.zeros((tokens, inner))
    for t in range(tokens):
        state = np.exp(dt[t][:, None] * a) * state + (dt[t] * x[t])[:, None] * b[t][None, :]
        y[t] = state @ c[t] + w["D"] * x[t]
    return (y * silu(z)) @ w["o"].T


def parallel(h, w, p, eps):
    """Two mixers read the same input; their outputs are added with a scale each."""
    left = chunked_attention(h, sub(w, "left."), p["left"], eps)
    right = selective_scan(h, sub(w, "right."), p["right"])
    return p["left_scale"] * left + p["right_scale"] * right


# --- feed-forwards ------------------------------------------------------------------------------------------
def dense_ffn(h, w):
    return np.maximum(h @ w["up"].T, 0.0) ** 2 @ w["down"].T


def route(scores, top, count, keep):
    """For one token: the ids of the ``top`` largest scores among the experts of the ``keep`` best groups (a group's
    score is its largest), lowest id first among equals."""
    experts = scores.shape[0]
    size = experts // count
    group_score = scores.reshape(count, size).max(axis=1)
    best = sorted(range(count), key=lambda g: (-group_score[g], g))[:keep]
    allowed = [e for e in range(experts) if e // size in best]
    return sorted(allowed, key=lambda e: (-scores[e], e))[:top]


def routing_gap(z, top, count, keep):
    """How far one token's router logits ``z`` are from another choice: the smallest difference between something
    chosen (a kept group's best logit, a chosen expert's logit) and the best thing of its kind that was not."""
    experts = z.shape[0]
    size = experts // count
    gap = np.inf
    groups = np.sort(z.reshape(count, size).max(axis=1))[::-1]
    if keep < count:
        gap = min(gap, groups[keep - 1] - groups[keep])
    chosen = route(z, top, count, keep)
    best = sorted(range(count), key=lambda g: (-z.reshape(count, size).max(axis=1)[g], g))[:keep]
    rest = [z[e] for e in range(experts) if e // size in best and e not in chosen]
    if rest:
        gap = min(gap, min(z[e] for e in chosen) - max(rest))
    return gap


def moe(h, w, p, gaps=None):
    router = p["router"]
    experts, top = router["experts"], router["top"]
    groups = router.get("groups") or {}
    count, keep = int(groups.get("count", 1)), int(groups.get("keep", groups.get("count", 1)))
    z = h @ w["router"].T
    if gaps is not None:
        gaps.append(np.array([routing_gap(z[t], top, count, keep) for t in range(h.shape[0])]))
    z = z - z.max(axis=-1, keepdims=True)
    scores = np.exp(z) / np.exp(z).sum(axis=-1, keepdims=True)
    out = np.zeros((h.shape[0], w["e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e in route(scores[t], top, count, keep):
            y = silu(w[f"e{e}.gate"] @ h[t]) * (w[f"e{e}.up"] @ h[t])
            out[t] += scores[t, e] * (w[f"e{e}.down"] @ y)
    return out


def token_side(x, tokens, table, layer, w, dim, eps):
    """What a layer adds from its own part of the per-token table, gated by the stream."""
    e = table[tokens][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ w["gate"].T) * e) @ w["proj"].T
    return norm_plain(y, w["norm"], eps)


# --- the model ----------------------------------------------------------------------------------------------
def sub(weights, prefix):
    return {name[len(prefix):]: value for name, value in weights.items() if name.startswith(prefix)}


def forward(config, weights, tokens, layers_out=None, gaps=None):
    """Logits ``[tokens, vocab]`` of one sequence from position 0; ``layers_out`` collects the stream after each layer,
    ``gaps`` per mixture of experts every token's :func:`routing_gap`."""
    tokens = np.asarray(tokens)
    eps = float(config["norm"]["eps"])
    x = weights["embed"][tokens] * float(config["embedding"]["scale"])
    side = config.get("token_side")
    for index, layer in enumerate(config["layers"]):
        w = sub(weights, f"l{index}.")
        h = norm_around_zero(x, w["norm1"], eps)
        if layer["type"] == "lightning":
            y = lightning(h, sub(w, "mix."), layer["mixer"], eps)
        elif layer["type"] == "parallel":
            y = parallel(h, sub(w, "mix."), layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + norm_around_zero(y, w["norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = norm_around_zero(x, w["norm2"], eps)
            y = dense_ffn(h, sub(w, "mlp.")) if mlp["kind"] == "dense" else moe(h, sub(w, "mlp."), mlp, gaps)
            x = x + norm_around_zero(y, w["norm2b"], eps)
        if side:
            x = x + token_side(x, tokens, weights["side.embed"], index, sub(w, "side."), int(side["dim"]), eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    return norm_around_zero(x, weights["final.norm"], eps) @ weights["head"].T
