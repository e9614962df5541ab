"""Plain, slow Zovozen forward pass: whole sequences, no cache, float64 NumPy.

One function per mechanism, written from the design's equations; nothing here
is shared with the engine (it reads a model folder with `json` and the
`safetensors` library and never touches a GPU).  Every engine path of the design
is compared with `forward()`.

Notation: x is the residual stream [T, width]; a linear weight W is stored
[out, in] and applied as x W^T; positions count from 0.
"""
import json
import math
from pathlib import Path

import numpy as np


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis (eps inside the root)."""
    x = np.asarray(x, np.float64)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def rmsnorm(x, weight, eps):
    return rms(x, eps) * np.asarray(weight, np.float64)


def linear(x, w, b=None):
    y = np.asarray(x, np.float64) @ np.asarray(w, np.float64).T
    return y if b is None else y + np.asarray(b, np.float64)


def sigmoid(z):
    z = np.asarray(z, np.float64)
    e = np.exp(-np.abs(z))
    return np.where(z >= 0, 1.0 / (1.0 + e), e / (1.0 + e))


def log_sigmoid(z):
    z = np.asarray(z, np.float64)
    return np.minimum(z, 0.0) - np.log1p(np.exp(-np.abs(z)))


def silu(z):
    return z * sigmoid(z)


# -- positions ----------------------------------------------------------------------------------------------------

def rotary_frequencies(rot):
    """Radians a position of pair i: base^(-2i/dims), all divided by the linear scaling factor."""
    dims = rot["dims"]
    f = np.asarray([rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)], np.float64)
    s = rot.get("scaling")
    return f if s is None else f / s["factor"]


def rotate_half(x, positions, rot):
    """x [T, heads, dim]: the first rot.dims coordinates of each head turn, pair (i, i + dims/2) by position * f_i."""
    x = np.array(x, np.float64)
    dims = rot["dims"]
    half = dims // 2
    a = np.asarray(positions, np.float64)[:, None] * rotary_frequencies(rot)[None, :]
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    u, v = x[..., :half].copy(), x[..., half:dims].copy()
    x[..., :half] = u * c - v * s
    x[..., half:dims] = v * c + u * s
    return x


# -- mixers -------------------------------------------------------------------------------------------------------

def chunk_visible(T, size):
    """visible[i, j]: j <= i and both in the same block of `size` positions counted from 0 (all j <= i without size)."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    seen = j <= i
    return seen if size is None else seen & (i // size == j // size)


def talking_attention(h, w, p, m, eps):
    """Softmax attention whose scores are mixed over the heads before the softmax, with a sink in the denominator."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rmsnorm(linear(h, w[p + ".q"], w[p + ".q.b"]), w[p + ".q.norm"], eps).reshape(T, H, D)
    k = rmsnorm(linear(h, w[p + ".k"], w[p + ".k.b"]), w[p + ".k.norm"], eps).reshape(T, G, D)
    v = rms(linear(h, w[p + ".v"], w[p + ".v.b"]).reshape(T, G, V), eps)
    if m.get("rot") is not None:
        q = rotate_half(q, np.arange(T), m["rot"])
        k = rotate_half(k, np.arange(T), m["rot"])
    temp = np.asarray(w[p + ".temp"], np.float64)
    scores = np.stack([(q[:, a] @ k[:, a // (H // G)].T) * m["scale"] * temp[a] for a in range(H)])      # [H, T, T]
    scores = np.einsum("hg,gij->hij", np.asarray(w[p + ".talk"], np.float64), scores)
    visible = chunk_visible(T, (m.get("mask") or {}).get("size"))
    sink = np.asarray(w[p + ".sink"], np.float64)
    out = np.zeros((T, H, V))
    for a in range(H):
        s = np.where(visible, scores[a], -np.inf)
        top = np.maximum(s.max(axis=1), sink[a])
        e = np.exp(s - top[:, None])
        out[:, a] = (e / (e.sum(axis=1) + np.exp(sink[a] - top))[:, None]) @ v[:, a // (H // G)]
    out = out.reshape(T, H * V) * sigmoid(linear(h, w[p + ".g"]))
    return linear(out, w[p + ".o"], w[p + ".o.b"])


def matrix_memory(h, w, p, m, eps, margins=None):
    """Matrix memory with exponential gates kept in range by a running maximum (starts at 0), per head:
    m_t = max(f + m, i); S = exp(f + m - m_t) S + exp(i - m_t) k v^T, n likewise with k alone;
    o = S^T q / (max(|n . q|, exp(-m_t)) + 1e-6).
    `margins`: a list that receives, per token, infinity but for the first: there a head's result is (k . q) v over its
    own size, that is plus or minus v's direction, and the entry is the smallest |cos(k, q)| over the heads, halved: how
    far the sign is from turning."""
    T = h.shape[0]
    H, D, V, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = linear(h, w[p + ".q"]).reshape(T, H, D) * D ** -0.5
    k = linear(h, w[p + ".k"]).reshape(T, H, D)
    v = linear(h, w[p + ".v"]).reshape(T, H, V)
    gi = cap * np.tanh(linear(h, w[p + ".i"], w[p + ".i.b"]) / cap)
    gf = log_sigmoid(cap * np.tanh(linear(h, w[p + ".f"], w[p + ".f.b"]) / cap))
    out = np.zeros((T, H, V))
    for a in range(H):
        S, n, top = np.zeros((D, V)), np.zeros(D), 0.0
        for t in range(T):
            new = max(gf[t, a] + top, gi[t, a])
            keep, take = math.exp(gf[t, a] + top - new), math.exp(gi[t, a] - new)
            S = keep * S + take * np.outer(k[t, a], v[t, a])
            n = keep * n + take * k[t, a]
            top = new
            out[t, a] = (q[t, a] @ S) / (max(abs(n @ q[t, a]), math.exp(-top)) + 1e-6)
    if margins is not None:
        sign = np.full(T, np.inf)
        sign[0] = 0.5 * min(abs(q[0, a] @ k[0, a]) / max(np.linalg.norm(q[0, a]) * np.linalg.norm(k[0, a]), 1e-300) for a in range(H))
        margins.append(sign)
    out = rms(out, eps).reshape(T, H * V) * np.asarray(w[p + ".norm"], np.float64) * sigmoid(linear(h, w[p + ".g"]))
    return linear(out, w[p + ".o"])


def parallel_mixer(h, w, p, m, eps, margins=None):
    return (m["left_scale"] * talking_attention(h, w, p + ".left", m["left"], eps)
            + m["right_scale"] * matrix_memory(h, w, p + ".right", m["right"], eps, margins))


# -- feed-forward -------------------------------------------------------------------------------------------------

def dense_ff(h, w, p):
    return linear(np.maximum(linear(h, w[p + ".up"], w[p + ".up.b"]), 0.0) ** 2, w[p + ".down"], w[p + ".down.b"])


def gated_expert(h, w, p):
    return linear(silu(linear(h, w[p + ".gate"])) * linear(h, w[p + ".up"]), w[p + ".down"])


def route(h, w, p, r, margins=None):
    """Per token the chosen outputs of the router and their weights.  Scores are a softmax over all outputs; the choice
    adds the correction and is held to the best `keep` of `count` groups of neighbours (a group's score is its largest
    choice score; the other groups count as minus infinity); the weights are the scores of the chosen, as they are.
    `margins`: a list that receives, per token, the smallest gap by which a choice was made (between the last group
    kept and the first one dropped, and between the last output chosen and the first one left out), as a share of the
    last one taken (about what the two differ by in the router's logits)."""
    z = linear(h, w[p + ".router"])
    e = np.exp(z - z.max(axis=1, keepdims=True))
    s = e / e.sum(axis=1, keepdims=True)
    choice = s + np.asarray(w[p + ".correction"], np.float64)
    T, n = choice.shape
    gap = np.full(T, np.inf)
    groups = r.get("groups")
    if groups is not None:
        count, keep = groups["count"], groups["keep"]
        per = n // count
        best = choice.reshape(T, count, per).max(axis=2)
        for t in range(T):
            order = np.argsort(-best[t], kind="stable")
            if keep < count:
                gap[t] = (best[t][order[keep - 1]] - best[t][order[keep]]) / max(abs(best[t][order[keep - 1]]), 1e-30)
            for g in order[keep:]:
                choice[t, g * per:(g + 1) * per] = -np.inf
    top = r["top"]
    picked = np.argsort(-choice, axis=1, kind="stable")[:, :top]
    if margins is not None:
        ordered = -np.sort(-choice, axis=1)
        if n > top:
            nxt = ordered[:, top]
            last = np.maximum(np.abs(ordered[:, top - 1]), 1e-30)
            gap = np.minimum(gap, np.where(np.isfinite(nxt), (ordered[:, top - 1] - np.where(np.isfinite(nxt), nxt, 0.0)) / last, np.inf))
        margins.append(gap)
    return picked, np.take_along_axis(s, picked, axis=1)


def mixture(h, w, p, mlp, margins=None):
    r = mlp["router"]
    real = r["experts"]
    picked, weights = route(h, w, p, r, margins)
    out = np.zeros_like(np.asarray(h, np.float64))
    for t in range(h.shape[0]):
        for e, g in zip(picked[t], weights[t]):
            out[t] += g * (gated_expert(h[t], w, f"{p}.e{e}") if e < real else h[t])
    if mlp.get("shared") is not None:
        out = out + gated_expert(h, w, p + ".shared")
    return out


# -- the model ----------------------------------------------------------------------------------------------------

def forward(cfg, w, tokens, layers_out=None, margins=None):
    """Logits [T, vocab] of a whole sequence.  `layers_out`: a list that receives the residual stream after every layer;
    `margins`: a list that receives every router's margins (route) and every memory's (matrix_memory): how far a
    position is from a decision that rounding could turn round."""
    eps = cfg["norm"]["eps"]
    x = np.asarray(w["embed"], np.float64)[np.asarray(tokens)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        if layer["type"] != "parallel":
            raise ValueError(f"layer type {layer['type']!r}")
        x = x + rmsnorm(parallel_mixer(x, w, p + ".mix", layer["mixer"], eps, margins), w[p + ".norm1"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            y = dense_ff(x, w, p + ".mlp") if mlp["kind"] == "dense" else mixture(x, w, p + ".mlp", mlp, margins)
            x = x + rmsnorm(y, w[p + ".norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    return linear(rmsnorm(x, w["final.norm"], eps), w["embed"])


def read_folder(folder):
    """(config.json as a dict, {name: float64 array}) of a model folder, read with the safetensors library."""
    import torch
    from safetensors.torch import load_file
    folder = Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    weights = {k: v.to(torch.float64).numpy() for k, v in load_file(str(folder / "model.safetensors")).items()}
    return cfg, weights


def greedy(cfg, w, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(np.argmax(forward(cfg, w, tokens)[-1])))
    return tokens[len(prompt):]
