"""Plain, slow Noresun forward pass: whole sequences, no cache, float64 NumPy.

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
    return np.where(z >= 0, 1.0 / (1.0 + np.exp(-np.abs(z))), np.exp(-np.abs(z)) / (1.0 + np.exp(-np.abs(z))))


def silu(z):
    return z * sigmoid(z)


# -- embedding ----------------------------------------------------------------------------------------------------

def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the bigram table for every token: a hash of (previous token, token); the last row for the first token."""
    tokens = [int(t) for t in tokens]
    return [buckets if i == 0 else (tokens[i - 1] * mul_prev + t * mul_cur) % buckets for i, t in enumerate(tokens)]


def embed(tokens, w, e):
    x = np.asarray(w["embed"], np.float64)[np.asarray(tokens)] * e["scale"]
    b = e.get("bigram")
    if b is not None:
        x = x + np.asarray(w["bigram"], np.float64)[bigram_rows(tokens, b["buckets"], b["mul_prev"], b["mul_cur"])]
    return x


# -- positions ----------------------------------------------------------------------------------------------------

def rotary_frequencies(rot):
    """Radians a position of each pair: base^(-2i/dims), the long wavelengths slowed down (Llama 3.1's rule)."""
    dims = rot["dims"]
    f = np.asarray([rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)], np.float64)
    s = rot.get("scaling")
    if s is None:
        return f
    out = f.copy()
    for i, fi in enumerate(f):
        wavelength = 2.0 * math.pi / fi
        if wavelength < s["original"] / s["high"]:
            continue
        if wavelength > s["original"] / s["low"]:
            out[i] = fi / s["factor"]
        else:
            t = (s["original"] / wavelength - s["low"]) / (s["high"] - s["low"])
            out[i] = (1.0 - t) * fi / s["factor"] + t * fi
    return out


def rotate_interleaved(x, positions, rot):
    """x [T, heads, dim]: the first rot.dims coordinates of each head turn, pair (2i, 2i + 1) by position * f_i."""
    x = np.array(x, np.float64)
    dims = rot["dims"]
    a = np.asarray(positions, np.float64)[:, None] * rotary_frequencies(rot)[None, :]      # [T, dims / 2]
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    u, v = x[..., 0:dims:2].copy(), x[..., 1:dims:2].copy()
    x[..., 0:dims:2] = u * c - v * s
    x[..., 1:dims:2] = v * c + u * s
    return x


# -- mixers -------------------------------------------------------------------------------------------------------

def min_gru(h, w, p, m, state=None):
    """S_t = (1 - z_t) S_(t-1) + z_t c_t element by element; z = sigmoid(Wz h + b), c = g(Wx h + b) with
    g(u) = u + 1/2 for u >= 0 and sigmoid(u) below; the result is Wo (S_t silu(Wg h))."""
    z = sigmoid(linear(h, w[p + ".z"], w[p + ".z.b"]))
    u = linear(h, w[p + ".x"], w[p + ".x.b"])
    cand = np.where(u >= 0, u + 0.5, sigmoid(u))
    S = np.zeros(m["width"]) if state is None else np.asarray(state, np.float64)
    states = np.zeros_like(z)
    for t in range(h.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        states[t] = S
    return linear(states * silu(linear(h, w[p + ".g"])), w[p + ".o"])


def attention_keys(h, w, p, m, eps):
    """What a layer caches: keys after the norm over the whole projection and the rotation, and values."""
    T = h.shape[0]
    G, D, V = m["kv_heads"], m["dim"], m["vdim"]
    k = rmsnorm(linear(h, w[p + ".k"]), w[p + ".k.norm"], eps).reshape(T, G, D)
    k = rotate_interleaved(k, np.arange(T), m["rot"])
    return k, linear(h, w[p + ".v"]).reshape(T, G, V)


def sigmoid_attention(h, w, p, m, eps, keys_values):
    """Attention without softmax: a visible key j (0 <= i - j < window) weighs sigmoid(q . k scale + b_head), and the
    weights are not normed over the keys."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rmsnorm(linear(h, w[p + ".q"]), w[p + ".q.norm"], eps).reshape(T, H, D)
    q = rotate_interleaved(q, np.arange(T), m["rot"])
    k, v = keys_values
    window = (m.get("mask") or {}).get("size")
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    visible = (j <= i) if window is None else (j <= i) & (i - j < window)
    out = np.zeros((T, H, V))
    bias = np.asarray(w[p + ".pb"], np.float64)
    for head in range(H):
        g = head // (H // G)
        scores = (q[:, head] @ k[:, g].T) * m["scale"] + bias[head]
        out[:, head] = np.where(visible, sigmoid(scores), 0.0) @ v[:, g]
    return linear(out.reshape(T, H * V), w[p + ".o"])


# -- feed-forward -------------------------------------------------------------------------------------------------

def routed_experts(h, w, p, mlp, margins=None):
    """Each token goes through the `top` experts with the largest router logits; their results are weighed by the
    softmax over those logits only.  An expert is Wdown relu(Wup h)^2.  `margins`: a list that receives, per token, how
    far the last chosen logit lies above the first one left out (infinite where every expert is chosen)."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    logits = linear(h, w[p + ".router"], w[p + ".router.b"])
    if margins is not None:
        ordered = -np.sort(-logits, axis=1)
        margins.append(ordered[:, top - 1] - ordered[:, top] if E > top else np.full(h.shape[0], np.inf))
    out = np.zeros((h.shape[0], np.asarray(w[p + ".e0.down"]).shape[0]))
    for t in range(h.shape[0]):
        chosen = np.argsort(-logits[t], kind="stable")[:top]
        weights = np.exp(logits[t][chosen] - logits[t][chosen].max())
        weights /= weights.sum()
        for e, g in zip(chosen, weights):
            a = np.maximum(linear(h[t], w[f"{p}.e{e}.up"]), 0.0) ** 2
            out[t] += g * linear(a, w[f"{p}.e{e}.down"])
    return out


# -- the model ----------------------------------------------------------------------------------------------------

def forward(cfg, w, tokens, layers_out=None, margins=None):
    """Logits [T, vocab] of a whole sequence.  `layers_out`: a list that receives the residual stream after every layer;
    `margins`: a list that receives every router's margins (routed_experts)."""
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    x = embed(tokens, w, cfg["embedding"])
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}", layer["mixer"]
        if layer["type"] == "mingru":
            y = min_gru(x, w, p + ".mix", m)
        elif layer["type"] == "attention":
            source = m.get("kv_from")
            if source is None:
                kept[i] = attention_keys(x, w, p + ".mix", m, eps)
            y = sigmoid_attention(x, w, p + ".mix", m, eps, kept[i if source is None else source])
        else:
            raise ValueError(f"layer type {layer['type']!r}")
        y = y * sigmoid(linear(x, w[p + ".rg1"], w[p + ".rg1.b"]))
        x = rmsnorm(alpha * x + y, w[p + ".norm1"], eps)
        if layer.get("mlp") is not None:
            y = routed_experts(x, w, p + ".mlp", layer["mlp"], margins)
            y = y * sigmoid(linear(x, w[p + ".rg2"], w[p + ".rg2.b"]))
            x = rmsnorm(alpha * x + y, w[p + ".norm2"], eps)
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
