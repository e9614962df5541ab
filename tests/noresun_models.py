"""Tiny Noresun configurations with weights of the tests' own making, written with the `safetensors` library (not the
engine's writer), and the plain implementation's logits for them.

The configurations differ from each other in every size and constant, and inside each the sizes that could be
confused are unequal: key and value sizes of a head, query and key/value heads, turning and other coordinates, experts
and chosen experts, windows of a layer and of the layer that reads its keys.  One has a width that is no multiple of
8, a single head, a window of one key, no table of token pairs and as many chosen experts as experts; one is drawn
sharp: scores with a spread of several units and biases far below zero, so that a query's result hangs on single keys,
and update gates close to zero, so that the recurrent state remembers the first tokens; one has no attention at all (no
pages); one has many heads whose keys and values have one size (nothing to pack) beside a layer that sees all keys.
"""
import json
from pathlib import Path

import numpy as np


def rot(base, dims, scaling=None):
    out = {"base": base, "dims": dims}
    if scaling is not None:
        out["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return out


def attention(heads, kv_heads, dim, vdim, scale, window, rotation, kv_from=None, mlp=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rotation}
    if window is not None:
        mixer["mask"] = {"size": window}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def mingru(width, mlp=None):
    return {"type": "mingru", "mixer": {"width": width}, "mlp": mlp}


def moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def config(vocab, width, alpha, eps, scale, bigram, layers):
    embedding = {"scale": scale}
    if bigram is not None:
        embedding["bigram"] = dict(zip(("buckets", "mul_prev", "mul_cur"), bigram))
    return {"architecture": "Noresun", "vocab": vocab, "width": width, "postln_alpha": alpha, "norm": {"eps": eps},
            "embedding": embedding, "layers": layers}


_R1 = rot(10000.0, 8, (4.0, 1.0, 4.0, 64))
_R2 = rot(500.0, 10)
_R3 = rot(100000.0, 16, (8.0, 2.0, 16.0, 128))
_R4 = rot(1000.0, 32, (2.0, 1.0, 2.0, 32))

CONFIGS = {
    # both mixers twice in an order of their own; the third layer reads the first one's keys over a longer window than
    # the first looks back over itself, and has no feed-forward
    "a": config(131, 64, 2.5, 1e-5, 8.0, (97, 17, 3), [
        attention(4, 2, 24, 16, 0.3, 20, _R1, mlp=moe(40, 6, 2)),
        mingru(48, moe(24, 3, 1)),
        attention(4, 2, 24, 16, 0.2, 37, _R1, kv_from=0),
        mingru(80, moe(32, 5, 3))]),
    # a width that is no multiple of 8, one head, a window of one key, values larger than keys, all coordinates turn,
    # no table of token pairs, every expert chosen, alpha 1
    "b": config(77, 100, 1.0, 1e-6, 3.0, None, [
        mingru(7, moe(12, 2, 2)),
        attention(1, 1, 10, 24, 0.5, 1, _R2, mlp=moe(20, 4, 1))]),
    # sharp (the weights' maker reads "sharp"): a window of 48, a layer that sees every key, and one that reads the
    # windowed layer's keys over a shorter window
    "s": config(97, 48, 3.0, 1e-5, 6.0, (61, 5, 11), [
        attention(4, 1, 32, 16, 0.35, 48, _R3, mlp=moe(32, 4, 2)),
        mingru(40, moe(24, 3, 2)),
        attention(2, 2, 16, 32, 0.5, None, _R1, mlp=moe(16, 2, 1)),
        attention(4, 1, 32, 16, 0.35, 29, _R3, kv_from=0),
        mingru(24)]),
    # no layer keeps pages: the cache manager has state slots only
    "g": config(53, 40, 2.0, 1e-5, 5.0, (31, 2, 7), [mingru(56, moe(16, 3, 2)), mingru(8)]),
    # twenty heads over four, keys and values of one size (nothing to pack), half of a head turns
    "w": config(211, 96, 4.0, 1e-5, 10.0, (128, 1, 1), [
        attention(20, 4, 64, 64, 0.125, 100, _R4, mlp=moe(48, 8, 2)),
        mingru(64, moe(48, 8, 4))]),
}
SEEDS = {"a": 21, "b": 22, "s": 23, "g": 24, "w": 25}


def tensor_shapes(c):
    H, V = c["width"], c["vocab"]
    shapes = {"embed": (V, H), "final.norm": (H,)}
    if "bigram" in c["embedding"]:
        shapes["bigram"] = (c["embedding"]["bigram"]["buckets"] + 1, H)
    for i, layer in enumerate(c["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        shapes.update({p + "norm1": (H,), p + "rg1": (H, H), p + "rg1.b": (H,)})
        if layer["type"] == "mingru":
            W = m["width"]
            shapes.update({p + "mix.z": (W, H), p + "mix.z.b": (W,), p + "mix.x": (W, H), p + "mix.x.b": (W,), p + "mix.g": (W, H),
                           p + "mix.o": (H, W)})
        else:
            nh, nkv, D, Vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            shapes.update({p + "mix.q": (nh * D, H), p + "mix.q.norm": (nh * D,), p + "mix.pb": (nh,), p + "mix.o": (H, nh * Vd)})
            if "kv_from" not in m:
                shapes.update({p + "mix.k": (nkv * D, H), p + "mix.v": (nkv * Vd, H), p + "mix.k.norm": (nkv * D,)})
        if layer["mlp"] is not None:
            F, E = layer["mlp"]["expert"]["ff"], layer["mlp"]["router"]["experts"]
            shapes.update({p + "norm2": (H,), p + "rg2": (H, H), p + "rg2.b": (H,), p + "mlp.router": (E, H), p + "mlp.router.b": (E,)})
            for j in range(E):
                shapes.update({f"{p}mlp.e{j}.up": (F, H), f"{p}mlp.e{j}.down": (H, F)})
    return shapes


def make_weights(c, seed, sharp=False):
    """Matrices N(0, 1/in) (so that every projection's output has a spread of about one), norm weights 1 + N(0, 0.1),
    biases N(0, 0.5), the attention's biases a head N(-1, 0.5), embedding rows N(0, 1) / scale, pair rows N(0, 1).
    `sharp`: the query norms' weights times 4 (scores with a spread of several units), the biases a head N(-5, 0.5) (a
    key that does not stand out weighs next to nothing), the update gate's bias N(-3, 0.5) (the state forgets slowly)."""
    import torch
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in sorted(tensor_shapes(c).items()):
        last = name.rsplit(".", 1)[-1]
        if last in ("norm", "norm1", "norm2"):
            w = 1.0 + 0.1 * rng.standard_normal(shape)
            if sharp and name.endswith("q.norm"):
                w = 4.0 * w
        elif last == "pb":
            w = (-5.0 if sharp else -1.0) + 0.5 * rng.standard_normal(shape)
        elif name.endswith("z.b") and sharp:
            w = -3.0 + 0.5 * rng.standard_normal(shape)
        elif last == "b":
            w = 0.5 * rng.standard_normal(shape)
        elif name == "embed":
            w = rng.standard_normal(shape) / c["embedding"]["scale"]
        elif name == "bigram":
            w = rng.standard_normal(shape)
        else:
            w = rng.standard_normal(shape) / np.sqrt(shape[-1])
        out[name] = torch.from_numpy(np.asarray(w, np.float32)).to(torch.bfloat16)
    return out


def write_folder(folder, c, seed, sharp=False):
    from safetensors.torch import save_file
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(c))
    save_file(make_weights(c, seed, sharp), str(folder / "model.safetensors"))
    return folder


_PLAIN = {}
CLOSE_CALL = 0.02     # a router's margin (its logits have a spread of about one) that bfloat16 rounding may turn round


def _plain(folder, tokens):
    import plain_noresun
    key = (str(folder), tuple(tokens))
    if key not in _PLAIN:
        cfg, w = _PLAIN.setdefault(("folder", str(folder)), plain_noresun.read_folder(folder))
        margins = []
        logits = plain_noresun.forward(cfg, w, list(tokens), margins=margins)
        _PLAIN[key] = (logits, np.min(margins, axis=0) if margins else np.full(len(tokens), np.inf))
    return _PLAIN[key]


def plain_logits(folder, tokens):
    """float64 logits [T, V] of the plain implementation, cached per (folder, tokens)."""
    return _plain(folder, tokens)[0]


def decided_rows(folder, tokens):
    """Which positions of a sequence have no close call in a router of their own: True where every
    router's margin at the position is at least CLOSE_CALL.  In bfloat16 a narrower margin may choose another expert
    than the float64 implementation does, which is no fault; such a position is compared in float32 only.  (A close
    call also reaches later positions through the recurrent state and the cached keys, but thinly: they stay in.)"""
    return _plain(folder, tokens)[1] >= CLOSE_CALL


def smallest_margins(folder, tokens):
    """For every position the smallest margin by which a router of the plain model decides there."""
    return _plain(folder, tokens)[1]


FLIP = 0.01           # a margin below which the rounding of a bfloat16 run that has come some layers far may choose otherwise


def decisive_tokens(folder, seed, n, vocab, margin=FLIP, tries=200):
    """`n` token ids drawn from `seed` at none of whose positions a router of the plain model decides by less than
    `margin`: the first position that does gets another token until none is left (a position's routers see only the
    tokens up to it, so what is settled stays settled).  A choice that bfloat16 rounding turns round changes the keys
    and states that later positions read, and no comparison should rest on one."""
    rng = np.random.default_rng(seed)
    tokens = [int(t) for t in rng.integers(0, vocab, n)]
    for _ in range(tries):
        margins = _plain(folder, tokens)[1]
        close = np.nonzero(margins < margin)[0]
        if not len(close):
            return tokens
        _PLAIN.pop((str(folder), tuple(tokens)), None)
        tokens[int(close[0])] = int(rng.integers(0, vocab))
    raise AssertionError(f"no sequence of {n} tokens without a close call after {tries} tries")
