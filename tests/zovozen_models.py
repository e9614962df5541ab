"""Tiny Zovozen configurations with weights of the tests' own making, written with the `safetensors` library (not the
engine's writer), and the plain implementation's logits for them.

The configurations differ from each other in every size and constant, and inside each the sizes that could be confused
are unequal: key and value sizes of a head, query and key/value heads, heads of the two mixers, turning and other
coordinates, experts, identity experts and chosen experts, blocks of positions of neighbouring layers.  One has a
width that is no multiple of 8, one head, blocks of a single position, all coordinates turning, one expert group and
every output chosen; one is drawn sharp (scores with a spread of several units, a layer that sees every key, forget
gates close to one); one has five query heads a key/value head and sixteen router outputs in four groups; one has no
rotation, no blocks, as many key/value heads as query heads and no identity experts.
"""
import json
from pathlib import Path

import numpy as np


def left(heads, kv_heads, dim, vdim, scale, chunk=None, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if chunk is not None:
        m["mask"] = {"size": chunk}
    if rot is not None:
        base, dims, factor = rot
        m["rot"] = {"base": base, "dims": dims}
        if factor is not None:
            m["rot"]["scaling"] = {"factor": factor}
    return m


def right(heads, dim, vdim, cap):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def layer(l, r, ls, rs, mlp=None):
    return {"type": "parallel", "mixer": {"left": l, "right": r, "left_scale": ls, "right_scale": rs}, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, identity=0, groups=None, shared=None):
    router = {"experts": experts, "top": top, "identity": identity}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def config(vocab, width, eps, layers):
    return {"architecture": "Zovozen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


CONFIGS = {
    # blocks of 20 and of 37 positions in neighbouring layers (two groups of pages), a layer without a feed-forward
    "a": config(131, 64, 1e-5, [
        layer(left(4, 2, 24, 16, 0.3, 20, (10000.0, 8, 2.0)), right(2, 8, 12, 8.0), 1.1, 0.7, dense(40)),
        layer(left(4, 2, 24, 16, 0.25, 37, (10000.0, 8, 2.0)), right(3, 16, 8, 5.0), 0.8, 1.3, moe(24, 6, 3, 2, (4, 2), 20)),
        layer(left(2, 1, 16, 32, 0.4, 20, (500.0, 16, None)), right(2, 8, 12, 8.0), 1.0, 1.0)]),
    # a width that is no multiple of 8, one head, blocks of one position (a row sees itself and the sink), every
    # coordinate turns, values larger than keys, every router output chosen, no groups, no shared expert
    "b": config(77, 100, 1e-6, [
        layer(left(1, 1, 10, 24, 0.5, 1, (500.0, 10, None)), right(1, 4, 5, 3.0), 0.5, 2.0, moe(12, 2, 2)),
        layer(left(1, 1, 10, 24, 0.5, 7, (500.0, 10, 3.0)), right(1, 4, 5, 3.0), 1.5, 0.25, dense(20))]),
    # sharp (the weights' maker reads "sharp"): blocks of 48, a layer that sees every key, identity experts
    "s": config(97, 48, 1e-5, [
        layer(left(4, 1, 32, 16, 0.35, 48, (100000.0, 16, 8.0)), right(2, 16, 16, 10.0), 1.0, 0.6, moe(32, 3, 2, 1, (2, 1), 16)),
        layer(left(2, 2, 16, 32, 0.5, None, (10000.0, 8, 2.0)), right(4, 8, 8, 6.0), 1.2, 0.9, dense(64))]),
    # twenty heads over four, keys and values of one size, half of a head turns; sixteen router outputs in four groups
    "w": config(211, 96, 1e-5, [
        layer(left(20, 4, 64, 64, 0.125, 100, (1000.0, 32, 2.0)), right(8, 32, 32, 15.0), 1.0, 1.0, moe(48, 14, 4, 2, (4, 2), 40)),
        layer(left(6, 6, 8, 8, 0.4, 64, (1000.0, 4, None)), right(5, 24, 40, 15.0), 0.9, 1.1, dense(136))]),
    # no rotation, no blocks, as many key/value heads as query heads, values larger than keys, one expert chosen
    "n": config(53, 40, 1e-5, [
        layer(left(3, 3, 16, 40, 0.25), right(2, 12, 20, 4.0), 1.3, 0.4, moe(16, 5, 1, 0, None, 8)),
        layer(left(3, 3, 16, 40, 0.25), right(2, 12, 20, 4.0), 0.7, 0.7)]),
}
SEEDS = {"a": 41, "b": 42, "s": 43, "w": 44, "n": 45}


def tensor_shapes(c):
    H, V = c["width"], c["vocab"]
    shapes = {"embed": (V, H), "final.norm": (H,)}
    for i, lay in enumerate(c["layers"]):
        p = f"l{i}."
        a, r = lay["mixer"]["left"], lay["mixer"]["right"]
        nh, nkv, D, Vd = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
        q = p + "mix.left."
        shapes.update({p + "norm1": (H,), q + "q": (nh * D, H), q + "q.b": (nh * D,), q + "k": (nkv * D, H), q + "k.b": (nkv * D,),
                       q + "v": (nkv * Vd, H), q + "v.b": (nkv * Vd,), q + "q.norm": (nh * D,), q + "k.norm": (nkv * D,),
                       q + "talk": (nh, nh), q + "temp": (nh,), q + "sink": (nh,), q + "g": (nh * Vd, H), q + "o": (H, nh * Vd),
                       q + "o.b": (H,)})
        q = p + "mix.right."
        rh, rd, rv = r["heads"], r["dim"], r["vdim"]
        shapes.update({q + "q": (rh * rd, H), q + "k": (rh * rd, H), q + "v": (rh * rv, H), q + "g": (rh * rv, H), q + "o": (H, rh * rv),
                       q + "norm": (rh * rv,), q + "i": (rh, H), q + "i.b": (rh,), q + "f": (rh, H), q + "f.b": (rh,)})
        mlp = lay["mlp"]
        if mlp is None:
            continue
        shapes[p + "norm2"] = (H,)
        q = p + "mlp."
        if mlp["kind"] == "dense":
            F = mlp["ff"]
            shapes.update({q + "up": (F, H), q + "up.b": (F,), q + "down": (H, F), q + "down.b": (H,)})
        else:
            F, E = mlp["expert"]["ff"], mlp["router"]["experts"]
            n = E + mlp["router"].get("identity", 0)
            shapes.update({q + "router": (n, H), q + "correction": (n,)})
            for j in range(E):
                shapes.update({f"{q}e{j}.gate": (F, H), f"{q}e{j}.up": (F, H), f"{q}e{j}.down": (H, F)})
            if "shared" in mlp:
                S = mlp["shared"]["ff"]
                shapes.update({q + "shared.gate": (S, H), q + "shared.up": (S, H), q + "shared.down": (H, S)})
    return shapes


def make_weights(c, seed, sharp=False):
    """Matrices N(0, 1/in), norm weights 1 + N(0, 0.1), biases N(0, 0.5), the heads' mix the identity + N(0, 0.3), a
    head's temperature 1 + N(0, 0.2), sinks N(0, 1), the routers' matrices N(0, 4/in) and corrections N(0, 0.03), the
    input gates' biases N(0, 1), the forget gates' N(2, 1), embedding rows N(0, 1).
    `sharp`: the query norms' weights times 4 (scores with a spread of several units: a query's result hangs on single
    keys), sinks N(-4, 0.5), forget gates' biases N(5, 0.5) (the memory keeps the first tokens)."""
    import torch
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in sorted(tensor_shapes(c).items()):
        last = name.rsplit(".", 1)[-1]
        if last in ("norm", "norm1", "norm2"):
            w = 1.0 + 0.1 * rng.standard_normal(shape)
            if sharp and name.endswith("q.norm"):
                w = 4.0 * w
        elif last == "talk":
            w = np.eye(shape[0]) + 0.3 * rng.standard_normal(shape)
        elif last == "temp":
            w = 1.0 + 0.2 * rng.standard_normal(shape)
        elif last == "sink":
            w = (-4.0 if sharp else 0.0) + (0.5 if sharp else 1.0) * rng.standard_normal(shape)
        elif last == "correction":
            w = 0.03 * rng.standard_normal(shape)
        elif name.endswith("f.b"):
            w = (5.0 if sharp else 2.0) + (0.5 if sharp else 1.0) * rng.standard_normal(shape)
        elif name.endswith("i.b"):
            w = rng.standard_normal(shape)
        elif last == "b":
            w = 0.5 * rng.standard_normal(shape)
        elif name == "embed":
            w = rng.standard_normal(shape)
        elif last == "router":
            w = 2.0 * rng.standard_normal(shape) / np.sqrt(shape[-1])
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
CLOSE_CALL = 0.1      # a router's margin (a share of the last score taken) that bfloat16 rounding may turn round


def _plain(folder, tokens):
    import plain_zovozen
    key = (str(folder), tuple(tokens))
    if key not in _PLAIN:
        cfg, w = _PLAIN.setdefault(("folder", str(folder)), plain_zovozen.read_folder(folder))
        margins = []
        logits = plain_zovozen.forward(cfg, w, list(tokens), margins=margins)
        _PLAIN[key] = (logits, np.min(margins, axis=0) if margins else np.full(len(tokens), np.inf))
    return _PLAIN[key]


def plain_logits(folder, tokens):
    """float64 logits [T, V] of the plain implementation, cached per (folder, tokens)."""
    return _plain(folder, tokens)[0]


def decided_rows(folder, tokens):
    """Which positions of a sequence have no close call of their own: True where every router's margin at the position is
    at least CLOSE_CALL, and, at a sequence's first position, no head of a matrix memory has a key and a query at
    nearly a right angle (the head's normed result is then plus or minus its value's direction, by the sign of k . q).
    In bfloat16 a narrower margin may choose another expert, or the other sign, than the float64 implementation does,
    which is no fault; such a position is compared in float32 only."""
    return _plain(folder, tokens)[1] >= CLOSE_CALL


FLIP = 0.05           # a margin below which the rounding of a bfloat16 run that has come some layers far may choose otherwise


def decisive_tokens(folder, seed, n, vocab, margin=FLIP, tries=300):
    """`n` token ids drawn from `seed` at none of whose positions a router of the plain model decides by less than
    `margin`: the first position that does gets another token until none is left (a position's routers see only the
    tokens up to it, so what is settled stays settled)."""
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
