"""The plain Zovozen implementation pinned by what fixes it beside the design's equations, and the framework's
declarations for the design (configuration, tensors, cache and state needs, rotary tables, pages given back, random
weights): everything that needs no GPU."""
import json
import math

import numpy as np
import pytest

import plain_zovozen as P
from zovozen_models import CONFIGS, SEEDS, tensor_shapes, write_folder


# -- the plain mechanisms -------------------------------------------------------------------------------------------

def test_split_half_rotation_is_a_complex_turn_of_part_of_a_head_with_positions_shrunk():
    rng = np.random.default_rng(1)
    r = {"base": 100.0, "dims": 6, "scaling": {"factor": 4.0}}
    x = rng.standard_normal((5, 2, 10))
    pos = np.array([0, 3, 4, 17, 100])
    got = P.rotate_half(x, pos, r)
    f = np.array([100.0 ** (-2 * i / 6) for i in range(3)]) / 4.0
    z = (x[..., 0:3] + 1j * x[..., 3:6]) * np.exp(1j * pos[:, None, None] * f)
    np.testing.assert_allclose(got[..., 0:3], z.real, atol=1e-12)
    np.testing.assert_allclose(got[..., 3:6], z.imag, atol=1e-12)
    np.testing.assert_array_equal(got[..., 6:], x[..., 6:])          # the rest of the head passes
    np.testing.assert_array_equal(got[0], x[0])                       # position 0 turns nothing
    np.testing.assert_allclose(P.rotary_frequencies({"base": 100.0, "dims": 6}), 4.0 * P.rotary_frequencies(r), rtol=1e-15)


def test_blocks_of_positions_count_from_zero():
    seen = P.chunk_visible(7, 3)
    assert seen[2].tolist() == [True, True, True, False, False, False, False]
    assert seen[3].tolist() == [False, False, False, True, False, False, False]      # a block's first row sees itself only
    assert seen[5].tolist() == [False, False, False, True, True, True, False]
    assert P.chunk_visible(4, None)[3].all()


def _attention_weights(heads=2, kv_heads=1, dim=4, vdim=3, T=6, seed=0):
    rng = np.random.default_rng(seed)
    H = 5
    w = {"a.q": rng.standard_normal((heads * dim, H)), "a.q.b": rng.standard_normal(heads * dim), "a.k": rng.standard_normal((kv_heads * dim, H)),
         "a.k.b": rng.standard_normal(kv_heads * dim), "a.v": rng.standard_normal((kv_heads * vdim, H)), "a.v.b": rng.standard_normal(kv_heads * vdim),
         "a.q.norm": 1 + 0.1 * rng.standard_normal(heads * dim), "a.k.norm": 1 + 0.1 * rng.standard_normal(kv_heads * dim),
         "a.talk": np.eye(heads), "a.temp": np.ones(heads), "a.sink": np.full(heads, -1e9), "a.g": np.zeros((heads * vdim, H)),
         "a.o": np.eye(heads * vdim), "a.o.b": np.zeros(heads * vdim)}
    return w, rng.standard_normal((T, H))


def test_attention_by_hand_sink_mix_and_temperature():
    heads, kv_heads, dim, vdim, T, eps = 2, 1, 4, 3, 6, 1e-6
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 0.5, "mask": {"size": 4}}
    w, h = _attention_weights()
    base = P.talking_attention(h, w, "a", m, eps) * 2.0              # (the gate is sigmoid(0) = 1/2)
    q = P.rmsnorm(h @ w["a.q"].T + w["a.q.b"], w["a.q.norm"], eps).reshape(T, heads, dim)
    k = P.rmsnorm(h @ w["a.k"].T + w["a.k.b"], w["a.k.norm"], eps).reshape(T, kv_heads, dim)
    v = (h @ w["a.v"].T + w["a.v.b"]).reshape(T, kv_heads, vdim)
    v = v / np.sqrt((v * v).mean(-1, keepdims=True) + eps)
    t = 5                                                            # sees positions 4 and 5 only
    for a in range(heads):
        s = np.array([q[t, a] @ k[j, 0] * 0.5 for j in (4, 5)])
        p = np.exp(s) / np.exp(s).sum()
        np.testing.assert_allclose(base[t, a * vdim:(a + 1) * vdim], p @ v[4:6, 0], rtol=1e-9)
    # a sink of score 0 is one more term in the denominator, without a value, not scaled and not times the temperature
    w2 = dict(w, **{"a.sink": np.zeros(heads), "a.temp": np.array([2.0, 0.5])})
    got = P.talking_attention(h, w2, "a", m, eps) * 2.0
    for a, temp in enumerate((2.0, 0.5)):
        s = np.array([q[t, a] @ k[j, 0] * 0.5 * temp for j in (4, 5)])
        np.testing.assert_allclose(got[t, a * vdim:(a + 1) * vdim], (np.exp(s) / (np.exp(s).sum() + 1.0)) @ v[4:6, 0], rtol=1e-9)
    # the mix: head 0 takes head 1's scores
    w3 = dict(w, **{"a.talk": np.array([[0.0, 1.0], [0.0, 1.0]])})
    got = P.talking_attention(h, w3, "a", m, eps) * 2.0
    np.testing.assert_allclose(got[:, :vdim], got[:, vdim:], rtol=1e-9)       # (one key/value head: equal scores, equal results)
    np.testing.assert_allclose(got[:, vdim:], base[:, vdim:], rtol=1e-9)


def test_matrix_memory_against_its_unrolled_sum_and_its_first_token():
    rng = np.random.default_rng(2)
    T, H, heads, dim, vdim, cap, eps = 7, 5, 2, 3, 4, 2.0, 1e-6
    w = {"m.q": rng.standard_normal((heads * dim, H)), "m.k": rng.standard_normal((heads * dim, H)), "m.v": rng.standard_normal((heads * vdim, H)),
         "m.g": np.zeros((heads * vdim, H)), "m.o": np.eye(heads * vdim), "m.norm": np.ones(heads * vdim),
         "m.i": 3 * rng.standard_normal((heads, H)), "m.i.b": rng.standard_normal(heads), "m.f": 3 * rng.standard_normal((heads, H)), "m.f.b": rng.standard_normal(heads)}
    h = rng.standard_normal((T, H))
    m = {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}
    got = P.matrix_memory(h, w, "m", m, eps) * 2.0
    gi = cap * np.tanh((h @ w["m.i"].T + w["m.i.b"]) / cap)
    gf = cap * np.tanh((h @ w["m.f"].T + w["m.f.b"]) / cap)
    gf = -np.log1p(np.exp(-gf))
    assert np.abs(gi).max() <= cap and (gf < 0).all()
    q = (h @ w["m.q"].T).reshape(T, heads, dim) / math.sqrt(dim)
    k, v = (h @ w["m.k"].T).reshape(T, heads, dim), (h @ w["m.v"].T).reshape(T, heads, vdim)
    for a in range(heads):
        top = 0.0
        for t in range(T):
            top = max(gf[t, a] + top, gi[t, a])
            # without the running maximum: weights exp(i_s + sum of later f), numerator and normalizer scaled alike
            wts = np.array([math.exp(gi[s, a] + gf[s + 1:t + 1, a].sum()) for s in range(t + 1)])
            num = sum(wts[s] * (k[s, a] @ q[t, a]) * v[s, a] for s in range(t + 1))
            den = abs(sum(wts[s] * (k[s, a] @ q[t, a]) for s in range(t + 1)))
            o = num * math.exp(-top) / (max(den * math.exp(-top), math.exp(-top)) + 1e-6)
            np.testing.assert_allclose(got[t, a * vdim:(a + 1) * vdim], o / math.sqrt((o * o).mean() + eps), rtol=1e-8, atol=1e-10)
    # the first token's result is plus or minus its value's direction
    for a in range(heads):
        u = v[0, a] / math.sqrt((v[0, a] ** 2).mean() + eps)
        np.testing.assert_allclose(np.abs(got[0, a * vdim:(a + 1) * vdim]), np.abs(u), rtol=1e-3)


def test_routing_by_scores_groups_correction_and_identity_experts():
    H = 4
    w = {"r.router": np.eye(6, H, k=0), "r.correction": np.zeros(6)}
    w["r.router"] = np.array([[2.0, 0, 0, 0], [0, 1.0, 0, 0], [0, 0, 1.5, 0], [0, 0, 0, 0.5], [1.0, 1.0, 0, 0], [0, 0, 1.0, 1.0]])
    h = np.array([[1.0, 0.2, 0.9, 0.1]])
    r = {"experts": 4, "identity": 2, "top": 2}
    z = h @ w["r.router"].T
    s = np.exp(z) / np.exp(z).sum()
    picked, weights = P.route(h, w, "r", r)
    assert picked[0].tolist() == list(np.argsort(-s[0])[:2])
    np.testing.assert_allclose(weights[0], s[0][picked[0]], rtol=1e-12)               # the scores as they are, not normed again
    assert weights.sum() < 1.0
    # a correction moves the choice and leaves the weights alone; it may be negative
    w2 = dict(w, **{"r.correction": np.array([-1.0, 0.0, -1.0, 0.5, -1.0, -1.0])})
    picked, weights = P.route(h, w2, "r", r)
    assert set(picked[0].tolist()) == {3, 1}
    np.testing.assert_allclose(weights[0], s[0][picked[0]], rtol=1e-12)
    # groups of neighbours: with every choice score negative a dropped group must count as minus infinity, not as zero
    w3 = dict(w, **{"r.correction": np.array([-1.0, -2.0, -1.5, -1.6, -3.0, -3.0])})
    picked, _ = P.route(h, w3, "r", dict(r, groups={"count": 3, "keep": 1}))
    best = (s[0] + w3["r.correction"]).reshape(3, 2).max(1).argmax()
    assert sorted(picked[0].tolist()) == [2 * best, 2 * best + 1]
    # an identity expert gives the input itself, times its weight
    wi = dict(w, **{"r.correction": np.array([-9.0, -9.0, -9.0, -9.0, 0.0, 0.0])})
    out = P.mixture(h, wi, "r", {"router": r, "expert": {"ff": 1}})
    np.testing.assert_allclose(out, (s[0][4] + s[0][5]) * h, rtol=1e-12)


def test_a_row_sees_nothing_later_and_the_cut_of_a_prompt_does_not_matter(tmp_path):
    folder = write_folder(tmp_path / "a", CONFIGS["a"], SEEDS["a"])
    cfg, w = P.read_folder(folder)
    tokens = list(np.random.default_rng(4).integers(0, cfg["vocab"], 40))
    whole = P.forward(cfg, w, tokens)
    np.testing.assert_allclose(P.forward(cfg, w, tokens[:25]), whole[:25], rtol=1e-9, atol=1e-9)
    other = tokens[:30] + [(tokens[30] + 1) % cfg["vocab"]] + tokens[31:]
    np.testing.assert_allclose(P.forward(cfg, w, other)[:30], whole[:30], rtol=1e-9, atol=1e-9)
    assert np.abs(P.forward(cfg, w, other)[30:] - whole[30:]).max() > 1e-3


# -- the framework's declarations -------------------------------------------------------------------------------------

@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_declared_tensors_and_needs(name):
    from runtime.engine.loading import build_from_config_dict
    from runtime.cache.pages import ChunkNeed, KVNeed
    raw = CONFIGS[name]
    arch, typed, model = build_from_config_dict(raw)
    assert arch.name == "Zovozen"
    assert {s.name: tuple(s.shape) for s in model.tensor_specs()} == tensor_shapes(raw)
    assert typed.to_dict() == json.loads(json.dumps(raw))
    caches, states = model.cache_needs(), model.state_needs()
    for i, layer in enumerate(raw["layers"]):
        a, r = layer["mixer"]["left"], layer["mixer"]["right"]
        pad = -(-max(a["dim"], a["vdim"]) // 8) * 8
        size = (a.get("mask") or {}).get("size")
        assert caches[i] == (KVNeed(a["kv_heads"], pad) if size is None else ChunkNeed(a["kv_heads"], pad, size, size))
        assert states[i].shape == (r["heads"] * r["dim"] * (r["vdim"] + 1) + r["heads"],) and states[i].dtype == "float32"


def test_blocks_give_back_every_page_before_the_block_of_the_next_token():
    from runtime.cache.manager import CacheManager
    from runtime.cache.pages import ChunkNeed, KVNeed
    need = ChunkNeed(2, 24, 20, 20)
    assert need.first_visible(39) == 20 and need.first_visible(40) == 40 and need.first_visible(0) == 0
    cache = CacheManager({0: need, 1: KVNeed(2, 24, 20)}, n_pages=16, page_size=4, max_requests=2)
    cache.create("r")
    cache.append_many([("r", 39)])
    cache.append_many([("r", 1)])                    # the token at 39 still sees 20..39
    blocks, window = cache.groups
    assert blocks.tables["r"][:6] == [-1] * 5 + [blocks.tables["r"][5]] and blocks.tables["r"][5] >= 0
    cache.append_many([("r", 1)])                    # the token at 40 starts a block: nothing before it is seen again
    assert all(p < 0 for p in blocks.tables["r"][:10]) and blocks.tables["r"][10] >= 0
    assert sum(p >= 0 for p in window.tables["r"]) == 6        # a window of 20 keys still holds 21..40
    for group in cache.groups:
        group.check()


def test_configuration_errors_name_their_place():
    from runtime.config import ConfigError, ZovozenConfig
    good = json.loads(json.dumps(CONFIGS["a"]))

    def broken(change):
        raw = json.loads(json.dumps(good))
        change(raw)
        with pytest.raises(ConfigError) as err:
            ZovozenConfig.from_dict(raw)
        return str(err.value)

    assert "layers[0].mixer.left" in broken(lambda r: r["layers"][0]["mixer"]["left"].pop("vdim"))
    assert "kv_heads" in broken(lambda r: r["layers"][0]["mixer"]["left"].update(heads=3))
    assert "layers[1].mixer.right" in broken(lambda r: r["layers"][1]["mixer"]["right"].pop("gate_cap"))
    assert "left_scale" in broken(lambda r: r["layers"][2]["mixer"].pop("left_scale"))
    assert "dense nor moe" in broken(lambda r: r["layers"][0]["mlp"].update(kind="glu"))
    assert "groups" in broken(lambda r: r["layers"][1]["mlp"]["router"]["groups"].update(count=3))
    assert "cannot be chosen" in broken(lambda r: r["layers"][1]["mlp"]["router"]["groups"].update(keep=1))
    assert "type" in broken(lambda r: r["layers"][1].update(type="serial"))
    assert "turning" in broken(lambda r: r["layers"][0]["mixer"]["left"]["rot"].update(dims=26))
    assert "scaling" in broken(lambda r: r["layers"][0]["mixer"]["left"]["rot"]["scaling"].update(factor=0))
    assert "norm" in broken(lambda r: r.pop("norm"))


def test_rotary_tables_of_the_framework_follow_the_plain_frequencies():
    from runtime.parts import RotaryEmbedding
    r = CONFIGS["s"]["layers"][0]["mixer"]["left"]["rot"]
    part = RotaryEmbedding(32, r["base"], 300, rotary_dim=r["dims"], pairing="split_half", scaling=r["scaling"])
    np.testing.assert_allclose(part.frequencies(), P.rotary_frequencies(r), rtol=1e-14)
    assert part.magnitude() == 1.0
    with pytest.raises(ValueError):
        RotaryEmbedding(8, 100.0, 8, scaling={"factor": 0.0})


def test_random_weights_mode_writes_a_folder_that_the_plain_implementation_reads(tmp_path):
    from runtime.engine import write_random_model
    from runtime.config import preset
    folder = write_random_model(tmp_path / "r", "zovozen-tiny", seed=3)
    cfg, w = P.read_folder(folder)
    assert {k: tuple(v.shape) for k, v in w.items()} == tensor_shapes(preset("zovozen-tiny"))
    logits = P.forward(cfg, w, [1, 2, 3, 4, 5])
    assert logits.shape == (5, cfg["vocab"]) and np.isfinite(logits).all()
