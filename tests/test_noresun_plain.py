"""The plain Noresun implementation pinned by what fixes it beside the design's equations, and the framework's
declarations for the design (configuration, tensors, schedule, cache and state needs, rotary tables, random weights):
everything that needs no GPU."""
import json
import math

import numpy as np
import pytest

import plain_noresun as P
from noresun_models import CONFIGS, SEEDS, tensor_shapes, write_folder


# -- the plain mechanisms -------------------------------------------------------------------------------------------

def test_min_gru_against_its_closed_form_and_its_carried_state():
    rng = np.random.default_rng(0)
    T, H, W = 9, 5, 4
    w = {"m.z": rng.standard_normal((W, H)), "m.z.b": rng.standard_normal(W), "m.x": rng.standard_normal((W, H)),
         "m.x.b": rng.standard_normal(W), "m.g": rng.standard_normal((W, H)), "m.o": np.eye(W)}
    h = rng.standard_normal((T, H))
    got = P.min_gru(h, w, "m", {"width": W})
    z = 1 / (1 + np.exp(-(h @ w["m.z"].T + w["m.z.b"])))
    u = h @ w["m.x"].T + w["m.x.b"]
    cand = np.where(u >= 0, u + 0.5, 1 / (1 + np.exp(-u)))
    g = h @ w["m.g"].T
    # closed form: S_t = sum_j z_j c_j prod_{j < i <= t} (1 - z_i)
    for t in range(T):
        S = sum(z[j] * cand[j] * np.prod(1 - z[j + 1:t + 1], axis=0) for j in range(t + 1))
        np.testing.assert_allclose(got[t], S * g[t] / (1 + np.exp(-g[t])), rtol=1e-12)
    # the candidate is continuous at zero and the state carries over a cut
    assert abs((0.0 + 0.5) - 1 / (1 + math.exp(-0.0))) < 1e-15
    first = P.min_gru(h[:4], w, "m", {"width": W})
    np.testing.assert_allclose(first, got[:4], rtol=1e-12)
    S4 = sum(z[j] * cand[j] * np.prod(1 - z[j + 1:4], axis=0) for j in range(4))
    np.testing.assert_allclose(P.min_gru(h[4:], w, "m", {"width": W}, state=S4), got[4:], rtol=1e-12)


def test_rotation_of_neighbouring_pairs_is_a_complex_turn_of_part_of_a_head():
    rng = np.random.default_rng(1)
    r = {"base": 100.0, "dims": 6}
    x = rng.standard_normal((5, 2, 10))
    pos = np.array([0, 3, 4, 17, 100])
    got = P.rotate_interleaved(x, pos, r)
    f = np.array([100.0 ** (-2 * i / 6) for i in range(3)])
    z = (x[..., 0:6:2] + 1j * x[..., 1:6:2]) * np.exp(1j * pos[:, None, None] * f)
    np.testing.assert_allclose(got[..., 0:6:2], z.real, atol=1e-12)
    np.testing.assert_allclose(got[..., 1:6:2], z.imag, atol=1e-12)
    np.testing.assert_array_equal(got[..., 6:], x[..., 6:])          # the rest of the head passes
    np.testing.assert_array_equal(got[0], x[0])                       # position 0 turns nothing


def test_frequencies_scaled_by_wavelength():
    r = {"base": 10000.0, "dims": 16, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 256}}
    plain = P.rotary_frequencies({"base": 10000.0, "dims": 16})
    got = P.rotary_frequencies(r)
    wavelength = 2 * math.pi / plain
    short, long = wavelength < 256 / 4.0, wavelength > 256 / 1.0
    assert short.any() and long.any() and (~short & ~long).any(), "the test wants pairs of all three kinds"
    np.testing.assert_array_equal(got[short], plain[short])
    np.testing.assert_allclose(got[long], plain[long] / 8.0, rtol=1e-15)
    mid = ~short & ~long
    assert ((got[mid] > plain[mid] / 8.0) & (got[mid] < plain[mid])).all()
    # at the borders the middle rule meets its neighbours
    for wl, want in ((256 / 4.0, 1.0), (256 / 1.0, 1 / 8.0)):
        s = (256 / wl - 1.0) / (4.0 - 1.0)
        assert abs(((1 - s) / 8.0 + s) - want) < 1e-15


def test_sigmoid_attention_by_hand_with_the_window_s_edge_and_grouped_heads():
    """Two query heads over one key head, keys and values of different sizes, identity projections, no rotation worth
    speaking of: every weight is a sigmoid of one product, keys outside the window weigh nothing, nothing is normed."""
    D, V, T = 2, 3, 6
    m = {"heads": 2, "kv_heads": 1, "dim": D, "vdim": V, "scale": 0.5, "mask": {"size": 3}, "rot": {"base": 10.0, "dims": 2}}
    rng = np.random.default_rng(2)
    h = rng.standard_normal((T, 4))
    w = {"a.q": rng.standard_normal((2 * D, 4)), "a.q.norm": np.ones(2 * D), "a.pb": np.array([-1.0, 0.5]), "a.o": np.eye(2 * V)}
    k = rng.standard_normal((T, 1, D))
    v = rng.standard_normal((T, 1, V))
    got = P.sigmoid_attention(h, w, "a", m, 1e-6, (k, v)).reshape(T, 2, V)
    qp = h @ w["a.q"].T
    q = (qp / np.sqrt((qp ** 2).mean(axis=1, keepdims=True) + 1e-6)).reshape(T, 2, D)      # one norm over both heads
    q = P.rotate_interleaved(q, np.arange(T), m["rot"])
    for i in range(T):
        for head in range(2):
            want = np.zeros(V)
            for j in range(T):
                if 0 <= i - j < 3:
                    want += v[j, 0] / (1 + math.exp(-(q[i, head] @ k[j, 0] * 0.5 + w["a.pb"][head])))
            np.testing.assert_allclose(got[i, head], want, rtol=1e-12)
    # one key more in the window changes a late row, and only rows that reach that far back
    wider = P.sigmoid_attention(h, w, "a", {**m, "mask": {"size": 4}}, 1e-6, (k, v)).reshape(T, 2, V)
    np.testing.assert_allclose(wider[:3], got[:3], rtol=1e-12)
    assert np.abs(wider[3:] - got[3:]).min() > 1e-6


def test_pair_rows_and_the_first_token():
    assert P.bigram_rows([5, 9, 9, 0], 7, 3, 2) == [7, (5 * 3 + 9 * 2) % 7, (9 * 3 + 9 * 2) % 7, (9 * 3) % 7]
    w = {"embed": np.arange(12.0).reshape(4, 3), "bigram": np.arange(100, 124.0).reshape(8, 3)}
    x = P.embed([2, 1], w, {"scale": 0.5, "bigram": {"buckets": 7, "mul_prev": 3, "mul_cur": 2}})
    np.testing.assert_allclose(x[0], w["embed"][2] * 0.5 + w["bigram"][7])
    np.testing.assert_allclose(x[1], w["embed"][1] * 0.5 + w["bigram"][(2 * 3 + 1 * 2) % 7])
    np.testing.assert_allclose(P.embed([3], w, {"scale": 2.0}), w["embed"][[3]] * 2.0)


def test_routed_experts_choose_by_logit_and_weigh_by_the_softmax_of_the_chosen():
    H, F = 3, 2
    w = {"f.router": np.array([[1.0, 0, 0], [0, 1.0, 0], [0, 0, 1.0], [1.0, 0, 0]]), "f.router.b": np.array([0.0, 0.1, -5.0, 0.0])}
    rng = np.random.default_rng(3)
    for e in range(4):
        w[f"f.e{e}.up"], w[f"f.e{e}.down"] = rng.standard_normal((F, H)), rng.standard_normal((H, F))
    h = np.array([[2.0, 1.0, 0.0], [0.0, 0.0, 9.0]])
    got = P.routed_experts(h, w, "f", {"router": {"experts": 4, "top": 2}})

    def expert(e, x):
        return w[f"f.e{e}.down"] @ (np.maximum(w[f"f.e{e}.up"] @ x, 0.0) ** 2)
    # row 0: logits (2, 1.1, -5, 2): experts 0 and 3 tie, the lower index first, equal weights
    np.testing.assert_allclose(got[0], 0.5 * expert(0, h[0]) + 0.5 * expert(3, h[0]), rtol=1e-12)
    # row 1: logits (0, 0.1, 4, 0): experts 2 and 1
    a, b = math.exp(4.0), math.exp(0.1)
    np.testing.assert_allclose(got[1], (a * expert(2, h[1]) + b * expert(1, h[1])) / (a + b), rtol=1e-12)


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
def test_declared_tensors_schedule_and_needs(name):
    from runtime.engine.loading import build_from_config_dict
    from runtime.cache import KVNeed
    raw = CONFIGS[name]
    arch, typed, model = build_from_config_dict(raw)
    assert arch.name == "Noresun"
    assert {s.name: tuple(s.shape) for s in model.tensor_specs()} == tensor_shapes(raw)
    assert typed.to_dict() == raw
    for i, layer in enumerate(raw["layers"]):
        assert model.schedule[i].reads == layer["mixer"].get("kv_from")
    states = model.state_needs()
    assert ("embedding" in states) == ("bigram" in raw["embedding"])
    for i, layer in enumerate(raw["layers"]):
        assert (i in states) == (layer["type"] == "mingru")
        if layer["type"] == "mingru":
            assert states[i].shape == (layer["mixer"]["width"],) and states[i].dtype == "float32"


def test_a_cache_keeps_what_its_furthest_reader_looks_back_over():
    from runtime.engine.loading import build_from_config_dict
    from runtime.cache import KVNeed
    _, _, model = build_from_config_dict(CONFIGS["a"])
    assert model.cache_needs() == {0: KVNeed(2, 24, 37)}            # layer 0 looks back over 20 keys, its reader over 37
    assert model.layers[0].mixer.window == 20 and model.layers[2].mixer.window == 37
    _, _, model = build_from_config_dict(CONFIGS["s"])
    assert model.cache_needs() == {0: KVNeed(1, 32, 48), 2: KVNeed(2, 32, None)}
    assert not build_from_config_dict(CONFIGS["g"])[2].cache_needs()


def test_configuration_errors_name_their_place():
    from runtime.config import ConfigError, NoresunConfig
    good = json.loads(json.dumps(CONFIGS["a"]))

    def broken(change):
        raw = json.loads(json.dumps(good))
        change(raw)
        with pytest.raises(ConfigError) as err:
            NoresunConfig.from_dict(raw)
        return str(err.value)

    assert "layers[0].mixer" in broken(lambda r: r["layers"][0]["mixer"].pop("vdim"))
    assert "kv_heads" in broken(lambda r: r["layers"][0]["mixer"].update(heads=3))
    assert "kv_from" in broken(lambda r: r["layers"][2]["mixer"].update(kv_from=1))          # layer 1 is no attention
    assert "kv_from" in broken(lambda r: r["layers"][0]["mixer"].update(kv_from=2))          # not an earlier layer
    assert "equal" in broken(lambda r: r["layers"][2]["mixer"].update(dim=32))
    assert "moe" in broken(lambda r: r["layers"][0]["mlp"].update(kind="dense"))
    assert "experts" in broken(lambda r: r["layers"][0]["mlp"]["router"].update(top=7))
    assert "type" in broken(lambda r: r["layers"][1].update(type="gru"))
    assert "turning" in broken(lambda r: r["layers"][0]["mixer"]["rot"].update(dims=26))
    assert "postln_alpha" in broken(lambda r: r.pop("postln_alpha"))
    assert "embedding.bigram" in broken(lambda r: r["embedding"]["bigram"].pop("buckets"))
    assert "scaling" in broken(lambda r: r["layers"][0]["mixer"]["rot"]["scaling"].update(low=9.0))


def test_rotary_tables_of_the_framework_follow_the_plain_frequencies():
    from runtime.parts import RotaryEmbedding
    r = CONFIGS["s"]["layers"][0]["mixer"]["rot"]
    part = RotaryEmbedding(r["dims"], r["base"], 300, rotary_dim=r["dims"], pairing="interleaved", scaling=r["scaling"])
    np.testing.assert_allclose(part.frequencies(), P.rotary_frequencies(r), rtol=1e-14)
    assert part.magnitude() == 1.0
    plain = RotaryEmbedding(10, 500.0, 8, pairing="interleaved")
    np.testing.assert_allclose(plain.frequencies(), P.rotary_frequencies({"base": 500.0, "dims": 10}), rtol=1e-14)
    with pytest.raises(ValueError):
        RotaryEmbedding(8, 100.0, 8, scaling={"factor": 2.0, "low": 4.0, "high": 1.0, "original": 64})


def test_random_weights_mode_writes_a_folder_that_the_plain_implementation_reads(tmp_path):
    from runtime.engine import write_random_model
    from runtime.config import preset
    folder = write_random_model(tmp_path / "r", "noresun-tiny", seed=3)
    cfg, w = P.read_folder(folder)
    assert {k: tuple(v.shape) for k, v in w.items()} == tensor_shapes(preset("noresun-tiny"))
    logits = P.forward(cfg, w, [1, 2, 3, 4, 5])
    assert logits.shape == (5, cfg["vocab"]) and np.isfinite(logits).all()
