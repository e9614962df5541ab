"""The Zovozen design on the GPU: every new kernel alone against plain float arithmetic of the same operands, then
whole models against the plain implementation (tests/plain_zovozen.py): layer by layer, prompt against token-by-token
decoding, portions down to two tokens, mixed batches with pages and state slots used again, batches against each
request alone, far keys and a block's edge in a model drawn sharp, the first tokens, long decoding, eager and
captured, generation through the scheduler, the replay program."""
import json

import numpy as np
import pytest
import torch

import plain_zovozen as P
import conftest
from conftest import random_tokens
from zovozen_models import CONFIGS, SEEDS, decided_rows, decisive_tokens, plain_logits, write_folder
from trace_tools import Trace

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("zovozen")
    return {name: write_folder(base / name, CONFIGS[name], SEEDS[name], sharp=name == "s") for name in CONFIGS}


def assert_close(got, want, dtype, what="", decided=None):
    """conftest.assert_close; in bfloat16 without the positions at which a router of the plain model has a close call."""
    if dtype == "bfloat16" and decided is not None:
        decided = np.asarray(decided, bool)
        assert decided.mean() > 0.3, f"{what}: too many close calls for the comparison to mean anything"
        got, want = np.asarray(got)[decided], np.asarray(want)[decided]
    conftest.assert_close(got, want, dtype, what)


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.asarray(a), dtype=dtype).cuda().contiguous()


def ints(a):
    return torch.as_tensor(np.asarray(a, dtype=np.int32)).cuda()


def close(got, want, tol=2e-5):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape
    assert np.isfinite(got).all()
    err = np.abs(got - want).max() / max(np.abs(want).max(), 1e-30)
    assert err < tol, f"differs by {err:.3e} (bound {tol})"


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def rounded(a, dtype):
    """The values a tensor of `dtype` holds of the array, as float64."""
    return torch.as_tensor(np.asarray(a), dtype=torch.float32).to(TORCH[dtype]).to(torch.float64).numpy()


# -- kernels alone ----------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, chunk, window, page_size, sink, gate", [
    (4, 2, 24, 16, 20, None, 16, True, True), (1, 1, 10, 24, 1, None, 16, True, False), (20, 4, 64, 64, 100, None, 8, True, True),
    (3, 3, 16, 40, None, None, 16, False, True), (6, 2, 8, 8, None, 33, 4, True, False), (40, 8, 32, 48, 70, None, 16, True, True),
    (16, 4, 128, 128, 128, None, 16, True, True), (32, 8, 96, 80, None, None, 32, False, True), (10, 5, 112, 72, 64, None, 16, True, False),
    (64, 16, 128, 64, 50, None, 16, True, True), (12, 12, 136, 160, 90, None, 16, True, True), (4, 2, 192, 256, 40, None, 16, True, True), (24, 8, 128, 120, 200, None, 16, True, True)])
def test_attention_with_mixed_scores_alone(dtype, heads, kv_heads, dim, vdim, chunk, window, page_size, sink, gate):
    """Rows of three requests (a long portion, a single token far into its sequence, a sequence's first tokens) against
    the plain sums; the pages lie scattered, pages before a row's block are not there (-1 in the table).  One query and
    one key far back in its block are scaled so that one score stands out among hundreds."""
    from runtime.kernels import ops
    rng = np.random.default_rng(heads * 100 + dim)
    pad = -(-max(dim, vdim) // 8) * 8
    lengths, new = [230, 301, 5], [70, 1, 5]                       # cached tokens after the step, rows of the step
    n_pages = sum(-(-n // page_size) for n in lengths) + 3
    order = rng.permutation(n_pages)
    width = max(-(-n // page_size) for n in lengths)
    tables = np.full((3, width), -1, np.int32)
    K = np.zeros((n_pages, kv_heads, page_size, pad))
    V = np.zeros((n_pages, kv_heads, pad, page_size))
    keys = [rng.standard_normal((n, kv_heads, dim)) for n in lengths]
    vals = [rng.standard_normal((n, kv_heads, vdim)) for n in lengths]
    rows = sum(new)
    q = np.zeros((rows, heads, pad))
    q[:, :, :dim] = rng.standard_normal((rows, heads, dim))
    positions = np.concatenate([np.arange(n - m, n) for n, m in zip(lengths, new)])
    seg_of_row = np.concatenate([np.full(m, s) for s, m in enumerate(new)])

    def first_seen(p):
        return p // chunk * chunk if chunk else max(0, p + 1 - window) if window else 0
    # a score that stands out: the last row of the first request and the key at the start of what it sees
    far = first_seen(lengths[0] - 1)
    keys[0][far] *= 2.0
    for h in range(heads):
        q[new[0] - 1, h, :dim] = 2.0 * keys[0][far, h // (heads // kv_heads)]
    used = 0
    for s, n in enumerate(lengths):
        dead = first_seen(n - new[s]) // page_size                  # pages that went back before this step
        for j in range(-(-n // page_size)):
            if j < dead:
                continue
            page = order[used]; used += 1
            tables[s, j] = page
            m = min(page_size, n - j * page_size)
            K[page, :, :m, :dim] = keys[s][j * page_size:j * page_size + m].transpose(1, 0, 2)
            V[page, :, :vdim, :m] = vals[s][j * page_size:j * page_size + m].transpose(1, 2, 0)
    mix = np.eye(heads) + 0.3 * rng.standard_normal((heads, heads))
    temp, sinks = 1 + 0.2 * rng.standard_normal(heads), rng.standard_normal(heads)
    gates = rng.standard_normal((rows, heads * vdim + 3))
    td = TORCH[dtype]
    out = torch.full((rows, heads * vdim), float("nan"), dtype=td, device="cuda")
    ops.attention_talking(dev(q.reshape(rows, -1), td), heads * pad, dev(K, td), dev(V, td), ints(tables), ints(seg_of_row), ints(positions), out,
                          heads, kv_heads, vdim, pad, page_size, dev(mix), 0.2, temp=dev(temp), sink=dev(sinks) if sink else None,
                          window=window, chunk=chunk, gate=dev(gates)[:, :heads * vdim] if gate else None)
    qr = rounded(q, dtype)
    want = np.zeros((rows, heads, vdim))
    group = heads // kv_heads
    stands_out = 0.0
    for r in range(rows):
        s, p = seg_of_row[r], positions[r]
        lo = first_seen(p)
        kk, vv = rounded(keys[s][lo:p + 1], dtype), rounded(vals[s][lo:p + 1], dtype)
        raw = np.stack([kk[:, h // group] @ qr[r, h, :dim] for h in range(heads)]) * 0.2 * rounded(temp, "float32")[:, None]
        sc = rounded(mix, "float32") @ raw
        for h in range(heads):
            top = max(sc[h].max(), sinks[h] if sink else -np.inf)
            e = np.exp(sc[h] - top)
            w = e / (e.sum() + (np.exp(rounded(sinks, "float32")[h] - top) if sink else 0.0))
            want[r, h] = w @ vv[:, h // group]
            if r == new[0] - 1 and lo == far:
                stands_out = max(stands_out, w[0])
    assert stands_out > 0.5 or chunk == 1, "the far key does not stand out"
    want = want.reshape(rows, -1)
    if gate:
        want = want * sigmoid(rounded(gates[:, :heads * vdim], "float32"))
    close(out.float().cpu().numpy(), want, 2e-5 if dtype == "float32" else 1.5e-2)
    # five blocks along a row's keys, merged (more blocks than some rows have tiles of keys)
    out.fill_(float("nan"))
    work = (torch.full((rows * heads * 5 * vdim,), float("nan"), device="cuda"), torch.full((rows * heads * 5 * 2,), float("nan"), device="cuda"))
    ops.attention_talking(dev(q.reshape(rows, -1), td), heads * pad, dev(K, td), dev(V, td), ints(tables), ints(seg_of_row), ints(positions), out,
                          heads, kv_heads, vdim, pad, page_size, dev(mix), 0.2, temp=dev(temp), sink=dev(sinks) if sink else None,
                          window=window, chunk=chunk, gate=dev(gates)[:, :heads * vdim] if gate else None, splits=5, workspace=work)
    close(out.float().cpu().numpy(), want, 2e-5 if dtype == "float32" else 1.5e-2)
    if ops.talking_tiles_ok(td, heads, kv_heads, vdim, pad, page_size):
        # the same rows as tiles of 16 on the matrix cores, the tiles in another order and padded with empty ones
        from runtime.kernels.attention import fill_tasks
        tasks = np.full((-(-rows // 16) + 3 + 2, 4), 0, np.int32)
        tasks[:, 0] = -1
        n = fill_tasks(tasks, new, 16, starts=[a - b for a, b in zip(lengths, new)])
        assert n == sum(-(-m // 16) for m in new)
        tiled = torch.full((rows, heads * vdim), float("nan"), dtype=td, device="cuda")
        ops.attention_talking_tiles(dev(q.reshape(rows, -1), td), dev(K, td), dev(V, td), ints(tables), ints(tasks), ints(positions), tiled,
                                    heads, kv_heads, vdim, pad, page_size, dev(mix), 0.2, temp=dev(temp), sink=dev(sinks) if sink else None,
                                    window=window, chunk=chunk, gate=dev(gates)[:, :heads * vdim] if gate else None)
        close(tiled.float().cpu().numpy(), want, 1.5e-2)
        # three blocks along a tile's keys, merged
        tiled.fill_(float("nan"))
        work = (torch.full((rows * heads * 3 * vdim,), float("nan"), device="cuda"), torch.full((rows * heads * 3 * 2,), float("nan"), device="cuda"))
        ops.attention_talking_tiles(dev(q.reshape(rows, -1), td), dev(K, td), dev(V, td), ints(tables), ints(tasks), ints(positions), tiled,
                                    heads, kv_heads, vdim, pad, page_size, dev(mix), 0.2, temp=dev(temp), sink=dev(sinks) if sink else None,
                                    window=window, chunk=chunk, gate=dev(gates)[:, :heads * vdim] if gate else None, splits=3, workspace=work)
        close(tiled.float().cpu().numpy(), want, 1.5e-2)


@pytest.mark.parametrize("heads, dim, vdim, piece", [(2, 8, 12, 0), (3, 16, 8, 64), (1, 4, 5, 0), (5, 24, 40, 64), (8, 32, 32, 128)])
def test_matrix_memory_over_segments_with_states_carried_and_slots_used_again(heads, dim, vdim, piece):
    """Three steps over four state slots: portions and single rows of several requests in one step, a slot zeroed and
    used again; the gates, the scan over vdim + 1 columns and the finish against the recurrence written out."""
    from runtime.kernels import ops
    rng = np.random.default_rng(heads + dim)
    K, W, C, cap, eps = heads * dim, heads * vdim, vdim + 1, 6.0, 1e-5
    bi, bf = rng.standard_normal(heads), 2 + rng.standard_normal(heads)
    weight = 1 + 0.1 * rng.standard_normal(W)
    state = torch.zeros(4, K * C + heads, device="cuda")
    kept = {s: (np.zeros((heads, dim, vdim)), np.zeros((heads, dim)), np.zeros(heads)) for s in range(4)}
    steps = [([7, 1, 150], [2, 0, 3]), ([1, 1, 1, 1], [3, 1, 0, 2]), ([90, 2, 5], [1, 2, 0])]
    for n, (counts, slots) in enumerate(steps):
        if n == 2:
            state[1].zero_()
            kept[1] = (np.zeros((heads, dim, vdim)), np.zeros((heads, dim)), np.zeros(heads))
        T = sum(counts)
        proj = rng.standard_normal((T, 2 * K + 2 * W + 2 * heads + 3))
        proj[:, 2 * K + 2 * W:2 * K + 2 * W + 2 * heads] *= 4.0                  # gates that reach their cap
        start = np.concatenate(([0], np.cumsum(counts)))
        dp = dev(proj)
        decay, step, top = (torch.empty(T, heads, device="cuda") for _ in range(3))
        vx = torch.empty(T, heads * C, device="cuda")
        g0 = 2 * K + 2 * W
        ops.mlstm_gates(dp[:, g0:g0 + heads], dp[:, g0 + heads:g0 + 2 * heads], dev(bi), dev(bf), dp[:, 2 * K:2 * K + W], decay, step, top, vx,
                        state[:, K * C:], ints(start), ints(slots), heads, vdim, cap, single_rows=all(c == 1 for c in counts))
        o = torch.full((T, heads * C), float("nan"), device="cuda")
        p = 0 if all(c == 1 for c in counts) else piece
        carry = None
        if p:
            sizes = ops.scan_carry(T, p, heads, dim, C, False)
            carry = (torch.empty(sizes[0], device="cuda"), torch.empty(sizes[1], device="cuda"))
        ops.linear_scan(dp[:, :K], dp[:, K:2 * K], vx, decay, o, state, ints(start), ints(slots), heads, dim, C, step=step,
                        q_scale=dim ** -0.5, piece=p, carry=carry)
        out = torch.full((T, W), float("nan"), device="cuda")
        ops.mlstm_finish(o, top, dp[:, 2 * K + W:2 * K + 2 * W], dev(weight), out, heads, vdim, eps)
        pr = rounded(proj, "float32")
        for s, slot in enumerate(slots):
            S, nn, m = (x.copy() for x in kept[slot])
            for t in range(start[s], start[s + 1]):
                gi = cap * np.tanh((pr[t, g0:g0 + heads] + rounded(bi, "float32")) / cap)
                gf = P.log_sigmoid(cap * np.tanh((pr[t, g0 + heads:g0 + 2 * heads] + rounded(bf, "float32")) / cap))
                row = np.zeros((heads, vdim))
                for h in range(heads):
                    qh, kh, vh = pr[t, h * dim:(h + 1) * dim] * dim ** -0.5, pr[t, K + h * dim:K + (h + 1) * dim], pr[t, 2 * K + h * vdim:2 * K + (h + 1) * vdim]
                    new = max(gf[h] + m[h], gi[h])
                    a, b = np.exp(gf[h] + m[h] - new), np.exp(gi[h] - new)
                    S[h] = a * S[h] + b * np.outer(kh, vh)
                    nn[h] = a * nn[h] + b * kh
                    m[h] = new
                    u = (qh @ S[h]) / (max(abs(nn[h] @ qh), np.exp(-new)) + 1e-6)
                    row[h] = u / np.sqrt(np.mean(u * u) + eps)
                want = row.reshape(-1) * rounded(weight, "float32") * sigmoid(pr[t, 2 * K + W:2 * K + 2 * W])
                got = out[t].cpu().numpy()
                assert np.abs(got - want).max() < 3e-5 * max(1.0, np.abs(want).max()), f"step {n}, row {t}"
            kept[slot] = (S, nn, m)
        for slot in range(4):
            S, nn, m = kept[slot]
            have = state[slot].cpu().numpy()
            close(have[:K * C].reshape(heads, dim, C)[:, :, :vdim] + 1.0, S + 1.0, 2e-5)
            close(have[:K * C].reshape(heads, dim, C)[:, :, vdim] + 1.0, nn + 1.0, 2e-5)
            close(have[K * C:] + 1.0, m + 1.0, 2e-5)


@pytest.mark.parametrize("rows, experts, identity, top, groups", [(1, 2, 0, 2, None), (9, 6, 2, 3, (4, 2)), (300, 14, 2, 4, (4, 2)), (70, 3, 1, 2, (2, 1)),
                                                                  (33, 5, 0, 1, None), (40, 4, 4, 3, (2, 2)), (4500, 6, 2, 3, (4, 2)), (50, 130, 6, 5, (8, 3))])
def test_routing_by_scores_with_a_correction_and_groups(rows, experts, identity, top, groups):
    """The choice and the weights against the plain routing (corrections that are negative as well, so that a dropped
    group must count as minus infinity and not as zero); the layout by expert holds every pair of an expert with
    matrices once and no pair of an identity expert.  Steps of few rows route a wave a row, many rows a thread a row."""
    from runtime.kernels import ops
    rng = np.random.default_rng(rows + experts)
    n = experts + identity
    logits = 2.0 * rng.standard_normal((rows, n + 3))
    correction = 0.1 * rng.standard_normal(n) - 0.2
    lg = dev(logits)[:, :n]
    tiles = ops.expert_tiles(rows, top, experts)
    chosen, weights = torch.empty(rows, top, dtype=torch.int32, device="cuda"), torch.empty(rows, top, device="cuda")
    places, tile_expert = torch.empty(tiles * 64, dtype=torch.int32, device="cuda"), torch.empty(tiles, dtype=torch.int32, device="cuda")
    ops.experts_route_scored(lg, dev(correction), top, chosen, weights, experts, groups, places, tile_expert)
    r = {"experts": experts, "identity": identity, "top": top}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    margins = []
    w = {"r.router": np.eye(n), "r.correction": rounded(correction, "float32")}
    picked, share = P.route(rounded(logits[:, :n], "float32"), w, "r", r, margins)
    sure = margins[0] > 1e-4
    assert sure.mean() > 0.9
    got, gw = chosen.cpu().numpy(), weights.cpu().numpy()
    np.testing.assert_array_equal(got[sure], picked[sure])
    close(gw[sure], share[sure], 1e-5)
    place = places.cpu().numpy()
    te = tile_expert.cpu().numpy()
    pairs = sorted(p for p in place if p >= 0)
    flat = got.reshape(-1)
    assert pairs == [i for i, e in enumerate(flat) if e < experts], "every pair of an expert with matrices once, no other"
    for pos, pair in enumerate(place):
        if pair >= 0:
            assert te[pos // 64] == flat[pair]


@pytest.mark.parametrize("dtype", DTYPES)
def test_weighted_sum_over_choices_with_identity_experts_and_the_shared_rows(dtype):
    from runtime.kernels import ops
    rng = np.random.default_rng(3)
    rows, top, dim, experts = 11, 3, 70, 4
    down, weights = rng.standard_normal((rows * top, dim)), rng.random((rows, top))
    chosen = rng.integers(0, experts + 2, (rows, top))
    x, shared = rng.standard_normal((rows, dim)), rng.standard_normal((rows, dim))
    d = dev(down)
    d[torch.as_tensor(chosen.reshape(-1) >= experts).cuda()] = float("nan")         # rows that no product wrote
    y = torch.empty(rows, dim, device="cuda")
    ops.experts_combine(d, dev(weights), ints(chosen), dev(x, TORCH[dtype]), y, experts, shared=dev(shared))
    xr = rounded(x, dtype)
    want = rounded(shared, "float32").copy()
    for r in range(rows):
        for k in range(top):
            want[r] += rounded(weights, "float32")[r, k] * (rounded(down, "float32")[r * top + k] if chosen[r, k] < experts else xr[r])
    close(y.cpu().numpy(), want, 1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim", [40, 1500, 5000])
def test_scaled_sum_of_two_results_normed_into_the_stream_with_its_copy(dtype, dim):
    from runtime.kernels import ops
    rng = np.random.default_rng(dim)
    rows = 5
    x, a, b, w = rng.standard_normal((rows, dim)), rng.standard_normal((rows, dim)), rng.standard_normal((rows, dim)), 1 + 0.1 * rng.standard_normal(dim)
    xs = dev(x)
    copy = torch.empty(rows, dim, dtype=TORCH[dtype], device="cuda")
    ops.post_norm_add(xs, dev(a), dev(w), 1e-5, 1.0, second=(dev(b), 1.2, 0.7), following=(None, 0.0, copy))
    y = 1.2 * rounded(a, "float32") + 0.7 * rounded(b, "float32")
    want = rounded(x, "float32") + y / np.sqrt((y * y).mean(1, keepdims=True) + 1e-5) * rounded(w, "float32")
    close(xs.cpu().numpy(), want, 1e-5)
    close(copy.float().cpu().numpy(), want, 1e-5 if dtype == "float32" else 5e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_squared_relu_behind_a_bias(dtype):
    from runtime.kernels import ops
    rng = np.random.default_rng(8)
    x, b = rng.standard_normal((7, 50)), rng.standard_normal(50)
    out = torch.empty(7, 50, dtype=TORCH[dtype], device="cuda")
    ops.bias_act(dev(x, TORCH[dtype]), dev(b), out, "relu2")
    close(out.float().cpu().numpy(), np.maximum(rounded(x, dtype) + rounded(b, "float32"), 0) ** 2, 1e-5 if dtype == "float32" else 5e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, rot", [(4, 2, 24, 16, 8), (1, 1, 10, 24, 10), (3, 3, 16, 40, 0)])
def test_biases_norm_over_the_projection_split_half_turn_and_normed_values_land_in_the_pages(dtype, heads, kv_heads, dim, vdim, rot):
    from runtime.kernels import ops
    rng = np.random.default_rng(dim)
    rows, page_size, pages, eps = 9, 4, 5, 1e-5
    pad = -(-max(dim, vdim) // 8) * 8
    nq, nk, nv = heads * dim, kv_heads * dim, kv_heads * vdim
    proj, bias = rng.standard_normal((rows, nq + nk + nv + 5)), 0.5 * rng.standard_normal(nq + nk + nv)
    qw, kw = 1 + 0.1 * rng.standard_normal(nq), 1 + 0.1 * rng.standard_normal(nk)
    positions = rng.integers(0, 50, rows)
    slots = rng.permutation(pages * page_size)[:rows]
    half = max(rot // 2, 1)
    freq = np.array([100.0 ** (-2 * i / max(rot, 2)) for i in range(half)]) if rot else np.zeros(1)
    ang = np.arange(64)[:, None] * freq[None, :]
    td = TORCH[dtype]
    q_out = torch.full((rows, heads * pad), float("nan"), dtype=td, device="cuda")
    kc = torch.zeros(pages, kv_heads, page_size, pad, dtype=td, device="cuda")
    vc = torch.zeros(pages, kv_heads, pad, page_size, dtype=td, device="cuda")
    ops.whole_norm_rope_scatter(dev(proj), dev(qw), dev(kw), ints(positions), ints(slots), dev(np.cos(ang)), dev(np.sin(ang)), q_out, kc, vc,
                                heads, kv_heads, dim, vdim, pad, page_size, eps, bias=dev(bias), split_half=True, value_norm=True)
    pr = rounded(proj[:, :nq + nk + nv], "float32") + rounded(bias, "float32")
    q = P.rmsnorm(pr[:, :nq], rounded(qw, "float32"), eps).reshape(rows, heads, dim)
    k = P.rmsnorm(pr[:, nq:nq + nk], rounded(kw, "float32"), eps).reshape(rows, kv_heads, dim)
    v = P.rms(pr[:, nq + nk:].reshape(rows, kv_heads, vdim), eps)
    if rot:
        r = {"base": 100.0, "dims": rot}
        q, k = np.stack([P.rotate_half(q[i:i + 1], [positions[i]], r)[0] for i in range(rows)]), np.stack([P.rotate_half(k[i:i + 1], [positions[i]], r)[0] for i in range(rows)])
    tol = 1e-5 if dtype == "float32" else 5e-3
    got = q_out.float().cpu().numpy().reshape(rows, heads, pad)
    close(got[:, :, :dim], q, tol)
    assert not got[:, :, dim:].any()
    kk, vv = kc.float().cpu().numpy(), vc.float().cpu().numpy()
    for i, slot in enumerate(slots):
        close(kk[slot // page_size, :, slot % page_size, :dim], k[i], tol)
        close(vv[slot // page_size, :, :vdim, slot % page_size], v[i], tol)


# -- whole models -----------------------------------------------------------------------------------------------------

def make_runner(folder, dtype, pages=40, page_size=16, max_requests=4, execution="eager"):
    from runtime.engine import load_model, ModelRunner
    return ModelRunner(load_model(folder, dtype=dtype), n_pages=pages, page_size=page_size, max_requests=max_requests, execution=execution)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_layers_one_by_one_and_a_whole_prompt(folders, name, dtype):
    from runtime.engine import StepEntry
    cfg, w = P.read_folder(folders[name])
    tokens = random_tokens(3, 45, cfg["vocab"])
    layers = []
    want = P.forward(cfg, w, tokens, layers)
    runner = make_runner(folders[name], dtype)
    seen = {}
    runner.layer_tap = lambda i, x: seen.__setitem__(i, x.float().cpu().numpy().copy())
    runner.create("r")
    got = runner.step([StepEntry("r", tokens, list(range(len(tokens))))]).cpu().numpy()
    ok = decided_rows(folders[name], tokens) if dtype == "bfloat16" else np.ones(len(tokens), bool)
    for i, x in enumerate(layers):
        close(seen[i][ok], x[ok], 2e-5 if dtype == "float32" else 4e-2)
    assert_close(got, want, dtype, "whole prompt", ok)


@pytest.mark.parametrize("execution", ["eager", "graph"])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_prompt_then_tokens_one_by_one_and_portions_down_to_two_tokens(folders, name, dtype, execution):
    from runtime.engine import StepEntry
    V = CONFIGS[name]["vocab"]
    tokens = random_tokens(4, 150, V)
    want = plain_logits(folders[name], tokens)
    runner = make_runner(folders[name], dtype, execution=execution)
    runner.create("d")
    got = [runner.step([StepEntry("d", tokens[:97], list(range(97)))]).cpu().numpy()]
    got += [runner.step([StepEntry("d", [t], [0])]).cpu().numpy() for t in tokens[97:]]      # a long run of single tokens
    ok = decided_rows(folders[name], tokens)
    assert_close(np.concatenate(got), want, dtype, "prompt, then decoded", ok)
    runner.release("d")
    runner.create("c")                                     # the same slot and pages once more, now in portions
    at, got = 0, []
    for n in [2, 3, 1, 2, 17, 2, 16, 31, 1, 5, 2, 33, 2, 100]:
        n = min(n, len(tokens) - at)
        got.append(runner.step([StepEntry("c", tokens[at:at + n], list(range(n)))]).cpu().numpy())
        at += n
    assert at == len(tokens)
    assert_close(np.concatenate(got), want, dtype, "portions", ok)
    runner.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_long_portion_walked_in_pieces(folders, dtype):
    """A portion long enough for the memory's scan to walk it in pieces side by side, after a shorter one that leaves a
    state, beside a second request's portion in the same step."""
    from runtime.engine import StepEntry
    from runtime.kernels import ops
    name = "a"
    V = CONFIGS[name]["vocab"]
    long, other = random_tokens(31, 700, V), random_tokens(32, 300, V)
    assert ops.scan_piece(600 + 300, False) > 0
    runner = make_runner(folders[name], dtype, pages=70)
    runner.create("l"); runner.create("o")
    got = [runner.step([StepEntry("l", long[:100], list(range(100)))]).cpu().numpy()]
    out = runner.step([StepEntry("l", long[100:], list(range(600))), StepEntry("o", other, list(range(300)))]).cpu().numpy()
    assert_close(np.concatenate([got[0], out[:600]]), plain_logits(folders[name], long), dtype, "pieces", decided_rows(folders[name], long))
    assert_close(out[600:], plain_logits(folders[name], other), dtype, "the second request", decided_rows(folders[name], other))


@pytest.mark.parametrize("name, dtype, execution", [("b", "float32", "graph"), ("a", "bfloat16", "graph"), ("s", "float32", "eager")])
def test_long_decoding_from_the_first_token(folders, name, dtype, execution):
    """A request decoded one token at a time from its very first token, over a dozen pages, beside a second request that
    joins late and leaves early (its slot and pages go back while the first goes on)."""
    from runtime.engine import StepEntry
    V = CONFIGS[name]["vocab"]
    first, second = random_tokens(61, 200, V), random_tokens(62, 40, V)
    runner = make_runner(folders[name], dtype, pages=24, execution=execution)
    runner.create("x")
    got, got2 = [], []
    for i, t in enumerate(first):
        entries = [StepEntry("x", [t], [0])]
        j = i - 50
        if j == 0:
            runner.create("y")
        if 0 <= j < len(second):
            entries.append(StepEntry("y", [second[j]], [0]))
        out = runner.step(entries).cpu().numpy()
        got.append(out[:1])
        if len(entries) == 2:
            got2.append(out[1:])
        if j == len(second) - 1:
            runner.release("y")
    assert_close(np.concatenate(got), plain_logits(folders[name], first), dtype, "decoded from the first token", decided_rows(folders[name], first))
    assert_close(np.concatenate(got2), plain_logits(folders[name], second), dtype, "the late one", decided_rows(folders[name], second))
    runner.cache.check()


def mixed(V, seed, lengths=(70, 33, 120, 9, 64, 97, 40, 130), live_at_once=4):
    """Up to `live_at_once` live requests: portions of some beside single tokens of others; requests end and new ones
    start on the pages and state slots they gave back; one request sits out some steps."""
    rng = np.random.default_rng(seed)
    seqs = {f"m{i}": random_tokens(seed * 100 + i, n, V) for i, n in enumerate(lengths)}
    waiting, live, fed, trace, step = list(seqs), [], {}, Trace(), 0
    while waiting or live:
        while waiting and len(live) < live_at_once:
            rid = waiting.pop(0); live.append(rid); fed[rid] = 0
        entries, ending = [], []
        for rid in list(live):
            remaining = len(seqs[rid]) - fed[rid]
            if rid == live[0] and step % 5 == 3 and len(live) > 1:
                continue
            if remaining > 12:
                n = max(1, min(int(rng.choice([2, 3, 7, 16, 21, 40])), remaining - 8))
                want = [n - 1] if rng.random() < 0.5 else list(range(n))
            else:
                n, want = 1, [0]
            entries.append((rid, seqs[rid][fed[rid]:fed[rid] + n], want))
            fed[rid] += n
            if fed[rid] == len(seqs[rid]):
                ending.append(rid); live.remove(rid)
        if entries:
            trace.add(entries, end=ending)
        step += 1
    return trace, seqs


@pytest.mark.parametrize("execution", ["eager", "graph"])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_mixed_batches_through_the_replay_program_with_pages_and_slots_used_again(folders, tmp_path, name, dtype, execution):
    from runtime.engine.replay import replay, MAX_LIVE
    V = CONFIGS[name]["vocab"]
    trace, seqs = mixed(V, seed=5)
    assert any(len(s["entries"]) == 4 for s in trace.steps)
    done = []
    runner = replay(folders[name], dtype, tmp_path, trace.peak, trace.lines(), echo=done.append, execution=execution)
    assert done == [f"done {i}" for i in range(len(trace.steps))]
    assert runner.cache.slots.n_slots == MAX_LIVE < len(seqs), "state slots must be used again"
    assert all(sum(-(-len(s) // 16) for s in seqs.values()) > g.pool.n_pages for g in runner.cache.groups), "pages must be used again"
    runner.cache.check()
    per_request = {}
    for step, rows in trace.expect.items():
        data = np.fromfile(tmp_path / f"{step}.f32", dtype="<f4").reshape(len(rows), V)
        for row, (rid, pos) in zip(data, rows):
            per_request.setdefault(rid, []).append((pos, row))
    for rid, items in per_request.items():
        pos = [p for p, _ in items]
        assert_close(np.stack([r for _, r in items]), plain_logits(folders[name], seqs[rid])[pos], dtype, f"request {rid}",
                     decided_rows(folders[name], seqs[rid])[pos])


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_batch_of_unequal_requests_gives_what_each_gives_alone(folders, dtype):
    from runtime.engine import StepEntry
    name = "w"
    V = CONFIGS[name]["vocab"]
    seqs = {k: decisive_tokens(folders[name], 50 + i, n, V, margin=0.01) for i, (k, n) in enumerate({"a": 61, "b": 5, "c": 1, "d": 30}.items())}
    alone = {}
    for k, toks in seqs.items():
        runner = make_runner(folders[name], dtype)
        runner.create(k)
        alone[k] = runner.step([StepEntry(k, toks, list(range(len(toks))))]).cpu().numpy()
    runner = make_runner(folders[name], dtype, max_requests=4)
    for k in seqs:
        runner.create(k)
    got = runner.step([StepEntry(k, toks, list(range(len(toks)))) for k, toks in seqs.items()]).cpu().numpy()
    at = 0
    for k, toks in seqs.items():
        piece = got[at:at + len(toks)]
        at += len(toks)
        err = np.abs(piece - alone[k]).max() / np.abs(alone[k]).max()
        assert err < (1e-5 if dtype == "float32" else 2e-2), f"request {k} differs from itself alone by {err:.2e}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_keys_a_block_s_edge_the_sink_and_old_state_in_a_model_drawn_sharp(folders, dtype):
    """In the sharp model a query's result hangs on single keys and the memory keeps the first tokens.  The test first
    shows that blocks one position longer or shorter, a sink left out and a memory that started late would each move
    the logits by many times the bound; then a prompt of many pages cut in the middle of a page and of a block, and
    tokens one by one over the borders of pages and blocks, hold the bound."""
    from runtime.engine import StepEntry
    name = "s"
    cfg, w = P.read_folder(folders[name])
    tokens = decisive_tokens(folders[name], 9, 410, cfg["vocab"])
    want = plain_logits(folders[name], tokens)
    scale = np.abs(want).max()
    for delta in (-1, 1):
        off = json.loads(json.dumps(cfg))
        off["layers"][0]["mixer"]["left"]["mask"]["size"] += delta
        assert np.abs(P.forward(off, w, tokens)[60:] - want[60:]).max() > 1e-3 * scale, "blocks one position off do not show"
    no_sink = dict(w)
    for i in range(len(cfg["layers"])):
        no_sink[f"l{i}.mix.left.sink"] = np.full_like(w[f"l{i}.mix.left.sink"], -1e9)
    assert np.abs(P.forward(cfg, no_sink, tokens) - want).max() > 1e-3 * scale, "a sink left out does not show"
    late = P.forward(cfg, w, tokens[192:])                  # (a start at a block's border: only the memory and the far keys differ)
    assert np.abs(late[-40:] - want[-40:]).max() > 0.01 * scale, "the first 192 tokens do not reach the last 40"
    runner = make_runner(folders[name], dtype, pages=60)
    runner.create("f")
    got = [runner.step([StepEntry("f", tokens[:201], list(range(201)))]).cpu().numpy(),
           runner.step([StepEntry("f", tokens[201:376], list(range(175)))]).cpu().numpy()]
    got += [runner.step([StepEntry("f", [t], [0])]).cpu().numpy() for t in tokens[376:]]
    got = np.concatenate(got)
    ok = decided_rows(folders[name], tokens)
    assert_close(got, want, dtype, "far keys", ok)
    assert_close(got[:3], want[:3], dtype, "the first tokens")
    assert_close(got[44:52], want[44:52], dtype, "around the first border of blocks", ok[44:52])
    assert_close(got[380:388], want[380:388], dtype, "decoded over a border of blocks", ok[380:388])


def test_blocks_give_their_pages_back(folders):
    """Model a sees blocks of 20 and of 37 positions, with two shapes of heads: three groups of pages, each keeping little
    more than a block.  A request far longer than any pool, decoded in portions and single tokens."""
    from runtime.engine import StepEntry
    name = "a"
    tokens = random_tokens(13, 330, CONFIGS[name]["vocab"])
    want = plain_logits(folders[name], tokens)
    runner = make_runner(folders[name], "float32", pages=8, page_size=16)       # 128 slots for 330 tokens
    assert len(runner.cache.groups) == 3
    runner.create("w")
    got, at = [], 0
    for n in [40, 33, 1, 1, 50, 2, 64, 1, 1, 1, 30, 60, 44, 1, 1]:
        got.append(runner.step([StepEntry("w", tokens[at:at + n], list(range(n)))]).cpu().numpy())
        at += n
    assert at == len(tokens)
    # A position at which a memory's sum nearly cancels before it is normed magnifies float rounding (here one, by a
    # factor of twenty, however the prompt is cut): all but two positions hold the bound, those stay within ten times it.
    got = np.concatenate(got)
    err = np.abs(got - want).max(axis=1) / np.abs(want).max()
    worst = np.argsort(-err)[:2]
    assert err[worst].max() < 10 * conftest.F32_TOL
    rest = np.ones(len(tokens), bool)
    rest[worst] = False
    assert_close(got[rest], want[rest], "float32", "blocks that give pages back")
    assert all(g.pool.used <= 3 for g in runner.cache.groups), "pages before the last block are given back"
    runner.cache.check()


@pytest.mark.parametrize("name, dtype, execution, overlap", [("a", "float32", "graph", True), ("a", "float32", "eager", False),
                                                             ("w", "bfloat16", "graph", True), ("n", "float32", "graph", True)])
def test_greedy_generation_through_the_scheduler(folders, name, dtype, execution, overlap):
    from runtime.engine.scheduler import Engine
    cfg, w = P.read_folder(folders[name])
    prompts = [random_tokens(70 + i, n, cfg["vocab"]) for i, n in enumerate([11, 3, 26, 1, 40])]
    engine = Engine.from_folder(folders[name], dtype=dtype, pages=24, page_size=16, execution=execution,
                                max_active=3, token_budget=24, prefill_chunk=9, overlap=overlap)
    got = engine.generate(prompts, max_new_tokens=10)
    for prompt, new in zip(prompts, got):
        assert len(new) == 10
        logits = P.forward(cfg, w, prompt + new)[len(prompt) - 1:-1]
        for row, token in zip(logits, new):       # every picked token is the plain model's best or within rounding of it, given the same past
            assert row.max() - row[token] < (1e-4 if dtype == "float32" else 0.05) * (row.max() - row.min())
    engine.runner.cache.check()
    assert not engine.runner.cache.lengths, "every request gave back what it held"


def test_command_line_serves_the_design(folders, tmp_path):
    """`python -m runtime` chooses the design by config.json: requests of a file against a folder, in float32, give the
    plain model's greedy tokens; the named configuration with random weights generates and reports its state slots."""
    import os, subprocess, sys
    from conftest import ROOT
    cfg, w = P.read_folder(folders["n"])
    requests = [{"key": "x", "prompt": [1, 2, 3, 4, 5, 6, 7], "max_new_tokens": 5}, {"key": "y", "prompt": [9], "max_new_tokens": 4}]
    (tmp_path / "requests.json").write_text(json.dumps(requests))
    env = dict(os.environ, PYTHONPATH=str(ROOT))
    proc = subprocess.run([sys.executable, "-m", "runtime", "--checkpoint", str(folders["n"]), "--dtype", "float32",
                           "--requests", str(tmp_path / "requests.json"), "--policy", "chunked", "--pages", "16",
                           "--token-budget", "6", "--prefill-chunk", "3"], capture_output=True, text=True, timeout=300, env=env, cwd=str(tmp_path))
    assert proc.returncode == 0, proc.stderr[-2000:]
    by_key = {r["key"]: r for r in json.loads(proc.stdout)["requests"]}
    assert by_key["x"]["generated"] == P.greedy(cfg, w, [1, 2, 3, 4, 5, 6, 7], 5)
    assert by_key["y"]["generated"] == P.greedy(cfg, w, [9], 4)
    proc = subprocess.run([sys.executable, "-m", "runtime", "--model", "zovozen-tiny", "--tokens", "5,6,7", "--max-new-tokens", "3",
                           "--overlap", "--report"], capture_output=True, text=True, timeout=300, env=env, cwd=str(tmp_path))
    assert proc.returncode == 0, proc.stderr[-2000:]
    out = json.loads(proc.stdout)
    assert out["weights"] == "random-zovozen-tiny" and len(out["requests"][0]["generated"]) == 3
    assert out["runner"]["replays"] >= 1 and out["runner"]["cache"][0]["resident_pages"] == 0


# -- configurations drawn at random -----------------------------------------------------------------------------------

def random_config(seed):
    """A configuration drawn at random: sizes, head counts, blocks of positions, rotation, constants, the kinds of
    feed-forward in an order of their own.  Every second draw has sizes of the order of a small real model (heads of 64
    to 128, a width of a few hundred, a dozen experts)."""
    from zovozen_models import config, dense, layer, left, moe, right
    rng = np.random.default_rng(1000 + seed)
    pick = lambda *values: values[int(rng.integers(len(values)))]
    big = seed % 2 == 1
    width = pick(192, 264, 384) if big else pick(40, 72, 100, 136)

    def feed_forward():
        kind = rng.random()
        if kind < 0.15:
            return None
        if kind < 0.4:
            return dense(pick(256, 520) if big else pick(24, 60, 100))
        count = pick(1, 2, 4)
        per = pick(2, 3, 4) if big else pick(1, 2, 3)
        outputs = count * per
        identity = min(pick(0, 0, 1, 2), outputs - 1)
        keep = int(rng.integers(1, count + 1))
        top = int(rng.integers(1, min(keep * per, 6) + 1))
        groups = None if count == 1 and rng.random() < 0.5 else (count, keep)
        return moe(pick(48, 80, 136) if big else pick(8, 20, 33), outputs - identity, top, identity, groups, pick(None, 16, 40))

    layers = []
    for _ in range(int(rng.integers(2, 6))):
        kv_heads = pick(1, 2, 3)
        heads = kv_heads * pick(1, 2, 4)
        dim = pick(64, 96, 128) if big else pick(6, 16, 24, 40)
        vdim = pick(dim, 32, 64, 80, 128) if big else pick(dim, 8, 12, 48)
        dims = pick(dim, dim // 2, 2, 4)
        rot = pick(None, (float(pick(50.0, 10000.0, 1e6)), dims - dims % 2 or 2, pick(None, 2.0, 8.0)))
        chunk = pick(None, 1, 2, 15, 16, 17, 33, 64, 90)
        mem_heads = pick(1, 2, 4, 6)
        layers.append(layer(left(heads, kv_heads, dim, vdim, float(rng.uniform(0.08, 0.4)), chunk, rot),
                            right(mem_heads, pick(32, 64) if big else pick(4, 8, 20), pick(32, 64, 100) if big else pick(5, 8, 16, 24), float(rng.uniform(2.0, 20.0))),
                            float(rng.uniform(0.3, 2.0)), float(rng.uniform(0.3, 2.0)), feed_forward()))
    return config(int(rng.integers(40, 700)), width, pick(1e-5, 1e-6), layers)


_DRAWN = {}


@pytest.fixture(scope="module")
def drawn(tmp_path_factory):
    """seed -> (configuration, folder, trace, sequences), made once for both dtypes."""
    def make(seed):
        if seed not in _DRAWN:
            cfg = random_config(seed)
            folder = write_folder(tmp_path_factory.mktemp(f"drawn{seed}") / "model", cfg, 300 + seed, sharp=seed % 3 == 0)
            lengths = (70, 33, 90, 9, 48) if seed % 2 else (70, 33, 120, 9, 64, 97)
            trace, seqs = mixed(cfg["vocab"], seed=40 + seed, lengths=lengths)
            _DRAWN[seed] = (cfg, folder, trace, seqs)
        return _DRAWN[seed]
    return make


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", range(16))
def test_configurations_drawn_at_random_in_mixed_batches(drawn, tmp_path, seed, dtype):
    """float32 holds its bound at every position but the few that the design itself magnifies (see
    test_blocks_give_their_pages_back).  In bfloat16 a router's close call, or a memory's sign at a first position, may
    fall otherwise than in float64 and reaches the positions after it through caches and states, so every position is
    compared alone: the median holds half the bound and at most a quarter of the positions miss it."""
    from runtime.engine.replay import replay
    cfg, folder, trace, seqs = drawn(seed)
    V = cfg["vocab"]
    done = []
    runner = replay(folder, dtype, tmp_path / "out", trace.peak, trace.lines(), echo=done.append, execution="graph" if seed % 2 else "eager")
    assert done == [f"done {i}" for i in range(len(trace.steps))]
    runner.cache.check()
    errs = []
    for step, rows in trace.expect.items():
        data = np.fromfile(tmp_path / "out" / f"{step}.f32", dtype="<f4").reshape(len(rows), V).astype(np.float64)
        for row, (rid, pos) in zip(data, rows):
            want = plain_logits(folder, seqs[rid])[pos]
            assert np.isfinite(row).all()
            if dtype == "float32":
                errs.append(np.abs(row - want).max() / np.abs(plain_logits(folder, seqs[rid])).max())
            else:
                errs.append(np.linalg.norm(row - want) / np.linalg.norm(want))
    errs = np.sort(np.asarray(errs))
    if dtype == "float32":
        assert errs[-1] < 20 * conftest.F32_TOL and errs[:-3].max() < conftest.F32_TOL, f"float32: worst {errs[-4:]}"
    else:
        assert (errs > conftest.BF16_RMSE).mean() <= 0.25 and np.median(errs) < 0.5 * conftest.BF16_RMSE, f"bfloat16: median {np.median(errs):.3e}, worst {errs[-4:]}"
