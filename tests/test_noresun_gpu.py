"""The Noresun design on the GPU: every new kernel alone against plain float arithmetic of the same operands, then
whole models against the plain implementation (tests/plain_noresun.py): layer by layer, prompt against token-by-token
decoding, portions down to two tokens, mixed batches with pages and state slots used again, batches against each
request alone, far keys and the window's edge in a model drawn sharp, the first tokens, long decoding, eager and
captured, generation through the scheduler, the command line, configurations drawn at random."""
import json
import math

import numpy as np
import pytest
import torch

import plain_noresun as P
import conftest
from conftest import random_tokens
from noresun_models import CONFIGS, SEEDS, decided_rows, decisive_tokens, plain_logits, smallest_margins, write_folder
from trace_tools import Trace

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("noresun")
    return {name: write_folder(base / name, CONFIGS[name], SEEDS[name], sharp=name == "s") for name in CONFIGS}


def assert_close(got, want, dtype, what="", decided=None):
    """conftest.assert_close; in bfloat16 without the positions at which a router of the plain model has a close call
    (`decided`: noresun_models.decided_rows of the compared positions), which must stay few."""
    if dtype == "bfloat16" and decided is not None:
        decided = np.asarray(decided, bool)
        assert decided.mean() > 0.7, f"{what}: too many close calls for the comparison to mean anything"
        got, want = np.asarray(got)[decided], np.asarray(want)[decided]
    conftest.assert_close(got, want, dtype, what)


def check_trace(trace, folder, out_dir, dtype, vocab, sequences):
    """Every row that a replay wrote against the plain implementation (trace_tools.Trace.check with this file's assert_close)."""
    per_request = {}
    for step, rows in trace.expect.items():
        data = np.fromfile(out_dir / f"{step}.f32", dtype="<f4").reshape(len(rows), vocab)
        for row, (rid, pos) in zip(data, rows):
            per_request.setdefault(rid, []).append((pos, row))
    assert {int(p.stem) for p in out_dir.glob("*.f32")} == set(trace.expect), "a step without wanted rows wrote a file, or a wanted one is missing"
    for rid, items in per_request.items():
        pos = [p for p, _ in items]
        assert_close(np.stack([r for _, r in items]), plain_logits(folder, sequences[rid])[pos], dtype, f"request {rid}",
                     decided_rows(folder, sequences[rid])[pos])


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


# -- kernels alone ----------------------------------------------------------------------------------------------------

def plain_scan(a, b, g, bz, bx, S):
    out = np.zeros_like(a)
    for t in range(a.shape[0]):
        z = sigmoid(a[t] + bz)
        u = b[t] + bx
        S = (1 - z) * S + z * np.where(u >= 0, u + 0.5, sigmoid(u))
        out[t] = S * g[t] * sigmoid(g[t])
    return out, S


@pytest.mark.parametrize("width, extra", [(5, 0), (64, 3), (200, 8)])
@pytest.mark.parametrize("piece", [0, 4, 64])
def test_min_gru_scan_over_segments_with_states_carried_and_slots_used_again(width, extra, piece):
    """Three steps over four state slots: portions and single rows of several requests in one step, a segment without
    rows, a slot zeroed and used again; whole segments and pieces give the same."""
    from runtime.kernels import ops
    rng = np.random.default_rng(width + piece)
    bz, bx = rng.standard_normal(width), rng.standard_normal(width)
    state = torch.zeros(4, width + 2, device="cuda")[:, :width]            # (rows of a wider buffer)
    kept = {s: np.zeros(width) for s in range(4)}
    steps = [([7, 1, 130], [2, 0, 3]), ([1, 1, 1, 1], [3, 1, 0, 2]), ([66, 0, 5], [1, 2, 0])]
    for n, (counts, slots) in enumerate(steps):
        if n == 2:
            state[1].zero_()
            kept[1] = np.zeros(width)
        T = sum(counts)
        proj = rng.standard_normal((T, 3 * width + extra))
        out = torch.full((T, width), float("nan"), device="cuda")
        start = np.concatenate(([0], np.cumsum(counts)))
        p = 0 if all(c == 1 for c in counts) else piece
        carry = torch.empty(2 * (T // p + len(counts)) * width, device="cuda") if p else None
        ops.mingru_scan(dev(proj), dev(bz), dev(bx), state, ints(start), ints(slots), out, width, piece=p, carry=carry)
        for s, slot in enumerate(slots):
            rows = slice(start[s], start[s + 1])
            if counts[s] == 0:
                continue
            want, kept[slot] = plain_scan(proj[rows, :width], proj[rows, width:2 * width], proj[rows, 2 * width:3 * width], bz, bx, kept[slot])
            close(out[rows].cpu().numpy(), want, 1e-5)
        for slot in range(4):
            close(state[slot].cpu().numpy() + 1.0, kept[slot] + 1.0, 1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows, experts, top, hidden, ff", [(1, 4, 1, 24, 16), (9, 5, 3, 20, 7), (150, 16, 2, 64, 40), (70, 3, 3, 100, 12), (8, 6, 2, 1040, 520),
                                                             (1100, 6, 3, 72, 136), (3000, 20, 1, 64, 48)])
def test_routed_experts_route_and_products(dtype, rows, experts, top, hidden, ff):
    """Choice and weights against a plain top-k (with a tie that the lower index wins); the layout by expert holds every
    pair once, in its expert's tiles; both products against plain arithmetic of the same operands.  The last two
    cases have rows enough for the form in which a block takes two tiles of one expert (runs of odd and even length, a
    product deeper than a whole number of steps)."""
    from runtime.kernels import ops
    rng = np.random.default_rng(rows + experts)
    td = TORCH[dtype]
    logits = rng.standard_normal((rows, experts + 5))
    if experts > 1:
        logits[0, 1] = logits[0, 0]                                      # a tie
    bias = rng.standard_normal(experts)
    if experts > 1:
        bias[1] = bias[0]
    lg = dev(logits)[:, :experts]
    tiles = ops.expert_tiles(rows, top, experts)
    chosen, weights = torch.empty(rows, top, dtype=torch.int32, device="cuda"), torch.empty(rows, top, device="cuda")
    places, tile_expert = torch.empty(tiles * 64, dtype=torch.int32, device="cuda"), torch.empty(tiles, dtype=torch.int32, device="cuda")
    ops.experts_route(lg, dev(bias), top, chosen, weights, places, tile_expert)
    full = lg.cpu().numpy().astype(np.float64) + bias.astype(np.float32).astype(np.float64)
    want = np.argsort(-full, axis=1, kind="stable")[:, :top]
    np.testing.assert_array_equal(chosen.cpu().numpy(), want)
    e = np.exp(np.take_along_axis(full, want, 1) - full.max(axis=1, keepdims=True))
    close(weights.cpu().numpy(), e / e.sum(axis=1, keepdims=True), 1e-5)
    pl, te = places.cpu().numpy(), tile_expert.cpu().numpy()
    assert sorted(pl[pl >= 0].tolist()) == list(range(rows * top))
    for pos in np.nonzero(pl >= 0)[0]:
        assert te[pos // 64] == want.reshape(-1)[pl[pos]]
    h = dev(rng.standard_normal((rows, hidden)), td)
    w_up = dev(rng.standard_normal((experts, ff, hidden)) / math.sqrt(hidden), td)
    w_down = dev(rng.standard_normal((experts, hidden, ff)) / math.sqrt(ff), td)
    up = torch.zeros(tiles * 64, ff, dtype=td, device="cuda")
    ops.experts_gemm(h, w_up, places, tile_expert, up, top=top, act=True)
    down = torch.full((rows * top, hidden), float("nan"), device="cuda")
    ops.experts_gemm(up, w_down, places, tile_expert, down, scatter=True)
    hf, uf, df = h.double().cpu().numpy(), w_up.double().cpu().numpy(), w_down.double().cpu().numpy()
    upn, down = up.double().cpu().numpy(), down.cpu()
    tol = 1e-5 if dtype == "float32" else 1e-2
    for pos in np.nonzero(pl >= 0)[0]:
        pair = pl[pos]
        ex = want.reshape(-1)[pair]
        close(upn[pos], np.maximum(uf[ex] @ hf[pair // top], 0.0) ** 2, tol)
        close(down[pair].cpu().numpy(), df[ex] @ upn[pos], tol)
    if ops.experts_rows_ok(h, w_up, rows * top) and ops.experts_rows_ok(up, w_down, rows * top):
        # steps of few rows: every pair streams its expert's matrices; the same numbers without the layout by expert
        up2 = ops.experts_rows(h, w_up, chosen, torch.empty(rows * top, ff, dtype=td, device="cuda"), top=top, act=True)
        down2 = ops.experts_rows(up2, w_down, chosen, torch.full((rows * top, hidden), float("nan"), device="cuda"))
        for pair in range(rows * top):
            ex = want.reshape(-1)[pair]
            close(up2[pair].double().cpu().numpy(), np.maximum(uf[ex] @ hf[pair // top], 0.0) ** 2, tol)
            close(down2[pair].cpu().numpy(), df[ex] @ up2[pair].double().cpu().numpy(), tol)
    else:
        assert dtype == "float32" or rows * top > ops.EXPERT_ROWS_PAIRS or hidden % 8 or ff % 8


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("top, gated", [(1, True), (3, True), (1, False)])
def test_the_norm_after_the_gated_sum(dtype, top, gated):
    from runtime.kernels import ops
    rng = np.random.default_rng(top)
    T, H, alpha, eps = 11, 70, 2.5, 1e-5
    x, w, gb = rng.standard_normal((T, H)), 1 + 0.1 * rng.standard_normal(H), rng.standard_normal(H)
    gate = rng.standard_normal((T, H + 9))
    xd = dev(x)
    cast = torch.empty(T, H, dtype=TORCH[dtype], device="cuda")
    if top > 1:
        rows, weights = rng.standard_normal((T * top, H)), rng.random((T, top))
        y = (rows.reshape(T, top, H) * weights[..., None]).sum(1)
        operand = ops.WeightedRows(dev(rows), dev(weights), top)
    else:
        y = rng.standard_normal((T, H))
        operand = dev(y)
    ops.gate_post_norm(xd, operand, dev(w), eps, alpha, gate=dev(gate)[:, 4:4 + H] if gated else None, gate_bias=dev(gb) if gated else None, cast=cast)
    v = alpha * x + y * (sigmoid(gate[:, 4:4 + H] + gb) if gated else 1.0)
    want = v / np.sqrt((v ** 2).mean(axis=1, keepdims=True) + eps) * w
    close(xd.cpu().numpy(), want, 1e-5)
    close(cast.float().cpu().numpy(), want, 1e-5 if dtype == "float32" else 1e-2)


@pytest.mark.parametrize("single", [False, True])
def test_embedding_with_hashed_pairs_and_the_token_kept_between_steps(single):
    from runtime.kernels import ops
    rng = np.random.default_rng(5)
    V, H, B, mp, mc, scale = 50, 12, 13, 40000, 70001, 3.0
    table, pairs = rng.standard_normal((V, H)), rng.standard_normal((B + 1, H))
    kept = torch.full((4,), 49, dtype=torch.int32, device="cuda")
    seqs = {0: list(rng.integers(0, V, 30)), 2: list(rng.integers(0, V, 30))}
    at = {0: 0, 2: 0}
    for counts in ([1, 1], [1, 1]) if single else ([5, 1], [2, 7], [1, 3]):
        tokens, positions, seg_of_row, slots = [], [], [], [0, 2]
        for s, (slot, n) in enumerate(zip(slots, counts)):
            tokens += seqs[slot][at[slot]:at[slot] + n]
            positions += list(range(at[slot], at[slot] + n))
            seg_of_row += [s] * n
        start = np.concatenate(([0], np.cumsum(counts)))
        out = torch.empty(sum(counts), H, device="cuda")
        ops.embedding_pairs(ints(tokens), ints(positions), ints(seg_of_row), ints(start), ints(slots), dev(table), out, scale=scale,
                            pairs=dev(pairs), last_token=kept, buckets=B, mul_prev=mp, mul_cur=mc,
                            single_rows=all(c == 1 for c in counts))
        row = 0
        for slot, n in zip(slots, counts):
            for i in range(at[slot], at[slot] + n):
                t = seqs[slot][i]
                b = B if i == 0 else (seqs[slot][i - 1] * mp + t * mc) % B
                close(out[row].cpu().numpy(), table[t].astype(np.float32) * scale + pairs[b].astype(np.float32), 1e-6)
                row += 1
            at[slot] += n
        assert kept.cpu().tolist() == [seqs[0][at[0] - 1], 49, seqs[2][at[2] - 1], 49]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, rot", [(4, 2, 24, 16, 8), (1, 1, 10, 24, 10), (3, 1, 8, 8, 2), (2, 2, 16, 40, 0)])
def test_queries_and_keys_normed_over_the_whole_projection_land_in_padded_heads_and_pages(dtype, heads, kv_heads, dim, vdim, rot):
    from runtime.kernels import ops
    rng = np.random.default_rng(heads * dim)
    td = TORCH[dtype]
    T, P_, pages, eps = 9, 8, 5, 1e-5
    pad = -(-max(dim, vdim) // 8) * 8
    nq, nk, nv = heads * dim, kv_heads * dim, kv_heads * vdim
    proj = rng.standard_normal((T, nq + nk + nv + 6))
    qw, kw = 1 + 0.1 * rng.standard_normal(nq), 1 + 0.1 * rng.standard_normal(nk)
    positions = rng.integers(0, 50, T)
    slots = rng.permutation(pages * P_)[:T]
    slots[3] = -1
    half = max(rot // 2, 1)
    angles = rng.standard_normal((50, half)) if rot else np.zeros((50, 1))
    cos, sin = np.cos(angles), np.sin(angles)
    q = torch.full((T, heads * pad), float("nan"), dtype=td, device="cuda")
    kc, vc = torch.zeros(pages, kv_heads, P_, pad, dtype=td, device="cuda"), torch.zeros(pages, kv_heads, pad, P_, dtype=td, device="cuda")
    ops.whole_norm_rope_scatter(dev(proj), dev(qw), dev(kw), ints(positions), ints(slots), dev(cos), dev(sin), q, kc, vc,
                                heads, kv_heads, dim, vdim, pad, P_, eps)

    def want(x, w, n_heads):
        x = x / np.sqrt((x ** 2).mean(axis=1, keepdims=True) + eps) * w
        x = x.reshape(T, n_heads, dim).copy()
        for i in range(rot // 2 if rot else 0):
            c, s = cos[positions, i][:, None], sin[positions, i][:, None]
            u, v = x[..., 2 * i].copy(), x[..., 2 * i + 1].copy()
            x[..., 2 * i], x[..., 2 * i + 1] = u * c - v * s, v * c + u * s
        return x
    tol = 1e-5 if dtype == "float32" else 1e-2
    qn = q.float().cpu().numpy().reshape(T, heads, pad)
    close(qn[..., :dim], want(proj[:, :nq], qw, heads), tol)
    assert (qn[..., dim:] == 0).all()
    kwant, vwant = want(proj[:, nq:nq + nk], kw, kv_heads), proj[:, nq + nk:nq + nk + nv].reshape(T, kv_heads, vdim)
    kn, vn = kc.float().cpu().numpy(), vc.float().cpu().numpy()
    for t in range(T):
        if slots[t] < 0:
            continue
        page, off = slots[t] // P_, slots[t] % P_
        close(kn[page, :, off, :dim], kwant[t], tol)
        close(vn[page, :, :vdim, off], vwant[t], tol)
        assert (kn[page, :, off, dim:] == 0).all() and (vn[page, :, vdim:, off] == 0).all()
    assert np.count_nonzero(kn.reshape(-1, pad).any(axis=1)) == (slots >= 0).sum() * kv_heads


def attention_case(dtype, heads, kv_heads, dim, lengths, new, window, page_size, seed):
    """Cached keys and values of several requests in shuffled pages, queries for the last `new[i]` positions of each."""
    rng = np.random.default_rng(seed)
    td = TORCH[dtype]
    n_pages = sum(-(-n // page_size) for n in lengths) + 2
    order = rng.permutation(n_pages)
    k = torch.zeros(n_pages, kv_heads, page_size, dim, dtype=td, device="cuda")
    v = torch.zeros(n_pages, kv_heads, dim, page_size, dtype=td, device="cuda")
    width = max(-(-n // page_size) for n in lengths)
    tables = np.full((len(lengths), width), -1, np.int32)
    keys, values, at = [], [], 0
    for s, n in enumerate(lengths):
        kk = dev(rng.standard_normal((n, kv_heads, dim)), td)
        vv = dev(rng.standard_normal((n, kv_heads, dim)), td)
        for j in range(-(-n // page_size)):
            page = int(order[at]); at += 1
            tables[s, j] = page
            rows = slice(j * page_size, min(n, (j + 1) * page_size))
            m = rows.stop - rows.start
            k[page, :, :m] = kk[rows].transpose(0, 1)
            v[page, :, :, :m] = vv[rows].permute(1, 2, 0)
        keys.append(kk.double().cpu().numpy()); values.append(vv.double().cpu().numpy())
    seg_of_row = [s for s, n in enumerate(new) for _ in range(n)]
    positions = [lengths[s] - n + i for s, n in enumerate(new) for i in range(n)]
    q = dev(rng.standard_normal((len(positions), heads * dim)) * 2.0, td)
    return k, v, ints(tables), ints(seg_of_row), ints(positions), q, keys, values


def plain_sigmoid_attention(q, keys, values, seg_of_row, positions, heads, kv_heads, dim, window, scale, bias):
    out = np.zeros((len(positions), heads, dim))
    for r, (s, p) in enumerate(zip(seg_of_row, positions)):
        lo = max(0, p - window + 1) if window else 0
        for h in range(heads):
            g = h // (heads // kv_heads)
            scores = keys[s][lo:p + 1, g] @ q[r, h] * scale + bias[h]
            out[r, h] = sigmoid(scores) @ values[s][lo:p + 1, g]
    return out.reshape(len(positions), heads * dim)


@pytest.mark.parametrize("dtype, heads, kv_heads, dim, window, page_size, splits", [
    ("float32", 4, 2, 24, 20, 16, 1), ("float32", 2, 1, 10, None, 8, 3), ("bfloat16", 6, 2, 20, 33, 4, 2), ("float32", 1, 1, 70, 1, 16, 1)])
def test_row_wise_attention_with_sigmoid_weights(dtype, heads, kv_heads, dim, window, page_size, splits):
    from runtime.kernels import ops
    lengths, new = [150, 37, 1], [40, 1, 1]
    k, v, tables, seg, pos, q, keys, values = attention_case(dtype, heads, kv_heads, dim, lengths, new, window, page_size, 7)
    bias = np.linspace(-2.0, 0.5, heads)
    out = torch.empty(q.shape[0], heads * dim, dtype=q.dtype, device="cuda")
    work = (torch.empty(q.shape[0] * heads * splits * dim, device="cuda"), torch.empty(q.shape[0] * heads * splits * 2, device="cuda")) if splits > 1 else None
    ops.attention_rowwise(q, heads * dim, k, v, tables, seg, pos, out, heads, kv_heads, dim, page_size, window, 0.3, splits, work,
                          head_bias=dev(bias))
    want = plain_sigmoid_attention(q.double().cpu().numpy().reshape(-1, heads, dim), keys, values, seg.cpu().tolist(), pos.cpu().tolist(),
                                   heads, kv_heads, dim, window, 0.3, bias)
    close(out.float().cpu().numpy(), want, 1e-5 if dtype == "float32" else 1e-2)


@pytest.mark.parametrize("heads, kv_heads, dim, window, page_size", [(4, 1, 128, 40, 16), (6, 2, 48, 100, 16), (20, 4, 64, None, 8), (2, 2, 24, 7, 16), (40, 2, 32, 64, 16)])
def test_matrix_core_attention_with_sigmoid_weights_as_tiles_and_as_rows(heads, kv_heads, dim, window, page_size):
    """Prompt rows as tiles from a task list, and single rows one block a row with their keys unsplit and split over
    blocks (whose partial results are plain sums): all against plain arithmetic, and against the row-wise kernel."""
    from runtime.kernels import ops
    from runtime.kernels.attention import fill_tasks
    lengths = [300, 77, 1, 130]
    bias = np.linspace(-3.0, 0.0, heads)
    hb = dev(bias)
    gc = min(heads // kv_heads, 16)
    for new, mode in (([200, 30, 1, 64], "tiles"), ([1, 1, 1, 1], "rows"), ([1, 1, 1, 1], "split")):
        k, v, tables, seg, pos, q, keys, values = attention_case("bfloat16", heads, kv_heads, dim, lengths, new, window, page_size, 11)
        T = q.shape[0]
        out = torch.full((T, heads * dim), float("nan"), dtype=torch.bfloat16, device="cuda")
        if mode == "tiles":
            per = 16 // gc
            tasks = np.zeros((-(-T // per) + len(new), 4), np.int32)
            n = fill_tasks(tasks, new, per, [l - c for l, c in zip(lengths, new)])
            tasks[n:] = (-1, 0, 0, 0)
            ops.attention_mfma(q, heads * dim, k, v, tables, seg, pos, out, heads, kv_heads, dim, page_size, window, 0.3,
                               tasks=ints(tasks), head_bias=hb)
        else:
            splits = 3 if mode == "split" else 1
            work = (torch.empty(T * heads * splits * dim, device="cuda"), torch.empty(T * heads * splits * 2, device="cuda")) if splits > 1 else None
            ops.attention_mfma(q, heads * dim, k, v, tables, seg, pos, out, heads, kv_heads, dim, page_size, window, 0.3,
                               splits=splits, workspace=work, head_bias=hb)
        want = plain_sigmoid_attention(q.double().cpu().numpy().reshape(-1, heads, dim), keys, values, seg.cpu().tolist(), pos.cpu().tolist(),
                                       heads, kv_heads, dim, window, 0.3, bias)
        close(out.float().cpu().numpy(), want, 1.5e-2)
        exact = torch.empty_like(out)
        ops.attention_rowwise(q, heads * dim, k, v, tables, seg, pos, exact, heads, kv_heads, dim, page_size, window, 0.3, head_bias=hb)
        close(out.float().cpu().numpy(), exact.float().cpu().numpy(), 1.5e-2)


# -- whole models -------------------------------------------------------------------------------------------------------

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
    """A portion long enough for the recurrent unit's scan to walk it in pieces side by side, after a shorter one that
    leaves a state, beside a second request's portion in the same step."""
    from runtime.engine import StepEntry
    from runtime.kernels import ops
    name = "a"
    V = CONFIGS[name]["vocab"]
    long, other = random_tokens(31, 700, V), random_tokens(32, 300, V)
    assert ops.mingru_piece(600 + 300, False) > 0
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
    long, short = random_tokens(21, 210, V), random_tokens(22, 40, V)
    want = {"l": plain_logits(folders[name], long), "s": plain_logits(folders[name], short)}
    runner = make_runner(folders[name], dtype, pages=17, execution=execution)
    runner.create("l")
    got = {"l": [], "s": []}
    for t, token in enumerate(long):
        entries = [StepEntry("l", [token], [0])]
        if 60 <= t < 100:
            if t == 60:
                runner.create("s")
            entries.append(StepEntry("s", [short[t - 60]], [0]))
        out = runner.step(entries).cpu().numpy()
        got["l"].append(out[0])
        if len(entries) == 2:
            got["s"].append(out[1])
        if t == 99:
            runner.release("s")
    assert_close(np.stack(got["l"]), want["l"], dtype, "long decoding", decided_rows(folders[name], long))
    assert_close(np.stack(got["s"]), want["s"], dtype, "the request that joined late", decided_rows(folders[name], short))
    runner.cache.check()


def mixed(V, seed, lengths=(70, 33, 120, 9, 64, 97, 40, 130), live_at_once=4, tokens_of=random_tokens):
    """Up to `live_at_once` live requests: portions of some beside single tokens of others; requests end and new ones
    start on the pages and state slots they gave back; one request sits out some steps."""
    rng = np.random.default_rng(seed)
    seqs = {f"m{i}": tokens_of(seed * 100 + i, n, V) for i, n in enumerate(lengths)}
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
    check_trace(trace, folders[name], tmp_path, dtype, V, seqs)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_batch_of_unequal_requests_gives_what_each_gives_alone(folders, dtype):
    from runtime.engine import StepEntry
    name = "a"
    V = CONFIGS[name]["vocab"]
    seqs = {k: random_tokens(50 + i, n, V) for i, (k, n) in enumerate({"a": 61, "b": 5, "c": 1, "d": 30}.items())}
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
def test_far_keys_the_window_s_edge_and_old_state_in_a_model_drawn_sharp(folders, dtype):
    """In the sharp model a query's result hangs on single keys and the recurrent state forgets slowly.  The test first
    shows that a window one key longer or shorter, and a state that started late, would move the logits by several
    times the bound; then a prompt of many pages cut in the middle of a page and of the window, and tokens one by one
    over page borders, hold the bound."""
    from runtime.engine import StepEntry
    name = "s"
    cfg, w = P.read_folder(folders[name])
    tokens = random_tokens(9, 410, cfg["vocab"])
    want = plain_logits(folders[name], tokens)
    scale = np.abs(want).max()
    for delta in (-1, 1):
        off = json.loads(json.dumps(cfg))
        for layer in (0, 3):
            off["layers"][layer]["mixer"]["mask"]["size"] += delta
        assert np.abs(P.forward(off, w, tokens)[60:] - want[60:]).max() > 1e-3 * scale, "a window one key off does not show"
    late = P.forward(cfg, w, tokens[200:])
    assert np.abs(late[-40:] - want[-40:]).max() > 0.01 * scale, "the first 200 tokens do not reach the last 40"
    runner = make_runner(folders[name], dtype, pages=60)
    runner.create("f")
    got = [runner.step([StepEntry("f", tokens[:201], list(range(201)))]).cpu().numpy(),
           runner.step([StepEntry("f", tokens[201:376], list(range(175)))]).cpu().numpy()]
    got += [runner.step([StepEntry("f", [t], [0])]).cpu().numpy() for t in tokens[376:]]
    got = np.concatenate(got)
    ok = decided_rows(folders[name], tokens)
    assert_close(got, want, dtype, "far keys", ok)
    assert_close(got[:3], want[:3], dtype, "the first tokens")
    assert_close(got[40:60], want[40:60], dtype, "around the window's first edge", ok[40:60])


def test_a_window_gives_its_pages_back_and_its_reader_still_sees_its_own(folders):
    """Layer 0 of model a looks back over 20 keys and layer 2 reads its cache over 37: the cache keeps 37.  A request far
    longer than the pool of a request that kept everything, decoded in portions and single tokens."""
    from runtime.engine import StepEntry
    name = "a"
    tokens = random_tokens(13, 330, CONFIGS[name]["vocab"])
    want = plain_logits(folders[name], tokens)
    runner = make_runner(folders[name], "float32", pages=10, page_size=16)       # 160 slots for 330 tokens
    runner.create("w")
    got, at = [], 0
    for n in [40, 33, 1, 1, 50, 2, 64, 1, 1, 1, 30, 60, 46]:
        got.append(runner.step([StepEntry("w", tokens[at:at + n], list(range(n)))]).cpu().numpy())
        at += n
    assert at == len(tokens)
    assert_close(np.concatenate(got), want, "float32", "a window beside its reader")
    runner.cache.check()


@pytest.mark.parametrize("name, dtype, execution, overlap", [("a", "float32", "graph", True), ("a", "float32", "eager", False),
                                                             ("w", "bfloat16", "graph", True), ("g", "float32", "graph", True)])
def test_greedy_generation_through_the_scheduler(folders, name, dtype, execution, overlap):
    """With overlapped ticks a request's last token is still on the device when its next step is launched: the table
    of token pairs takes it from the request's state slot."""
    from runtime.engine.scheduler import Engine
    cfg, w = P.read_folder(folders[name])
    prompts = [random_tokens(70 + i, n, cfg["vocab"]) for i, n in enumerate([11, 3, 26, 1, 40])]
    engine = Engine.from_folder(folders[name], dtype=dtype, pages=24, page_size=16, execution=execution,
                                max_active=3, token_budget=24, prefill_chunk=9, overlap=overlap)
    got = engine.generate(prompts, max_new_tokens=10)
    for prompt, new in zip(prompts, got):
        assert len(new) == 10
        if dtype == "float32":
            assert new == P.greedy(cfg, w, prompt, 10)
        else:       # bfloat16: every picked token is the plain model's best or within rounding of it, given the same past
            logits = P.forward(cfg, w, prompt + new)[len(prompt) - 1:-1]
            for row, token in zip(logits, new):
                assert row.max() - row[token] < 0.05 * (row.max() - row.min())
    engine.runner.cache.check()
    assert not engine.runner.cache.lengths, "every request gave back what it held"


def test_command_line_serves_the_design(folders, tmp_path):
    """`python -m runtime` chooses the design by config.json: requests of a file against a folder, in float32, give the
    plain model's greedy tokens; the named configuration with random weights generates and reports its state slots."""
    import os, subprocess, sys
    from conftest import ROOT
    cfg, w = P.read_folder(folders["a"])
    requests = [{"key": "x", "prompt": [1, 2, 3, 4, 5, 6, 7], "max_new_tokens": 5}, {"key": "y", "prompt": [9], "max_new_tokens": 4}]
    (tmp_path / "requests.json").write_text(json.dumps(requests))
    env = dict(os.environ, PYTHONPATH=str(ROOT))
    proc = subprocess.run([sys.executable, "-m", "runtime", "--checkpoint", str(folders["a"]), "--dtype", "float32",
                           "--requests", str(tmp_path / "requests.json"), "--policy", "chunked", "--pages", "16",
                           "--token-budget", "6", "--prefill-chunk", "3"], capture_output=True, text=True, timeout=300, env=env, cwd=str(tmp_path))
    assert proc.returncode == 0, proc.stderr[-2000:]
    by_key = {r["key"]: r for r in json.loads(proc.stdout)["requests"]}
    assert by_key["x"]["generated"] == P.greedy(cfg, w, [1, 2, 3, 4, 5, 6, 7], 5)
    assert by_key["y"]["generated"] == P.greedy(cfg, w, [9], 4)
    proc = subprocess.run([sys.executable, "-m", "runtime", "--model", "noresun-tiny", "--tokens", "5,6,7", "--max-new-tokens", "3",
                           "--overlap", "--report"], capture_output=True, text=True, timeout=300, env=env, cwd=str(tmp_path))
    assert proc.returncode == 0, proc.stderr[-2000:]
    out = json.loads(proc.stdout)
    assert out["weights"] == "random-noresun-tiny" and len(out["requests"][0]["generated"]) == 3
    assert out["runner"]["replays"] >= 1 and out["runner"]["cache"][0]["resident_pages"] == 0


def random_config(seed):
    """A configuration drawn at random: sizes, head counts, the order of the layers, windows, constants; some attention
    layers read the keys of an earlier one over a window of their own, some layers have no feed-forward.  Every second
    draw has sizes of the order of a small real model (heads of 64 to 128, a width of a few hundred, a dozen experts)."""
    from noresun_models import attention, config, mingru, moe, rot
    rng = np.random.default_rng(seed)
    pick = lambda *values: values[int(rng.integers(len(values)))]
    big = seed % 2 == 1
    width = pick(192, 264, 384) if big else pick(40, 72, 100, 136)

    def feed_forward():
        if rng.random() < 0.2:
            return None
        experts = pick(8, 12, 32) if big else pick(2, 3, 5, 7)
        return moe(pick(48, 80, 136) if big else pick(8, 20, 33), experts, min(experts, pick(1, 2, 3, 4, 6)))

    layers, owners = [], []
    for i in range(int(rng.integers(2, 7))):
        if rng.random() < 0.4:
            layers.append(mingru(pick(96, 200, 320) if big else pick(3, 16, 50, 96), feed_forward()))
            continue
        window = pick(None, 1, 2, 15, 16, 17, 33, 64, 90)
        scale = float(rng.uniform(0.08, 0.4))
        if owners and rng.random() < 0.4:
            j = pick(*owners)
            m = layers[j]["mixer"]
            layers.append(attention(m["heads"], m["kv_heads"], m["dim"], m["vdim"], scale, window, m["rot"], kv_from=j, mlp=feed_forward()))
            continue
        kv_heads = pick(1, 2, 3)
        dim = pick(64, 96, 128) if big else pick(6, 16, 24, 40)
        vdim = pick(dim, 32, 64, 128) if big else pick(dim, 8, 12, 48)
        dims = pick(dim, dim // 2, 2, 4)
        scaling = pick(None, (pick(2.0, 8.0, 32.0), pick(1.0, 2.0), pick(4.0, 8.0), pick(16, 128, 1024)))
        layers.append(attention(kv_heads * pick(1, 2, 4), kv_heads, dim, vdim, scale, window, rot(float(pick(50.0, 10000.0, 1e6)), dims - dims % 2 or 2, scaling),
                                mlp=feed_forward()))
        owners.append(i)
    bigram = pick(None, (int(rng.integers(5, 700)), int(rng.integers(0, 50)), int(rng.integers(1, 50))))
    return config(int(rng.integers(40, 700)), width, float(rng.uniform(0.5, 4.0)), pick(1e-5, 1e-6), float(rng.uniform(2.0, 20.0)), bigram, layers)


def check_trace_row_by_row(trace, folder, out_dir, dtype, vocab, sequences, doubtful=0.05, share=0.1):
    """check_trace for models whose routers decide often: float32 is compared as ever.  In bfloat16 the rounding that
    has gathered over some layers turns a choice with a margin of a few hundredths round now and then, and what that
    position leaves in the caches and states reaches the ones after it.  So every position is compared alone: before
    a request's first position with a margin under `doubtful` each must hold the bound; from there on one may miss
    it, and over the whole trace at most `share` of the positions do."""
    if dtype == "float32":
        return check_trace(trace, folder, out_dir, dtype, vocab, sequences)
    held = missed = 0
    for step, rows in trace.expect.items():
        data = np.fromfile(out_dir / f"{step}.f32", dtype="<f4").reshape(len(rows), vocab).astype(np.float64)
        for row, (rid, pos) in zip(data, rows):
            want = plain_logits(folder, sequences[rid])[pos]
            assert np.isfinite(row).all()
            err = np.linalg.norm(row - want) / np.linalg.norm(want)
            if err < conftest.BF16_RMSE:
                held += 1
                continue
            doubt = np.nonzero(smallest_margins(folder, sequences[rid])[:pos + 1] < doubtful)[0]
            assert len(doubt), f"request {rid}, position {pos}: bfloat16 differs by {err:.3e} and no choice before it was close"
            missed += 1
    assert missed <= share * (held + missed), f"{missed} of {held + missed} positions differ"


_DRAWN = {}


@pytest.fixture(scope="module")
def drawn(tmp_path_factory):
    """seed -> (configuration, folder, trace, sequences), made once for both dtypes (the sequences are decisive_tokens:
    the plain model's routers decide every position of them clearly)."""
    def make(seed):
        if seed not in _DRAWN:
            cfg = random_config(seed)
            folder = write_folder(tmp_path_factory.mktemp(f"drawn{seed}") / "model", cfg, 200 + seed, sharp=seed % 3 == 0)
            lengths = (70, 33, 90, 9, 48) if seed % 2 else (70, 33, 120, 9, 64, 97)
            trace, seqs = mixed(cfg["vocab"], seed=40 + seed, lengths=lengths, tokens_of=lambda s, n, V: decisive_tokens(folder, s, n, V))
            _DRAWN[seed] = (cfg, folder, trace, seqs)
        return _DRAWN[seed]
    return make


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random_in_mixed_batches(drawn, tmp_path, seed, dtype):
    from runtime.engine.replay import replay
    cfg, folder, trace, seqs = drawn(seed)
    done = []
    runner = replay(folder, dtype, tmp_path / "out", trace.peak, trace.lines(), echo=done.append, execution="graph" if seed % 2 else "eager")
    assert done == [f"done {i}" for i in range(len(trace.steps))]
    runner.cache.check()
    check_trace_row_by_row(trace, folder, tmp_path / "out", dtype, cfg["vocab"], seqs)
