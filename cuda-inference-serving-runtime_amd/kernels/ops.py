"""Checked Python entry points of the HIP kernels.

Every function validates device, dtype, contiguity and shapes on the host
before the launch, because a kernel that reads out of bounds can take the GPU
down.  Tensors are torch tensors on the GPU; launches go to torch's current
stream, so they are ordered with torch's own work and can be captured into a
graph.  Nothing here computes on the CPU.  One kind of call leaves the kernels of this repository: large bf16
products of more than 64 rows, which go to the vendor's library through torch.mm (see library_ok).
"""
import ctypes as C

import torch

from . import library

F32, BF16 = 0, 1
MFMA_HEAD_PADS = library.ATTENTION_PADS
SKINNY_ROWS = 64   # products with at most this many rows run the weight-streaming kernel
_DT = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


_configured = False


def lib():
    global _configured
    handle = library.load()
    if not _configured:
        _declare(handle)
        _configured = True
    return handle


def _declare(h):
    p, i, f, ll = C.c_void_p, C.c_int, C.c_float, C.c_longlong
    sig = {
        "cisr_embedding": [p, p, p, i, i, i, i, p],
        "cisr_rmsnorm": [p, p, p, p, i, i, f, i, p],
        "cisr_add_rmsnorm": [p, p, p, p, i, i, f, i, p],
        "cisr_residual_add": [p, p, ll, i, p],
        "cisr_swiglu": [p, p, i, i, i, p],
        "cisr_rope_scatter": [p, p, p, p, p, p, p, i, i, i, i, i, i, i, i, i, i, p],
        "cisr_page_copy": [p, p, p, i, i, ll, ll, p],
        "cisr_f32_to_bf16": [p, p, ll, p],
        "cisr_bias_add": [p, p, ll, i, i, i, p],
        "cisr_attn_rowwise": [p, i, p, p, p, p, p, p, p, p, i, i, i, i, i, i, i, f, i, i, p],
        "cisr_gemm_f32": [p, i, p, i, p, i, p, i, i, i, i, p],
        "cisr_gemm_bf16": [p, i, p, i, p, i, p, i, i, i, i, i, p],
        "cisr_gemm_bf16_swiglu": [p, i, p, i, p, i, i, i, i, i, p],
        "cisr_gemm_bf16_tile": [p, i, p, i, p, i, p, i, i, i, i, i, i, p],
        "cisr_gemm_bf16_swiglu_tile": [p, i, p, i, p, i, i, i, i, i, i, p],
        "cisr_gemm_skinny_bf16": [p, i, p, i, p, i, p, i, i, i, i, i, i, p, f, p, p],
        "cisr_qkv_rope_skinny": [p, i, p, i, p, i, i, i, p, f, p, p, p, p, p, p, i, i, i, i, i, p],
        "cisr_attn_merge": [p, p, p, i, i, i, i, p, p],
        "cisr_argmax": [p, p, p, i, p, p, i, i, p],
        "cisr_sample": [p, p, p, p, p, p, i, i, i, p],
        "cisr_take_tokens": [p, p, p, i, i, p],
        "cisr_gemm_wide_bf16": [p, i, p, i, p, i, p, i, i, i, i, i, i, p, C.c_longlong, p],
        "cisr_gemm_wide_partials_bf16": [p, i, p, i, i, i, i, p, C.c_longlong, p],
        "cisr_rmsnorm_partials": [p, p, i, p, p, i, i, f, i, p],
        "cisr_add_rmsnorm_bf16": [p, p, p, p, i, i, f, i, p],
        "cisr_qkv_rope_wide": [p, i, p, i, p, i, i, i, p, p, p, p, p, p, i, i, i, i, i, p, C.c_longlong, p],
        "cisr_gemm_merged_bf16": [p, p, i, i, i, p, i, p, i, p, i, i, i, p],
        "cisr_gemm_merged_ok": [i, i, i, i, i],
        "cisr_gemm_skinny_bf16_gated": [p, i, p, i, p, i, i, i, i, i, f, f, f, p],
        "cisr_gemm_wide_bf16_gated": [p, i, p, i, p, i, i, i, i, i, f, f, f, p, C.c_longlong, p],
        "cisr_gemm_bf16_gated": [p, i, p, i, p, i, i, i, i, i, f, f, f, p],
        "cisr_post_norm_add": [p, p, p, p, p, p, i, i, f, f, p, f, p, i, i, i, f, f, p, p],
        "cisr_glu_clamped": [p, p, i, i, f, f, f, i, p],
        "cisr_qk_norm_scatter": [p, i, p, p, p, p, p, p, i, i, i, i, i, i, i, f, i, p],
        "cisr_head_gate": [p, p, i, p, i, i, i, i, i, p],
        "cisr_layernorm": [p, p, p, p, p, i, i, f, i, p],
        "cisr_rms_slice": [p, i, i, p, p, i, i, f, i, p],
        "cisr_latent_keys": [p, i, i, p, p, i, p, p, p, p, p, p, p, i, i, i, i, i, i, i, i, i, i, f, i, p],
        "cisr_heads_product": [p, i, i, p, p, i, i, p, i, i, i, i, i, i, p],
        "cisr_gelu": [p, p, ll, i, i, p],
        "cisr_gemm_bf16_heads": [p, i, i, p, p, i, i, p, i, i, i, i, i, i, p],
        "cisr_gemm_skinny_bf16_act": [p, i, p, i, p, i, i, i, i, i, i, p],
        "cisr_gemm_bf16_act": [p, i, p, i, p, i, i, i, i, i, i, p],
        "cisr_attn_rowwise_sigmoid": [p, i, p, p, p, p, p, p, p, p, i, i, i, i, i, i, i, f, i, i, p, p],
        "cisr_attn_merge_sum": [p, p, i, i, i, i, p, p],
        "cisr_embedding_pairs": [p, p, p, p, p, p, p, p, p, p, i, i, i, i, f, i, ll, ll, i, i, i, p],
        "cisr_gate_post_norm": [p, p, i, p, p, i, p, p, p, i, i, f, f, i, p],
        "cisr_whole_norm_rope_scatter": [p, i, p, p, p, p, p, p, p, i, i, p, p, p, i, i, i, i, i, i, i, f, i, i, i, i, p],
        "cisr_attn_talking": [p, i, p, p, p, p, p, p, p, p, p, i, p, i, i, i, i, i, i, i, i, i, f, i, p, p, i, p],
        "cisr_experts_route": [p, i, p, p, p, i, i, i, i, p, p, p],
        "cisr_experts_gemm": [p, i, p, p, p, i, i, p, i, i, i, i, i, i, i, p],
        "cisr_experts_rows": [p, i, p, p, i, p, i, i, i, i, i, i, i, p],
        "cisr_experts_route_scored": [p, i, p, p, p, i, i, i, i, i, i, i, p, p, p],
        "cisr_experts_combine": [p, p, p, p, i, p, p, i, i, i, i, p],
        "cisr_bias_act": [p, p, p, ll, i, i, i, p],
        "cisr_experts_rows_ok": [i, i, i],
    }
    for name, args in sig.items():
        fn = getattr(h, name)
        fn.argtypes = args
        fn.restype = C.c_int
    h.cisr_gemm_wide_workspace.argtypes = [i, i, i, i]
    h.cisr_gemm_wide_workspace.restype = C.c_longlong
    h.cisr_gemv_ok.argtypes = [i, i, i]
    h.cisr_gemv_ok.restype = C.c_int
    h.cisr_gemv_set.argtypes = [i, ll]
    h.cisr_gemv_set.restype = None


_attention_entries = {}


def _attention_entry(dpad, law="softmax"):
    """The matrix-core attention entry point for a padded head size (its shared object is built and loaded
    at the first use of that size).  `law` "sigmoid": the build whose weights are sigmoid(score + a bias a head), not
    normed over the keys; its entry takes the biases as a last argument."""
    fn = _attention_entries.get((dpad, law))
    if fn is None:
        p, i, f = C.c_void_p, C.c_int, C.c_float
        sigmoid = law == "sigmoid"
        fn = getattr(library.load_attention(dpad, law), f"cisr_attn_mfma_sig_d{dpad}" if sigmoid else f"cisr_attn_mfma_d{dpad}")
        fn.argtypes = [p, i, p, p, p, i, p, i, p, p, p, p, p, i, i, i, i, i, f, i, i, i, i, p] + ([p] if sigmoid else [])
        fn.restype = C.c_int
        _attention_entries[(dpad, law)] = fn
    return fn


def prepare(units=()):
    """Build, side by side, the core and the further shared objects `units` (names of library.units(): what the
    parts of a model say they need, `kernel_units`), and load the core."""
    library.ensure([library.CORE] + [u for u in dict.fromkeys(units) if u != library.CORE])
    lib()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_current_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The handle of the current stream of the current device.  Every launch asks for it: torch's short way where it has
    one (a prompt step run kernel by kernel asks 240 times; `torch.cuda.current_stream()` takes 9 us a call, 2 ms a step)."""
    if _raw_stream is not None and _current_device is not None:
        return _raw_stream(_current_device())
    return torch.cuda.current_stream().cuda_stream


def _check(code, what):
    if code != 0:
        raise KernelError(f"{what}: HIP error {code}")


def _dev(t, name, dtype=None, shape=None):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name}: expected a GPU tensor")
    if not t.is_contiguous():
        raise KernelError(f"{name}: tensor must be contiguous")
    if dtype is not None:
        allowed = dtype if isinstance(dtype, (tuple, list)) else (dtype,)
        if t.dtype not in allowed:
            raise KernelError(f"{name}: dtype {t.dtype}, expected {allowed}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name}: shape {tuple(t.shape)}, expected {tuple(shape)}")
    return t.data_ptr()


def _storage(t, name):
    if t.dtype not in _DT:
        raise KernelError(f"{name}: storage dtype {t.dtype} is not float32 or bfloat16")
    return _DT[t.dtype]


def embedding(tokens, table, out):
    """out[r] = table[tokens[r]] widened to float.  tokens int32 [T], table [V, H], out float [T, H]."""
    rows = tokens.shape[0]
    vocab, dim = table.shape
    _check(lib().cisr_embedding(_dev(tokens, "tokens", torch.int32, (rows,)), _dev(table, "table"),
                                _dev(out, "out", torch.float32, (rows, dim)), rows, dim, vocab,
                                _storage(table, "table"), _stream()), "embedding")
    return out


def rmsnorm(x, weight, out, eps, rows=None):
    """out = rmsnorm(x[rows]) * weight.  x float [T, H]; weight float [H]; out [R, H] float or bf16."""
    dim = x.shape[1]
    n_out = out.shape[0]
    if rows is None and n_out != x.shape[0]:
        raise KernelError("rmsnorm: out rows differ from input rows")
    rp = None if rows is None else _dev(rows, "rows", torch.int32, (n_out,))
    _check(lib().cisr_rmsnorm(_dev(x, "x", torch.float32), _dev(weight, "weight", torch.float32, (dim,)),
                              _dev(out, "out", None, (n_out, dim)), rp, n_out, dim, float(eps),
                              _storage(out, "out"), _stream()), "rmsnorm")
    return out


def partials_ok(x):
    """Whether add_partials / rmsnorm_partials take the float rows x."""
    return (x.dtype == torch.float32 and x.is_contiguous() and x.shape[1] % 4 == 0 and x.shape[1] <= 8192
            and x.data_ptr() % 16 == 0)


def add_partials(x, partials):
    """x += what gemm_unfinished left (float rows, in place): the partial sums in slice order, or (slices 0) the
    bf16 product."""
    parts, slices = partials
    rows, dim = x.shape
    if slices == 0:
        return residual_add(x, parts)
    if not partials_ok(x) or parts.numel() < slices * rows * dim:
        raise KernelError("add_partials: contiguous float rows of a multiple of 4 (at most 8192) and their partial sums")
    _check(lib().cisr_rmsnorm_partials(x.data_ptr(), _dev(parts, "partials", torch.float32), int(slices), None, None, rows, dim,
                                       0.0, _DT[torch.float32], _stream()), "add_partials")
    return x


def rmsnorm_partials(x, partials, weight, out, eps):
    """x += what gemm_unfinished left (in place), out = rmsnorm(x) * weight: one kernel."""
    parts, slices = partials
    rows, dim = x.shape
    if not partials_ok(x) or out.data_ptr() % 16:
        raise KernelError("rmsnorm_partials: contiguous float rows of a multiple of 4 (at most 8192)")
    wp, op = _dev(weight, "weight", torch.float32, (dim,)), _dev(out, "out", None, (rows, dim))
    if slices == 0:
        _check(lib().cisr_add_rmsnorm_bf16(x.data_ptr(), _dev(parts, "product", torch.bfloat16, (rows, dim)), wp, op, rows, dim,
                                           float(eps), _storage(out, "out"), _stream()), "rmsnorm_partials")
        return out
    if parts.numel() < slices * rows * dim:
        raise KernelError("rmsnorm_partials: too few partial sums")
    _check(lib().cisr_rmsnorm_partials(x.data_ptr(), _dev(parts, "partials", torch.float32), int(slices), wp, op,
                                       rows, dim, float(eps), _storage(out, "out"), _stream()), "rmsnorm_partials")
    return out


def add_rmsnorm(x, delta, weight, out, eps):
    """x += delta (float residual, in place), out = rmsnorm(x) * weight."""
    rows, dim = x.shape
    dt = _storage(delta, "delta")
    if out.dtype != delta.dtype:
        raise KernelError("add_rmsnorm: out and delta must share a dtype")
    _check(lib().cisr_add_rmsnorm(_dev(x, "x", torch.float32), _dev(delta, "delta", None, (rows, dim)),
                                  _dev(weight, "weight", torch.float32, (dim,)), _dev(out, "out", None, (rows, dim)),
                                  rows, dim, float(eps), dt, _stream()), "add_rmsnorm")
    return out


def residual_add(x, delta):
    """x += delta, x float, delta float or bf16 of the same shape."""
    if x.shape != delta.shape:
        raise KernelError("residual_add: shapes differ")
    _check(lib().cisr_residual_add(_dev(x, "x", torch.float32), _dev(delta, "delta"), x.numel(),
                                   _storage(delta, "delta"), _stream()), "residual_add")
    return x


def swiglu(gate_up, out):
    """out[r, i] = silu(gate_up[r, i]) * gate_up[r, I + i]."""
    rows, two_i = gate_up.shape
    if two_i % 2:
        raise KernelError("swiglu: input width must be even")
    inter = two_i // 2
    _check(lib().cisr_swiglu(_dev(gate_up, "gate_up"), _dev(out, "out", gate_up.dtype, (rows, inter)), rows, inter,
                             _storage(gate_up, "gate_up"), _stream()), "swiglu")
    return out


def bias_add(x, bias):
    """x[r, c] += bias[c], in place (added in float).  x [T, N] float or bf16, contiguous; bias [N] float or bf16."""
    rows, cols = x.shape
    _check(lib().cisr_bias_add(_dev(x, "x"), _dev(bias, "bias", None, (cols,)), rows, cols, _storage(x, "x"), _storage(bias, "bias"),
                               _stream()), "bias_add")
    return x


def rope_scatter(qkv, positions, slots, cos, sin, kcache, vcache, heads, kv_heads, dim, page_size, interleaved=False):
    """Rotate q (in place) and k of the fused projection rows, write k and v into
    the cache at `slots`.  kcache/vcache None: q only (a layer reading another's cache).
    Pair i of a head is coordinates (i, i + rot/2), or with `interleaved` (2i, 2i + 1).
    qkv [T, (heads + 2 kv_heads) * dim] (or [T, heads * dim] without a cache);
    cos/sin float [max_pos, rot/2]; keys [pages, kv_heads, page_size, dim],
    values transposed in a page: [pages, kv_heads, dim, page_size]."""
    rows = qkv.shape[0]
    has_kv = kcache is not None
    width = (heads + (2 * kv_heads if has_kv else 0)) * dim
    dt = _storage(qkv, "qkv")
    max_pos, half = cos.shape
    rot = 2 * half
    if rot > dim or rot <= 0:
        raise KernelError(f"rope_scatter: rotary size {rot} does not fit head size {dim}")
    kp = vp = sp = None
    if has_kv:
        pages = kcache.shape[0]
        kp = _dev(kcache, "kcache", qkv.dtype, (pages, kv_heads, page_size, dim))
        vp = _dev(vcache, "vcache", qkv.dtype, (pages, kv_heads, dim, page_size))
        sp = _dev(slots, "slots", torch.int32, (rows,))
    _check(lib().cisr_rope_scatter(_dev(qkv, "qkv", None, (rows, width)), _dev(positions, "positions", torch.int32, (rows,)),
                                   sp, _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32, (max_pos, half)),
                                   kp, vp, rows, heads, kv_heads, dim, rot, page_size, max_pos, int(has_kv),
                                   int(bool(interleaved)), dt, _stream()), "rope_scatter")


def page_copy(pool, src, dst, slabs, pages_per_slab):
    """pool viewed as [slabs, pages_per_slab, page]: page dst[i] := page src[i] in every slab."""
    n = src.shape[0]
    total = pool.numel() * pool.element_size()
    if total % (slabs * pages_per_slab):
        raise KernelError("page_copy: pool does not divide into slabs and pages")
    slab_bytes = total // slabs
    page_bytes = slab_bytes // pages_per_slab
    _check(lib().cisr_page_copy(_dev(pool, "pool"), _dev(src, "src", torch.int32, (n,)), _dev(dst, "dst", torch.int32, (n,)),
                                n, slabs, page_bytes, slab_bytes, _stream()), "page_copy")


def f32_to_bf16(x, out):
    _check(lib().cisr_f32_to_bf16(_dev(x, "x", torch.float32), _dev(out, "out", torch.bfloat16, x.shape), x.numel(),
                                  _stream()), "f32_to_bf16")
    return out


ROWWISE_MAX_HEAD = 640     # the row-wise attention kernel's largest head (the matrix-core kernels stop at 256)


def attention_rowwise(q, q_row_stride, kcache, vcache, tables, seg_of_row, positions, out, heads, kv_heads, dim,
                      page_size, window, scale, splits=1, workspace=None, head_bias=None):
    """Each row attends to its request's cached keys lo..position.  q is a view
    into a row-major buffer with `q_row_stride` elements per row; out [T, heads*dim].
    `head_bias` (float [heads]): the weight of a visible key is sigmoid(score + head_bias[head]) instead of its share
    of a softmax, and the weights are not normed over the keys."""
    rows = out.shape[0]
    dt = _storage(out, "out")
    if dim % 2 or dim > ROWWISE_MAX_HEAD:
        raise KernelError(f"attention: head size {dim} must be even and at most {ROWWISE_MAX_HEAD}")
    if heads % kv_heads:
        raise KernelError(f"attention: {heads} query heads do not divide into {kv_heads} key heads")
    pages = kcache.shape[0]
    width = tables.shape[1]
    if q.dtype != out.dtype or kcache.dtype != out.dtype:
        raise KernelError("attention: q, cache and out must share a dtype")
    if q.numel() < (rows - 1) * q_row_stride + heads * dim:
        raise KernelError("attention: q buffer too small for its stride")
    po = pm = None
    if splits > 1:
        if workspace is None:
            raise KernelError("attention: split runs need a workspace")
        part_o, part_ml = workspace
        po = _dev(part_o, "part_o", torch.float32)
        pm = _dev(part_ml, "part_ml", torch.float32)
        if part_o.numel() < rows * heads * splits * dim or part_ml.numel() < rows * heads * splits * 2:
            raise KernelError("attention: split workspace too small")
    args = (q.data_ptr(), q_row_stride, _dev(kcache, "kcache", None, (pages, kv_heads, page_size, dim)),
            _dev(vcache, "vcache", None, (pages, kv_heads, dim, page_size)),
            _dev(tables, "tables", torch.int32), _dev(seg_of_row, "seg_of_row", torch.int32, (rows,)),
            _dev(positions, "positions", torch.int32, (rows,)), _dev(out, "out", None, (rows, heads * dim)),
            po, pm, rows, heads, kv_heads, dim, page_size, width, int(window or 0), float(scale), int(splits), dt)
    if head_bias is not None:
        _check(lib().cisr_attn_rowwise_sigmoid(*args, _dev(head_bias, "head_bias", torch.float32, (heads,)), _stream()), "attention_rowwise")
    else:
        _check(lib().cisr_attn_rowwise(*args, _stream()), "attention_rowwise")
    return out


# Large bf16 products of many rows go to the vendor's library through torch.mm (the reference's linears are
# library calls too: cuBLAS through runtime/blas.py:44-56, or CuPy's matmul, runtime/model.py:108): from this many rows on, with weights of at least LIBRARY_MIN_BYTES;
# the residual sum or the activation is then a kernel after the product.  Measured on an MI355X at 2048 rows:
# 1,270-1,480 TFLOP/s against 830-920 of the tiled kernel here on the 8B shapes (a prompt step of 30.6 against
# 39.9 ms); at 65-255 rows with weights streamed from HBM it is up to 2.5 times as fast on narrow outputs with
# a long inner size, which leave the tiled kernel few tiles (it does not cut K).  With at most 64 rows the
# weight-streaming kernels here are as fast or faster (8 rows: 50 against 67 us for gate and up of the 8B
# sizes), as are all products of small weights, and both save the kernel after the product.  The least weights are
# those of the 1.7B sizes' output projection (8 MB: 10.7 against 13.9 us at 128 rows, 29 against 33 at 2,048, the
# residual sum included; the products of the 135M sizes, 0.7 to 3.5 MB, are as fast or faster here).  0 rows: never.
LIBRARY_MIN_ROWS = 65
LIBRARY_MIN_BYTES = 8 << 20
LIBRARY_GATED_MIN_ROWS, LIBRARY_GATED_MIN_BYTES = 33, 64 << 20


def attention_talking(q, q_row_stride, kcache, vcache, tables, seg_of_row, positions, out, heads, kv_heads, vdim, pad, page_size,
                      mix, scale, temp=None, sink=None, window=None, chunk=None, gate=None, splits=1, workspace=None):
    """Attention whose scores are mixed over the heads before the softmax: s_h = sum_g mix[h, g] temp[g] scale (q_g . k),
    weights exp(s_h) / (exp(sink_h) + sum over the visible keys), out_h = sum w_h v of the head's key/value head, times
    sigmoid(gate) element by element.  A row at position p sees the keys of its block of `chunk` positions up to itself
    (or the last `window`, or all).  q [T, >= heads * pad] and the pages hold heads of `pad` coordinates, the rest zero;
    out [T, heads * vdim]; mix float [heads, heads], temp and sink float [heads] or None; gate a float view
    [T, heads * vdim] or None.  `splits` > 1: that many blocks share a row's keys and leave their sums in `workspace` =
    (float [T * heads * splits * vdim], float [T * heads * splits * 2]) for a merge kernel behind them."""
    rows = out.shape[0]
    pages = kcache.shape[0]
    po = pm = None
    if splits > 1:
        if workspace is None or workspace[0].numel() < rows * heads * splits * vdim or workspace[1].numel() < rows * heads * splits * 2:
            raise KernelError("attention_talking: split keys need a workspace for their sums")
        po, pm = _dev(workspace[0], "part_o", torch.float32), _dev(workspace[1], "part_ml", torch.float32)
    gp, ldg = None, 0
    if gate is not None:
        if gate.dtype != torch.float32 or tuple(gate.shape) != (rows, heads * vdim) or gate.stride(1) != 1 or not gate.is_cuda:
            raise KernelError("attention_talking: the gate must be float [T, heads * vdim] with unit stride")
        gp, ldg = gate.data_ptr(), gate.stride(0)
    if q.dim() != 2 or q.shape[0] != rows or q.stride(1) != 1 or q.shape[1] < heads * pad or q.dtype != out.dtype or not q.is_cuda:
        raise KernelError("attention_talking: q must be [T, >= heads * pad] of the output's dtype")
    width = tables.shape[1]
    _check(lib().cisr_attn_talking(q.data_ptr(), int(q_row_stride), _dev(kcache, "kcache", out.dtype, (pages, kv_heads, page_size, pad)),
                                   _dev(vcache, "vcache", out.dtype, (pages, kv_heads, pad, page_size)),
                                   _dev(tables, "tables", torch.int32), _dev(seg_of_row, "seg_of_row", torch.int32, (rows,)),
                                   _dev(positions, "positions", torch.int32, (rows,)), _dev(mix, "mix", torch.float32, (heads, heads)),
                                   None if temp is None else _dev(temp, "temp", torch.float32, (heads,)),
                                   None if sink is None else _dev(sink, "sink", torch.float32, (heads,)), gp, ldg,
                                   _dev(out, "out", None, (rows, heads * vdim)), rows, heads, kv_heads, vdim, pad, page_size, width,
                                   int(window or 0), int(chunk or 0), float(scale), int(splits), po, pm, _storage(out, "out"), _stream()),
           "attention_talking")
    return out


_talking = None


def _talk():
    global _talking
    if _talking is None:
        h = library.load(library.TALKING)
        p, i, f = C.c_void_p, C.c_int, C.c_float
        h.cisr_attn_talking_tiles.argtypes = [p, i, p, p, p, p, i, p, p, p, p, p, i, p, i, i, i, i, i, i, i, i, f, i, i, p, p, p]
        h.cisr_attn_talking_tiles.restype = C.c_int
        _talking = h
    return _talking


TALKING_TILE_ROWS = 16     # rows of a tile of attention_talking_tiles


def talking_tiles_ok(dtype, heads, kv_heads, vdim, pad, page_size):
    """Whether attention_talking_tiles takes these sizes: bfloat16, at most 32 heads of at most 128 coordinates, pages
    of a multiple of 8 keys."""
    return (dtype == torch.bfloat16 and 0 < heads <= 32 and kv_heads > 0 and heads % kv_heads == 0 and 0 < pad <= 128 and pad % 8 == 0
            and 0 < vdim <= pad and page_size > 0 and page_size % 8 == 0)


def attention_talking_tiles(q, kcache, vcache, tables, tasks, positions, out, heads, kv_heads, vdim, pad, page_size, mix, scale,
                            temp=None, sink=None, window=None, chunk=None, gate=None, splits=1, workspace=None):
    """attention_talking on the matrix cores for bfloat16: `tasks` int32 [n, 4] lists tiles of up to 16 consecutive rows of
    one segment (segment, first row, rows, anything; segment -1: no tile); a block takes a tile with all its heads.
    `splits` > 1: that many blocks share a tile's keys and leave their sums in `workspace` = (float [T * heads * splits *
    vdim], float [T * heads * splits * 2]) for a merge kernel that runs behind them."""
    rows = out.shape[0]
    pages = kcache.shape[0]
    if not talking_tiles_ok(out.dtype, heads, kv_heads, vdim, pad, page_size):
        raise KernelError("attention_talking_tiles: sizes not supported")
    gp, ldg = None, 0
    if gate is not None:
        if gate.dtype != torch.float32 or tuple(gate.shape) != (rows, heads * vdim) or gate.stride(1) != 1 or not gate.is_cuda:
            raise KernelError("attention_talking_tiles: the gate must be float [T, heads * vdim] with unit stride")
        gp, ldg = gate.data_ptr(), gate.stride(0)
    if q.dim() != 2 or q.shape[0] != rows or q.stride(1) != 1 or q.shape[1] < heads * pad or q.dtype != out.dtype or not q.is_cuda or q.stride(0) % 8:
        raise KernelError("attention_talking_tiles: q must be bf16 [T, >= heads * pad] with rows of 16-byte chunks")
    if tasks.dtype != torch.int32 or tasks.dim() != 2 or tasks.shape[1] != 4 or not tasks.is_contiguous() or not tasks.is_cuda:
        raise KernelError("attention_talking_tiles: tasks must be int32 [n, 4]")
    po = pm = None
    if splits > 1:
        if workspace is None or workspace[0].numel() < rows * heads * splits * vdim or workspace[1].numel() < rows * heads * splits * 2:
            raise KernelError("attention_talking_tiles: split keys need a workspace for their sums")
        po, pm = _dev(workspace[0], "part_o", torch.float32), _dev(workspace[1], "part_ml", torch.float32)
    _check(_talk().cisr_attn_talking_tiles(q.data_ptr(), q.stride(0), _dev(kcache, "kcache", out.dtype, (pages, kv_heads, page_size, pad)),
                                           _dev(vcache, "vcache", out.dtype, (pages, kv_heads, pad, page_size)), _dev(tables, "tables", torch.int32),
                                           tasks.data_ptr(), tasks.shape[0], _dev(positions, "positions", torch.int32, (rows,)),
                                           _dev(mix, "mix", torch.float32, (heads, heads)),
                                           None if temp is None else _dev(temp, "temp", torch.float32, (heads,)),
                                           None if sink is None else _dev(sink, "sink", torch.float32, (heads,)), gp, ldg,
                                           _dev(out, "out", torch.bfloat16, (rows, heads * vdim)), heads, kv_heads, vdim, pad, page_size,
                                           tables.shape[1], int(window or 0), int(chunk or 0), float(scale), rows, int(splits), po, pm,
                                           _stream()), "attention_talking_tiles")
    return out


class ScratchPool:
    """Device memory that some products need beyond their inputs and outputs: the library's bf16 product before its
    sum into the residual, the wide kernel's partial sums, the slice winners of the argmax.  A buffer is handed out
    again to every later call that it is large enough for, and none is freed before `clear`: captured programs keep
    the addresses.  A step function owns one pool (calls on its stream are ordered, so they can share buffers);
    calls that name no pool share DEFAULT_SCRATCH."""

    def __init__(self):
        self.buffers = {}   # (kind, device, dtype) -> [tensors]

    def get(self, kind, elements, dtype, device):
        pool = self.buffers.setdefault((kind, device, dtype), [])
        for buf in pool:
            if buf.numel() >= elements:
                return buf
        pool.append(torch.empty(1 << max(int(elements) - 1, 0).bit_length(), dtype=dtype, device=device))
        return pool[-1]

    def bytes(self):
        return sum(t.numel() * t.element_size() for pool in self.buffers.values() for t in pool)

    def clear(self):
        self.buffers.clear()


DEFAULT_SCRATCH = ScratchPool()


def library_ok(m, w, gated=False):
    """`gated`: the product of gate and up, whose activation is a kernel of its own after the library's product.  With
    weights of 64 MB and more it goes there from 33 rows on: 64 rows against the 8B sizes' 235 MB take 60.7 us there and
    69.7 in the wide kernel here (58.4 against 63.0 at 33 rows; 23.0 against 26.5 at the 1.7B sizes), the activation
    included; the other products of 33 to 64 rows are as fast here."""
    least = LIBRARY_MIN_ROWS
    if gated and w.numel() * 2 >= LIBRARY_GATED_MIN_BYTES:
        least = min(least, LIBRARY_GATED_MIN_ROWS)
    return (LIBRARY_MIN_ROWS > 0 and m >= least and w.dtype == torch.bfloat16 and w.is_contiguous()
            and w.numel() * 2 >= LIBRARY_MIN_BYTES)


def _scratch_bf16(scratch, device, rows, cols):
    return (scratch or DEFAULT_SCRATCH).get("library", rows * cols, torch.bfloat16, device)[:rows * cols].view(rows, cols)


def gemm(a, w, out, residual=None, after_norm=False, scratch=None):
    """out[M, N] = a[M, K] . w[N, K]^T (+ residual).  float operands run the true
    32-bit kernel; bf16 operands run on the matrix cores with float accumulation.
    out may be float or (bf16 operands only) bf16; residual is float and may be `out`.
    `after_norm`: a hint for the choice of kernel, see wide_ok.  `scratch`: the ScratchPool of the caller's steps."""
    m, k = a.shape
    n, k2 = w.shape
    if k != k2:
        raise KernelError(f"gemm: inner sizes differ ({k} vs {k2})")
    if a.dtype != w.dtype:
        raise KernelError(f"gemm: operand dtypes differ ({a.dtype} vs {w.dtype})")
    if a.stride(1) != 1 or w.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm: rows must be contiguous")
    if tuple(out.shape) != (m, n) or not out.is_cuda or not a.is_cuda or not w.is_cuda:
        raise KernelError("gemm: bad output shape or device")
    rp, ldr = None, 0
    if residual is not None:
        if residual.dtype != torch.float32 or out.dtype != torch.float32 or tuple(residual.shape) != (m, n) or residual.stride(1) != 1:
            raise KernelError("gemm: residual needs float [M, N] and a float output")
        rp, ldr = residual.data_ptr(), residual.stride(0)
    if a.dtype == torch.float32:
        if out.dtype != torch.float32:
            raise KernelError("gemm: float operands need a float output")
        code = lib().cisr_gemm_f32(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0),
                                   rp, ldr, m, n, k, _stream())
    elif (a.dtype == torch.bfloat16 and library_ok(m, w) and a.is_contiguous() and out.is_contiguous()
          and (residual is None or residual is out)):
        if residual is None:
            # (float results are the library's float accumulators as they are: 2,048 rows against 10,240 x 2,048 take 83 us
            # there and 193 in the tiled kernel here)
            if out.dtype == torch.float32:
                torch.mm(a, w.t(), out_dtype=torch.float32, out=out)
            else:
                torch.mm(a, w.t(), out=out)
            return out
        product = _scratch_bf16(scratch, a.device, m, n)
        torch.mm(a, w.t(), out=product)
        return residual_add(out, product)
    elif a.dtype == torch.bfloat16 and m <= SKINNY_ROWS and _skinny_ok(a, w) and wide_ok(m, w, after_norm=after_norm):
        return _gemm_wide(a, w, out, residual, False, "gemm", scratch)
    elif a.dtype == torch.bfloat16 and m <= SKINNY_ROWS and _skinny_ok(a, w):
        code = lib().cisr_gemm_skinny_bf16(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(),
                                           out.stride(0), rp, ldr, m, n, k, _storage(out, "out"), 0, None, 0.0, None,
                                           _stream())
    elif a.dtype == torch.bfloat16:
        code = lib().cisr_gemm_bf16(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0),
                                    rp, ldr, m, n, k, _storage(out, "out"), _stream())
    else:
        raise KernelError(f"gemm: unsupported dtype {a.dtype}")
    _check(code, "gemm")
    return out


# Weights of at least this many bytes are streamed by the kernel that keeps the activations in registers
# (norm, rotary embedding and cache write are then kernels of their own); smaller ones by the kernels that
# fuse them, which cost fewer launches.  Measured on an MI355X against the other kernel in captured graphs:
# with at most 16 rows the activations are a small part of the traffic and the fused kernels hold out up to
# about 64 MB; with 17 to 32 rows the wide kernel wins from about 12 MB on, with more from about 30 MB on
# (a block then holds so much of the activations that it needs many rows of W to spread their cost over).
WIDE_MIN_BYTES_FEW_ROWS = 64 << 20
WIDE_MIN_BYTES = 12 << 20
WIDE_MIN_BYTES_MANY_ROWS = 30 << 20
_wide_plans = {}


def wide_ok(m, w, swiglu=False, after_norm=False):
    """Whether a product of m rows with the bf16 weights w runs the wide weight-streaming kernel.
    `after_norm`: the rows are the output of an RMSNorm, which the other kernel would fuse (it then reads the
    float residual and the norm's weights for every 16 rows of W, which costs it more than bf16 rows do)."""
    n, k = w.shape
    if gemv_ok(m, n, k):   # up to four rows against large weights: the matrix-vector kernel takes them
        return False
    least = WIDE_MIN_BYTES_FEW_ROWS if m <= 16 else WIDE_MIN_BYTES if m <= 32 else WIDE_MIN_BYTES_MANY_ROWS
    if m <= 16 and n < 16 * _compute_units(w.device) and k >= 4096:
        # a narrow output with a long inner size: the fused kernels have a block for every 16 columns and
        # cannot fill the GPU; this one cuts K as well
        least = min(least, max(WIDE_MIN_BYTES, 16 << 20))
    if m >= 4 and after_norm and k >= 2048:     # (one or two rows of the residual cost the fused kernel next to nothing)
        least = min(least, max(WIDE_MIN_BYTES, 24 << 20))
    if (w.dtype != torch.bfloat16 or not 0 < m <= SKINNY_ROWS or w.numel() * 2 < least or k % 8 or w.stride(0) % 8
            or w.data_ptr() % 16 or w.stride(1) != 1):
        return False
    return _wide_plan(m, n // 2 if swiglu else n, k, swiglu) >= 0


GEMV_ROWS, GEMV_MIN_BYTES = 4, 4 << 20


def gemv_ok(m, n, k):
    """Whether a product of m rows with weights [n, k] runs the matrix-vector kernel (up to four rows against weights
    of 4 MB and more with an inner size of at least 1024: a wave owns whole rows of the weights; see csrc/gemv.hip
    and the measurements in csrc/gemm_skinny.hip).  The weight-streaming entry points choose it themselves; callers ask only to know that
    the wide kernel and its separate norm are not wanted."""
    return bool(lib().cisr_gemv_ok(int(m), int(n), int(k)))


def set_gemv(rows=GEMV_ROWS, least_bytes=GEMV_MIN_BYTES):
    """The most rows (0 to 8; 0 switches it off) and the least bytes of weights that the matrix-vector kernel is given
    (least_bytes 0 also lifts the rule's least inner size): for measurements and tests.  Without arguments: the rule
    as it is."""
    lib().cisr_gemv_set(int(rows), int(least_bytes))


_units = {}


def _compute_units(device):
    if device not in _units:
        _units[device] = torch.cuda.get_device_properties(device).multi_processor_count
    return _units[device]


def _wide_plan(m, n, k, swiglu):
    key = ((m + 15) // 16, m, n, k, swiglu)
    need = _wide_plans.get(key)
    if need is None:
        need = _wide_plans[key] = int(lib().cisr_gemm_wide_workspace(m, n, k, n if swiglu else 0))
    return need


def _wide_workspace(scratch, device, floats):
    if floats <= 0:
        return None
    return (scratch or DEFAULT_SCRATCH).get("wide", floats, torch.float32, device)


def _gemm_wide(a, w, out, residual, swiglu, what, scratch=None):
    m, k = a.shape
    n = w.shape[0] // 2 if swiglu else w.shape[0]
    need = _wide_plan(m, n, k, swiglu)
    if need < 0 or a.stride(0) % 8 or a.data_ptr() % 16:
        raise KernelError(f"{what}: shape not supported by the wide kernel")
    work = _wide_workspace(scratch, a.device, need)
    rp, ldr = (residual.data_ptr(), residual.stride(0)) if residual is not None else (None, 0)
    _check(lib().cisr_gemm_wide_bf16(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0),
                                     rp, ldr, m, n, k, _storage(out, "out"), n if swiglu else 0,
                                     None if work is None else work.data_ptr(), 0 if work is None else work.numel(),
                                     _stream()), what)
    return out


def gemm_unfinished(a, w, residual, scratch=None):
    """The product a . w^T that is to be added to the float rows `residual`, left unfinished where adding it takes a
    kernel of its own: the wide kernel's partial sums of a product cut into slices, (partial sums [slices, M, N],
    slices), or the library's bf16 product, (product [M, N], 0); rmsnorm_partials or add_partials then are that
    kernel.  None (nothing done) for every other product: call gemm."""
    m, k = a.shape
    n = w.shape[0]
    if (a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.shape[1] != k or tuple(residual.shape) != (m, n)
            or not partials_ok(residual)):
        return None
    if library_ok(m, w):
        if not a.is_contiguous():
            return None
        product = _scratch_bf16(scratch, a.device, m, n)
        torch.mm(a, w.t(), out=product)
        return product, 0
    if not 0 < m <= SKINNY_ROWS or not _skinny_ok(a, w) or not wide_ok(m, w):
        return None
    need = _wide_plan(m, n, k, False)
    if need <= 0:
        return None
    work = _wide_workspace(scratch, a.device, need)
    _check(lib().cisr_gemm_wide_partials_bf16(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), m, n, k,
                                              work.data_ptr(), work.numel(), _stream()), "gemm_unfinished")
    return work, need // (m * n)


def _skinny_ok(a, w):
    k = a.shape[1]
    return (k % 8 == 0 and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def _norm_args(x, norm, k):
    """(weight pointer, eps, rows pointer, number of output rows) for a fused RMSNorm prologue."""
    weight, eps, rows = norm
    if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dtype != torch.float32 or x.dim() != 2 or x.stride(1) != 1:
        raise KernelError("fused norm: expected float GPU rows with unit column stride (a view of wider rows will do)")
    if x.shape[1] != k or x.stride(0) % 8 or x.data_ptr() % 16:
        raise KernelError("fused norm: the residual rows must be 32-byte aligned floats of the product's inner size")
    wp = _dev(weight, "norm weight", torch.float32, (k,))
    rp = None if rows is None else _dev(rows, "rows", torch.int32)
    return wp, float(eps), rp, (x.shape[0] if rows is None else rows.shape[0])


def fused_norm_ok(x, w, rows_out):
    """Whether the weight-streaming kernel can take RMSNorm(x) . w^T with the norm fused (and large weights
    do not make the norm as a kernel of its own and the wide kernel the better choice)."""
    return (not wide_ok(rows_out, w, after_norm=True) and w.dtype == torch.bfloat16 and rows_out <= SKINNY_ROWS and x.dtype == torch.float32 and x.shape[1] % 8 == 0
            and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0)


def swiglu_fused_ok(a, w_gate_up):
    """Whether gemm_swiglu runs as one kernel for these operands (no scratch buffer needed): bf16 with
    16-byte aligned rows; few rows take the weight-streaming kernel, more the tiled one."""
    return a.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16 and a.is_cuda and _skinny_ok(a, w_gate_up)


def gemm_normed(x, norm, w, out):
    """out[R, N] = RMSNorm(x[rows]) . w^T with the norm applied inside the product's kernel.
    x float [T, K]; norm = (weight float [K], eps, rows int32 [R] or None); w bf16 [N, K]; out float or bf16."""
    n, k = w.shape
    wp, eps, rp, m = _norm_args(x, norm, k)
    if not fused_norm_ok(x, w, m) or tuple(out.shape) != (m, n) or out.stride(1) != 1:
        raise KernelError("gemm_normed: shape not supported by the fused kernel")
    _check(lib().cisr_gemm_skinny_bf16(x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0),
                                       None, 0, m, n, k, _storage(out, "out"), 0, wp, eps, rp, _stream()), "gemm_normed")
    return out


def gemm_swiglu(a, w_gate_up, out, gate_up=None, norm=None, scratch=None, law=None):
    """out[M, I] = silu(a . Wg^T) * (a . Wu^T) with w_gate_up = [Wg; Wu] ([2I, K]); with `law` = (limit, slope, shift)
    the activation is g sigmoid(slope g) (u + shift), g = min(gate, limit), u = clamp(up, -limit, limit) instead.
    Few rows of bf16 run one fused weight-streaming kernel (with `norm` = (weight, eps, None), `a` is the float
    residual and RMSNorm is fused too); otherwise the product goes to `gate_up` [M, 2I] and the activation is
    a second kernel.  `scratch`: the ScratchPool of the caller's steps."""
    m, k = a.shape
    two_i, k2 = w_gate_up.shape
    inter = two_i // 2
    if k != k2 or two_i % 2 or tuple(out.shape) != (m, inter) or not out.is_contiguous():
        raise KernelError("gemm_swiglu: shapes do not fit")
    if norm is not None:
        if law is not None:
            raise KernelError("gemm_swiglu: the fused norm comes with the silu law only")
        wp, eps, rp, _ = _norm_args(a, norm, k)
        if not fused_norm_ok(a, w_gate_up, m) or out.dtype != torch.bfloat16:
            raise KernelError("gemm_swiglu: shape not supported by the fused kernel")
        _check(lib().cisr_gemm_skinny_bf16(a.data_ptr(), a.stride(0), w_gate_up.data_ptr(), w_gate_up.stride(0),
                                           out.data_ptr(), out.stride(0), None, 0, m, inter, k, BF16, inter, wp, eps, rp,
                                           _stream()), "gemm_swiglu")
        return out
    if out.dtype != a.dtype or a.dtype != w_gate_up.dtype:
        raise KernelError("gemm_swiglu: dtypes differ")
    activate = swiglu if law is None else (lambda gu, o: glu_clamped(gu, o, *law))
    if a.dtype == torch.bfloat16 and library_ok(m, w_gate_up, gated=True) and a.is_contiguous():
        product = _scratch_bf16(scratch, a.device, m, two_i)
        torch.mm(a, w_gate_up.t(), out=product)
        return activate(product, out)
    if swiglu_fused_ok(a, w_gate_up) and law is not None:
        # the same kernels with the activation's law given
        lim, slope, shift = (float(x) for x in law)
        if m <= SKINNY_ROWS and wide_ok(m, w_gate_up, True, after_norm=True):
            need = _wide_plan(m, inter, k, True)
            if need < 0 or a.stride(0) % 8 or a.data_ptr() % 16:
                raise KernelError("gemm_swiglu: shape not supported by the wide kernel")
            work = _wide_workspace(scratch, a.device, need)
            code = lib().cisr_gemm_wide_bf16_gated(a.data_ptr(), a.stride(0), w_gate_up.data_ptr(), w_gate_up.stride(0), out.data_ptr(),
                                                   out.stride(0), m, inter, k, inter, lim, slope, shift,
                                                   None if work is None else work.data_ptr(), 0 if work is None else work.numel(), _stream())
        elif m <= SKINNY_ROWS:
            code = lib().cisr_gemm_skinny_bf16_gated(a.data_ptr(), a.stride(0), w_gate_up.data_ptr(), w_gate_up.stride(0), out.data_ptr(),
                                                     out.stride(0), m, inter, k, inter, lim, slope, shift, _stream())
        else:
            code = lib().cisr_gemm_bf16_gated(a.data_ptr(), a.stride(0), w_gate_up.data_ptr(), w_gate_up.stride(0), out.data_ptr(),
                                              out.stride(0), m, inter, k, inter, lim, slope, shift, _stream())
        _check(code, "gemm_swiglu")
        return out
    if swiglu_fused_ok(a, w_gate_up):
        if m <= SKINNY_ROWS and wide_ok(m, w_gate_up, True, after_norm=True):
            return _gemm_wide(a, w_gate_up, out, None, True, "gemm_swiglu", scratch)
        if m <= SKINNY_ROWS:
            _check(lib().cisr_gemm_skinny_bf16(a.data_ptr(), a.stride(0), w_gate_up.data_ptr(), w_gate_up.stride(0),
                                               out.data_ptr(), out.stride(0), None, 0, m, inter, k, BF16, inter, None, 0.0,
                                               None, _stream()), "gemm_swiglu")
        else:   # many rows: the tiled product with the activation as its epilogue
            _check(lib().cisr_gemm_bf16_swiglu(a.data_ptr(), a.stride(0), w_gate_up.data_ptr(), w_gate_up.stride(0),
                                               out.data_ptr(), out.stride(0), m, inter, k, inter, _stream()), "gemm_swiglu")
        return out
    if gate_up is None:
        raise KernelError("gemm_swiglu: this shape needs a buffer [M, 2I] for the product of gate and up")
    gemm(a, w_gate_up, gate_up, scratch=scratch)
    return activate(gate_up, out)


def qkv_rope_fused_ok(a, w, head_dim, cos, normed):
    """Whether the fused projection + rotary + scatter kernel takes this shape."""
    m, k = a.shape
    if normed and wide_ok(m, w, after_norm=True):      # large weights: the norm is a kernel of its own, the projection the wide kernel
        return False
    return (w.dtype == torch.bfloat16 and m <= SKINNY_ROWS and k % 8 == 0 and head_dim % 16 == 0
            and 2 * cos.shape[1] == head_dim and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0
            and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0
            and a.dtype == (torch.float32 if normed else torch.bfloat16))


def qkv_rope(a, w, q_out, positions, slots, cos, sin, kcache, vcache, heads, kv_heads, dim, page_size, norm=None, scratch=None):
    """One kernel for a decode step's projections: (RMSNorm of the float residual `a` if `norm` = (weight, eps),
    else `a` is bf16 and normed), product with w = [Wq; Wk; Wv], rotary embedding of q and k, q into
    q_out [M, heads*dim], k and v into the cache at `slots`.  kcache None: w = Wq only (a layer reading
    another layer's cache)."""
    m, k = a.shape
    has_kv = kcache is not None
    n_kv = kv_heads if has_kv else 0
    if not qkv_rope_fused_ok(a, w, dim, cos, norm is not None) or tuple(w.shape) != ((heads + 2 * n_kv) * dim, k):
        raise KernelError("qkv_rope: shape not supported by the fused kernel")
    wp, eps = (None, 0.0)
    if norm is not None:
        wp, eps = _dev(norm[0], "norm weight", torch.float32, (k,)), float(norm[1])
    kp = vp = sp = None
    if has_kv:
        pages = kcache.shape[0]
        kp = _dev(kcache, "kcache", torch.bfloat16, (pages, kv_heads, page_size, dim))
        vp = _dev(vcache, "vcache", torch.bfloat16, (pages, kv_heads, dim, page_size))
        sp = _dev(slots, "slots", torch.int32, (m,))
    max_pos = cos.shape[0]
    if norm is None and wide_ok(m, w, after_norm=True):
        need = _wide_plan(m, w.shape[0], k, False)
        work = _wide_workspace(scratch, a.device, need)
        _check(lib().cisr_qkv_rope_wide(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0),
                                        _dev(q_out, "q_out", torch.bfloat16, (m, heads * dim)), heads * dim, m, k,
                                        _dev(positions, "positions", torch.int32, (m,)), sp,
                                        _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32, (max_pos, dim // 2)),
                                        kp, vp, heads, n_kv, dim, page_size, max_pos,
                                        None if work is None else work.data_ptr(), 0 if work is None else work.numel(),
                                        _stream()), "qkv_rope")
        return q_out
    _check(lib().cisr_qkv_rope_skinny(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0),
                                      _dev(q_out, "q_out", torch.bfloat16, (m, heads * dim)), heads * dim, m, k, wp, eps,
                                      _dev(positions, "positions", torch.int32, (m,)), sp,
                                      _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32, (max_pos, dim // 2)),
                                      kp, vp, heads, n_kv, dim, page_size, max_pos, _stream()), "qkv_rope")
    return q_out


def attention_mfma(q, q_row_stride, kcache, vcache, tables, seg_of_row, positions, out, heads, kv_heads, dim,
                   page_size, window, scale, tasks=None, splits=1, workspace=None, waves=4, block_tiles=False,
                   item_tiles=1, row_ids=None, merge=True, key_groups=1, stream_loads=False, head_bias=None):
    """Matrix-core attention (bf16).  tasks int32 [n, 4] = (segment, first row, rows, 0) runs tiles of
    prompt rows: one tile of 16/GC rows a block whose waves share the keys (with item_tiles=2, head sizes up to
    64: 32/GC rows, two item tiles a wave), or with `block_tiles` (head sizes up to 128) one tile of
    64 item_tiles / GC rows a block whose four waves own different rows and share keys and values through LDS
    (GC = query heads per key head, at most 16); tasks None runs one block
    per row (decode) of `waves` wavefronts (4 or 8) with `splits` blocks along the keys; splits > 1 needs
    workspace = (partials float, statistics float) and a merge.  `row_ids` (int32 [n], with tasks None): only
    the rows it lists are computed and written (negative entries are skipped): the decode rows of a mixed step.
    `merge` False (rows mode with splits > 1): the partial outputs are left unmerged in the workspace, whose first
    buffer is then bfloat16, for gemm_merged; `out` is not written.  `key_groups` 2 (block_tiles 32): a block is two
    halves that take the even and the odd 32-key steps of its items and merge at the end.  `stream_loads` (rows mode):
    keys and values are read with non-temporal loads, which the caches do not keep.
    `head_bias` (float [heads]): the sigmoid law (see attention_rowwise); the tile and row forms have it, the block
    tiles do not, and the partial results of split keys are plain sums that only this function merges."""
    rows = out.shape[0]
    if head_bias is not None and (block_tiles or not merge):
        raise KernelError("attention_mfma: the sigmoid law runs as tiles and rows, merged here")
    if not mfma_attention_supported(out.dtype, dim, page_size):
        raise KernelError(f"attention_mfma: head size {dim} / page size {page_size} / dtype {out.dtype} not supported")
    if heads % kv_heads:
        raise KernelError(f"attention: {heads} query heads do not divide into {kv_heads} key heads")
    if not scale > 0:
        raise KernelError("attention_mfma: the score scale must be positive (the maximum is taken before scaling)")
    if q.dtype != out.dtype or kcache.dtype != out.dtype or q_row_stride % 8 or q.data_ptr() % 16:
        raise KernelError("attention_mfma: q, cache and out must be bfloat16 with 16-byte aligned rows")
    if q.numel() < (rows - 1) * q_row_stride + heads * dim:
        raise KernelError("attention: q buffer too small for its stride")
    pages = kcache.shape[0]
    if kcache.numel() >= 2 ** 31 or vcache.numel() >= 2 ** 31:
        raise KernelError("attention_mfma: a layer's keys (or values) must be fewer than 2^31 elements (32-bit byte offsets)")
    dpad = -(-dim // 32) * 32
    fn = _attention_entry(dpad, "softmax" if head_bias is None else "sigmoid")
    law = () if head_bias is None else (_dev(head_bias, "head_bias", torch.float32, (heads,)),)
    po = pm = tp = None
    if tasks is not None:
        if item_tiles not in ((1, 2, 3, 4) if block_tiles == 32 else (1, 2)) or (item_tiles == 2 and dim > 64 and not block_tiles):
            raise KernelError("attention_mfma: two item tiles a wave need a head size of at most 64")
        if block_tiles and dpad > 128:
            raise KernelError("attention_mfma: block tiles need a head size of at most 128")
        n_tasks, splits = tasks.shape[0], 1
        mode = (2 if item_tiles == 1 else 4) if block_tiles else (3 if item_tiles == 2 else 0)
        if block_tiles == 32:
            # the 32 x 32 matrix instruction: 128/GC rows a block and four waves (item_tiles 2), or 64/GC rows and two
            if out.numel() >= 2 ** 31:
                raise KernelError("attention_mfma: the output must be fewer than 2^31 elements (32-bit offsets)")
            if page_size < 8 or dpad > 128:
                raise KernelError("attention_mfma: 32 x 32 block tiles need pages of at least 8 keys and a head size of at most 128")
            if key_groups not in (1, 2) or (key_groups == 2 and item_tiles >= 3):
                raise KernelError("attention_mfma: one or two key groups, two with 64 or 128 items a block")
            if dpad > 64 and (item_tiles == 4 or (item_tiles == 2 and key_groups == 2)):
                raise KernelError("attention_mfma: blocks of more than eight waves need a head size of at most 64")
            mode = {(1, 1): 6, (2, 1): 5, (3, 1): 10, (4, 1): 7, (1, 2): 8, (2, 2): 9}[(item_tiles, key_groups)]
        tp = _dev(tasks, "tasks", torch.int32, (n_tasks, 4))
    else:
        n_tasks, mode = rows, 1
        if row_ids is not None:
            n_tasks = row_ids.numel()
            tp = _dev(row_ids, "row_ids", torch.int32, (n_tasks,))
        if splits > 1:
            if workspace is None:
                raise KernelError("attention: split runs need a workspace")
            part_o, part_ml = workspace
            po, pm = _dev(part_o, "part_o", torch.float32 if merge else torch.bfloat16), _dev(part_ml, "part_ml", torch.float32)
            if part_o.numel() < n_tasks * heads * splits * dim or part_ml.numel() < n_tasks * heads * splits * 2:
                raise KernelError("attention: split workspace too small")
    _check(fn(q.data_ptr(), q_row_stride, _dev(kcache, "kcache", None, (pages, kv_heads, page_size, dim)),
              _dev(vcache, "vcache", None, (pages, kv_heads, dim, page_size)), _dev(tables, "tables", torch.int32),
              tables.shape[1], tp, n_tasks, _dev(seg_of_row, "seg_of_row", torch.int32, (rows,)),
              _dev(positions, "positions", torch.int32, (rows,)), _dev(out, "out", None, (rows, heads * dim)), po, pm,
              heads, kv_heads, dim, page_size.bit_length() - 1, int(window or 0), float(scale), int(splits),
              11 if mode == 1 and stream_loads else mode, int(waves),
              int(mode == 1 and splits > 1 and not merge), _stream(), *law), "attention_mfma")
    if mode == 1 and splits > 1 and merge:
        if head_bias is not None:
            _check(lib().cisr_attn_merge_sum(po, out.data_ptr(), n_tasks, heads, dim, int(splits), tp, _stream()), "attention_merge")
        else:
            _check(lib().cisr_attn_merge(po, pm, out.data_ptr(), n_tasks, heads, dim, int(splits), tp, _stream()), "attention_merge")
    return out


def gemm_merged_ok(m, w, heads, dim, splits):
    """Whether gemm_merged takes m rows of `splits` partial attention results of heads x dim against the bf16 weights w."""
    return (w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] == heads * dim and w.stride(1) == 1 and w.stride(0) % 8 == 0
            and w.data_ptr() % 16 == 0 and bool(lib().cisr_gemm_merged_ok(int(m), int(w.shape[0]), int(heads), int(dim), int(splits))))


def gemm_merged(partials, heads, dim, w, out, residual):
    """out[M, N] = residual + merge(partials) . w^T in float: the output projection of a decode step whose attention
    was split over `splits` blocks along the keys and left unmerged (attention_mfma with merge=False).
    partials = (bf16 [M, heads, splits, dim] normalised partial outputs, float [M, heads, splits, 2] statistics, splits)."""
    part_o, part_ml, splits = partials
    m, n = out.shape
    if not gemm_merged_ok(m, w, heads, dim, splits) or w.shape[0] != n:
        raise KernelError("gemm_merged: shape not supported by the fused kernel")
    if out.dtype != torch.float32 or out.stride(1) != 1 or tuple(residual.shape) != (m, n) or residual.dtype != torch.float32 or residual.stride(1) != 1:
        raise KernelError("gemm_merged: float output and residual [M, N]")
    if part_o.numel() < m * heads * splits * dim or part_ml.numel() < m * heads * splits * 2:
        raise KernelError("gemm_merged: partial results too small")
    _check(lib().cisr_gemm_merged_bf16(_dev(part_o, "part_o", torch.bfloat16), _dev(part_ml, "part_ml", torch.float32), int(splits),
                                       int(heads), int(dim), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0),
                                       residual.data_ptr(), residual.stride(0), m, n, _stream()), "gemm_merged")
    return out


def mfma_attention_supported(dtype, dim, page_size):
    return (dtype == torch.bfloat16 and dim % 8 == 0 and dim <= 256 and page_size >= 8
            and page_size & (page_size - 1) == 0)



def _scatter(out, index, rows):
    """(pointer of index or None, length of out) for a token choice that writes out[index[r]]."""
    if index is None:
        _dev(out, "out", torch.int32, (rows,))
        return None, rows
    _dev(out, "out", torch.int32)
    return _dev(index, "index", torch.int32, (rows,)), out.numel()


def argmax(logits, out, index=None, scratch=None):
    """out[r] = index of the largest logit of row r (the lowest index wins a tie).  With `index`
    (int32 [R]) the result of row r goes to out[index[r]] instead, or nowhere if that is no place of out."""
    rows, vocab = logits.shape
    pool = scratch or DEFAULT_SCRATCH
    val = pool.get("argmax", rows * 32, torch.float32, logits.device)
    idx = pool.get("argmax", rows * 32, torch.int32, logits.device)
    where, out_n = _scatter(out, index, rows)
    _check(lib().cisr_argmax(_dev(logits, "logits", torch.float32), out.data_ptr(), where, out_n,
                             val.data_ptr(), idx.data_ptr(), rows, vocab, _stream()), "argmax")
    return out


def sample(logits, temperature, seeds, counters, out, index=None):
    """Temperature sampling per row; temperature <= 0 is greedy.  seeds/counters int64 [R].
    `index` as for argmax."""
    rows, vocab = logits.shape
    where, out_n = _scatter(out, index, rows)
    _check(lib().cisr_sample(_dev(logits, "logits", torch.float32), _dev(temperature, "temperature", torch.float32, (rows,)),
                             _dev(seeds, "seeds", torch.int64, (rows,)), _dev(counters, "counters", torch.int64, (rows,)),
                             out.data_ptr(), where, out_n, rows, vocab, _stream()), "sample")
    return out


def take_tokens(tokens, source, sampled):
    """tokens[r] = sampled[source[r]] for the rows whose source is a place of `sampled` (all int32)."""
    rows = tokens.numel()
    _check(lib().cisr_take_tokens(_dev(tokens, "tokens", torch.int32), _dev(source, "source", torch.int32, (rows,)),
                                  _dev(sampled, "sampled", torch.int32), rows, sampled.numel(), _stream()), "take_tokens")
    return tokens


# -- layers that norm a sublayer's output, clamped gates, normed and gated attention ----------------------------------

class Partials:
    """A product [rows, cols] that the wide kernel cut along its inner size and left as partial sums: `parts` float
    [slices * rows * cols], to be added in slice order by the kernel that reads the product next (post_norm_add)."""

    def __init__(self, parts, slices, rows, cols):
        self.parts, self.slices, self.rows, self.cols = parts, int(slices), int(rows), int(cols)


PARTIALS_MAX_COLS = 4096      # rows that post_norm_add holds in registers: only those take partial sums


def gemm_for_norm(a, w, out, make_buffer, scratch=None):
    """a . w^T for a reader that can add partial sums (post_norm_add): where the wide kernel cuts the product along
    its inner size, its slices' partial sums are left in a buffer of the caller's (`make_buffer(floats)`: not the
    shared scratch, which the next wide product would overwrite) and a Partials is returned; every other product is
    finished into `out` (float [M, N]) and `out` is returned."""
    m, k = a.shape
    n = w.shape[0]
    if (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and 0 < m <= SKINNY_ROWS and n <= PARTIALS_MAX_COLS
            and not library_ok(m, w) and _skinny_ok(a, w) and wide_ok(m, w)):
        need = _wide_plan(m, n, k, False)
        if need > 0:
            work = make_buffer(need)
            _check(lib().cisr_gemm_wide_partials_bf16(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), m, n, k,
                                                      _dev(work, "partial sums", torch.float32), work.numel(), _stream()), "gemm_for_norm")
            return Partials(work, need // (m * n), m, n)
    return gemm(a, w, out, scratch=scratch)


class Biased:
    """Float rows [T, N] that still lack a bias a column (float [N]): a product's result whose bias is left to the kernel
    that reads it next (post_norm_add adds it on the way)."""

    def __init__(self, rows, bias):
        self.rows, self.bias = rows, bias


def post_norm_add(x, y, weight, eps, mult, second=None, following=None):
    """x += mult * rmsnorm(y) * weight, in place (all float, [T, H]).  With `second` = (y2, w1, w2) the row that is
    normed is (rmsnorm(y) w1 + rmsnorm(y2) w2) / 2: two sublayers side by side; with `second` = (y2, c1, c2), two
    numbers, it is the plain sum c1 y + c2 y2.  `weight` None: no outer norm,
    x += mult * row.  `following` = (weight float [H], eps, out [T, H] float or bf16): the norm that reads x next is made
    by the same kernel, out = rmsnorm(x) * weight; a weight of None: out is the new x itself in out's type.
    y (and y2) may be a Partials of [T, H]: its slices are added on the way."""
    rows, dim = x.shape
    xp = _dev(x, "x", torch.float32)
    bias_p = None
    if isinstance(y, Biased):          # (y + bias, added as the rows are read)
        bias_p, y = _dev(y.bias, "bias of y", torch.float32, (dim,)), y.rows

    def operand(t, name):
        if isinstance(t, Partials):
            if (t.rows, t.cols) != (rows, dim) or dim > PARTIALS_MAX_COLS or t.parts.numel() < t.slices * rows * dim:
                raise KernelError(f"post_norm_add: {name} is not the partial sums of a product [{rows}, {dim}]")
            return _dev(t.parts, name, torch.float32), t.slices
        return _dev(t, name, torch.float32, (rows, dim)), 0

    yp, slices_a = operand(y, "y")
    slices_b = 0
    wp = None if weight is None else _dev(weight, "weight", torch.float32, (dim,))
    ap = bp = w2p = None
    ca = cb = 0.0
    if second is not None:
        y2, w1, w2 = second
        bp, slices_b = operand(y2, "y2")
        if isinstance(w1, torch.Tensor):
            ap, w2p = _dev(w1, "w1", torch.float32, (dim,)), _dev(w2, "w2", torch.float32, (dim,))
        else:
            ca, cb = float(w1), float(w2)
    np_, neps, op, odt = None, 0.0, None, F32
    if following is not None:
        nw, neps, out = following
        np_ = None if nw is None else _dev(nw, "following weight", torch.float32, (dim,))
        op, odt = _dev(out, "following out", None, (rows, dim)), _storage(out, "following out")
    _check(lib().cisr_post_norm_add(xp, yp, ap, bp, w2p, wp, rows, dim, float(eps), float(mult), np_, float(neps), op, odt,
                                    slices_a, slices_b, ca, cb, bias_p, _stream()), "post_norm_add")
    return x


def glu_clamped(gate_up, out, limit, slope=1.702, shift=1.0):
    """out[r, i] = g sigmoid(slope g) (u + shift), g = min(gate_up[r, i], limit), u = clamp(gate_up[r, I + i], -limit, limit)."""
    rows, two_i = gate_up.shape
    if two_i % 2:
        raise KernelError("glu_clamped: input width must be even")
    inter = two_i // 2
    _check(lib().cisr_glu_clamped(_dev(gate_up, "gate_up"), _dev(out, "out", gate_up.dtype, (rows, inter)), rows, inter,
                                  float(limit), float(slope), float(shift), _storage(gate_up, "gate_up"), _stream()), "glu_clamped")
    return out


def qk_norm_scatter(qkv, q_norm, k_norm, q_out, kcache, vcache, slots, heads, kv_heads, dim, vdim, pad, page_size, eps):
    """Rows of a fused projection [q: heads x dim | k: kv_heads x dim | v: kv_heads x vdim | ...]: queries and keys
    RMS-normed per head (weights float [dim], or None: left as they are), queries into q_out [T, heads * pad], keys and
    values into the cache at `slots`, all as heads of `pad` coordinates whose rest is zero (keys [pages, kv_heads,
    page_size, pad], values transposed in a page, [pages, kv_heads, pad, page_size])."""
    rows, ld = qkv.shape
    if dim > pad or vdim > pad or pad > 256 or ld < (heads + kv_heads) * dim + kv_heads * vdim:
        raise KernelError(f"qk_norm_scatter: heads of {dim} / {vdim} do not fit rows of {ld} or pages of {pad}")
    pages = kcache.shape[0]
    wq = None if q_norm is None else _dev(q_norm, "q_norm", torch.float32, (dim,))
    wk = None if k_norm is None else _dev(k_norm, "k_norm", torch.float32, (dim,))
    _check(lib().cisr_qk_norm_scatter(_dev(qkv, "qkv"), ld, wq, wk, _dev(q_out, "q_out", qkv.dtype, (rows, heads * pad)),
                                      _dev(kcache, "kcache", qkv.dtype, (pages, kv_heads, page_size, pad)),
                                      _dev(vcache, "vcache", qkv.dtype, (pages, kv_heads, pad, page_size)),
                                      _dev(slots, "slots", torch.int32, (rows,)), rows, heads, kv_heads, dim, vdim, pad,
                                      page_size, float(eps), _storage(qkv, "qkv"), _stream()), "qk_norm_scatter")
    return q_out


def head_gate(attn, gates, out, heads, vdim, pad):
    """out[t, h, :] = attn[t, h, :vdim] * sigmoid(gates[t, h]); attn [T, heads * pad], gates a view [T, heads] of a
    row-major buffer (or None: no gate, the heads are only packed), out [T, heads * vdim]."""
    rows = attn.shape[0]
    gp, ldg = None, 0
    if gates is not None:
        if gates.dtype != attn.dtype or tuple(gates.shape) != (rows, heads) or gates.stride(1) != 1 or not gates.is_cuda:
            raise KernelError("head_gate: gates must be [T, heads] of the activations' dtype with unit stride")
        gp, ldg = gates.data_ptr(), gates.stride(0)
    _check(lib().cisr_head_gate(_dev(attn, "attn", None, (rows, heads * pad)), gp, ldg,
                                _dev(out, "out", attn.dtype, (rows, heads * vdim)), rows, heads, vdim, pad,
                                _storage(attn, "attn"), _stream()), "head_gate")
    return out


# -- layers with a centred norm, latent attention, an ungated feed-forward (csrc/elementwise_latent.hip) --------------

def layernorm(x, weight, out, eps, rows=None, bias=None):
    """out = (x[rows] - mean) / sqrt(var + eps) * weight (+ bias), var the mean of the squared deviations.
    x float [T, H]; weight, bias float [H]; out [R, H] float or bf16."""
    dim = x.shape[1]
    n_out = out.shape[0]
    if rows is None and n_out != x.shape[0]:
        raise KernelError("layernorm: out rows differ from input rows")
    rp = None if rows is None else _dev(rows, "rows", torch.int32, (n_out,))
    bp = None if bias is None else _dev(bias, "bias", torch.float32, (dim,))
    _check(lib().cisr_layernorm(_dev(x, "x", torch.float32), _dev(weight, "weight", torch.float32, (dim,)), bp,
                                _dev(out, "out", None, (n_out, dim)), rp, n_out, dim, float(eps), _storage(out, "out"),
                                _stream()), "layernorm")
    return out


def rms_slice(x, weight, out, eps):
    """out = x / sqrt(mean(x^2) + eps) * weight over the columns of the float view x [T, n] of a row-major buffer;
    weight float [n]; out [T, n] float or bf16."""
    rows, n = x.shape
    xp, ld = _rows_of(x, "x")
    _check(lib().cisr_rms_slice(xp, ld, 0, _dev(weight, "weight", torch.float32, (n,)), _dev(out, "out", None, (rows, n)),
                                rows, n, float(eps), _storage(out, "out"), _stream()), "rms_slice")
    return out


def latent_keys(down, weight, q, q_out, kcache, vcache, positions, slots, cos, sin, heads, dim, rot_dim, rank, pad,
                page_size, eps, interleaved=False):
    """Rows of a latent attention's down-projection `down` (a float view [T, rank + rot_dim]): the first `rank` columns
    RMS-normed with `weight` are the latent c, the last `rot_dim` the key part that turns with the position (its first
    2 * cos.shape[1] coordinates; pair i is (i, i + pairs) or, `interleaved`, (2i, 2i + 1)).  Written at `slots` as one
    key head [c | turned | 0] of `pad` coordinates (kcache [pages, 1, page_size, pad]) and one value head [c | 0]
    (vcache [pages, 1, pad, page_size]).  q [T, heads * (dim + rot_dim)]: the last rot_dim coordinates of each head are
    turned alike and written to q_out[t, h, rank : rank + rot_dim], zeros behind them; q_out[t, h, :rank] is left to
    the caller (the query's product with the key up-projection)."""
    rows = q_out.shape[0]
    dp, ld = _rows_of(down, "down", rank + rot_dim)
    max_pos, half = cos.shape
    if rank + rot_dim > pad or 2 * half > rot_dim or half <= 0:
        raise KernelError(f"latent_keys: {rank} + {rot_dim} coordinates do not fit heads of {pad}, or {2 * half} turn among {rot_dim}")
    if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] != heads * (dim + rot_dim) or q.shape[0] != rows or q.dtype != q_out.dtype:
        raise KernelError("latent_keys: q must be [T, heads * (dim + rot_dim)] of the cache's dtype")
    pages = kcache.shape[0]
    sp = None if slots is None else _dev(slots, "slots", torch.int32, (rows,))
    _check(lib().cisr_latent_keys(dp, ld, 0, _dev(weight, "weight", torch.float32, (rank,)), q.data_ptr(), q.stride(0),
                                  _dev(q_out, "q_out", None, (rows, heads * pad)),
                                  _dev(kcache, "kcache", q_out.dtype, (pages, 1, page_size, pad)),
                                  _dev(vcache, "vcache", q_out.dtype, (pages, 1, pad, page_size)),
                                  _dev(positions, "positions", torch.int32, (rows,)), sp,
                                  _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32, (max_pos, half)),
                                  rows, heads, dim, rot_dim, 2 * half, rank, pad, page_size, max_pos, int(bool(interleaved)),
                                  float(eps), _storage(q_out, "q_out"), _stream()), "latent_keys")
    return q_out


def heads_product(a, a_head, w, out, out_head, gate=None):
    """out[t, h * out_head + n] = sum_k a[t, h * a_head + k] w[h, n, k], times sigmoid(gate[t, h]) if `gate` (a float view
    [T, heads]) is given: a small matrix of its own for every head.  a, out row-major views of the compute dtype with
    unit column stride; w [heads, N, K] contiguous."""
    heads, n, k = w.shape
    rows = a.shape[0]
    if (not a.is_cuda or not out.is_cuda or a.dim() != 2 or out.dim() != 2 or a.dtype != w.dtype or out.dtype != w.dtype
            or a.stride(1) != 1 or out.stride(1) != 1 or out.shape[0] != rows):
        raise KernelError("heads_product: GPU operands of one dtype with contiguous rows")
    if a.shape[1] < (heads - 1) * a_head + k or out.shape[1] < (heads - 1) * out_head + n:
        raise KernelError("heads_product: rows too short for their heads")
    gp, ldg = (None, 0) if gate is None else _rows_of(gate, "gate", heads)
    if gate is not None and gate.shape[0] != rows:
        raise KernelError("heads_product: gates differ in rows")
    if w.dtype == torch.bfloat16:
        # the tiled matrix-core product, a launch for all heads (grid.y), the gate in its epilogue
        _check(lib().cisr_gemm_bf16_heads(a.data_ptr(), a.stride(0), int(a_head), _dev(w, "w"), out.data_ptr(), out.stride(0),
                                          int(out_head), gp, ldg, rows, n, k, heads, BF16, _stream()), "heads_product")
        return out
    _check(lib().cisr_heads_product(a.data_ptr(), a.stride(0), int(a_head), _dev(w, "w"), out.data_ptr(), out.stride(0),
                                    int(out_head), gp, ldg, rows, heads, n, k, _storage(w, "w"), _stream()), "heads_product")
    return out


GELU_KINDS = {"gelu": 0, "gelu_erf": 0, "gelu_tanh": 1, "relu2": 2}      # ungated activations (relu2: relu(z)^2)


def gemm_gelu(a, w, out, kind="gelu", scratch=None, product=None):
    """out[M, N] = gelu(a . w^T), out of the operands' dtype.  bf16 products of this repository's own kernels (few rows
    against weights that the wide kernel does not take; many rows against weights that the library does not take) apply
    the activation as their epilogue; the others run the product into `product` ([M, N], a buffer of the caller's) and
    the activation as a kernel after it, as the gated feed-forwards do beside the library's product."""
    if kind not in GELU_KINDS:
        raise KernelError(f"gelu: unknown form {kind!r}")
    m, k = a.shape
    n = w.shape[0]
    fused = (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and tuple(out.shape) == (m, n)
             and w.shape[1] == k and a.stride(1) == 1 and w.stride(1) == 1 and out.stride(1) == 1 and not library_ok(m, w))
    act = 1 + GELU_KINDS[kind]
    if fused and m <= SKINNY_ROWS and _skinny_ok(a, w) and not wide_ok(m, w):
        _check(lib().cisr_gemm_skinny_bf16_act(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0),
                                               m, n, k, BF16, act, _stream()), "gemm_gelu")
        return out
    if fused and m > SKINNY_ROWS:
        _check(lib().cisr_gemm_bf16_act(a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), out.stride(0),
                                        m, n, k, BF16, act, _stream()), "gemm_gelu")
        return out
    if product is None:
        raise KernelError("gemm_gelu: this product needs a buffer for its result before the activation")
    return gelu(gemm(a, w, product, scratch=scratch), out, kind)


def bias_act(x, bias, out, kind):
    """out = act(x + bias[column]): the activation of a product with a bias (float [N]); x, out [M, N] of one dtype."""
    if kind not in GELU_KINDS:
        raise KernelError(f"bias_act: unknown activation {kind!r}")
    _check(lib().cisr_bias_act(_dev(x, "x"), _dev(bias, "bias", torch.float32, (x.shape[1],)), _dev(out, "out", x.dtype, x.shape), x.numel(),
                               x.shape[1], GELU_KINDS[kind], _storage(x, "x"), _stream()), "bias_act")
    return out


def gelu(x, out, kind="gelu"):
    """out = gelu(x): "gelu" the exact form with the error function, "gelu_tanh" the tanh form."""
    if kind not in GELU_KINDS:
        raise KernelError(f"gelu: unknown form {kind!r}")
    _check(lib().cisr_gelu(_dev(x, "x"), _dev(out, "out", x.dtype, x.shape), x.numel(), GELU_KINDS[kind], _storage(x, "x"),
                           _stream()), "gelu")
    return out


# -- mixers with a state per request (the kernels of csrc/recurrence.hip, a shared object of their own) ---------------

_recurrence = None


def _rec():
    global _recurrence
    if _recurrence is None:
        h = library.load(library.RECURRENCE)
        p, i, f, ll = C.c_void_p, C.c_int, C.c_float, C.c_longlong
        sig = {
            "cisr_linear_scan": [p, i, p, i, p, i, p, i, i, p, i, p, i, p, ll, p, p, i, i, i, i, i, f, i, i, i, p, p, p],
            "cisr_conv_silu": [p, i, i, p, p, p, ll, p, p, p, p, i, i, i, i, i, i, p, p, p, p, i, p],
            "cisr_decay_gate": [p, i, p, p, i, i, f, p],
            "cisr_decay_gate_low_rank": [p, i, i, p, p, p, i, i, f, p],
            "cisr_group_norm_gate": [p, p, i, p, i, p, i, p, i, p, i, i, i, f, i, i, p],
            "cisr_delta_scan": [p, i, p, i, p, i, p, i, p, i, p, i, p, ll, p, p, i, i, i, i, i, f, i, p],
            "cisr_unit_heads": [p, i, i, i, i, i, f, f, p],
            "cisr_mingru_scan": [p, i, p, p, p, i, p, p, p, i, i, i, i, p, i, i, p],
            "cisr_mlstm_gates": [p, i, p, i, p, p, p, i, p, p, p, p, p, ll, p, p, i, i, i, i, f, i, p],
            "cisr_mlstm_finish": [p, p, p, i, p, p, i, i, i, f, f, i, p],
        }
        for name, args in sig.items():
            fn = getattr(h, name)
            fn.argtypes = args
            fn.restype = C.c_int
        h.cisr_linear_scan_carry.argtypes = [i, i, i, i, i, i, C.POINTER(ll)]
        h.cisr_linear_scan_carry.restype = ll
        _recurrence = h
    return _recurrence


def _rows_of(t, name, cols=None):
    """(pointer, row stride) of a float matrix view with unit column stride."""
    if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != torch.float32 or t.dim() != 2 or t.stride(1) != 1:
        raise KernelError(f"{name}: expected a float GPU matrix with contiguous rows")
    if cols is not None and t.shape[1] != cols:
        raise KernelError(f"{name}: {t.shape[1]} columns, expected {cols}")
    return t.data_ptr(), t.stride(0)


def scan_piece(rows, decode_only):
    """Rows of a piece where the linear scan walks long segments in pieces side by side (0: a wave walks a whole
    segment).  A step of single tokens has nothing to cut; a portion is cut so that its pieces fill the GPU, at the
    price of walking every piece but the last twice (once for its end state, once for its results)."""
    if decode_only or rows < 128:
        return 0
    return 128 if rows >= 1024 else 64


def scan_columns(runs, heads, cols):
    """Columns of the state that one wave of the linear scan owns (16, 8 or 4): fewer columns make more waves of the
    same head, until the launch has about a wave for every SIMD of the GPU (wider tiles read the state in longer runs).  `runs`: segments, or pieces of them."""
    for width in (16, 8, 4):
        if runs * heads * -(-cols // width) >= 1024 or width == 4:
            return width


def scan_carry(rows, piece, heads, rows_of_state, cols_of_state, vector):
    """(floats of carry, floats of carry_decay) that linear_scan needs for a step of `rows` rows cut into pieces."""
    decay = C.c_longlong(0)
    n = _rec().cisr_linear_scan_carry(int(rows), int(piece), int(heads), int(rows_of_state), int(cols_of_state), int(vector), C.byref(decay))
    return int(n), int(decay.value)


def linear_scan(q, k, v, decay, out, state, seg_start, state_slots, heads, rows_of_state, cols_of_state, share=1,
                step=None, q_scale=1.0, columns=None, piece=0, carry=None):
    """Per segment and head: S_t = diag(a_t) S_(t-1) + k_t (v_t step_t)^T, o_t = q_scale S_t^T q_t over the segment's
    rows in order, S [rows_of_state, cols_of_state] read from and written back to the segment's state slot.
    q, k float views [T, heads / share * R]; v, out [T, heads * C]; decay [T, heads * R] (a vector a head) or
    [T, heads] (a number a head); step None or [T, heads]; state float [slots, >= heads * R * C] (a view whose rows
    start with the state); seg_start int32 [S + 1]; state_slots int32 [S].
    `piece` > 0: segments longer than that many rows are walked in pieces side by side (three launches: the pieces'
    end states from zero, the states at their starts in order, the results), with `carry` = (float buffer, float
    buffer) of at least scan_carry(...) elements."""
    R, Cc = int(rows_of_state), int(cols_of_state)
    T = v.shape[0]
    segments = state_slots.shape[0]
    if heads % share or R > 256:
        raise KernelError("linear_scan: heads must divide into their groups and a state has at most 256 rows")
    qp, ldq = _rows_of(q, "q", heads // share * R)
    kp, ldk = _rows_of(k, "k", heads // share * R)
    vp, ldv = _rows_of(v, "v", heads * Cc)
    op, ldo = _rows_of(out, "out", heads * Cc)
    if decay.shape[1] not in (heads, heads * R):
        raise KernelError("linear_scan: decays are one a head or one a state row")
    vec = decay.shape[1] != heads
    ap, lda = _rows_of(decay, "decay")
    sp, lds = (None, 0) if step is None else _rows_of(step, "step", heads)
    if any(t.shape[0] != T for t in (q, k, decay, out)) or (step is not None and step.shape[0] != T):
        raise KernelError("linear_scan: operands differ in rows")
    if state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < heads * R * Cc or not state.is_cuda:
        raise KernelError("linear_scan: the state must be float [slots, >= heads * R * C]")
    cp = dp = None
    if piece:
        need = scan_carry(T, piece, heads, R, Cc, vec)
        if carry is None or carry[0].numel() < need[0] or carry[1].numel() < need[1]:
            raise KernelError("linear_scan: pieces need the carry buffers that scan_carry sizes")
        cp, dp = _dev(carry[0], "carry", torch.float32), _dev(carry[1], "carry_decay", torch.float32)
    cols = int(columns or scan_columns(-(-T // piece) if piece else segments, heads, Cc))
    while columns is None and cols > 4 and -(-R // (128 // cols)) > 16:
        cols //= 2         # (at most 16 rows of its two columns a lane, where the tile can be narrower: registers)
    _check(_rec().cisr_linear_scan(qp, ldq, kp, ldk, vp, ldv, ap, lda, int(vec), sp, lds, op, ldo, state.data_ptr(),
                                   state.stride(0), _dev(seg_start, "seg_start", torch.int32, (segments + 1,)),
                                   _dev(state_slots, "state_slots", torch.int32, (segments,)), segments, heads, R, Cc,
                                   int(share), float(q_scale), cols, T, int(piece), cp, dp, _stream()), "linear_scan")
    return out


def conv_silu(x, taps_weight, bias, conv_state, out, seg_of_row, seg_start, state_slots, gates=None, single_rows=False):
    """out[t, c] = silu(bias[c] + sum_j w[c, j] input(t - (K - 1) + j)[c]) over the rows of each segment, the K - 1 inputs
    before a segment's first row taken from its state slot, which then moves on to the last K - 1 inputs.
    x float view [T, channels]; taps_weight float [channels, K]; conv_state float view [slots, >= (K - 1) * channels].
    `gates` = (dt view [T, heads], dt_bias [heads], a_log [heads], step out [T, heads], decay out [T, heads]):
    step = softplus(dt + dt_bias), decay = exp(-exp(a_log) step), made by the same launch.
    `single_rows`: the caller vouches that no segment has more than one row (a step of single tokens); the state then
    moves on in the same launch instead of a second one."""
    T, channels = x.shape
    K = taps_weight.shape[1]
    segments = state_slots.shape[0]
    xp, ld = _rows_of(x, "x")
    if conv_state.dtype != torch.float32 or conv_state.stride(1) != 1 or conv_state.shape[1] < (K - 1) * channels:
        raise KernelError("conv_silu: the state must be float [slots, >= (K - 1) * channels]")
    heads, dtp, dt_first, bp2, alp, stp, dcp = 0, None, 0, None, None, None, None
    if gates is not None:
        dt, dt_bias, a_log, step, decay = gates
        heads = dt.shape[1]
        dp, ldd = _rows_of(dt, "dt")
        if ldd != ld or (dp - xp) % 4:
            raise KernelError("conv_silu: the step sizes must be columns of the rows that hold the convolution's inputs")
        dt_first = (dp - xp) // 4
        bp2, alp = _dev(dt_bias, "dt_bias", torch.float32, (heads,)), _dev(a_log, "a_log", torch.float32, (heads,))
        stp, dcp = _dev(step, "step", torch.float32, (T, heads)), _dev(decay, "decay", torch.float32, (T, heads))
    _check(_rec().cisr_conv_silu(xp, ld, 0, _dev(taps_weight, "taps", torch.float32, (channels, K)),
                                 None if bias is None else _dev(bias, "bias", torch.float32, (channels,)),
                                 conv_state.data_ptr(), conv_state.stride(0), _dev(out, "out", torch.float32, (T, channels)),
                                 _dev(seg_of_row, "seg_of_row", torch.int32, (T,)),
                                 _dev(seg_start, "seg_start", torch.int32, (segments + 1,)),
                                 _dev(state_slots, "state_slots", torch.int32, (segments,)), T, segments, channels, K, heads,
                                 dt_first, bp2, alp, stp, dcp, int(bool(single_rows)), _stream()), "conv_silu")
    return out


def decay_gate(z, bias, out, tau):
    """out = sigmoid(z + bias)^(1 / tau) in float; z a float view [T, N], bias float [N] or None, out float [T, N]."""
    T, n = z.shape
    zp, ld = _rows_of(z, "z")
    _check(_rec().cisr_decay_gate(zp, ld, None if bias is None else _dev(bias, "bias", torch.float32, (n,)),
                                  _dev(out, "out", torch.float32, (T, n)), T, n, float(tau), _stream()), "decay_gate")
    return out


def decay_gate_low_rank(low, up, bias, out, tau):
    """out = sigmoid(low . up + bias)^(1 / tau) in float: low a float view [T, rank] (the first half of a low-rank
    projection), up float [rank, N] (the second half's matrix, transposed), bias float [N] or None, out float [T, N]."""
    T, rank = low.shape
    n = up.shape[1]
    lp, ld = _rows_of(low, "low")
    _check(_rec().cisr_decay_gate_low_rank(lp, ld, rank, _dev(up, "up", torch.float32, (rank, n)),
                                           None if bias is None else _dev(bias, "bias", torch.float32, (n,)),
                                           _dev(out, "out", torch.float32, (T, n)), T, n, float(tau), _stream()), "decay_gate_low_rank")
    return out


def group_norm_gate(y, gate, weight, out, groups, eps, gate_first, shared_weight=False, skip=None):
    """Rows of y float [T, groups * size] in `groups` equal parts, each divided by its own root mean square, times
    `weight` ([size] if shared by the parts, else [groups * size]), with silu(gate) multiplied in before the norm
    (`gate_first`) or after it; `skip` = (d [n], x view [T, groups * size]) adds d[i // (groups * size / n)] x[t, i]
    first.  gate a float view [T, groups * size]; out [T, groups * size] float or bf16."""
    T, width = y.shape
    if width % groups:
        raise KernelError("group_norm_gate: the row does not divide into its parts")
    size = width // groups
    gp, ldg = _rows_of(gate, "gate", width)
    wp = _dev(weight, "weight", torch.float32, (size if shared_weight else width,))
    dp, span, xp, ldx = None, 0, None, 0
    if skip is not None:
        d, x = skip
        if width % d.shape[0]:
            raise KernelError("group_norm_gate: the skip weights do not divide the row")
        dp, span = _dev(d, "skip", torch.float32), width // d.shape[0]
        xp, ldx = _rows_of(x, "x", width)
    _check(_rec().cisr_group_norm_gate(_dev(y, "y", torch.float32), gp, ldg, wp, int(shared_weight), dp, span, xp, ldx,
                                       _dev(out, "out", None, (T, width)), T, groups, size, float(eps), int(bool(gate_first)),
                                       _storage(out, "out"), _stream()), "group_norm_gate")
    return out


def unit_heads(x, heads, dim, scale=1.0, eps=1e-6):
    """The float view x [T, heads * dim] in place: every head becomes x / sqrt(sum(x^2) + eps) * scale."""
    xp, ld = _rows_of(x, "x", heads * dim)
    _check(_rec().cisr_unit_heads(xp, ld, 0, x.shape[0], heads, dim, float(eps), float(scale), _stream()), "unit_heads")
    return x


def delta_columns(segments, heads, cols):
    """Columns of the state that one wave of the delta rule owns (32, 16 or 8): wide tiles read and write the state in
    long runs (steps of many single tokens), narrow ones make more waves of the same head, until the launch has about
    a wave for every SIMD of the GPU (a prompt's one segment is walked in order by every wave)."""
    for width in (32, 16, 8):
        if segments * heads * -(-cols // width) >= 1024 or width == 8:
            return width


def delta_scan(q, k, v, decay, write, out, state, seg_start, state_slots, heads, rows_of_state, cols_of_state, share=1,
               q_scale=1.0, columns=None):
    """Per segment and head, over the segment's rows in order: S <- g S; u = sigmoid(b) (v - S^T k); S <- S + k u^T;
    o = q_scale S^T q, S [rows_of_state, cols_of_state] read from and written back to the segment's state slot.
    q, k float views [T, heads / share * R]; v, out [T, heads * C]; decay (g) and write (b) [T, heads]; state float
    [slots, >= heads * R * C]; seg_start int32 [S + 1]; state_slots int32 [S]."""
    R, Cc = int(rows_of_state), int(cols_of_state)
    T = v.shape[0]
    segments = state_slots.shape[0]
    if heads % share or R > 256:
        raise KernelError("delta_scan: heads must divide into their groups and a state has at most 256 rows")
    qp, ldq = _rows_of(q, "q", heads // share * R)
    kp, ldk = _rows_of(k, "k", heads // share * R)
    vp, ldv = _rows_of(v, "v", heads * Cc)
    op, ldo = _rows_of(out, "out", heads * Cc)
    gp, ldg = _rows_of(decay, "decay", heads)
    bp, ldb = _rows_of(write, "write", heads)
    if any(t.shape[0] != T for t in (q, k, decay, write, out)):
        raise KernelError("delta_scan: operands differ in rows")
    if state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < heads * R * Cc or not state.is_cuda:
        raise KernelError("delta_scan: the state must be float [slots, >= heads * R * C]")
    cols = int(columns or delta_columns(segments, heads, Cc))
    while columns is None and cols > 8 and -(-R // (128 // cols)) > 32:
        cols //= 2         # (at most 32 rows of its two columns a lane)
    _check(_rec().cisr_delta_scan(qp, ldq, kp, ldk, vp, ldv, gp, ldg, bp, ldb, op, ldo, state.data_ptr(), state.stride(0),
                                  _dev(seg_start, "seg_start", torch.int32, (segments + 1,)),
                                  _dev(state_slots, "state_slots", torch.int32, (segments,)), segments, heads, R, Cc,
                                  int(share), float(q_scale), cols, _stream()), "delta_scan")
    return out


# -- layers that norm after the sum, hashed token pairs, whole-projection norms (csrc/elementwise_postnorm.hip) --------

def embedding_pairs(tokens, positions, seg_of_row, seg_start, state_slots, table, out, scale=1.0, pairs=None, last_token=None,
                    buckets=0, mul_prev=0, mul_cur=0, cast=None, single_rows=False):
    """out[r] = table[tokens[r]] * scale (+ pairs[(previous token * mul_prev + token * mul_cur) mod buckets], or row
    `buckets` of `pairs` at position 0), float [T, H].  The token before a segment's first row is last_token[state slot]
    (int32 [slots]), which afterwards holds the segment's last token.  `cast`: a copy of the rows in the table's type.
    `single_rows`: every segment brings one row (one launch instead of two)."""
    rows = tokens.shape[0]
    vocab, dim = table.shape
    segments = state_slots.shape[0]
    pp = lp = None
    if pairs is not None:
        if last_token is None or buckets <= 0 or pairs.dtype != table.dtype:
            raise KernelError("embedding_pairs: the pair table needs its buckets, the kept tokens and the table's dtype")
        pp = _dev(pairs, "pairs", None, (buckets + 1, dim))
        lp = _dev(last_token, "last_token", torch.int32)
        if last_token.numel() < 1:
            raise KernelError("embedding_pairs: no kept tokens")
    cp, cdt = None, _storage(table, "table")
    if cast is not None:
        cp, cdt = _dev(cast, "cast", None, (rows, dim)), _storage(cast, "cast")
        if cast.dtype != table.dtype:
            raise KernelError("embedding_pairs: the copy has the table's dtype")
    _check(lib().cisr_embedding_pairs(_dev(tokens, "tokens", torch.int32, (rows,)), _dev(positions, "positions", torch.int32, (rows,)),
                                      _dev(seg_of_row, "seg_of_row", torch.int32, (rows,)),
                                      _dev(seg_start, "seg_start", torch.int32, (segments + 1,)),
                                      _dev(state_slots, "state_slots", torch.int32, (segments,)), lp, _dev(table, "table"), pp,
                                      _dev(out, "out", torch.float32, (rows, dim)), cp, rows, segments, dim, vocab, float(scale),
                                      int(buckets), int(mul_prev), int(mul_cur), int(bool(single_rows)), _storage(table, "table"), cdt,
                                      _stream()), "embedding_pairs")
    return out


class WeightedRows:
    """A sublayer's result as `top` rows a step row, to be summed with weights by the kernel that reads it next
    (gate_post_norm): rows float [T * top, H], weights float [T, top]."""

    def __init__(self, rows, weights, top):
        self.rows, self.weights, self.top = rows, weights, int(top)


def gate_post_norm(x, y, weight, eps, alpha, gate=None, gate_bias=None, cast=None):
    """x <- rmsnorm(alpha x + y * sigmoid(gate + gate_bias)) * weight, in place (float [T, H]); y float [T, H] or a
    WeightedRows; `gate` a float view [T, H] with unit column stride (None: no gate); `cast` [T, H]: a copy of the
    new rows in the activations' type."""
    rows, dim = x.shape
    top, yw = 1, None
    if isinstance(y, WeightedRows):
        top = y.top
        yp = _dev(y.rows, "y", torch.float32, (rows * top, dim))
        yw = _dev(y.weights, "y weights", torch.float32, (rows, top))
    else:
        yp = _dev(y, "y", torch.float32, (rows, dim))
    gp, ldg, gb = None, 0, None
    if gate is not None:
        if gate.dtype != torch.float32 or tuple(gate.shape) != (rows, dim) or gate.stride(1) != 1 or not gate.is_cuda:
            raise KernelError("gate_post_norm: the gate is a float view [T, H] with unit column stride")
        gp, ldg = gate.data_ptr(), gate.stride(0)
        gb = None if gate_bias is None else _dev(gate_bias, "gate_bias", torch.float32, (dim,))
    cp, cdt = None, F32
    if cast is not None:
        cp, cdt = _dev(cast, "cast", None, (rows, dim)), _storage(cast, "cast")
    _check(lib().cisr_gate_post_norm(_dev(x, "x", torch.float32), yp, top, yw, gp, ldg, gb, _dev(weight, "weight", torch.float32, (dim,)),
                                     cp, rows, dim, float(eps), float(alpha), cdt, _stream()), "gate_post_norm")
    return x


def whole_norm_rope_scatter(proj, q_norm, k_norm, positions, slots, cos, sin, q_out, kcache, vcache, heads, kv_heads, dim, vdim,
                            pad, page_size, eps, bias=None, split_half=False, value_norm=False):
    """Rows of a projection with float results [q: heads x dim | k: kv_heads x dim | v: kv_heads x vdim | ...]: q and k
    RMS-normed over all their heads at once (weights float [heads * dim], [kv_heads * dim]), the first 2 * cos.shape[1]
    coordinates of every head turned in neighbouring pairs by the position (cos / sin float [max_pos, pairs]), q into
    q_out [T, heads * pad], k and v into the pages at `slots` as heads of `pad` coordinates whose rest is zero.
    kcache None: the rows have queries only (a layer that reads another's cache).  `bias`: float over the q, k and v
    columns, added before everything else; `split_half`: the pairs are (i, i + pairs) instead of neighbours;
    `value_norm`: each head's value is divided by its root mean square over vdim (eps, no weight) before it is stored."""
    rows, ld = proj.shape
    has_kv = kcache is not None
    bp = None if bias is None else _dev(bias, "bias", torch.float32, (heads * dim + (kv_heads * (dim + vdim) if has_kv else 0),))
    if proj.dtype != torch.float32 or proj.stride(1) != 1 or not proj.is_cuda:
        raise KernelError("whole_norm_rope_scatter: a float projection with contiguous rows")
    if dim > pad or vdim > pad or ld < heads * dim + (kv_heads * (dim + vdim) if has_kv else 0):
        raise KernelError(f"whole_norm_rope_scatter: heads of {dim} / {vdim} do not fit rows of {ld} or pages of {pad}")
    max_pos, half = cos.shape
    if 2 * half > dim:
        raise KernelError(f"whole_norm_rope_scatter: {2 * half} turning coordinates in heads of {dim}")
    kp = vp = sp = kw = None
    if has_kv:
        pages = kcache.shape[0]
        kp = _dev(kcache, "kcache", q_out.dtype, (pages, kv_heads, page_size, pad))
        vp = _dev(vcache, "vcache", q_out.dtype, (pages, kv_heads, pad, page_size))
        sp = _dev(slots, "slots", torch.int32, (rows,))
        kw = _dev(k_norm, "k_norm", torch.float32, (kv_heads * dim,))
    _check(lib().cisr_whole_norm_rope_scatter(proj.data_ptr(), proj.stride(0), bp, _dev(q_norm, "q_norm", torch.float32, (heads * dim,)), kw,
                                              _dev(positions, "positions", torch.int32, (rows,)), sp,
                                              _dev(cos, "cos", torch.float32), _dev(sin, "sin", torch.float32, (max_pos, half)),
                                              half, max_pos, _dev(q_out, "q_out", None, (rows, heads * pad)), kp, vp, rows, heads,
                                              kv_heads, dim, vdim, pad, page_size, float(eps), int(has_kv), int(bool(split_half)),
                                              int(bool(value_norm)), _storage(q_out, "q_out"), _stream()), "whole_norm_rope_scatter")
    return q_out


# -- routed experts (csrc/experts.hip) -----------------------------------------------------------------------------

EXPERT_TILE = 64      # rows of a tile of the experts' products: every expert's rows are padded to a multiple


def expert_tiles(rows, top, experts):
    """Tiles that the rows of a step can take at most once ordered by expert (every expert's run padded to whole tiles)."""
    return -(-rows * top // EXPERT_TILE) + experts


def experts_route(logits, bias, top, chosen, weights, pair_of_pos=None, tile_expert=None):
    """logits: a float view [T, E] with unit column stride (+ bias float [E]) -> chosen int32 [T, top] (largest first,
    the lowest index wins a tie), weights float [T, top] (softmax over the chosen logits), and, unless pair_of_pos is
    None, the (row, choice) pairs ordered by expert: pair_of_pos int32 [tiles * 64] (-1: padding), tile_expert int32
    [tiles] (-1: none)."""
    rows, experts = logits.shape
    if logits.dtype != torch.float32 or logits.stride(1) != 1 or not logits.is_cuda:
        raise KernelError("experts_route: float logits with contiguous rows")
    if not 0 < top <= min(experts, 16):
        raise KernelError(f"experts_route: {top} of {experts} experts")
    tiles, pp, tp = 0, None, None
    if pair_of_pos is not None:
        tiles = tile_expert.shape[0]
        if tiles < expert_tiles(rows, top, experts):
            raise KernelError(f"experts_route: {tiles} tiles for {rows} rows x {top} of {experts} experts")
        pp, tp = _dev(pair_of_pos, "pair_of_pos", torch.int32, (tiles * EXPERT_TILE,)), _dev(tile_expert, "tile_expert", torch.int32, (tiles,))
    _check(lib().cisr_experts_route(logits.data_ptr(), logits.stride(0), None if bias is None else _dev(bias, "bias", torch.float32, (experts,)),
                                    _dev(chosen, "chosen", torch.int32, (rows, top)), _dev(weights, "weights", torch.float32, (rows, top)),
                                    rows, experts, top, tiles, pp, tp, _stream()), "experts_route")
    return chosen, weights


def experts_route_scored(logits, correction, top, chosen, weights, experts, groups=None, pair_of_pos=None, tile_expert=None):
    """Routing by scores: logits a float view [T, outputs]; s = softmax over all outputs; the choice goes by s + correction
    (float [outputs] or None), held to the best `groups[1]` of `groups[0]` equal groups of neighbours (a group's score is
    its largest choice score); chosen int32 [T, top] (the lowest index wins a tie), weights float [T, top] = s of the
    chosen, not normed again.  The first `experts` outputs have matrices: only their pairs are ordered by expert into
    pair_of_pos / tile_expert (as experts_route does), the others are left to the caller."""
    rows, outputs = logits.shape
    if logits.dtype != torch.float32 or logits.stride(1) != 1 or not logits.is_cuda:
        raise KernelError("experts_route_scored: float logits with contiguous rows")
    count, keep = groups or (0, 0)
    if not 0 < top <= min(outputs, 16) or not 0 < experts <= outputs or count > 64:
        raise KernelError(f"experts_route_scored: {top} of {outputs} outputs, {experts} with matrices, {count} groups")
    tiles, pp, tp = 0, None, None
    if pair_of_pos is not None:
        tiles = tile_expert.shape[0]
        if tiles < expert_tiles(rows, top, experts):
            raise KernelError(f"experts_route_scored: {tiles} tiles for {rows} rows x {top} of {experts} experts")
        pp, tp = _dev(pair_of_pos, "pair_of_pos", torch.int32, (tiles * EXPERT_TILE,)), _dev(tile_expert, "tile_expert", torch.int32, (tiles,))
    _check(lib().cisr_experts_route_scored(logits.data_ptr(), logits.stride(0),
                                           None if correction is None else _dev(correction, "correction", torch.float32, (outputs,)),
                                           _dev(chosen, "chosen", torch.int32, (rows, top)), _dev(weights, "weights", torch.float32, (rows, top)),
                                           rows, outputs, int(experts), top, int(count), int(keep), tiles, pp, tp, _stream()), "experts_route_scored")
    return chosen, weights


def experts_combine(down, weights, chosen, x, y, experts, shared=None):
    """y[r] = sum_k weights[r, k] * (down[r * top + k] if chosen[r, k] < experts else x[r]) + shared[r]: the weighted sum
    over a row's choices (a choice without matrices is the input x itself) plus the rows every token goes through.
    down [T * top, H], shared and y [T, H] are float, x [T, H] float or bf16."""
    rows, top = weights.shape
    dim = y.shape[1]
    _check(lib().cisr_experts_combine(_dev(down, "down", torch.float32, (rows * top, dim)), _dev(weights, "weights", torch.float32),
                                      _dev(chosen, "chosen", torch.int32, (rows, top)), _dev(x, "x", None, (rows, dim)), _storage(x, "x"),
                                      None if shared is None else _dev(shared, "shared", torch.float32, (rows, dim)),
                                      _dev(y, "y", torch.float32, (rows, dim)), rows, dim, top, int(experts), _stream()), "experts_combine")
    return y


EXPERT_ROWS_PAIRS = 32     # steps of at most this many (row, choice) pairs stream each pair's matrices (experts_rows)


def experts_rows_ok(a, w, pairs):
    """Whether experts_rows takes the product: bf16, few pairs, rows of 16-byte chunks that a wave holds in registers."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and 0 < pairs <= EXPERT_ROWS_PAIRS and a.stride(1) == 1
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and bool(lib().cisr_experts_rows_ok(int(w.shape[2]), int(a.stride(0)), int(pairs))))


def experts_rows(a, w, chosen, out, top=0, act=False):
    """out[pair] = act(a[pair // top, or pair with top 0] . w[chosen[pair]]^T) for every (row, choice) pair of a step of
    few rows: a pair's block streams its expert's matrix (no layout by expert).  w [experts, N, K] bf16; chosen int32
    [T, top] flattened to pairs; out [pairs, N]."""
    experts, n, k = w.shape
    pairs = chosen.numel()
    if not experts_rows_ok(a, w, pairs) or a.shape[1] != k or tuple(out.shape) != (pairs, n) or not out.is_contiguous():
        raise KernelError("experts_rows: shape not supported")
    if a.shape[0] < (-(-pairs // top) if top > 0 else pairs):
        raise KernelError("experts_rows: too few operand rows")
    _check(lib().cisr_experts_rows(a.data_ptr(), a.stride(0), _dev(w, "w"), _dev(chosen, "chosen", torch.int32), int(top), _dev(out, "out"),
                                   out.stride(0), pairs, n, k, int(bool(act)), _storage(out, "out"), int(experts), _stream()), "experts_rows")
    return out


def experts_gemm(a, w, pair_of_pos, tile_expert, out, top=0, scatter=False, act=False):
    """out[row of place] = act(a[row of place] . w[expert of the place's tile]^T) over the places that experts_route
    laid out.  w [experts, N, K]; `top` > 0: a place's operand is row pair // top of `a` (the step's rows), else the
    place's own row; `scatter`: the result goes to row `pair` of out, else to the place's own row.  `act`: relu(.)^2."""
    experts, n, k = w.shape
    tiles = tile_expert.shape[0]
    places = tiles * EXPERT_TILE
    if a.dtype != w.dtype or a.dim() != 2 or a.shape[1] != k or a.stride(1) != 1 or not w.is_contiguous():
        raise KernelError("experts_gemm: operands of one dtype, [rows, K] against [experts, N, K]")
    if out.dim() != 2 or out.shape[1] != n or not out.is_contiguous() or (a.dtype == torch.float32 and out.dtype != torch.float32):
        raise KernelError("experts_gemm: out is [rows, N], float for float operands")
    if pair_of_pos.numel() != places:
        raise KernelError("experts_gemm: the places do not fit the tiles")
    if (top <= 0 and a.shape[0] < places) or (not scatter and out.shape[0] < places):
        raise KernelError("experts_gemm: operands by place need a row a place")
    _check(lib().cisr_experts_gemm(_dev(a, "a") if a.is_contiguous() else a.data_ptr(), a.stride(0), _dev(w, "w"),
                                   _dev(tile_expert, "tile_expert", torch.int32), _dev(pair_of_pos, "pair_of_pos", torch.int32),
                                   int(top), int(bool(scatter)), _dev(out, "out"), out.stride(0), tiles, n, k, int(bool(act)),
                                   _storage(a, "a"), _storage(out, "out"), _stream()), "experts_gemm")
    return out


def mlstm_gates(zi, zf, bias_i, bias_f, v, decay, step, top, vx, top_state, seg_start, state_slots, heads, vdim, cap, single_rows=False):
    """The operands of the matrix memory's scan from the projections' float results: log gates i = cap tanh((zi + bi) /
    cap), f = logsigmoid(cap tanh((zf + bf) / cap)) (zi, zf float views [T, heads]); along every segment's rows the
    running maximum m' = max(f + m, i), from `top_state`[slot, head] and back into it; decay = exp(f + m - m'), step =
    exp(i - m') and top = m', float [T, heads]; vx [T, heads * (vdim + 1)] = the values v (a float view [T, heads *
    vdim]) with a column of ones a head.  `single_rows`: every segment has one row (row t is segment t; rows past the
    segments are padding): one kernel makes the gates and moves the maxima on."""
    T = v.shape[0]
    segments = state_slots.shape[0]
    ip, ldi = _rows_of(zi, "zi", heads)
    fp, ldf = _rows_of(zf, "zf", heads)
    vp, ldv = _rows_of(v, "v", heads * vdim)
    if top_state.dtype != torch.float32 or top_state.dim() != 2 or top_state.stride(1) != 1 or top_state.shape[1] < heads or not top_state.is_cuda:
        raise KernelError("mlstm_gates: the running maxima are float [slots, >= heads]")
    _check(_rec().cisr_mlstm_gates(ip, ldi, fp, ldf, _dev(bias_i, "bias_i", torch.float32, (heads,)), _dev(bias_f, "bias_f", torch.float32, (heads,)),
                                   vp, ldv, _dev(decay, "decay", torch.float32, (T, heads)), _dev(step, "step", torch.float32, (T, heads)),
                                   _dev(top, "top", torch.float32, (T, heads)), _dev(vx, "vx", torch.float32, (T, heads * (vdim + 1))),
                                   top_state.data_ptr(), top_state.stride(0), _dev(seg_start, "seg_start", torch.int32, (segments + 1,)),
                                   _dev(state_slots, "state_slots", torch.int32, (segments,)), T, segments, heads, vdim, float(cap), int(bool(single_rows)),
                                   _stream()), "mlstm_gates")


def mlstm_finish(o, top, gate, weight, out, heads, vdim, eps, floor=1e-6):
    """The matrix memory's result from its scan's: o float [T, heads * (vdim + 1)], the last column of a head n . q;
    out[t, h] = rms(o_h / (max(|n . q|, exp(-top)) + floor)) * weight * sigmoid(gate), rms over vdim with eps; gate a
    float view [T, heads * vdim], weight float [heads * vdim], out [T, heads * vdim] float or bf16."""
    T = o.shape[0]
    gp, ldg = _rows_of(gate, "gate", heads * vdim)
    _check(_rec().cisr_mlstm_finish(_dev(o, "o", torch.float32, (T, heads * (vdim + 1))), _dev(top, "top", torch.float32, (T, heads)), gp, ldg,
                                    _dev(weight, "weight", torch.float32, (heads * vdim,)), _dev(out, "out", None, (T, heads * vdim)),
                                    T, heads, vdim, float(eps), float(floor), _storage(out, "out"), _stream()), "mlstm_finish")
    return out


def mingru_piece(rows, decode_only):
    """Rows of a piece where the minimal gated unit's scan walks long segments in pieces side by side (0: a thread walks
    a whole segment)."""
    if decode_only or rows < 256:
        return 0
    return 64 if rows < 4096 else 128


def mingru_scan(proj, bias_z, bias_x, state, seg_start, state_slots, out, width, piece=0, carry=None):
    """Element by element over `width` channels: z = sigmoid(a + bias_z), c = cand(b + bias_x), S <- (1 - z) S + z c,
    out = S silu(g), with [a | b | g] the first 3 width columns of proj (a float view with contiguous rows) and
    cand(u) = u + 1/2 for u >= 0, sigmoid(u) below.  S: state float [slots, >= width] rows of a view, read from and
    written back to each segment's slot.  `piece` > 0: segments are walked in pieces of that many rows (three
    launches); carry float [2 * (rows // piece + segments) * width]."""
    rows = proj.shape[0]
    segments = state_slots.shape[0]
    pp, ld = _rows_of(proj, "proj")
    sp, sld = _rows_of(state, "state")
    if proj.shape[1] < 3 * width or state.shape[1] < width or tuple(out.shape) != (rows, width):
        raise KernelError("mingru_scan: shapes do not fit the width")
    cp, pieces = None, 0
    if piece > 0:
        pieces = rows // piece + segments
        if carry is None or carry.numel() < 2 * pieces * width:
            raise KernelError("mingru_scan: pieces need a carry buffer")
        cp = _dev(carry, "carry", torch.float32)
    _check(_rec().cisr_mingru_scan(pp, ld, _dev(bias_z, "bias_z", torch.float32, (width,)), _dev(bias_x, "bias_x", torch.float32, (width,)),
                                   sp, sld, _dev(seg_start, "seg_start", torch.int32, (segments + 1,)),
                                   _dev(state_slots, "state_slots", torch.int32, (segments,)), _dev(out, "out", None, (rows, width)),
                                   rows, segments, width, int(piece), cp, pieces, _storage(out, "out"), _stream()), "mingru_scan")
    return out
