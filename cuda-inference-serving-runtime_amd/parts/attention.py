"""Grouped-query attention over the paged cache.

q = h Wq^T, k = h Wk^T, v = h Wv^T; q and k take the position encoding; k and v
go into the cache at the step's slots; every row then attends to its request's
cached keys up to its own position (or the last `window` of them), scale
1/sqrt(head_dim) unless given; the result goes through Wo and is added to the
residual (reference: runtime/model.py:110-115).  The three projections run as
one product against the concatenated weight [q; k; v] (a layout choice only).

A mixer built with `own_kv` False has no k/v projections: it attends to
the cache another layer wrote.  With `bias` the q/k/v projections add
`<name>.{q,k,v}_proj.bias` before the position encoding, with `out_bias` the output
projection adds `<name>.o_proj.bias`: the products run as they are and a small kernel
adds the bias (the fused projection kernels have no bias and are not used then).
"""
import math

import torch

from ..cache.pages import ChunkNeed, KVNeed
from ..kernels import attention as kernel, ops
from .base import Mixer, TensorSpec, matrix_operand, register_part


class PagedAttention(Mixer):
    def __init__(self, name, hidden, heads, kv_heads, head_dim, position, window=None, scale=None, own_kv=True,
                 bias=False, out_bias=False, tuning=None):
        if heads % kv_heads:
            raise ValueError(f"{heads} query heads are not a multiple of {kv_heads} key/value heads")
        if head_dim % 2 or head_dim > 256:
            raise ValueError(f"head size {head_dim} must be even and at most 256")
        self.name, self.hidden, self.heads, self.kv_heads, self.head_dim = name, hidden, heads, kv_heads, head_dim
        self.position, self.window, self.own_kv = position, window, own_kv
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.bias, self.out_bias = bool(bias), bool(out_bias)
        self.w_in = self.w_out = self.b_in = self.b_out = None
        self.tuning = tuning if tuning is not None else kernel.DEFAULT_TUNING   # what the kernel's launch rules may be told

    def kernel_units(self, dtype):
        return kernel.kernel_units(self.head_dim, dtype)

    def step_arrays(self):
        return [kernel.SingleRows(self.tuning.split_single_from), kernel.RowsLongestFirst()]

    def cache_need(self):
        return KVNeed(self.kv_heads, self.head_dim, self.window) if self.own_kv else None

    def cache_read(self):
        return None if self.own_kv else KVNeed(self.kv_heads, self.head_dim, self.window)

    def tensor_specs(self):
        n, H, D = self.name, self.hidden, self.head_dim
        specs = [TensorSpec(f"{n}.q_proj.weight", (self.heads * D, H))]
        if self.own_kv:
            specs += [TensorSpec(f"{n}.k_proj.weight", (self.kv_heads * D, H)),
                      TensorSpec(f"{n}.v_proj.weight", (self.kv_heads * D, H))]
        specs.append(TensorSpec(f"{n}.o_proj.weight", (H, self.heads * D)))
        if self.bias:
            specs.append(TensorSpec(f"{n}.q_proj.bias", (self.heads * D,)))
            if self.own_kv:
                specs += [TensorSpec(f"{n}.k_proj.bias", (self.kv_heads * D,)), TensorSpec(f"{n}.v_proj.bias", (self.kv_heads * D,))]
        if self.out_bias:
            specs.append(TensorSpec(f"{n}.o_proj.bias", (H,)))
        return specs

    def bind(self, tensors, dtype):
        names = ["q_proj"] + (["k_proj", "v_proj"] if self.own_kv else [])
        parts = [matrix_operand(tensors[f"{self.name}.{p}.weight"], dtype) for p in names]
        self.w_in = torch.cat(parts, dim=0).contiguous() if len(parts) > 1 else parts[0]
        self.w_out = matrix_operand(tensors[f"{self.name}.o_proj.weight"], dtype)
        if self.bias:   # (a bias keeps the type it is stored in; it is added in float)
            self.b_in = torch.cat([tensors[f"{self.name}.{p}.bias"] for p in names], dim=0).contiguous()
        if self.out_bias:
            self.b_out = tensors[f"{self.name}.o_proj.bias"].contiguous()

    def prepare(self, device, dtype):
        self.position.prepare(device, dtype)

    @property
    def _interleaved(self):
        return getattr(self.position, "pairing", "split_half") == "interleaved"

    def _fused_projection_ok(self, a, normed):
        cos, _ = self.position.tables()
        # (the fused kernels turn split-half pairs only; another pairing takes the general rotary kernel)
        return not self._interleaved and not self.bias and ops.qkv_rope_fused_ok(a, self.w_in, self.head_dim, cos, normed)

    def fuses_norm(self, norm, residual, ctx):
        return getattr(norm, "fusable_as", None) == "rms" and self._fused_projection_ok(residual, True)

    def forward(self, h, residual, ctx, site, norm=None):
        T = residual.shape[0]
        D, nh, nkv = self.head_dim, self.heads, self.kv_heads
        gid, kcache, vcache = ctx.cache.pages_of_site(site)
        view = ctx.kv[gid]
        cos, sin = self.position.tables()
        if not self.own_kv:
            kcache_w = vcache_w = slots = None
        else:
            kcache_w, vcache_w, slots = kcache, vcache, view.slots
        if norm is not None or self._fused_projection_ok(h, False):
            # few rows: norm, projections, rotary embedding and the cache write are one kernel
            q, q_stride = ctx.buffer("attn.q", (T, nh * D), ctx.dtype), nh * D
            ops.qkv_rope(residual if norm is not None else h, self.w_in, q, ctx.positions, slots, cos, sin,
                         kcache_w, vcache_w, nh, nkv, D, view.page_size,
                         norm=(norm.weight, norm.eps) if norm is not None else None, scratch=ctx.scratch)
        else:
            q_stride = (nh + (2 * nkv if self.own_kv else 0)) * D
            q = ctx.buffer("attn.qkv", (T, q_stride), ctx.dtype)
            ops.gemm(h, self.w_in, q, scratch=ctx.scratch)
            if self.b_in is not None:
                ops.bias_add(q, self.b_in)
            ops.rope_scatter(q, ctx.positions, slots, cos, sin, kcache_w, vcache_w, nh, nkv, D, view.page_size,
                             interleaved=self._interleaved)
        out = ctx.buffer("attn.out", (T, nh * D), ctx.dtype)
        # a decode step of few rows may leave the partial results of its split keys to the output projection
        unmerged = kernel.paged_attention(ctx, q, q_stride, kcache, vcache, view, out, nh, nkv, D, self.window, self.scale,
                                          defer_merge=lambda splits: ops.gemm_merged_ok(T, self.w_out, nh, D, splits),
                                          tuning=self.tuning)
        if unmerged is not None:
            residual = ops.gemm_merged(unmerged, nh, D, self.w_out, residual, residual)
        else:
            residual = ctx.add_product(out, self.w_out, residual)
        if self.b_out is not None:
            ops.bias_add(residual, self.b_out)   # (sums commute: slices of the product that a later norm adds may still be out)
        return residual


class NormedGatedAttention(Mixer):
    """Grouped-query softmax attention over the paged cache whose positions do not enter the scores: queries and keys
    are RMS-normed per head (a weight of size `dim` each, shared by the heads; `qk_norm` False: not normed), the score
    is (q . k) * scale, keys and values may differ in size (`dim`, `vdim`), and each head's result is multiplied by
    sigmoid of a projection of the mixer's input, one number a head (`head_gate`).

    The pages hold heads of `pad` = max(dim, vdim) coordinates (rounded up to a multiple of 8), the rest zero: zero
    coordinates add nothing to a score and give result coordinates that are not read, so the attention kernels
    of the framework serve as they are.  `names`: the tensors' names under `name` (q, k, v, o, gate, q norm, k norm)."""

    NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "gate": "g", "q_norm": "q.norm", "k_norm": "k.norm"}

    def __init__(self, name, hidden, heads, kv_heads, dim, vdim, scale, eps, qk_norm=True, head_gate=True, window=None,
                 names=None, tuning=None):
        if heads % kv_heads:
            raise ValueError(f"{heads} query heads are not a multiple of {kv_heads} key/value heads")
        self.pad = -(-max(dim, vdim) // 8) * 8
        if self.pad > 256:
            raise ValueError(f"head sizes {dim} / {vdim}: at most 256")
        if not scale > 0:
            raise ValueError("the score scale must be positive")
        self.name, self.hidden, self.heads, self.kv_heads, self.dim, self.vdim = name, hidden, heads, kv_heads, dim, vdim
        self.scale, self.eps, self.qk_norm, self.head_gate, self.window = float(scale), float(eps), bool(qk_norm), bool(head_gate), window
        self.names = {**self.NAMES, **(names or {})}
        self.tuning = tuning or kernel.DEFAULT_TUNING
        self.w_in = self.w_out = self.q_weight = self.k_weight = None

    def _tensor(self, which):
        return f"{self.name}.{self.names[which]}"

    def kernel_units(self, dtype):
        return kernel.kernel_units(self.pad, dtype)

    def step_arrays(self):
        return [kernel.SingleRows(self.tuning.split_single_from), kernel.RowsLongestFirst()]

    def cache_need(self):
        return KVNeed(self.kv_heads, self.pad, self.window)

    def tensor_specs(self):
        H, nh, nkv, D, V = self.hidden, self.heads, self.kv_heads, self.dim, self.vdim
        specs = [TensorSpec(self._tensor("q"), (nh * D, H)), TensorSpec(self._tensor("k"), (nkv * D, H)),
                 TensorSpec(self._tensor("v"), (nkv * V, H)), TensorSpec(self._tensor("o"), (H, nh * V))]
        if self.head_gate:
            specs.append(TensorSpec(self._tensor("gate"), (nh, H)))
        if self.qk_norm:
            specs += [TensorSpec(self._tensor("q_norm"), (D,), init="one_plus_normal"),
                      TensorSpec(self._tensor("k_norm"), (D,), init="one_plus_normal")]
        return specs

    def bind(self, tensors, dtype):
        parts = [matrix_operand(tensors[self._tensor(p)], dtype) for p in (("q", "k", "v", "gate") if self.head_gate else ("q", "k", "v"))]
        rows = sum(p.shape[0] for p in parts)
        if rows % 8:      # rows of the fused projection are a multiple of 16 bytes: zero rows at the end
            parts.append(torch.zeros(8 - rows % 8, self.hidden, dtype=parts[0].dtype, device=parts[0].device))
        self.w_in = torch.cat(parts, dim=0).contiguous()
        self.w_out = matrix_operand(tensors[self._tensor("o")], dtype)
        if self.qk_norm:
            self.q_weight = tensors[self._tensor("q_norm")].to(torch.float32).contiguous()
            self.k_weight = tensors[self._tensor("k_norm")].to(torch.float32).contiguous()

    def output(self, h, ctx, site):
        """The mixer's result, float [T, hidden], without the residual sum."""
        T = h.shape[0]
        nh, nkv, D, V, pad = self.heads, self.kv_heads, self.dim, self.vdim, self.pad
        gid, kcache, vcache = ctx.cache.pages_of_site(site)
        view = ctx.kv[gid]
        qkv = ops.gemm(h, self.w_in, ctx.buffer("gattn.qkv", (T, self.w_in.shape[0]), ctx.dtype), scratch=ctx.scratch)
        q = ops.qk_norm_scatter(qkv, self.q_weight, self.k_weight, ctx.buffer("gattn.q", (T, nh * pad), ctx.dtype), kcache, vcache,
                                view.slots, nh, nkv, D, V, pad, view.page_size, self.eps)
        out = ctx.buffer("gattn.out", (T, nh * pad), ctx.dtype)
        kernel.paged_attention(ctx, q, nh * pad, kcache, vcache, view, out, nh, nkv, pad, self.window, self.scale, tuning=self.tuning)
        first_gate = (nh + nkv) * D + nkv * V
        gates = qkv[:, first_gate:first_gate + nh] if self.head_gate else None
        act = ops.head_gate(out, gates, ctx.buffer("gattn.act", (T, nh * V), ctx.dtype), nh, V, pad)
        return ctx.product_for_norm(act, self.w_out, "gattn.y")

    def forward(self, h, residual, ctx, site, norm=None):
        from .block import add_sublayer
        return add_sublayer(residual, self.output(h, ctx, site), None, 1.0)


class LatentAttention(Mixer):
    """Softmax attention whose keys and values are made from one latent a token (multi-head latent attention).

    Per token the cache holds c = rms(Wdkv h)[:rank] * w (the latent) and kr = rot(Wdkv h [rank:]) (a key part that
    turns with the position, one for every head).  Head j's key is [Wuk_j c | kr], its value Wuv_j c, its query
    [q_j | rot(qr_j)] with `dim` plain and `rot_dim` turning coordinates; score = (q_j . Wuk_j c + rot(qr_j) . kr) scale,
    softmax over the visible keys (all earlier ones, or the last `window`).  Queries come from one projection, or with
    `q_rank` through a normed latent of their own: q = Wuq (rms(Wdq h) wq).  With `head_gate` a head's result is
    multiplied by sigmoid((Wg h)_j).  Then the output projection.

    The keys' up-projection is moved to the query's side: q'_j = Wuk_j^T q_j has `rank` coordinates, and the attention
    is that of `heads` query heads [q'_j | rot(qr_j)] over ONE key head [c | kr] and one value head [c] of
    pad = rank + rot_dim coordinates (rounded up to 8, the rest zero), which the framework's paged attention kernels
    run as they are; the weighted sum of latents then goes through Wuv_j.  The pages therefore hold what the design
    says must be kept, c and kr, and nothing a head.  Up to 256 coordinates the matrix-core kernels serve (bfloat16); a
    larger latent (up to 640 with its turning part) runs the exact row-wise kernel in both dtypes.  `position` turns the first `position.rotary_dim` of the rot_dim
    coordinates.  `names`: the tensors' names under `name`."""

    NAMES = {"q": "q", "dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk",
             "uv": "uv", "gate": "g", "o": "o"}

    def __init__(self, name, hidden, heads, dim, rot_dim, vdim, kv_rank, scale, eps, position, q_rank=None, window=None,
                 head_gate=True, names=None, tuning=None):
        self.pad = -(-(kv_rank + rot_dim) // 8) * 8
        if self.pad > ops.ROWWISE_MAX_HEAD:
            raise ValueError(f"a latent of {kv_rank} and {rot_dim} turning coordinates: at most {ops.ROWWISE_MAX_HEAD} together")
        if not scale > 0:
            raise ValueError("the score scale must be positive")
        if position.rotary_dim > rot_dim:
            raise ValueError(f"{position.rotary_dim} coordinates turn, the queries and keys have {rot_dim} for it")
        self.name, self.hidden, self.heads, self.dim, self.rot_dim, self.vdim = name, hidden, heads, dim, rot_dim, vdim
        self.kv_rank, self.scale, self.eps, self.position = kv_rank, float(scale), float(eps), position
        self.q_rank, self.window, self.head_gate = q_rank, window, bool(head_gate)
        self.names = {**self.NAMES, **(names or {})}
        self.tuning = tuning or kernel.DEFAULT_TUNING
        self.w_q = self.w_small = self.w_absorb = self.w_value = self.w_out = None

    def _tensor(self, which):
        return f"{self.name}.{self.names[which]}"

    def kernel_units(self, dtype):
        return kernel.kernel_units(self.pad, dtype)

    def step_arrays(self):
        return [kernel.SingleRows(self.tuning.split_single_from), kernel.RowsLongestFirst()]

    def cache_need(self):
        return KVNeed(1, self.pad, self.window)

    def tensor_specs(self):
        H, nh, D, R, V, r, t = self.hidden, self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank, self._tensor
        if self.q_rank is None:
            specs = [TensorSpec(t("q"), (nh * (D + R), H))]
        else:
            specs = [TensorSpec(t("dq"), (self.q_rank, H)), TensorSpec(t("dq_norm"), (self.q_rank,), init="one_plus_normal"),
                     TensorSpec(t("uq"), (nh * (D + R), self.q_rank))]
        specs += [TensorSpec(t("dkv"), (r + R, H)), TensorSpec(t("dkv_norm"), (r,), init="one_plus_normal"),
                  TensorSpec(t("uk"), (nh * D, r)), TensorSpec(t("uv"), (nh * V, r)), TensorSpec(t("o"), (H, nh * V))]
        if self.head_gate:
            specs.append(TensorSpec(t("gate"), (nh, H)))
        return specs

    def bind(self, tensors, dtype):
        nh, D, V, r, t = self.heads, self.dim, self.vdim, self.kv_rank, self._tensor
        # one product with float results for everything small that reads the mixer's input: the latents before their
        # norms, the key part that turns, the gates; the queries' own (large) product gives the compute dtype
        small = ([] if self.q_rank is None else ["dq"]) + ["dkv"] + (["gate"] if self.head_gate else [])
        parts = [matrix_operand(tensors[t(p)], dtype) for p in small]
        rows = sum(p.shape[0] for p in parts)
        if rows % 8:
            parts.append(torch.zeros(8 - rows % 8, self.hidden, dtype=parts[0].dtype, device=parts[0].device))
        self.w_small = torch.cat(parts, dim=0).contiguous()
        self.w_q = matrix_operand(tensors[t("q" if self.q_rank is None else "uq")], dtype)
        self.w_absorb = matrix_operand(tensors[t("uk")], dtype).view(nh, D, r).transpose(1, 2).contiguous()   # [heads, rank, dim]
        self.w_value = matrix_operand(tensors[t("uv")], dtype).view(nh, V, r).contiguous()                    # [heads, vdim, rank]
        self.w_out = matrix_operand(tensors[t("o")], dtype)
        self.kv_weight = tensors[t("dkv_norm")].to(torch.float32).contiguous()
        self.q_weight = None if self.q_rank is None else tensors[t("dq_norm")].to(torch.float32).contiguous()
        self.q_size = 0
        if self.q_rank is not None:        # (the query latent's size may be the file's to say: both halves must agree)
            self.q_size = tensors[t("dq")].shape[0]
            if self.w_q.shape[1] != self.q_size or self.q_weight.shape[0] != self.q_size:
                raise ValueError(f"{self.name}: the query latent's projections and norm disagree about its size")

    def prepare(self, device, dtype):
        self.position.prepare(device, dtype)

    def forward(self, h, residual, ctx, site, norm=None):
        T = h.shape[0]
        nh, D, R, V, r, pad = self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank, self.pad
        gid, kcache, vcache = ctx.cache.pages_of_site(site)
        view = ctx.kv[gid]
        cos, sin = self.position.tables()
        small = ops.gemm(h, self.w_small, ctx.buffer("lat.small", (T, self.w_small.shape[0]), torch.float32), scratch=ctx.scratch)
        first = 0
        if self.q_rank is not None:
            first = self.q_size
        q = ctx.buffer("lat.q", (T, nh * (D + R)), ctx.dtype)
        if self.q_rank is not None and ops.fused_norm_ok(small[:, :first], self.w_q, T):
            # few rows: the query latent's norm rides in the product that reads it
            ops.gemm_normed(small[:, :first], (self.q_weight, self.eps, None), self.w_q, q)
        else:
            if self.q_rank is not None:
                h = ops.rms_slice(small[:, :first], self.q_weight, ctx.buffer("lat.cq", (T, first), ctx.dtype), self.eps)
            ops.gemm(h, self.w_q, q, scratch=ctx.scratch)
        qa = ctx.buffer("lat.qa", (T, nh * pad), ctx.dtype)
        ops.latent_keys(small[:, first:first + r + R], self.kv_weight, q, qa, kcache, vcache, ctx.positions, view.slots, cos, sin,
                        nh, D, R, r, pad, view.page_size, self.eps, interleaved=self.position.pairing == "interleaved")
        ops.heads_product(q, D + R, self.w_absorb, qa, pad)
        out = ctx.buffer("lat.out", (T, nh * pad), ctx.dtype)
        kernel.paged_attention(ctx, qa, nh * pad, kcache, vcache, view, out, nh, 1, pad, self.window, self.scale, tuning=self.tuning)
        gates = small[:, first + r + R:first + r + R + nh] if self.head_gate else None
        act = ops.heads_product(out, pad, self.w_value, ctx.buffer("lat.act", (T, nh * V), ctx.dtype), V, gate=gates)
        return ctx.add_product(act, self.w_out, residual)


class SigmoidAttention(Mixer):
    """Grouped-query attention over the paged cache without a softmax: a visible key weighs sigmoid(q . k scale +
    b_head), one number `<name>.pb`[head] added to the score, and the weights are not normed over the keys.  Queries
    and keys are RMS-normed over the whole projection (all heads at once, a weight an element) before `position` turns
    the first `position.rotary_dim` coordinates of every head in neighbouring pairs; keys and values may differ in
    size (`dim`, `vdim`); a row sees itself and the `window` - 1 keys before it (None: all).

    The pages hold heads of `pad` = max(dim, vdim) coordinates (rounded up to a multiple of 8), the rest zero, so the
    framework's attention kernels run with their sigmoid law (`head_bias`) and nothing else changed.  `own_kv` False:
    the layer has no key and value tensors and reads the cache another layer wrote.  `keep`: the window the layer's
    own cache keeps, where layers that read it look further back than it does itself (None with a window: its own).
    `ride(weight)`: further rows for the input product, whose float results are then `rider`.
    `names`: the tensors' names under `name`."""

    NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "bias": "pb"}

    def __init__(self, name, hidden, heads, kv_heads, dim, vdim, scale, eps, position, window=None, keep="own", own_kv=True,
                 names=None, tuning=None):
        if heads % kv_heads:
            raise ValueError(f"{heads} query heads are not a multiple of {kv_heads} key/value heads")
        self.pad = -(-max(dim, vdim) // 8) * 8
        if self.pad > 256:
            raise ValueError(f"head sizes {dim} / {vdim}: at most 256")
        if not scale > 0:
            raise ValueError("the score scale must be positive")
        if getattr(position, "pairing", "split_half") != "interleaved" or position.rotary_dim > dim:
            raise ValueError("the position part must turn neighbouring pairs of at most `dim` coordinates")
        self.name, self.hidden, self.heads, self.kv_heads, self.dim, self.vdim = name, hidden, heads, kv_heads, dim, vdim
        self.scale, self.eps, self.position, self.window, self.own_kv = float(scale), float(eps), position, window, bool(own_kv)
        self.keep = window if keep == "own" else keep
        if self.keep is not None and (window is None or window > self.keep):
            raise ValueError("a layer's cache keeps at least the keys the layer itself looks back over")
        self.names = {**self.NAMES, **(names or {})}
        self.tuning = tuning or kernel.DEFAULT_TUNING
        self.w_in = self.w_own = self.w_out = self.q_weight = self.k_weight = self.head_bias = self.rider = None
        self.rider_rows = 0

    def _tensor(self, which):
        return f"{self.name}.{self.names[which]}"

    def kernel_units(self, dtype):
        return kernel.kernel_units(self.pad, dtype, "sigmoid")

    def step_arrays(self):
        return [kernel.SingleRows(self.tuning.split_single_from), kernel.RowsLongestFirst()]

    def cache_need(self):
        return KVNeed(self.kv_heads, self.pad, self.keep) if self.own_kv else None

    def cache_read(self):
        return None if self.own_kv else KVNeed(self.kv_heads, self.pad, self.window)

    def tensor_specs(self):
        H, nh, nkv, D, V = self.hidden, self.heads, self.kv_heads, self.dim, self.vdim
        specs = [TensorSpec(self._tensor("q"), (nh * D, H)), TensorSpec(self._tensor("q_norm"), (nh * D,), init="one_plus_normal")]
        if self.own_kv:
            specs += [TensorSpec(self._tensor("k"), (nkv * D, H)), TensorSpec(self._tensor("v"), (nkv * V, H)),
                      TensorSpec(self._tensor("k_norm"), (nkv * D,), init="one_plus_normal")]
        return specs + [TensorSpec(self._tensor("bias"), (nh,)), TensorSpec(self._tensor("o"), (H, nh * V))]

    def _join(self, extra=None):
        parts = list(self.w_own) + ([] if extra is None else [extra])
        rows = sum(p.shape[0] for p in parts)
        if rows % 8:      # rows of the fused projection are a multiple of 8: zero rows at the end
            parts.append(torch.zeros(8 - rows % 8, self.hidden, dtype=parts[0].dtype, device=parts[0].device))
        self.w_in = torch.cat(parts, dim=0).contiguous()

    def bind(self, tensors, dtype):
        self.w_own = [matrix_operand(tensors[self._tensor(p)], dtype) for p in (("q", "k", "v") if self.own_kv else ("q",))]
        self.own_rows = sum(p.shape[0] for p in self.w_own)
        self._join()
        self.w_out = matrix_operand(tensors[self._tensor("o")], dtype)
        self.q_weight = tensors[self._tensor("q_norm")].to(torch.float32).contiguous()
        self.k_weight = tensors[self._tensor("k_norm")].to(torch.float32).contiguous() if self.own_kv else None
        self.head_bias = tensors[self._tensor("bias")].to(torch.float32).contiguous()

    def ride(self, weight):
        self.rider_rows = weight.shape[0]
        self._join(weight)

    def prepare(self, device, dtype):
        self.position.prepare(device, dtype)

    def output(self, h, ctx, site):
        """The mixer's result, float [T, hidden], without the residual sum."""
        T = h.shape[0]
        nh, nkv, D, V, pad = self.heads, self.kv_heads, self.dim, self.vdim, self.pad
        gid, kcache, vcache = ctx.cache.pages_of_site(site)
        view = ctx.kv[gid]
        cos, sin = self.position.tables()
        # queries, keys and values before their norm are float (the norms' statistics are): one product with float results
        proj = ops.gemm(h, self.w_in, ctx.buffer("sattn.proj", (T, self.w_in.shape[0]), torch.float32), scratch=ctx.scratch)
        self.rider = proj[:, self.own_rows:self.own_rows + self.rider_rows] if self.rider_rows else None
        q = ctx.buffer("sattn.q", (T, nh * pad), ctx.dtype)
        if self.own_kv:
            ops.whole_norm_rope_scatter(proj, self.q_weight, self.k_weight, ctx.positions, view.slots, cos, sin, q, kcache, vcache,
                                        nh, nkv, D, V, pad, view.page_size, self.eps)
        else:
            ops.whole_norm_rope_scatter(proj, self.q_weight, None, ctx.positions, None, cos, sin, q, None, None,
                                        nh, nkv, D, V, pad, view.page_size, self.eps)
        out = ctx.buffer("sattn.out", (T, nh * pad), ctx.dtype)
        kernel.paged_attention(ctx, q, nh * pad, kcache, vcache, view, out, nh, nkv, pad, self.window, self.scale,
                               tuning=self.tuning, head_bias=self.head_bias)
        act = out if pad == V else ops.head_gate(out, None, ctx.buffer("sattn.act", (T, nh * V), ctx.dtype), nh, V, pad)
        return ops.gemm(act, self.w_out, ctx.buffer("sattn.y", (T, self.hidden), torch.float32), scratch=ctx.scratch)

    def forward(self, h, residual, ctx, site, norm=None):
        from .block import add_sublayer
        return add_sublayer(residual, self.output(h, ctx, site), None, 1.0)


class TalkingAttention(Mixer):
    """Grouped-query softmax attention over the paged cache whose scores are mixed over the heads before the softmax:
    s_h = sum_g `talk`[h, g] (`temp`[g] scale q_g . k), a learned number a head (`sink`) in every softmax's denominator
    (a key without a value), and the heads' results gated element by element by sigmoid(W_g h) before the output
    projection.  Queries and keys are RMS-normed over the whole projection (all heads at once, a weight an element)
    before `position` turns the first `position.rotary_dim` coordinates of every head (split-half pairs); each head's
    value is divided by its root mean square and cached so; keys and values may differ in size (`dim`, `vdim`);
    projections have biases (`<tensor>.b`) where `bias` names them.  A row sees the keys of its own block of `chunk`
    positions up to itself (blocks counted from position 0; None: all keys before it).

    The pages hold heads of `pad` = max(dim, vdim) coordinates (rounded up to a multiple of 8), the rest zero; with a
    `chunk` the cache keeps the last `chunk` keys (ChunkNeed: pages before a row's block go back).  The scores of all
    heads of a row meet in one kernel (ops.attention_talking).  `names`: the tensors' names under `name`."""

    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "talk": "talk",
             "temp": "temp", "sink": "sink"}

    def __init__(self, name, hidden, heads, kv_heads, dim, vdim, scale, eps, position, chunk=None, bias=("q", "k", "v", "o"),
                 temp=True, sink=True, gate=True, value_norm=True, names=None):
        if heads % kv_heads:
            raise ValueError(f"{heads} query heads are not a multiple of {kv_heads} key/value heads")
        self.pad = -(-max(dim, vdim) // 8) * 8
        if not scale > 0:
            raise ValueError("the score scale must be positive")
        if getattr(position, "pairing", "split_half") != "split_half" or getattr(position, "rotary_dim", 0) > dim:
            raise ValueError("the position part must turn split-half pairs of at most `dim` coordinates")
        if chunk is not None and chunk <= 0:
            raise ValueError("a block of positions holds at least one")
        self.name, self.hidden, self.heads, self.kv_heads, self.dim, self.vdim = name, hidden, heads, kv_heads, dim, vdim
        self.scale, self.eps, self.position, self.chunk = float(scale), float(eps), position, chunk
        self.bias, self.has_temp, self.has_sink, self.has_gate, self.value_norm = tuple(bias), bool(temp), bool(sink), bool(gate), bool(value_norm)
        self.names = {**self.NAMES, **(names or {})}
        self.w_in = self.w_out = self.b_in = self.b_out = self.q_weight = self.k_weight = self.talk = self.temp = self.sink = None
        self.rider, self.rider_rows = None, 0

    def _tensor(self, which):
        return f"{self.name}.{self.names[which]}"

    def kernel_units(self, dtype):
        return kernel.talking_units(dtype, self.heads, self.kv_heads, self.vdim, self.pad)

    def step_arrays(self):
        return [kernel.TileTasks(ops.TALKING_TILE_ROWS)]

    def cache_need(self):
        return KVNeed(self.kv_heads, self.pad) if self.chunk is None else ChunkNeed(self.kv_heads, self.pad, self.chunk, self.chunk)

    def tensor_specs(self):
        H, nh, nkv, D, V = self.hidden, self.heads, self.kv_heads, self.dim, self.vdim
        t = self._tensor
        rows = {"q": nh * D, "k": nkv * D, "v": nkv * V, "o": H}
        specs = [TensorSpec(t("q"), (nh * D, H)), TensorSpec(t("k"), (nkv * D, H)), TensorSpec(t("v"), (nkv * V, H)),
                 TensorSpec(t("q_norm"), (nh * D,), init="one_plus_normal"), TensorSpec(t("k_norm"), (nkv * D,), init="one_plus_normal"),
                 TensorSpec(t("talk"), (nh, nh)), TensorSpec(t("o"), (H, nh * V))]
        specs += [TensorSpec(t(p) + ".b", (rows[p],)) for p in self.bias]
        if self.has_temp:
            specs.append(TensorSpec(t("temp"), (nh,), init="one_plus_normal"))
        if self.has_sink:
            specs.append(TensorSpec(t("sink"), (nh,)))
        if self.has_gate:
            specs.append(TensorSpec(t("g"), (nh * V, H)))
        return specs

    def bind(self, tensors, dtype):
        t = self._tensor
        inputs = ("q", "k", "v") + (("g",) if self.has_gate else ())
        parts = self.w_own = [matrix_operand(tensors[t(p)], dtype) for p in inputs]
        self.own_rows = sum(p.shape[0] for p in parts)
        self._join()
        self.w_out = matrix_operand(tensors[t("o")], dtype)

        def f32(x):
            return x.to(torch.float32).contiguous()
        if any(p in self.bias for p in ("q", "k", "v")):
            sizes = {"q": self.heads * self.dim, "k": self.kv_heads * self.dim, "v": self.kv_heads * self.vdim}
            ref = parts[0]
            self.b_in = torch.cat([f32(tensors[t(p) + ".b"]) if p in self.bias else torch.zeros(sizes[p], dtype=torch.float32, device=ref.device)
                                   for p in ("q", "k", "v")]).contiguous()
        self.b_out = f32(tensors[t("o") + ".b"]) if "o" in self.bias else None
        self.q_weight, self.k_weight, self.talk = f32(tensors[t("q_norm")]), f32(tensors[t("k_norm")]), f32(tensors[t("talk")])
        self.temp = f32(tensors[t("temp")]) if self.has_temp else None
        self.sink = f32(tensors[t("sink")]) if self.has_sink else None

    def _join(self, extra=None):
        parts = list(self.w_own) + ([] if extra is None else [extra])
        rows = sum(p.shape[0] for p in parts)
        if rows % 8:      # rows of the fused projection are a multiple of 8: zero rows at the end
            parts.append(torch.zeros(8 - rows % 8, self.hidden, dtype=parts[0].dtype, device=parts[0].device))
        self.w_in = torch.cat(parts, dim=0).contiguous()

    def ride(self, weight):
        """Further rows for the input product (a neighbour that reads the same h); their float results are `rider`
        after `output`."""
        self.rider_rows = weight.shape[0]
        self._join(weight)

    def prepare(self, device, dtype):
        self.position.prepare(device, dtype)

    def output(self, h, ctx, site):
        """The mixer's result, float [T, hidden] (an ops.Biased where the output projection has a bias), without the
        residual sum."""
        T = h.shape[0]
        nh, nkv, D, V, pad = self.heads, self.kv_heads, self.dim, self.vdim, self.pad
        gid, kcache, vcache = ctx.cache.pages_of_site(site)
        view = ctx.kv[gid]
        cos, sin = self.position.tables()
        # queries, keys and values before their norms are float (the norms' statistics are), and so is the gate
        proj = ops.gemm(h, self.w_in, ctx.buffer("tattn.proj", (T, self.w_in.shape[0]), torch.float32), scratch=ctx.scratch)
        self.rider = proj[:, self.own_rows:self.own_rows + self.rider_rows] if self.rider_rows else None
        q = ctx.buffer("tattn.q", (T, nh * pad), ctx.dtype)
        ops.whole_norm_rope_scatter(proj, self.q_weight, self.k_weight, ctx.positions, view.slots, cos, sin, q, kcache, vcache,
                                    nh, nkv, D, V, pad, view.page_size, self.eps, bias=self.b_in, split_half=True, value_norm=self.value_norm)
        first = nh * D + nkv * (D + V)
        act = ctx.buffer("tattn.act", (T, nh * V), ctx.dtype)
        kernel.talking_attention(ctx, q, kcache, vcache, view, act, nh, nkv, V, pad, self.talk, self.scale, temp=self.temp, sink=self.sink,
                                 chunk=self.chunk, gate=proj[:, first:first + nh * V] if self.has_gate else None)
        y = ops.gemm(act, self.w_out, ctx.buffer("tattn.y", (T, self.hidden), torch.float32), scratch=ctx.scratch)
        return y if self.b_out is None else ops.Biased(y, self.b_out)       # (the kernel that adds the result adds the bias)

    def forward(self, h, residual, ctx, site, norm=None):
        from .block import add_sublayer
        return add_sublayer(residual, self.output(h, ctx, site), None, 1.0)


register_part("mixer", "talking_attention", TalkingAttention)
register_part("mixer", "attention", PagedAttention)
register_part("mixer", "sigmoid_attention", SigmoidAttention)
register_part("mixer", "latent_attention", LatentAttention)
register_part("mixer", "normed_gated_attention", NormedGatedAttention)
