"""Mixers that keep a state of fixed size per request instead of keys and values.

Both are the same recurrence per head, S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, run by one kernel
(ops.linear_scan) over the rows of a step as they come (portions and single tokens of several requests), with
the state in the cache manager's state slots, in float in every mode:

  GatedLinearAttention   a_t a vector over the key channels, sigmoid(z_t)^(1/tau), z_t from a low-rank projection
                         with a bias; q scaled by dim^(-1/2); each head's result RMS-normed over vdim with a weight
                         shared by the heads, times silu of a gate projection, then the output projection.
  StateSpaceDuality      (Mamba-2) a_t one number a head, exp(-exp(A_log) dt_t) with dt_t = softplus(dt + dt_bias);
                         k = B_t, q = C_t (shared by the heads of a group), v = dt_t x_t; x, B and C come out of a short
                         causal convolution with silu whose last inputs are part of the state; y = o + D x, times
                         silu(z), RMS-normed in equal parts of the row, then the output projection.

  GatedDeltaRule         S <- g_t S; u = beta_t (v_t - S^T k_t); S <- S + k_t u^T; o_t = S^T q_t, a kernel of its own
                         (ops.delta_scan): g_t = exp(-exp(A_log) softplus(a_t + dt_bias)) and beta_t = sigmoid(b_t) one
                         number a head; q, k, v come out of a short causal convolution with silu (its last inputs are
                         part of the state), q and k are made unit vectors per head, q scaled by dim^(-1/2); each
                         head's result RMS-normed, times silu of a gate projection, then the output projection.

  MinGRU                 no heads and no matrix state: S_t = (1 - z_t) S_(t-1) + z_t c_t element by element over `width`
                         channels, z_t = sigmoid(Wz h + bz), c_t = cand(Wx h + bx) with cand(u) = u + 1/2 for u >= 0 and
                         sigmoid(u) below (the gates read the current token only); the result is Wo (S_t silu(Wg h)).
                         A kernel of its own (ops.mingru_scan).

The projections and the convolution's inputs are products with float results; decays, step sizes, gates of the
recurrence and the norms are float arithmetic; the operands of the output projections are the compute dtype.
"""
import torch

from ..cache.pages import StateNeed
from ..kernels import library, ops
from ..weights.loader import AnySize
from .base import Mixer, TensorSpec, matrix_operand, register_part


def _float(t):
    return t.to(torch.float32).contiguous()


def _scan(ctx, tag, q, k, v, decay, out, state, heads, rows, cols, **kw):
    """ops.linear_scan over the step's segments; the segments of a step with long portions are walked in pieces."""
    T = v.shape[0]
    piece = ops.scan_piece(T, ctx.decode_only)
    carry = None
    if piece:
        n, n_decay = ops.scan_carry(T, piece, heads, rows, cols, decay.shape[1] != heads)
        carry = (ctx.buffer(tag + ".carry", (n,), torch.float32), ctx.buffer(tag + ".carry_decay", (n_decay,), torch.float32))
    return ops.linear_scan(q, k, v, decay, out, state, ctx.seg_start, ctx.state_slots, heads, rows, cols, piece=piece, carry=carry, **kw)


class GatedLinearAttention(Mixer):
    NAMES = {"q": "q", "k": "k", "v": "v", "gate": "g", "o": "o", "norm": "norm", "down": "a1", "up": "a2", "bias": "a2.b"}

    def __init__(self, name, hidden, heads, dim, vdim, tau, eps, rank=16, names=None):
        """`rank`: the inner size of the decay's low-rank projection where no file says it (the files decide)."""
        if not tau > 0:
            raise ValueError("tau must be positive")
        self.name, self.hidden, self.heads, self.dim, self.vdim = name, hidden, heads, dim, vdim
        self.tau, self.eps, self.rank = float(tau), float(eps), int(rank)
        self.names = {**self.NAMES, **(names or {})}

    def _tensor(self, which):
        return f"{self.name}.{self.names[which]}"

    def kernel_units(self, dtype):
        return [library.RECURRENCE]

    def state_need(self):
        return StateNeed((self.heads, self.dim, self.vdim), "float32")

    def tensor_specs(self):
        H, K, V = self.hidden, self.heads * self.dim, self.heads * self.vdim
        return [TensorSpec(self._tensor("q"), (K, H)), TensorSpec(self._tensor("k"), (K, H)), TensorSpec(self._tensor("v"), (V, H)),
                TensorSpec(self._tensor("gate"), (V, H)), TensorSpec(self._tensor("o"), (H, V)),
                TensorSpec(self._tensor("norm"), (self.vdim,), init="one_plus_normal"),
                TensorSpec(self._tensor("down"), (AnySize(self.rank), H)), TensorSpec(self._tensor("up"), (K, AnySize(self.rank))),
                TensorSpec(self._tensor("bias"), (K,))]

    def bind(self, tensors, dtype):
        # one product for q, k, v, the gate and the first half of the decay's low-rank projection; its second half is a
        # few multiplications a decay, done in float by the kernel that makes the decays
        parts = [matrix_operand(tensors[self._tensor(p)], dtype) for p in ("q", "k", "v", "gate", "down")]
        self.low_rank = parts[-1].shape[0]
        self.w_up = _float(tensors[self._tensor("up")].t())          # [rank, heads * dim]: the decays' kernel reads it by columns
        if self.low_rank != self.w_up.shape[0]:
            raise ValueError(f"{self.name}: the decay's projections disagree about their inner size "
                             f"({self.low_rank} and {self.w_up.shape[0]})")
        self.w_in = torch.cat(parts, dim=0).contiguous()
        self.w_out = matrix_operand(tensors[self._tensor("o")], dtype)
        self.norm_weight, self.bias = _float(tensors[self._tensor("norm")]), _float(tensors[self._tensor("bias")])

    def output(self, h, ctx, site):
        T = h.shape[0]
        K, V = self.heads * self.dim, self.heads * self.vdim
        proj = ops.gemm(h, self.w_in, ctx.buffer("gla.proj", (T, self.w_in.shape[0]), torch.float32), scratch=ctx.scratch)
        decay = ops.decay_gate_low_rank(proj[:, 2 * K + 2 * V:], self.w_up, self.bias, ctx.buffer("gla.decay", (T, K), torch.float32), self.tau)
        state = ctx.cache.state_storage[site]
        o = ctx.buffer("gla.o", (T, V), torch.float32)
        _scan(ctx, "gla", proj[:, :K], proj[:, K:2 * K], proj[:, 2 * K:2 * K + V], decay, o, state.view(state.shape[0], -1),
              self.heads, self.dim, self.vdim, q_scale=self.dim ** -0.5)
        act = ops.group_norm_gate(o, proj[:, 2 * K + V:2 * K + 2 * V], self.norm_weight, ctx.buffer("gla.act", (T, V), ctx.dtype),
                                  self.heads, self.eps, gate_first=False, shared_weight=True)
        return ctx.product_for_norm(act, self.w_out, "gla.y")

    def forward(self, h, residual, ctx, site, norm=None):
        from .block import add_sublayer
        return add_sublayer(residual, self.output(h, ctx, site), None, 1.0)


class StateSpaceDuality(Mixer):
    NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "a_log": "A_log", "skip": "D",
             "norm": "norm", "o": "o"}
    MAX_TAPS = 16

    def __init__(self, name, hidden, heads, vdim, state, groups, taps, norm_groups, eps, names=None):
        if heads % groups:
            raise ValueError(f"{heads} heads do not divide into {groups} groups")
        if (heads * vdim) % norm_groups:
            raise ValueError(f"{heads} x {vdim} channels do not divide into {norm_groups} equal parts")
        if not 1 <= taps <= self.MAX_TAPS:
            raise ValueError(f"a convolution of {taps} taps: 1 to {self.MAX_TAPS}")
        self.name, self.hidden, self.heads, self.vdim, self.state, self.groups = name, hidden, heads, vdim, state, groups
        self.taps, self.norm_groups, self.eps = int(taps), int(norm_groups), float(eps)
        self.inner = heads * vdim
        self.channels = self.inner + 2 * groups * state          # what the convolution runs over: x, B, C
        self.names = {**self.NAMES, **(names or {})}

    def _tensor(self, which):
        return f"{self.name}.{self.names[which]}"

    def kernel_units(self, dtype):
        return [library.RECURRENCE]

    def state_need(self):
        """One float row a request: the heads' states [heads, state, vdim], then the convolution's last taps - 1 inputs
        [taps - 1, channels]."""
        return StateNeed((self.heads * self.state * self.vdim + (self.taps - 1) * self.channels,), "float32")

    def tensor_specs(self):
        H, t = self.hidden, self._tensor
        return [TensorSpec(t("in"), (2 * self.inner + 2 * self.groups * self.state + self.heads, H)),
                TensorSpec(t("conv"), (self.channels, self.taps)), TensorSpec(t("conv_bias"), (self.channels,)),
                TensorSpec(t("dt_bias"), (self.heads,)), TensorSpec(t("a_log"), (self.heads,)), TensorSpec(t("skip"), (self.heads,)),
                TensorSpec(t("norm"), (self.inner,), init="one_plus_normal"), TensorSpec(t("o"), (H, self.inner))]

    def bind(self, tensors, dtype):
        t = self._tensor
        self.w_in, self.w_out = matrix_operand(tensors[t("in")], dtype), matrix_operand(tensors[t("o")], dtype)
        self.conv, self.conv_bias = _float(tensors[t("conv")]), _float(tensors[t("conv_bias")])
        self.dt_bias, self.a_log, self.skip = _float(tensors[t("dt_bias")]), _float(tensors[t("a_log")]), _float(tensors[t("skip")])
        self.norm_weight = _float(tensors[t("norm")])

    def output(self, h, ctx, site):
        T = h.shape[0]
        inner, GN, ch, nh = self.inner, self.groups * self.state, self.channels, self.heads
        proj = ops.gemm(h, self.w_in, ctx.buffer("ssd.proj", (T, 2 * inner + 2 * GN + nh), torch.float32), scratch=ctx.scratch)
        state = ctx.cache.state_storage[site]
        heads_state = nh * self.state * self.vdim
        xbc = ctx.buffer("ssd.xbc", (T, ch), torch.float32)
        step, decay = ctx.buffer("ssd.step", (T, nh), torch.float32), ctx.buffer("ssd.decay", (T, nh), torch.float32)
        ops.conv_silu(proj[:, inner:inner + ch], self.conv, self.conv_bias, state[:, heads_state:], xbc, ctx.seg_of_row,
                      ctx.seg_start, ctx.state_slots, gates=(proj[:, inner + ch:], self.dt_bias, self.a_log, step, decay),
                      single_rows=ctx.decode_only)
        y = ctx.buffer("ssd.o", (T, inner), torch.float32)
        _scan(ctx, "ssd", xbc[:, inner + GN:], xbc[:, inner:inner + GN], xbc[:, :inner], decay, y, state,
              nh, self.state, self.vdim, share=nh // self.groups, step=step)
        act = ops.group_norm_gate(y, proj[:, :inner], self.norm_weight, ctx.buffer("ssd.act", (T, inner), ctx.dtype),
                                  self.norm_groups, self.eps, gate_first=True, skip=(self.skip, xbc[:, :inner]))
        return ctx.product_for_norm(act, self.w_out, "ssd.y")

    def forward(self, h, residual, ctx, site, norm=None):
        from .block import add_sublayer
        return add_sublayer(residual, self.output(h, ctx, site), None, 1.0)


class GatedDeltaRule(Mixer):
    """The gated delta rule.  `kv_heads` heads of q and k (`dim` each) serve `heads` heads of v (`vdim` each), head j
    using q/k head j // (heads / kv_heads).  `names`: the tensors' names under `name`; the convolutions' taps are
    `<projection>.conv`, [channels, taps]; tap n - 1 weighs the newest input."""

    NAMES = {"q": "q", "k": "k", "v": "v", "write": "b", "decay": "a", "dt_bias": "dt_bias", "a_log": "A_log", "gate": "g",
             "norm": "norm", "o": "o", "conv": "conv"}
    MAX_TAPS = 16

    def __init__(self, name, hidden, heads, kv_heads, dim, vdim, taps, eps, unit_eps=1e-6, names=None):
        if heads % kv_heads:
            raise ValueError(f"{heads} heads are not a multiple of {kv_heads} query/key heads")
        if not 1 <= taps <= self.MAX_TAPS:
            raise ValueError(f"a convolution of {taps} taps: 1 to {self.MAX_TAPS}")
        if dim > 256:
            raise ValueError(f"query/key heads of {dim}: at most 256")
        self.name, self.hidden, self.heads, self.kv_heads, self.dim, self.vdim = name, hidden, heads, kv_heads, dim, vdim
        self.taps, self.eps, self.unit_eps = int(taps), float(eps), float(unit_eps)
        self.qk, self.inner = kv_heads * dim, heads * vdim
        self.channels = 2 * self.qk + self.inner           # what the convolution runs over: q, k, v
        self.names = {**self.NAMES, **(names or {})}

    def _tensor(self, which):
        return f"{self.name}.{self.names[which]}"

    def kernel_units(self, dtype):
        return [library.RECURRENCE]

    def state_need(self):
        """One float row a request: the heads' states [heads, dim, vdim], then the convolution's last taps - 1 inputs
        [taps - 1, channels]."""
        return StateNeed((self.heads * self.dim * self.vdim + (self.taps - 1) * self.channels,), "float32")

    def tensor_specs(self):
        H, t, conv = self.hidden, self._tensor, self.names["conv"]
        return [TensorSpec(t("q"), (self.qk, H)), TensorSpec(t("k"), (self.qk, H)), TensorSpec(t("v"), (self.inner, H)),
                TensorSpec(f"{t('q')}.{conv}", (self.qk, self.taps)), TensorSpec(f"{t('k')}.{conv}", (self.qk, self.taps)),
                TensorSpec(f"{t('v')}.{conv}", (self.inner, self.taps)),
                TensorSpec(t("write"), (self.heads, H)), TensorSpec(t("decay"), (self.heads, H)),
                TensorSpec(t("dt_bias"), (self.heads,)), TensorSpec(t("a_log"), (self.heads,)),
                TensorSpec(t("gate"), (self.inner, H)), TensorSpec(t("norm"), (self.vdim,), init="one_plus_normal"),
                TensorSpec(t("o"), (H, self.inner))]

    def bind(self, tensors, dtype):
        t, conv = self._tensor, self.names["conv"]
        # one product with float results: [q | k | v | decay | write | gate] (everything that enters the recurrence is float)
        parts = [matrix_operand(tensors[t(p)], dtype) for p in ("q", "k", "v", "decay", "write", "gate")]
        rows = sum(p.shape[0] for p in parts)
        if rows % 8:
            parts.append(torch.zeros(8 - rows % 8, self.hidden, dtype=parts[0].dtype, device=parts[0].device))
        self.w_in = torch.cat(parts, dim=0).contiguous()
        self.w_out = matrix_operand(tensors[t("o")], dtype)
        self.conv = torch.cat([_float(tensors[f"{t(p)}.{conv}"]) for p in ("q", "k", "v")], dim=0).contiguous()
        self.dt_bias, self.a_log = _float(tensors[t("dt_bias")]), _float(tensors[t("a_log")])
        self.norm_weight = _float(tensors[t("norm")])

    def _normed_result(self, h, ctx, site):
        """The operand of the output projection [T, heads * vdim]; moves the request's state on."""
        T = h.shape[0]
        qk, inner, ch, nh = self.qk, self.inner, self.channels, self.heads
        proj = ops.gemm(h, self.w_in, ctx.buffer("delta.proj", (T, self.w_in.shape[0]), torch.float32), scratch=ctx.scratch)
        state = ctx.cache.state_storage[site]
        heads_state = nh * self.dim * self.vdim
        qkv = ctx.buffer("delta.qkv", (T, ch), torch.float32)
        step, decay = ctx.buffer("delta.step", (T, nh), torch.float32), ctx.buffer("delta.decay", (T, nh), torch.float32)
        ops.conv_silu(proj[:, :ch], self.conv, None, state[:, heads_state:], qkv, ctx.seg_of_row, ctx.seg_start, ctx.state_slots,
                      gates=(proj[:, ch:ch + nh], self.dt_bias, self.a_log, step, decay), single_rows=ctx.decode_only)
        ops.unit_heads(qkv[:, :2 * qk], 2 * self.kv_heads, self.dim, eps=self.unit_eps)
        o = ctx.buffer("delta.o", (T, inner), torch.float32)
        ops.delta_scan(qkv[:, :qk], qkv[:, qk:2 * qk], qkv[:, 2 * qk:], decay, proj[:, ch + nh:ch + 2 * nh], o, state,
                       ctx.seg_start, ctx.state_slots, nh, self.dim, self.vdim, share=nh // self.kv_heads, q_scale=self.dim ** -0.5)
        act = ops.group_norm_gate(o, proj[:, ch + 2 * nh:ch + 2 * nh + inner], self.norm_weight, ctx.buffer("delta.act", (T, inner), ctx.dtype),
                                  nh, self.eps, gate_first=False, shared_weight=True)
        return act

    def output(self, h, ctx, site):
        """The mixer's result, float [T, hidden], without the residual sum."""
        return ctx.product_for_norm(self._normed_result(h, ctx, site), self.w_out, "delta.y")

    def forward(self, h, residual, ctx, site, norm=None):
        return ctx.add_product(self._normed_result(h, ctx, site), self.w_out, residual)


class MinGRU(Mixer):
    """The minimal gated recurrent unit over `width` channels (see the module's text).  State: float [width] a request,
    zero at the start.  `ride(weight)`: further rows for the input product, whose float results are then `rider`.
    `names`: the tensors' names under `name` (biases are `<projection>.b`)."""

    NAMES = {"z": "z", "x": "x", "gate": "g", "o": "o"}

    def __init__(self, name, hidden, width, names=None):
        self.name, self.hidden, self.width = name, hidden, int(width)
        self.names = {**self.NAMES, **(names or {})}
        self.rider, self.rider_rows = None, 0

    def _tensor(self, which):
        return f"{self.name}.{self.names[which]}"

    def kernel_units(self, dtype):
        return [library.RECURRENCE]

    def state_need(self):
        return StateNeed((self.width,), "float32")

    def tensor_specs(self):
        H, W, t = self.hidden, self.width, self._tensor
        return [TensorSpec(t("z"), (W, H)), TensorSpec(t("z") + ".b", (W,)), TensorSpec(t("x"), (W, H)), TensorSpec(t("x") + ".b", (W,)),
                TensorSpec(t("gate"), (W, H)), TensorSpec(t("o"), (H, W))]

    def _join(self, extra=None):
        parts = list(self.w_own) + ([] if extra is None else [extra])
        rows = sum(p.shape[0] for p in parts)
        if rows % 8:
            parts.append(torch.zeros(8 - rows % 8, self.hidden, dtype=parts[0].dtype, device=parts[0].device))
        self.w_in = torch.cat(parts, dim=0).contiguous()

    def bind(self, tensors, dtype):
        t = self._tensor
        # one product with float results: [z | x | gate] (everything that enters the recurrence is float)
        self.w_own = [matrix_operand(tensors[t(p)], dtype) for p in ("z", "x", "gate")]
        self._join()
        self.w_out = matrix_operand(tensors[t("o")], dtype)
        self.bias_z, self.bias_x = _float(tensors[t("z") + ".b"]), _float(tensors[t("x") + ".b"])

    def ride(self, weight):
        self.rider_rows = weight.shape[0]
        self._join(weight)

    def output(self, h, ctx, site):
        """The mixer's result, float [T, hidden], without the residual sum; moves the request's state on."""
        T, W = h.shape[0], self.width
        proj = ops.gemm(h, self.w_in, ctx.buffer("mingru.proj", (T, self.w_in.shape[0]), torch.float32), scratch=ctx.scratch)
        self.rider = proj[:, 3 * W:3 * W + self.rider_rows] if self.rider_rows else None
        piece = ops.mingru_piece(T, ctx.decode_only)
        carry = ctx.buffer("mingru.carry", (2 * (T // piece + ctx.n_segments) * W,), torch.float32) if piece else None
        act = ops.mingru_scan(proj, self.bias_z, self.bias_x, ctx.cache.state_storage[site], ctx.seg_start, ctx.state_slots,
                              ctx.buffer("mingru.act", (T, W), ctx.dtype), W, piece=piece, carry=carry)
        return ops.gemm(act, self.w_out, ctx.buffer("mingru.y", (T, self.hidden), torch.float32), scratch=ctx.scratch)

    def forward(self, h, residual, ctx, site, norm=None):
        from .block import add_sublayer
        return add_sublayer(residual, self.output(h, ctx, site), None, 1.0)


class MatrixMemory(Mixer):
    """The matrix memory of xLSTM (mLSTM): per head a state S [dim, vdim], a normalizer n [dim] and a running maximum m
    (all zero at a sequence's start), with log gates i = cap tanh((Wi h + bi) / cap) and f = logsigmoid(cap tanh((Wf h +
    bf) / cap)):  m' = max(f + m, i);  S <- exp(f + m - m') S + exp(i - m') k v^T, n likewise with k alone;
    o = S^T q / (max(|n . q|, exp(-m')) + 1e-6), q scaled by dim^(-1/2).  Each head's o is divided by its root mean
    square, times a weight an element, times sigmoid(Wg h), then the output projection.

    n rides in the state as one more column (a value that is always 1), so the recurrence is the linear scan with a
    decay a head and a step size (ops.linear_scan); the gates, the walk of m and the finish are kernels of their own
    (ops.mlstm_gates, ops.mlstm_finish).  The state slot holds [heads, dim, vdim + 1] and then m [heads], float."""

    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "i": "i", "f": "f"}

    def __init__(self, name, hidden, heads, dim, vdim, gate_cap, eps, floor=1e-6, names=None):
        if not gate_cap > 0:
            raise ValueError("the gates' cap must be positive")
        self.name, self.hidden, self.heads, self.dim, self.vdim = name, hidden, heads, dim, vdim
        self.cap, self.eps, self.floor = float(gate_cap), float(eps), float(floor)
        self.names = {**self.NAMES, **(names or {})}

    def _tensor(self, which):
        return f"{self.name}.{self.names[which]}"

    def kernel_units(self, dtype):
        return [library.RECURRENCE]

    def state_need(self):
        return StateNeed((self.heads * self.dim * (self.vdim + 1) + self.heads,), "float32")

    def tensor_specs(self):
        H, K, V, t = self.hidden, self.heads * self.dim, self.heads * self.vdim, self._tensor
        return [TensorSpec(t("q"), (K, H)), TensorSpec(t("k"), (K, H)), TensorSpec(t("v"), (V, H)), TensorSpec(t("g"), (V, H)),
                TensorSpec(t("o"), (H, V)), TensorSpec(t("norm"), (V,), init="one_plus_normal"),
                TensorSpec(t("i"), (self.heads, H)), TensorSpec(t("i") + ".b", (self.heads,)),
                TensorSpec(t("f"), (self.heads, H)), TensorSpec(t("f") + ".b", (self.heads,))]

    def bind(self, tensors, dtype):
        t = self._tensor
        parts = [matrix_operand(tensors[t(p)], dtype) for p in ("q", "k", "v", "g", "i", "f")]
        rows = sum(p.shape[0] for p in parts)
        if rows % 8:
            parts.append(torch.zeros(8 - rows % 8, self.hidden, dtype=parts[0].dtype, device=parts[0].device))
        self.w_in = torch.cat(parts, dim=0).contiguous()
        self.w_out = matrix_operand(tensors[t("o")], dtype)
        self.norm_weight = _float(tensors[t("norm")])
        self.bias_i, self.bias_f = _float(tensors[t("i") + ".b"]), _float(tensors[t("f") + ".b"])

    def input_weight(self):
        """The matrix of the input product, for a neighbour that reads the same h and makes both products as one (its
        float results then come back as `proj` of `output`)."""
        return self.w_in

    def output(self, h, ctx, site, proj=None):
        T = h.shape[0]
        nh, R, V = self.heads, self.dim, self.vdim
        K, W, C = nh * R, nh * V, V + 1
        if proj is None:
            proj = ops.gemm(h, self.w_in, ctx.buffer("mm.proj", (T, self.w_in.shape[0]), torch.float32), scratch=ctx.scratch)
        state = ctx.cache.state_storage[site]
        state = state.view(state.shape[0], -1)
        decay, step, top = (ctx.buffer("mm." + n, (T, nh), torch.float32) for n in ("decay", "step", "top"))
        vx = ctx.buffer("mm.vx", (T, nh * C), torch.float32)
        gates = 2 * K + 2 * W
        ops.mlstm_gates(proj[:, gates:gates + nh], proj[:, gates + nh:gates + 2 * nh], self.bias_i, self.bias_f, proj[:, 2 * K:2 * K + W],
                        decay, step, top, vx, state[:, K * C:], ctx.seg_start, ctx.state_slots, nh, V, self.cap, single_rows=ctx.decode_only)
        o = ctx.buffer("mm.o", (T, nh * C), torch.float32)
        _scan(ctx, "mm", proj[:, :K], proj[:, K:2 * K], vx, decay, o, state, nh, R, C, step=step, q_scale=R ** -0.5)
        act = ops.mlstm_finish(o, top, proj[:, 2 * K + W:2 * K + 2 * W], self.norm_weight, ctx.buffer("mm.act", (T, W), ctx.dtype),
                               nh, V, self.eps, self.floor)
        return ops.gemm(act, self.w_out, ctx.buffer("mm.y", (T, self.hidden), torch.float32), scratch=ctx.scratch)

    def forward(self, h, residual, ctx, site, norm=None):
        from .block import add_sublayer
        return add_sublayer(residual, self.output(h, ctx, site), None, 1.0)


class SideBySide(Mixer):
    """Two mixers that read the same input; the result is half the sum of theirs, each RMS-normed over the model
    width with a weight of its own (`<name>.<first_out>` / `<name>.<second_out>`), or, with `scales` = (a, b), the plain
    sum a first + b second without norms or tensors of its own.  At most one of the two keeps pages and at most one a
    state: a site of the cache has one need of each kind."""

    def __init__(self, name, hidden, first, second, eps, first_out="left.out", second_out="right.out", scales=None):
        for kind in ("cache_need", "state_need"):
            if getattr(first, kind)() is not None and getattr(second, kind)() is not None:
                raise ValueError(f"both mixers of {name} declare a {kind}: a layer keeps one")
        self.name, self.hidden, self.first, self.second, self.eps = name, hidden, first, second, float(eps)
        self.scales = None if scales is None else (float(scales[0]), float(scales[1]))
        self.out_names = (f"{name}.{first_out}", f"{name}.{second_out}") if scales is None else ()

    def mixers(self):
        return [self.first, self.second]

    def kernel_units(self, dtype):
        return [u for m in self.mixers() if hasattr(m, "kernel_units") for u in m.kernel_units(dtype)]

    def step_arrays(self):
        return [a for m in self.mixers() if hasattr(m, "step_arrays") for a in m.step_arrays()]

    def cache_need(self):
        return self.first.cache_need() or self.second.cache_need()

    def state_need(self):
        return self.first.state_need() or self.second.state_need()

    def tensor_specs(self):
        return ([s for m in self.mixers() for s in m.tensor_specs()]
                + [TensorSpec(n, (self.hidden,), init="one_plus_normal") for n in self.out_names])

    def bind(self, tensors, dtype):
        for m in self.mixers():
            m.bind(tensors, dtype)
        self.out_weights = [_float(tensors[n]) for n in self.out_names]
        # both read the same h: where the first takes further rows into its input product and the second can be handed
        # its projection, the two products are one
        self.joined = self.scales is not None and hasattr(self.first, "ride") and hasattr(self.second, "input_weight")
        if self.joined:
            self.first.ride(self.second.input_weight())

    def prepare(self, device, dtype):
        for m in self.mixers():
            m.prepare(device, dtype)

    def output(self, h, ctx, site):
        from .block import NormedMean, ScaledSum
        if self.scales is not None:
            first = self.first.output(h, ctx, site)
            second = self.second.output(h, ctx, site, proj=self.first.rider) if self.joined else self.second.output(h, ctx, site)
            return ScaledSum(first, self.scales[0], second, self.scales[1])
        return NormedMean(self.first.output(h, ctx, site), self.out_weights[0], self.second.output(h, ctx, site),
                          self.out_weights[1], self.eps)

    def forward(self, h, residual, ctx, site, norm=None):
        from .block import add_sublayer
        return add_sublayer(residual, self.output(h, ctx, site), None, 1.0)


register_part("mixer", "gated_linear_attention", GatedLinearAttention)
register_part("mixer", "state_space_duality", StateSpaceDuality)
register_part("mixer", "side_by_side", SideBySide)
register_part("mixer", "gated_delta_rule", GatedDeltaRule)
register_part("mixer", "mingru", MinGRU)
register_part("mixer", "matrix_memory", MatrixMemory)
