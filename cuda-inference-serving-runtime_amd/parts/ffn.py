"""Gated feed-forward (SwiGLU): x + (silu(h Wg^T) * (h Wu^T)) Wd^T
(reference: runtime/model.py:116-119).  Gate and up run as one product against
the concatenated weight [gate; up].  With `bias` every projection adds `<name>.*_proj.bias`:
the products run as they are and a small kernel adds the bias (no fused activation then)."""
import torch

from ..kernels import ops
from .base import FeedForward, TensorSpec, matrix_operand, register_part


class GatedMLP(FeedForward):
    def __init__(self, name, hidden, intermediate, activation="silu", bias=False, names=None):
        """`names` = (gate, up, down): the matrices' full names under `name` where they are not `<x>_proj.weight`
        (no biases then)."""
        if activation != "silu":
            raise ValueError(f"activation {activation!r}: only silu has a kernel")
        if names is not None and bias:
            raise ValueError("biases come with the default tensor names")
        self.name, self.hidden, self.intermediate = name, hidden, intermediate
        self.bias = bool(bias)
        self.names = tuple(names) if names is not None else ("gate_proj.weight", "up_proj.weight", "down_proj.weight")
        self.w_gate_up = self.w_down = self.b_gate_up = self.b_down = None

    def tensor_specs(self):
        n, H, I = self.name, self.hidden, self.intermediate
        specs = [TensorSpec(f"{n}.{self.names[0]}", (I, H)), TensorSpec(f"{n}.{self.names[1]}", (I, H)),
                 TensorSpec(f"{n}.{self.names[2]}", (H, I))]
        if self.bias:
            specs += [TensorSpec(f"{n}.gate_proj.bias", (I,)), TensorSpec(f"{n}.up_proj.bias", (I,)), TensorSpec(f"{n}.down_proj.bias", (H,))]
        return specs

    def bind(self, tensors, dtype):
        gate = matrix_operand(tensors[f"{self.name}.{self.names[0]}"], dtype)
        up = matrix_operand(tensors[f"{self.name}.{self.names[1]}"], dtype)
        self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = matrix_operand(tensors[f"{self.name}.{self.names[2]}"], dtype)
        if self.bias:   # (a bias keeps the type it is stored in; it is added in float)
            self.b_gate_up = torch.cat([tensors[f"{self.name}.gate_proj.bias"], tensors[f"{self.name}.up_proj.bias"]], dim=0).contiguous()
            self.b_down = tensors[f"{self.name}.down_proj.bias"].contiguous()

    def fuses_norm(self, norm, residual, ctx):
        return not self.bias and getattr(norm, "fusable_as", None) == "rms" and ops.fused_norm_ok(residual, self.w_gate_up, residual.shape[0])

    def forward(self, h, residual, ctx, norm=None):
        T = residual.shape[0]
        act = ctx.buffer("ffn.act", (T, self.intermediate), ctx.dtype)
        if self.bias:
            gate_up = ops.gemm(h, self.w_gate_up, ctx.buffer("ffn.gate_up", (T, 2 * self.intermediate), ctx.dtype), scratch=ctx.scratch)
            ops.swiglu(ops.bias_add(gate_up, self.b_gate_up), act)
            return ops.bias_add(ctx.add_product(act, self.w_down, residual), self.b_down)
        if norm is not None:
            ops.gemm_swiglu(residual, self.w_gate_up, act, norm=(norm.weight, norm.eps, None), scratch=ctx.scratch)
        elif ops.swiglu_fused_ok(h, self.w_gate_up):
            ops.gemm_swiglu(h, self.w_gate_up, act, scratch=ctx.scratch)   # one kernel: product and activation
        else:
            ops.gemm_swiglu(h, self.w_gate_up, act, gate_up=ctx.buffer("ffn.gate_up", (T, 2 * self.intermediate), ctx.dtype), scratch=ctx.scratch)
        return ctx.add_product(act, self.w_down, residual)

    def output(self, h, ctx, tag="ffn"):
        """The feed-forward's result, float [T, hidden], without the residual sum (no biases)."""
        if self.bias:
            raise NotImplementedError("the result without the residual sum is made for the form without biases")
        T = h.shape[0]
        act = ctx.buffer(tag + ".act", (T, self.intermediate), ctx.dtype)
        if ops.swiglu_fused_ok(h, self.w_gate_up):
            ops.gemm_swiglu(h, self.w_gate_up, act, scratch=ctx.scratch)
        else:
            ops.gemm_swiglu(h, self.w_gate_up, act, gate_up=ctx.buffer(tag + ".gate_up", (T, 2 * self.intermediate), ctx.dtype), scratch=ctx.scratch)
        return ops.gemm(act, self.w_down, ctx.buffer(tag + ".out", (T, self.hidden), torch.float32), scratch=ctx.scratch)


class ClampedGLU(FeedForward):
    """y = (g sigmoid(slope g) (u + shift)) Wd^T with g = min(h Wg^T, limit), u = clamp(h Wu^T, -limit, limit).
    Gate and up run as one product against [gate; up]; `names` = (gate, up, down), the tensors' names under `name`."""

    def __init__(self, name, hidden, intermediate, limit, slope=1.702, shift=1.0, names=("gate", "up", "down")):
        if not limit > 0:
            raise ValueError("the clamp's limit must be positive")
        self.name, self.hidden, self.intermediate = name, hidden, intermediate
        self.limit, self.slope, self.shift, self.names = float(limit), float(slope), float(shift), tuple(names)
        self.w_gate_up = self.w_down = None

    def _tensor(self, which):
        return f"{self.name}.{self.names[which]}"

    def tensor_specs(self):
        H, I = self.hidden, self.intermediate
        return [TensorSpec(self._tensor(0), (I, H)), TensorSpec(self._tensor(1), (I, H)), TensorSpec(self._tensor(2), (H, I))]

    def bind(self, tensors, dtype):
        gate, up = (matrix_operand(tensors[self._tensor(i)], dtype) for i in (0, 1))
        self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = matrix_operand(tensors[self._tensor(2)], dtype)

    def output(self, h, ctx):
        """The feed-forward's result, float [T, hidden], without the residual sum."""
        T = h.shape[0]
        law = (self.limit, self.slope, self.shift)
        act = ctx.buffer("ffn.act", (T, self.intermediate), ctx.dtype)
        if ops.swiglu_fused_ok(h, self.w_gate_up):
            ops.gemm_swiglu(h, self.w_gate_up, act, scratch=ctx.scratch, law=law)      # the product and the activation are one kernel
        else:
            ops.gemm_swiglu(h, self.w_gate_up, act, gate_up=ctx.buffer("ffn.gate_up", (T, 2 * self.intermediate), ctx.dtype),
                            scratch=ctx.scratch, law=law)
        return ctx.product_for_norm(act, self.w_down, "ffn.out")

    def forward(self, h, residual, ctx, norm=None):
        from .block import add_sublayer
        return add_sublayer(residual, self.output(h, ctx), None, 1.0)


class DenseMLP(FeedForward):
    """y = act(h Wu^T) Wd^T, one matrix up and one down, no gate.  `activation`: "gelu" (the exact form, with the error
    function), "gelu_tanh" or "relu2" (the square of relu).  `names` = (up, down), the tensors' names under `name`.
    `bias`: both products add `<tensor>.b` (the up product's activation is then a kernel after the bias, not its epilogue)."""

    def __init__(self, name, hidden, intermediate, activation="gelu", names=("up", "down"), bias=False):
        if activation not in ops.GELU_KINDS:
            raise ValueError(f"activation {activation!r}: one of {sorted(ops.GELU_KINDS)}")
        self.name, self.hidden, self.intermediate, self.activation = name, hidden, intermediate, activation
        self.names, self.bias = tuple(names), bool(bias)
        self.w_up = self.w_down = self.b_up = self.b_down = None

    def _tensor(self, which):
        return f"{self.name}.{self.names[which]}"

    def tensor_specs(self):
        specs = [TensorSpec(self._tensor(0), (self.intermediate, self.hidden)), TensorSpec(self._tensor(1), (self.hidden, self.intermediate))]
        if self.bias:
            specs += [TensorSpec(self._tensor(0) + ".b", (self.intermediate,)), TensorSpec(self._tensor(1) + ".b", (self.hidden,))]
        return specs

    def bind(self, tensors, dtype):
        self.w_up, self.w_down = (matrix_operand(tensors[self._tensor(i)], dtype) for i in (0, 1))
        if self.bias:
            self.b_up, self.b_down = (tensors[self._tensor(i) + ".b"].to(torch.float32).contiguous() for i in (0, 1))

    def _activations(self, h, ctx):
        T = h.shape[0]
        if self.bias:
            up = ops.gemm(h, self.w_up, ctx.buffer("ffn.up", (T, self.intermediate), ctx.dtype), scratch=ctx.scratch)
            return ops.bias_act(up, self.b_up, ctx.buffer("ffn.act", (T, self.intermediate), ctx.dtype), self.activation)
        # the activation is the epilogue of the product where a kernel of this repository runs it
        return ops.gemm_gelu(h, self.w_up, ctx.buffer("ffn.act", (T, self.intermediate), ctx.dtype), self.activation, scratch=ctx.scratch,
                             product=ctx.buffer("ffn.up", (T, self.intermediate), ctx.dtype))

    def output(self, h, ctx):
        """The feed-forward's result, float [T, hidden], without the residual sum."""
        if self.bias:
            y = ops.gemm(self._activations(h, ctx), self.w_down, ctx.buffer("ffn.out", (h.shape[0], self.hidden), torch.float32), scratch=ctx.scratch)
            return ops.Biased(y, self.b_down)          # (the kernel that adds the result adds the bias)
        return ctx.product_for_norm(self._activations(h, ctx), self.w_down, "ffn.out")

    def forward(self, h, residual, ctx, norm=None):
        if self.bias:
            from .block import add_sublayer
            return add_sublayer(residual, self.output(h, ctx), None, 1.0)
        return ctx.add_product(self._activations(h, ctx), self.w_down, residual)


class RoutedExperts(FeedForward):
    """A mixture of `experts` small feed-forwards of which every row uses `top`: router logits W_r h + b in float, the
    `top` largest chosen (the lowest index wins a tie), their weights the softmax over the chosen logits only; an
    expert is W_down relu(W_up h)^2 without biases, and the result is the weighted sum of the chosen experts'.

    The rows of a step are ordered by expert on the device (ops.experts_route) and each expert's matrix meets only its
    own rows, in tiles (ops.experts_gemm); the down products are left as `top` rows a step row for the kernel that
    adds the sublayer's result (ops.WeightedRows).  `ride(weight)`: further rows for the router's product, whose
    float results are then `rider`.  `names`: (router, expert prefix, up, down), the tensors' names under `name`;
    expert j's matrices are `<name>.<prefix>j.<up|down>`."""

    def __init__(self, name, hidden, intermediate, experts, top, names=("router", "e", "up", "down")):
        if not 0 < top <= min(experts, 16):
            raise ValueError(f"{top} of {experts} experts: between 1 and min(experts, 16)")
        self.name, self.hidden, self.intermediate, self.experts, self.top = name, hidden, intermediate, int(experts), int(top)
        self.names = tuple(names)
        self.rider, self.rider_rows = None, 0

    def _expert(self, j, which):
        return f"{self.name}.{self.names[1]}{j}.{self.names[2 + which]}"

    def tensor_specs(self):
        H, I, router = self.hidden, self.intermediate, f"{self.name}.{self.names[0]}"
        specs = [TensorSpec(router, (self.experts, H)), TensorSpec(router + ".b", (self.experts,))]
        for j in range(self.experts):
            specs += [TensorSpec(self._expert(j, 0), (I, H)), TensorSpec(self._expert(j, 1), (H, I))]
        return specs

    def _join(self, extra=None):
        parts = [self.w_router] + ([] if extra is None else [extra])
        rows = sum(p.shape[0] for p in parts)
        if rows % 8:
            parts.append(torch.zeros(8 - rows % 8, self.hidden, dtype=parts[0].dtype, device=parts[0].device))
        self.w_in = torch.cat(parts, dim=0).contiguous()

    def bind(self, tensors, dtype):
        router = f"{self.name}.{self.names[0]}"
        self.w_router = matrix_operand(tensors[router], dtype)
        self.router_bias = tensors[router + ".b"].to(torch.float32).contiguous()
        self._join()
        self.w_up = torch.stack([matrix_operand(tensors[self._expert(j, 0)], dtype) for j in range(self.experts)]).contiguous()
        self.w_down = torch.stack([matrix_operand(tensors[self._expert(j, 1)], dtype) for j in range(self.experts)]).contiguous()

    def ride(self, weight):
        self.rider_rows = weight.shape[0]
        self._join(weight)

    def output(self, h, ctx):
        """The feed-forward's result as ops.WeightedRows (float [T * top, hidden] and the weights [T, top])."""
        T, E, top = h.shape[0], self.experts, self.top
        logits = ops.gemm(h, self.w_in, ctx.buffer("moe.logits", (T, self.w_in.shape[0]), torch.float32), scratch=ctx.scratch)
        self.rider = logits[:, E:E + self.rider_rows] if self.rider_rows else None
        chosen, weights = ctx.buffer("moe.chosen", (T, top), torch.int32), ctx.buffer("moe.weights", (T, top), torch.float32)
        down = ctx.buffer("moe.down", (T * top, self.hidden), torch.float32)
        if ops.experts_rows_ok(h, self.w_up, T * top) and ops.experts_rows_ok(h, self.w_down, T * top):
            # few rows (decoding): every (row, choice) pair streams its expert's two matrices
            ops.experts_route(logits[:, :E], self.router_bias, top, chosen, weights)
            up = ops.experts_rows(h, self.w_up, chosen, ctx.buffer("moe.up", (T * top, self.intermediate), ctx.dtype), top=top, act=True)
            ops.experts_rows(up, self.w_down, chosen, down)
            return ops.WeightedRows(down, weights, top)
        tiles = ops.expert_tiles(T, top, E)
        places, tile_expert = ctx.buffer("moe.places", (tiles * ops.EXPERT_TILE,), torch.int32), ctx.buffer("moe.tiles", (tiles,), torch.int32)
        ops.experts_route(logits[:, :E], self.router_bias, top, chosen, weights, places, tile_expert)
        up = ops.experts_gemm(h, self.w_up, places, tile_expert, ctx.buffer("moe.up", (tiles * ops.EXPERT_TILE, self.intermediate), ctx.dtype),
                              top=top, act=True)
        ops.experts_gemm(up, self.w_down, places, tile_expert, down, scatter=True)
        return ops.WeightedRows(down, weights, top)

    def forward(self, h, residual, ctx, norm=None):
        return _add_weighted(residual, self.output(h, ctx))


class ScoredExperts(FeedForward):
    """A mixture of experts routed by scores: s = softmax(W_r h) over all router outputs, in float; the choice goes by
    s + `correction` (a tensor; the weights use s without it), optionally held to the best `groups[1]` of `groups[0]`
    equal groups of neighbouring outputs (a group's score is its largest choice score; the others count as minus
    infinity); the `top` largest are chosen and weigh s itself, not normed again.  The first `experts` outputs are gated
    feed-forwards W_down (silu(W_gate h) * (W_up h)) without biases; the last `identity` outputs have no tensors: their
    result is the input itself.  `shared`: a feed-forward part (with `output`) that every row goes through, added.

    The rows of a step are ordered by expert on the device and each expert's matrices meet only their own rows
    (ops.experts_gemm; steps of few rows stream each pair's matrices, ops.experts_rows); gate and up are one product over
    [gate; up] a expert, followed by the activation.  `names`: (router, correction, expert prefix, gate, up, down)."""

    def __init__(self, name, hidden, intermediate, experts, top, identity=0, groups=None, shared=None, correction=True,
                 names=("router", "correction", "e", "gate", "up", "down")):
        outputs = experts + identity
        if not 0 < top <= min(outputs, 16) or experts <= 0 or identity < 0:
            raise ValueError(f"{top} of {experts} + {identity} router outputs: between 1 and min(outputs, 16)")
        if groups is not None:
            count, keep = groups
            if count <= 0 or count > 64 or outputs % count or not 0 < keep <= count or keep * (outputs // count) < top:
                raise ValueError(f"{outputs} router outputs in {count} groups of which {keep} are kept, for {top} choices")
        if shared is not None and not hasattr(shared, "output"):
            raise ValueError("the shared feed-forward must give its result without the residual sum (output)")
        self.name, self.hidden, self.intermediate = name, hidden, intermediate
        self.experts, self.identity, self.outputs, self.top = int(experts), int(identity), outputs, int(top)
        self.groups, self.shared, self.has_correction, self.names = groups, shared, bool(correction), tuple(names)

    def _expert(self, j, which):
        return f"{self.name}.{self.names[2]}{j}.{self.names[3 + which]}"

    def tensor_specs(self):
        H, I = self.hidden, self.intermediate
        specs = [TensorSpec(f"{self.name}.{self.names[0]}", (self.outputs, H))]
        if self.has_correction:
            specs.append(TensorSpec(f"{self.name}.{self.names[1]}", (self.outputs,)))
        for j in range(self.experts):
            specs += [TensorSpec(self._expert(j, 0), (I, H)), TensorSpec(self._expert(j, 1), (I, H)), TensorSpec(self._expert(j, 2), (H, I))]
        return specs + ([] if self.shared is None else self.shared.tensor_specs())

    def bind(self, tensors, dtype):
        router = matrix_operand(tensors[f"{self.name}.{self.names[0]}"], dtype)
        if router.shape[0] % 8:      # rows of the router's product are a multiple of 8: zero rows at the end
            router = torch.cat([router, torch.zeros(8 - router.shape[0] % 8, self.hidden, dtype=router.dtype, device=router.device)])
        self.w_router = router.contiguous()
        self.correction = tensors[f"{self.name}.{self.names[1]}"].to(torch.float32).contiguous() if self.has_correction else None
        self.w_gate_up = torch.stack([torch.cat([matrix_operand(tensors[self._expert(j, 0)], dtype), matrix_operand(tensors[self._expert(j, 1)], dtype)])
                                      for j in range(self.experts)]).contiguous()
        self.w_down = torch.stack([matrix_operand(tensors[self._expert(j, 2)], dtype) for j in range(self.experts)]).contiguous()
        if self.shared is not None:
            self.shared.bind(tensors, dtype)

    def prepare(self, device, dtype):
        if self.shared is not None:
            self.shared.prepare(device, dtype)

    def output(self, h, ctx):
        """The feed-forward's result, float [T, hidden], without the residual sum."""
        T, E, top, I = h.shape[0], self.experts, self.top, self.intermediate
        logits = ops.gemm(h, self.w_router, ctx.buffer("moe.logits", (T, self.w_router.shape[0]), torch.float32), scratch=ctx.scratch)
        chosen, weights = ctx.buffer("moe.chosen", (T, top), torch.int32), ctx.buffer("moe.weights", (T, top), torch.float32)
        down = ctx.buffer("moe.down", (T * top, self.hidden), torch.float32)
        if ops.experts_rows_ok(h, self.w_gate_up, T * top) and ops.experts_rows_ok(h, self.w_down, T * top):
            # few rows (decoding): every (row, choice) pair streams its expert's matrices
            ops.experts_route_scored(logits[:, :self.outputs], self.correction, top, chosen, weights, E, self.groups)
            gate_up = ops.experts_rows(h, self.w_gate_up, chosen, ctx.buffer("moe.gate_up", (T * top, 2 * I), ctx.dtype), top=top)
            act = ops.swiglu(gate_up, ctx.buffer("moe.act", (T * top, I), ctx.dtype))
            ops.experts_rows(act, self.w_down, chosen, down)
        else:
            tiles = ops.expert_tiles(T, top, E)
            places, tile_expert = ctx.buffer("moe.places", (tiles * ops.EXPERT_TILE,), torch.int32), ctx.buffer("moe.tiles", (tiles,), torch.int32)
            ops.experts_route_scored(logits[:, :self.outputs], self.correction, top, chosen, weights, E, self.groups, places, tile_expert)
            gate_up = ops.experts_gemm(h, self.w_gate_up, places, tile_expert, ctx.buffer("moe.gate_up", (tiles * ops.EXPERT_TILE, 2 * I), ctx.dtype), top=top)
            act = ops.swiglu(gate_up, ctx.buffer("moe.act", (tiles * ops.EXPERT_TILE, I), ctx.dtype))
            ops.experts_gemm(act, self.w_down, places, tile_expert, down, scatter=True)
        also = None if self.shared is None else self.shared.output(h, ctx, tag="moe.shared")
        return ops.experts_combine(down, weights, chosen, h, ctx.buffer("moe.y", (T, self.hidden), torch.float32), E, shared=also)

    def forward(self, h, residual, ctx, norm=None):
        from .block import add_sublayer
        return add_sublayer(residual, self.output(h, ctx), None, 1.0)


def _add_weighted(residual, y):
    """residual += sum_k weights[:, k] * rows[k]: for an arrangement that adds a feed-forward's result itself (torch's own
    kernels: no arrangement of this package takes this way)."""
    rows, dim = residual.shape
    residual += (y.rows.view(rows, y.top, dim) * y.weights.unsqueeze(-1)).sum(dim=1)
    return residual


register_part("ffn", "routed_experts", RoutedExperts)
register_part("ffn", "scored_experts", ScoredExperts)
register_part("ffn", "gated_mlp", GatedMLP)
register_part("ffn", "dense_mlp", DenseMLP)
register_part("ffn", "clamped_glu", ClampedGLU)
