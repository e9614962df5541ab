"""Arrangement of parts in a layer.  PreNormBlock is the Llama arrangement
(reference: runtime/model.py:106-119): x = x + mixer(norm1(x)); x = x + ffn(norm2(x)),
the residual stream x kept in float.  SandwichBlock norms each sublayer's result as well
and scales it: x = x + m norm1b(mixer(norm1(x))); x = x + m norm2b(ffn(norm2(x))); without the norms in front
(`reads_stream`) its sublayers read x itself: x = x + m norm1b(mixer(x)).  PostNormBlock norms after the
sum, and its sublayers read the stream itself: x = norm1(a x + g1 mixer(x)); x = norm2(a x + g2 ffn(x)), with
optional gates g = sigmoid(W x + b) element by element."""
import torch

from ..kernels import ops
from .base import CAST, Part, TensorSpec, matrix_operand, register_part


class PreNormBlock(Part):
    def __init__(self, mixer_norm, mixer, ffn_norm=None, ffn=None):
        """`ffn` None (and no `ffn_norm`): a layer without a feed-forward."""
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a feed-forward comes with the norm before it, or not at all")
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def parts(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def tensor_specs(self):
        return [s for p in self.parts() for s in p.tensor_specs()]

    def bind(self, tensors, dtype):
        for p in self.parts():
            p.bind(tensors, dtype)

    def prepare(self, device, dtype):
        for p in self.parts():
            p.prepare(device, dtype)

    # What the block keeps between steps, asked of the block (not of a part inside it): one mixer here, so one need
    # of each kind; an arrangement with more parts that keep something answers for all of them.
    def cache_need(self):
        return self.mixer.cache_need()

    def cache_read(self):
        return self.mixer.cache_read() if hasattr(self.mixer, "cache_read") else None

    def state_need(self):
        return self.mixer.state_need()

    def kernel_units(self, dtype):
        """Shared objects beside the core that the parts need (names of kernels.library.units())."""
        return [u for p in self.parts() if hasattr(p, "kernel_units") for u in p.kernel_units(dtype)]

    def step_arrays(self):
        """Step arrays that the parts want every step's metadata to carry from the start (engine.context.StepArray)."""
        return [a for p in self.parts() if hasattr(p, "step_arrays") for a in p.step_arrays()]

    def first_norm(self):
        """The norm that reads the residual stream first: the block before may leave its last product to it."""
        return self.mixer_norm

    def forward(self, residual, ctx, site):
        # ctx.next_norm names the norm that reads the residual stream after the part that runs: a part's last
        # product may be left to it (ctx.add_product); on entry it is the norm after this block
        after = ctx.next_norm
        ffn_fuses = self.ffn is not None and self.ffn.fuses_norm(self.ffn_norm, residual, ctx)
        ctx.next_norm = after if self.ffn is None else None if ffn_fuses else self.ffn_norm
        if self.mixer.fuses_norm(self.mixer_norm, residual, ctx):
            ctx.settle(residual)
            residual = self.mixer.forward(None, residual, ctx, site, norm=self.mixer_norm)
        else:
            residual = self.mixer.forward(self.mixer_norm.forward(residual, ctx), residual, ctx, site)
        if self.ffn is None:
            return residual
        if ffn_fuses:
            ctx.settle(residual)
            ctx.next_norm = after
            return self.ffn.forward(None, residual, ctx, norm=self.ffn_norm)
        h = self.ffn_norm.forward(residual, ctx)
        ctx.settle(residual)       # (a norm that adds no partial sums)
        ctx.next_norm = after
        return self.ffn.forward(h, residual, ctx)


class NormedMean:
    """What a mixer made of two mixers side by side hands to the arrangement around it: half the sum of two results,
    each RMS-normed over the width with a weight of its own (float [T, H] each, or the partial sums of a cut product).  The arrangement's kernel that adds
    a sublayer's result to the residual stream makes the mean on the way (ops.post_norm_add)."""

    def __init__(self, first, first_weight, second, second_weight, eps):
        self.first, self.first_weight, self.second, self.second_weight, self.eps = first, first_weight, second, second_weight, eps


class ScaledSum:
    """What a mixer made of two mixers side by side may hand to the arrangement around it instead: a first + b second,
    two float results [T, H] and two numbers.  The kernel that adds the sublayer's result makes the sum on the way."""

    def __init__(self, first, first_scale, second, second_scale):
        self.first, self.first_scale, self.second, self.second_scale = first, float(first_scale), second, float(second_scale)


def add_sublayer(residual, result, norm, mult, eps=None, following=None):
    """residual += mult * norm(result) (norm None: mult * result); `result` float rows, a NormedMean or a ScaledSum.
    `following` = (norm part, out): the RMS norm that reads the residual stream next is made by the same kernel; with
    CAST as the norm, `out` receives the new rows themselves in its type."""
    weight = None if norm is None else norm.weight
    eps = norm.eps if norm is not None else eps
    then = None
    if following is not None:
        then = (None, 0.0, following[1]) if following[0] is CAST else (following[0].weight, following[0].eps, following[1])
    if isinstance(result, ScaledSum):
        return ops.post_norm_add(residual, result.first, weight, 0.0 if eps is None else eps, mult,
                                 second=(result.second, result.first_scale, result.second_scale), following=then)
    if isinstance(result, NormedMean):
        if eps is not None and eps != result.eps:
            raise ValueError("the norms inside a mean of two results and the norm around it must share their eps (one kernel)")
        return ops.post_norm_add(residual, result.first, weight, result.eps, mult,
                                 second=(result.second, result.first_weight, result.second_weight), following=then)
    return ops.post_norm_add(residual, result, weight, 0.0 if eps is None else eps, mult, following=then)


class SandwichBlock(Part):
    """A norm before and after each sublayer, the normed result times `mult` added to the float residual stream.
    Its mixer and feed-forward give their result without the residual sum (`output`); `ffn` None: a layer without
    a feed-forward.  The norms after the sublayers are RMS norms (`weight`, `eps`); the sum, the norm and the scale
    are one kernel.  `reads_stream`: there are no norms in front (`mixer_norm`, `ffn_norm` None) and the sublayers read
    the residual stream itself, in the activations' type (that copy is made by the kernel that wrote the stream last)."""

    def __init__(self, mixer_norm, mixer, mixer_post, ffn_norm=None, ffn=None, ffn_post=None, mult=1.0, reads_stream=False):
        self.reads_stream = bool(reads_stream)
        if self.reads_stream:
            if mixer_norm is not None or ffn_norm is not None or (ffn is None) != (ffn_post is None):
                raise ValueError("sublayers that read the stream itself have no norm in front; a feed-forward comes with the norm after it")
        elif (ffn is None) != (ffn_norm is None) or (ffn is None) != (ffn_post is None):
            raise ValueError("a feed-forward comes with the norms before and after it, or not at all")
        for post in (mixer_post, ffn_post):
            if post is not None and getattr(post, "fusable_as", None) != "rms":
                raise ValueError("the norm after a sublayer must be an RMS norm (weight, eps)")
        if not hasattr(mixer, "output") or (ffn is not None and not hasattr(ffn, "output")):
            raise ValueError("the sublayers of this arrangement must give their result without the residual sum (output)")
        self.mixer_norm, self.mixer, self.mixer_post = mixer_norm, mixer, mixer_post
        self.ffn_norm, self.ffn, self.ffn_post = ffn_norm, ffn, ffn_post
        self.mult = float(mult)

    def parts(self):
        return [p for p in (self.mixer_norm, self.mixer, self.mixer_post, self.ffn_norm, self.ffn, self.ffn_post) if p is not None]

    def tensor_specs(self):
        return [s for p in self.parts() for s in p.tensor_specs()]

    def bind(self, tensors, dtype):
        for p in self.parts():
            p.bind(tensors, dtype)

    def prepare(self, device, dtype):
        for p in self.parts():
            p.prepare(device, dtype)

    def cache_need(self):
        return self.mixer.cache_need()

    def cache_read(self):
        return self.mixer.cache_read()

    def state_need(self):
        return self.mixer.state_need()

    def kernel_units(self, dtype):
        return [u for p in self.parts() if hasattr(p, "kernel_units") for u in p.kernel_units(dtype)]

    def step_arrays(self):
        return [a for p in self.parts() if hasattr(p, "step_arrays") for a in p.step_arrays()]

    def first_norm(self):
        return CAST if self.reads_stream else self.mixer_norm

    @staticmethod
    def _plain_rms(norm):
        return norm is not None and getattr(norm, "fusable_as", None) == "rms"

    def _forward_stream(self, residual, ctx, site):
        """The layer whose sublayers read the stream itself: h is x in the activations' type (x itself in float32)."""
        after = ctx.next_norm
        ctx.next_norm = None
        ctx.settle(residual)
        narrow = ctx.dtype != torch.float32
        T, H = residual.shape

        def following(reader, tag):
            # the copy of the new rows for whoever reads the stream next: this block's feed-forward, or the next block
            if reader is CAST:
                return (CAST, ctx.buffer(tag, (T, H), ctx.dtype)) if narrow else None
            return (reader, ctx.buffer(tag, (T, H), ctx.dtype)) if self._plain_rms(reader) else None

        def leave(then):
            if then is not None:
                ctx.leave_normed(after, residual, then[1])
            elif after is CAST:
                ctx.leave_normed(CAST, residual, residual)

        h = ctx.take_normed(CAST, residual)
        if h is None:
            h = ops.f32_to_bf16(residual, ctx.buffer("stream.cast", (T, H), ctx.dtype)) if narrow else residual
        last = self.ffn is None
        then = following(after if last else CAST, "norm.ahead" if last else "norm.inside")
        add_sublayer(residual, self.mixer.output(h, ctx, site), self.mixer_post, self.mult, following=then)
        if last:
            leave(then)
            return residual
        h = then[1] if then is not None else residual
        then = following(after, "norm.ahead")
        add_sublayer(residual, self.ffn.output(h, ctx), self.ffn_post, self.mult, following=then)
        leave(then)
        return residual

    def forward(self, residual, ctx, site):
        if self.reads_stream:
            return self._forward_stream(residual, ctx, site)
        # the kernel that adds a sublayer's result also makes the norm that reads the residual stream next, where that
        # is an RMS norm over all rows: this block's second norm, or the following block's first (ctx.next_norm), which
        # finds its rows waiting in ctx.normed
        after = ctx.next_norm
        ctx.next_norm = None          # (no product of this block is left to a later norm)
        h = ctx.take_normed(self.mixer_norm, residual)
        if h is None:
            h = self.mixer_norm.forward(residual, ctx)
            ctx.settle(residual)
        T = residual.shape[0]
        last = self.ffn is None

        def following(norm, tag):
            return (norm, ctx.buffer(tag, (T, residual.shape[1]), ctx.dtype)) if self._plain_rms(norm) else None

        then = following(after if last else self.ffn_norm, "norm.ahead" if last else "norm.inside")
        add_sublayer(residual, self.mixer.output(h, ctx, site), self.mixer_post, self.mult, following=then)
        if last:
            if then is not None:
                ctx.leave_normed(after, residual, then[1])
            return residual
        h = then[1] if then is not None else self.ffn_norm.forward(residual, ctx)
        then = following(after, "norm.ahead")
        add_sublayer(residual, self.ffn.output(h, ctx), self.ffn_post, self.mult, following=then)
        if then is not None:
            ctx.leave_normed(after, residual, then[1])
        return residual


class PostNormBlock(Part):
    """The norm after the sum: x <- norm1(alpha x + mixer(x)), then x <- norm2(alpha x + ffn(x)); the sublayers read x
    itself (in the activations' type).  With `gated` each sublayer's result is first multiplied element by element by
    sigmoid(W x + b), W = `<name>.<gate names[i]>` [H, H] and b = `<...>.b`.  The sum, the gate, the norm and the copy of
    the new rows in the activations' type are one kernel (ops.gate_post_norm); a feed-forward that gives its result as
    weighted rows (ops.WeightedRows: routed experts) has them summed on the way.  The gate's product rides in the
    sublayer's own first product where the sublayer offers that (`ride(weight)`, then `rider` after `output`: a float view
    [T, H]); otherwise it is a product of its own.  `ffn` None: a layer without a feed-forward (no second norm)."""

    def __init__(self, name, hidden, mixer_norm, mixer, ffn_norm=None, ffn=None, alpha=1.0, gated=False, gate_names=("rg1", "rg2")):
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a feed-forward comes with the norm after it, or not at all")
        for norm in (mixer_norm, ffn_norm):
            if norm is not None and getattr(norm, "fusable_as", None) != "rms":
                raise ValueError("the norm after a sum must be an RMS norm (weight, eps)")
        if not hasattr(mixer, "output") or (ffn is not None and not hasattr(ffn, "output")):
            raise ValueError("the sublayers of this arrangement must give their result without the residual sum (output)")
        self.name, self.hidden, self.alpha, self.gated = name, hidden, float(alpha), bool(gated)
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn
        self.gate_names = tuple(gate_names)
        self.gates = {}       # sublayer index -> (weight or None if it rides, bias float)

    def parts(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def _gated(self):
        return [(i, sub) for i, sub in enumerate((self.mixer, self.ffn)) if self.gated and sub is not None]

    def tensor_specs(self):
        specs = [s for p in self.parts() for s in p.tensor_specs()]
        for i, _ in self._gated():
            gate = f"{self.name}.{self.gate_names[i]}"
            specs += [TensorSpec(gate, (self.hidden, self.hidden)), TensorSpec(gate + ".b", (self.hidden,))]
        return specs

    def bind(self, tensors, dtype):
        for p in self.parts():
            p.bind(tensors, dtype)
        for i, sub in self._gated():
            gate = f"{self.name}.{self.gate_names[i]}"
            weight = matrix_operand(tensors[gate], dtype)
            bias = tensors[gate + ".b"].to(torch.float32).contiguous()
            if hasattr(sub, "ride"):
                sub.ride(weight)          # the sublayer's first product makes the gate's too
                weight = None
            self.gates[i] = (weight, bias)

    def prepare(self, device, dtype):
        for p in self.parts():
            p.prepare(device, dtype)

    def cache_need(self):
        return self.mixer.cache_need()

    def cache_read(self):
        return self.mixer.cache_read() if hasattr(self.mixer, "cache_read") else None

    def state_need(self):
        return self.mixer.state_need()

    def kernel_units(self, dtype):
        return [u for p in self.parts() if hasattr(p, "kernel_units") for u in p.kernel_units(dtype)]

    def step_arrays(self):
        return [a for p in self.parts() if hasattr(p, "step_arrays") for a in p.step_arrays()]

    def _sum_and_norm(self, x, h, result, which, sub, norm, ctx):
        """x <- norm(alpha x + gate * result) in place; returns the new rows in the activations' type."""
        if isinstance(result, ops.Biased):
            result = ops.bias_add(result.rows, result.bias)
        if isinstance(result, ops.Partials):
            raise TypeError("a sublayer of this arrangement gives finished rows (or weighted rows), no partial sums")
        gate = bias = None
        if which in self.gates:
            weight, bias = self.gates[which]
            gate = sub.rider if weight is None else ops.gemm(h, weight, ctx.buffer(f"post.gate{which}", x.shape, torch.float32), scratch=ctx.scratch)
        cast = None if ctx.dtype == torch.float32 else ctx.buffer(f"post.cast{which}", x.shape, ctx.dtype)
        ops.gate_post_norm(x, result, norm.weight, norm.eps, self.alpha, gate=gate, gate_bias=bias, cast=cast)
        return x if cast is None else cast

    def forward(self, residual, ctx, site):
        ctx.next_norm = None          # (no product of this block is left to a later norm)
        ctx.settle(residual)
        h = ctx.take_normed(CAST, residual)
        if h is None:
            h = residual if ctx.dtype == torch.float32 else ops.f32_to_bf16(residual, ctx.buffer("post.cast", residual.shape, ctx.dtype))
        h = self._sum_and_norm(residual, h, self.mixer.output(h, ctx, site), 0, self.mixer, self.mixer_norm, ctx)
        if self.ffn is not None:
            h = self._sum_and_norm(residual, h, self.ffn.output(h, ctx), 1, self.ffn, self.ffn_norm, ctx)
        ctx.leave_normed(CAST, residual, h)
        return residual


register_part("block", "postnorm", PostNormBlock)
register_part("block", "prenorm", PreNormBlock)
register_part("block", "sandwich", SandwichBlock)
