"""Token embedding and output head.

x0[r] = E[token_r] with no scaling (reference: runtime/model.py:105), or with PairHashEmbedding
E[token_r] * scale + B[hash(token before, token_r)]; logits =
h . W^T with W the head's own matrix or, when tied, the embedding matrix
(reference: runtime/checkpoint.py:38-39).  Logits are always float.
"""
import torch

from ..kernels import ops
from .base import Part, TensorSpec, matrix_operand


class TokenEmbedding(Part):
    def __init__(self, name, vocab, hidden, tensor=None):
        """`tensor`: the table's full name where it is not `<name>.weight`."""
        self.name, self.vocab, self.hidden = name, vocab, hidden
        self.tensor = tensor if tensor is not None else name + ".weight"
        self.weight = None

    def tensor_specs(self):
        return [TensorSpec(self.tensor, (self.vocab, self.hidden))]

    def bind(self, tensors, dtype):
        self.weight = matrix_operand(tensors[self.tensor], dtype)

    def forward(self, ctx):
        out = ctx.buffer("residual", (ctx.tokens.shape[0], self.hidden), torch.float32)
        return ops.embedding(ctx.tokens, self.weight, out)


STATE_SITE = "embedding"      # the key of the embedding's state among the cache manager's state sites


class PairHashEmbedding(TokenEmbedding):
    """x[r] = E[token_r] * scale + B[(token before * mul_prev + token_r * mul_cur) mod buckets], B a second table of
    `buckets` + 1 rows whose last row serves a sequence's first token (`buckets` None: no second table, only the scale).
    The token before a portion's first one is the last token of the request's step before: part of the request's state,
    one int32 in its state slot, written on the device (so a token that was picked on the device and has not reached
    the host yet serves as well).  The rows are also left in the activations' type for a layer whose sublayers read
    the stream itself (parts.base.CAST)."""

    def __init__(self, name, vocab, hidden, scale=1.0, buckets=None, mul_prev=0, mul_cur=0, tensor=None, pairs_tensor=None):
        super().__init__(name, vocab, hidden, tensor=tensor)
        if buckets is not None and (buckets <= 0 or mul_prev < 0 or mul_cur < 0):
            raise ValueError("a table of token pairs needs a positive number of buckets and multipliers >= 0")
        self.scale, self.buckets, self.mul_prev, self.mul_cur = float(scale), buckets, int(mul_prev), int(mul_cur)
        self.pairs_tensor = pairs_tensor if pairs_tensor is not None else name + ".pairs"
        self.pairs = None

    def tensor_specs(self):
        specs = super().tensor_specs()
        if self.buckets is not None:
            specs.append(TensorSpec(self.pairs_tensor, (self.buckets + 1, self.hidden)))
        return specs

    def bind(self, tensors, dtype):
        super().bind(tensors, dtype)
        if self.buckets is not None:
            self.pairs = matrix_operand(tensors[self.pairs_tensor], dtype)

    def state_need(self):
        from ..cache.pages import StateNeed
        return StateNeed((1,), "int32") if self.buckets is not None else None

    def forward(self, ctx):
        from .base import CAST
        T = ctx.tokens.shape[0]
        out = ctx.buffer("residual", (T, self.hidden), torch.float32)
        cast = ctx.buffer("residual.cast", (T, self.hidden), ctx.dtype) if ctx.dtype != torch.float32 else None
        kept = ctx.cache.state_storage[STATE_SITE].view(-1) if self.buckets is not None else None
        ops.embedding_pairs(ctx.tokens, ctx.positions, ctx.seg_of_row, ctx.seg_start, ctx.state_slots, self.weight, out,
                            scale=self.scale, pairs=self.pairs, last_token=kept, buckets=self.buckets or 0,
                            mul_prev=self.mul_prev, mul_cur=self.mul_cur, cast=cast, single_rows=ctx.decode_only)
        ctx.leave_normed(CAST, out, out if cast is None else cast)
        return out


class LMHead(Part):
    def __init__(self, name, vocab, hidden, tied_to=None, tensor=None):
        self.name, self.vocab, self.hidden, self.tied_to = name, vocab, hidden, tied_to
        self.tensor = tensor if tensor is not None else name + ".weight"
        self.weight = None

    def tensor_specs(self):
        return [] if self.tied_to is not None else [TensorSpec(self.tensor, (self.vocab, self.hidden))]

    def bind(self, tensors, dtype):
        self.weight = self.tied_to.weight if self.tied_to is not None else matrix_operand(tensors[self.tensor], dtype)

    def fuses_norm(self, norm, residual, rows):
        return getattr(norm, "fusable_as", None) == "rms" and ops.fused_norm_ok(residual, self.weight, rows.shape[0])

    def forward(self, h, ctx, norm=None, residual=None):
        """Logits of the normed rows h; or, with `norm`, of RMSNorm(residual[ctx.logit_rows]) in one kernel."""
        n = ctx.logit_rows.shape[0] if norm is not None else h.shape[0]
        logits = ctx.buffer("logits", (n, self.vocab), torch.float32)
        if norm is not None:
            return ops.gemm_normed(residual, (norm.weight, norm.eps, ctx.logit_rows), self.weight, logits)
        return ops.gemm(h, self.weight, logits, after_norm=True, scratch=ctx.scratch)
