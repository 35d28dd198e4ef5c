"""The two ends of a model: the embedding table and the output head.

Embedding without multiplier (crates/backends/backend_common/src/generic_model.rs:104-111; `scale` is a
parameter for families that have one);
the head is the final norm of the wanted rows only and a product with
lm_head, or with the embedding table when the two are tied
(generic_model.rs:266-283; loader_common.rs:1851-1872).
"""
import torch

from ..kernels import ops
from ..weights import TensorNeed
from .base import Part
from .linear import Linear
from .registry import build, register


@register("embedding", "table")
class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, vocab_size, hidden_size, weight, shared=None, norm=None, scale=None):
        """norm: a PartSpec of a norm that the gathered rows pass before they are the residual stream
        (it must offer forward_in_place), or None. scale: the gathered rows times this constant (a head
        tied to the table uses the table as it is)."""
        self.scale = None if scale is None or float(scale) == 1.0 else float(scale)
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.weight_name = weight
        self.table = None
        self.norm = build("norm", norm) if norm is not None else None

    def tensor_needs(self):
        needs = {self.weight_name: TensorNeed((self.vocab_size, self.hidden_size), "table")}
        if self.norm is not None:
            needs.update(self.norm.tensor_needs())
        return needs

    def load(self, tensors, rt, shared_with_head=False):
        """shared_with_head: the table is also the head's matrix; it is then kept in the order the
        head's kernels want, and rows are gathered from that order."""
        self.linear = Linear(rt.weight(tensors[self.weight_name]), pack=shared_with_head, scratch=rt.scratch)
        self.table = self.linear.weight
        if self.norm is not None:
            self.norm.load(tensors, rt)

    def forward(self, ctx, token_ids):
        x = ctx.rt.buffer("residual", (token_ids.shape[0], self.hidden_size), torch.float32)
        ops.embed(token_ids, self.table, x, packed=self.linear.packed)
        if self.scale is not None:
            ops.scale(x, self.scale)
        if self.norm is not None:
            self.norm.forward_in_place(ctx, x)
        return x


@register("head", "linear")
class OutputHead(Part):
    graph_safe = True

    def __init__(self, vocab_size, hidden_size, weight, tied_to_embedding, norm, shared=None, logit_scale=None):
        """weight: the head's tensor name; tied_to_embedding: use the embedding table instead;
        logit_scale: the logits are the product times this constant (None: as they are)."""
        self.logit_scale = None if logit_scale is None or float(logit_scale) == 1.0 else float(logit_scale)
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.weight_name = weight
        self.tied = bool(tied_to_embedding)
        self.norm = norm                  # a built norm part
        self.proj = None

    def tensor_needs(self):
        needs = dict(self.norm.tensor_needs())
        if not self.tied:
            needs[self.weight_name] = TensorNeed((self.vocab_size, self.hidden_size))
        return needs

    def load(self, tensors, rt, embedding=None):
        self.norm.load(tensors, rt)
        if self.tied:
            self.proj = embedding.linear
        else:
            self.proj = Linear(rt.weight(tensors[self.weight_name]), scratch=rt.scratch)

    def forward(self, ctx, x, rows):
        y = self.norm.forward(ctx, x, rows, name="head_normed")
        shape = (rows.shape[0], self.vocab_size)
        logits = ctx.logits_out
        if logits is None:
            logits = torch.empty(shape, dtype=torch.float32, device=x.device)
        elif tuple(logits.shape) != shape or logits.dtype != torch.float32 or not logits.is_contiguous():
            raise ValueError(f"the caller's logits are {tuple(logits.shape)} {logits.dtype}, the step's {shape} float32")
        self.proj.forward(y, logits)
        if self.logit_scale is not None:
            ops.scale(logits, self.logit_scale)
        return logits
