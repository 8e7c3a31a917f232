"""The two ends of a model: the embedding table and the output head.

Embedding without multiplier (crates/backends/backend_common/src/generic_model.rs:104-111);
the head is the final norm of the wanted rows only and a product with
lm_head, or with the embedding table when the two are tied
(generic_model.rs:266-283; loader_common.rs:1851-1872).
"""
import torch

from ..kernels import ops
from ..weights import TensorNeed
from .base import Part
from .linear import Linear
from .registry import register


@register("embedding", "table")
class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, vocab_size, hidden_size, weight, shared=None):
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.weight_name = weight
        self.table = None

    def tensor_needs(self):
        return {self.weight_name: TensorNeed((self.vocab_size, self.hidden_size), "table")}

    def load(self, tensors, rt, shared_with_head=False):
        """shared_with_head: the table is also the head's matrix; it is then kept in the order the
        head's kernels want, and rows are gathered from that order."""
        self.linear = Linear(rt.weight(tensors[self.weight_name]), pack=shared_with_head, scratch=rt.scratch)
        self.table = self.linear.weight

    def forward(self, ctx, token_ids):
        x = ctx.rt.buffer("residual", (token_ids.shape[0], self.hidden_size), torch.float32)
        ops.embed(token_ids, self.table, x, packed=self.linear.packed)
        return x


@register("head", "linear")
class OutputHead(Part):
    graph_safe = True

    def __init__(self, vocab_size, hidden_size, weight, tied_to_embedding, norm, shared=None):
        """weight: the head's tensor name; tied_to_embedding: use the embedding table instead."""
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
        return logits
