"""What every part has in common, and the context a step hands to the parts.

Interfaces (x is the float32 residual stream [T, hidden], y a normed copy of it
in the compute dtype; T counts the tokens of the step, packed over sequences):

  norm          forward(ctx, x, rows=None) -> y            (rows: gather these rows only)
  mixer         forward(ctx, y, x)                         adds its output to x
  feed_forward  forward(ctx, y, x)                         adds its output to x
  position      rotation() -> (cos, sin, rotary_dims) or None, tables on the GPU
  block         forward(ctx, x)                            runs one layer on x in place
  embedding     forward(ctx, token_ids) -> x
  head          forward(ctx, x, rows) -> float32 logits [len(rows), vocab]

Every part also has
  tensor_needs() -> {tensor name: TensorNeed}   the tensors it reads from the weight files
  load(tensors, rt)                             take them (converted as its kernels need)
and a mixer has
  cache_need() -> None, KVNeed, StateNeed or a tuple of them.
A part whose forward() only enqueues GPU work sets `graph_safe = True`.
"""
from dataclasses import dataclass
from typing import Any

import torch


def _not_while_recording(device, what):
    """Memory is never allocated while a step is recorded into a graph (it would belong to that
    graph's pool): the step has to run outside a recording first."""
    if device.type == "cuda" and torch.cuda.is_current_stream_capturing():
        from ..errors import NeedsEagerStep
        raise NeedsEagerStep(f"{what} would have to be allocated while a graph is recorded")


class Part:
    kind = "?"
    # True if forward() only enqueues GPU work (no host synchronisation, no host-side copies):
    # a step made of such parts may be captured into a HIP graph and replayed.
    graph_safe = False

    def tensor_needs(self):
        return {}

    def load(self, tensors, rt):
        pass

    def cache_need(self):
        return None


class Runtime:
    """Compute dtype, device and the scratch buffers that all layers share."""

    def __init__(self, dtype, device):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError("compute dtype must be float32 or bfloat16")
        self.dtype = dtype
        self.device = torch.device(device)
        self._buffers = {}
        self._views = {}         # (name, dtype, shape) -> the view of the buffer that was handed out last
        self._outgrown = []      # never freed: a captured graph may hold their addresses
        self._scratch = None

    @property
    def scratch(self):
        """The kernels' own scratch memory (K slices of products, partial results of the decode
        attention) of this runtime's owner: see kernels.mfma.Scratch."""
        if self._scratch is None:
            from ..kernels.mfma import Scratch
            self._scratch = Scratch()
        return self._scratch

    @property
    def exact(self):
        """True in the all-float32 mode."""
        return self.dtype == torch.float32

    def buffer(self, name, shape, dtype=None):
        """A scratch tensor of at least this size, reused from call to call under its name. A
        buffer that has become too small is replaced by one at least twice as large and kept all
        the same (a captured graph may still write to it): what is kept is less than what is in use."""
        dtype = dtype or self.dtype
        shape = tuple(shape)
        view = self._views.get((name, dtype, shape))      # the same request as before: the same tensor
        if view is not None:
            return view
        n = 1
        for s in shape:
            n *= int(s)
        key = (name, dtype)
        buf = self._buffers.get(key)
        if buf is None or buf.numel() < n:
            _not_while_recording(self.device, f"the scratch buffer {name!r}")
            if buf is not None:
                self._outgrown.append(buf)
                n_new = max(n, 2 * buf.numel())
            else:
                n_new = max(n, 1)
            buf = torch.empty(n_new, dtype=dtype, device=self.device)
            self._buffers[key] = buf
            for old in [k for k in self._views if k[0] == name and k[1] == dtype]:
                del self._views[old]                       # views of the buffer that was replaced
        if len(self._views) > 4096:
            self._views.clear()
        view = self._views[(name, dtype, shape)] = buf[:n].view(*shape)
        return view

    def weight(self, t, matrix=True):
        """A stored tensor as the kernels read it: matrices in the compute dtype, scales in float32."""
        t = t.to(self.device)
        return t.to(self.dtype if matrix else torch.float32).contiguous()


@dataclass
class NormedRows:
    """An RMSNorm of the residual stream x that the product which last added to x has prepared.
    Half done (squares given): xg = bfloat16(x * norm.w), and squares[b, m] = the sum of x[m]^2 over
    the b-th block of 16 columns (its rows padded to a power of two); a product that reads xg and
    scales its rows by 1 / sqrt(sum of squares / width + eps) gives what it would give for norm(x).
    Whole (squares None): xg is norm(x). No norm kernel runs in either case."""
    norm: Any
    entry: int           # the schedule entry whose part may use it
    x: Any
    xg: Any
    squares: Any

    def row_scale(self):
        return self.squares, self.norm.eps

    def leave(self):
        return self.norm.w, self.xg, self.squares, self.norm.eps


@dataclass
class StepContext:
    """What one step hands down to the parts."""
    rt: Runtime
    meta: Any            # engine.batch.BatchMeta
    cache: Any           # cache.Cache
    entry: int = 0       # the schedule entry that is running
    cache_entry: int = 0  # the entry whose cache it uses
    owns_cache: bool = True
    # A norm handed from part to part (NormedRows). The block sets `handed` to what the part that
    # runs may use in place of norm(x), and `norm_ahead` to (norm, entry): the norm that x meets
    # after this part. A part whose last product into x can do so calls leave_norm and passes the
    # result to that product; parts that know nothing of this are served by the norm's own kernel.
    handed: Any = None
    norm_ahead: Any = None
    left: Any = None
    norm_after_block: Any = None     # set by the model: (first norm of the next entry's block, entry)
    logits_out: Any = None           # where the head is to write, if the caller owns the logits

    def leave_norm(self, linear, x):
        """For a part, just before `linear` adds its last product into x: a NormedRows that product
        is to fill (Linear.forward(..., leave=rows.leave())), or None."""
        if self.norm_ahead is None:
            return None
        norm, entry = self.norm_ahead
        if norm is None or not getattr(norm, "hands_on", False):
            return None
        how = linear.norm_handoff(x.shape[0])
        if how is None:
            return None
        rows, width = x.shape
        squares = None
        xg = self.rt.buffer("handed_rows", (rows, width), torch.bfloat16)
        if how == "half":
            squares = self.rt.buffer("handed_squares", ((width + 15) // 16, linear.handed_rows(rows)), torch.float32)
        self.left = NormedRows(norm, entry, x, xg, squares)
        return self.left

    def take_handed(self, linear, x):
        """For a part that starts with `linear` on norm(x): the NormedRows to use instead, or None."""
        h = self.handed
        if h is None or not linear.finishes_norm(x.shape[0]):
            return None
        return h
