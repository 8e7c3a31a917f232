"""Grouped-query attention over the paged cache.

Formulas as the reference computes them (`bc/` = crates/backends/backend_common/src/):
q, k, v projections without bias (bc/generic_attention/prefill/mod.rs:73-77),
optional RMSNorm of every head with one weight [head_dim]
(bc/generic_attention/mod.rs:62-76), rotation at absolute positions
(prefill/mod.rs:189-210), keys and values appended to the cache (:232), scores
scaled by 1/sqrt(head_dim) (bc/generic_attention/decode.rs:126), consecutive
query heads sharing a kv head (decode.rs:131-140), causal by count
(prefill/kernel_f32.rs:65-67), output projection added to the residual
(prefill/mod.rs:293, bc/generic_layer.rs:1234-1236).
A window (keys of the last `window` positions only) is a parameter that the
reference does not have.
"""
import math

import torch

from ..cache import KVNeed
from ..kernels import mfma, ops
from ..weights import TensorNeed
from .base import Part
from .linear import Linear
from .registry import register


@register("mixer", "attention")
class Attention(Part):
    graph_safe = True

    def __init__(self, hidden_size, num_heads, num_kv_heads, head_dim, eps, position, names,
                 qk_norm=True, window=None, scale=None, shared=None, reads_cache_only=False):
        """names: dict with q, k, v, o (and q_norm, k_norm when qk_norm) -> tensor names.
        reads_cache_only: the part has no k / v projections and attends over a cache that
        another entry of the schedule fills."""
        if num_heads % num_kv_heads:
            raise ValueError("num_heads must be divisible by num_kv_heads")
        self.hidden_size = int(hidden_size)
        self.nq = int(num_heads)
        self.nkv = int(num_kv_heads)
        self.hd = int(head_dim)
        self.eps = float(eps)
        self.qk_norm = bool(qk_norm)
        self.window = int(window) if window else None
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.hd)
        self.names = dict(names)
        self.reads_cache_only = bool(reads_cache_only)
        self.position = shared.position(position)
        self.qkv = self.o = self.q_norm_w = self.k_norm_w = None

    @property
    def q_dim(self):
        return self.nq * self.hd

    @property
    def kv_dim(self):
        return self.nkv * self.hd

    def tensor_needs(self):
        n = self.names
        needs = {n["q"]: TensorNeed((self.q_dim, self.hidden_size)),
                 n["o"]: TensorNeed((self.hidden_size, self.q_dim))}
        if not self.reads_cache_only:
            needs[n["k"]] = TensorNeed((self.kv_dim, self.hidden_size))
            needs[n["v"]] = TensorNeed((self.kv_dim, self.hidden_size))
        if self.qk_norm:
            needs[n["q_norm"]] = TensorNeed((self.hd,), "scale")
            if not self.reads_cache_only:
                needs[n["k_norm"]] = TensorNeed((self.hd,), "scale")
        return needs

    def cache_need(self):
        if self.reads_cache_only:
            return None
        return KVNeed(self.nkv, self.hd, self.window)

    def load(self, tensors, rt):
        n = self.names
        rows = [tensors[n["q"]]]
        if not self.reads_cache_only:
            rows += [tensors[n["k"]], tensors[n["v"]]]
        # one fused projection [q rows | k rows | v rows]: the activations are read once
        self.qkv = Linear(rt.weight(torch.cat([r.to(rt.device) for r in rows], 0)), scratch=rt.scratch)
        self.o = Linear(rt.weight(tensors[n["o"]]), scratch=rt.scratch)
        if self.qk_norm:
            self.q_norm_w = rt.weight(tensors[n["q_norm"]], matrix=False)
            if not self.reads_cache_only:
                self.k_norm_w = rt.weight(tensors[n["k_norm"]], matrix=False)

    def forward_from_residual(self, ctx, x, norm):
        """With few rows and bfloat16 weights no norm kernel runs: the projection takes what the
        product before left of the norm, or else does the norm itself on the way."""
        handed = ctx.take_handed(self.qkv, x)
        if handed is not None:
            self.forward(ctx, handed.xg, x, row_scale=handed.row_scale())
            return True
        if not (hasattr(norm, "w") and hasattr(norm, "eps") and self.qkv.fuses_norm(x)):
            return False
        self.forward(ctx, None, x, fused_norm=norm)
        return True

    def project_out(self, ctx, attn, x):
        """x += attn @ Wo^T, the part's last product into the residual stream."""
        left = ctx.leave_norm(self.o, x)
        self.o.forward(attn, x, accumulate=True, leave=None if left is None else left.leave())

    def forward(self, ctx, y, x, fused_norm=None, row_scale=None):
        rt = ctx.rt
        T = x.shape[0]
        kv = ctx.cache.kv_view(ctx.cache_entry)
        write_kv = not self.reads_cache_only
        width = self.q_dim + (2 * self.kv_dim if write_kv else 0)
        rot = self.position.rotation()
        cos, sin, rot_dims = rot if rot is not None else (None, None, 0)
        if write_kv and fused_norm is None and row_scale is None and rt.dtype == torch.bfloat16:
            if mfma.gemm_qkv_fusable(y, self.qkv.weight, ctx.meta, kv, self.nq, self.nkv, self.hd, rot_dims):
                # a long prompt: the projection norms, rotates and writes the cache in its epilogue
                q = rt.buffer("q", (T, self.q_dim))
                mfma.gemm_qkv(y, self.qkv.weight, self.qkv.packed, self.q_norm_w, self.k_norm_w, cos, sin, ctx.meta,
                              kv, q, self.nq, self.nkv, self.hd, self.eps)
                attn = rt.buffer("attn", (T, self.q_dim))
                self.attend(ctx, q, kv, attn)
                self.project_out(ctx, attn, x)
                return
        qkv = rt.buffer("qkv", (T, width), torch.float32)
        fused_decode = False
        if write_kv and rt.dtype == torch.bfloat16:
            fused_decode = mfma.decode_fusable(ctx.meta, kv, self.nq, self.nkv, self.hd, rot_dims, rt.dtype)
        slices = None
        if fused_norm is not None:
            self.qkv.forward_normed(x, fused_norm.w, fused_norm.eps, qkv)
        else:
            # (the fused decode kernel of heads of 128 and the rotation kernel of bfloat16 prompts add
            # up slices of K themselves)
            defer = (fused_decode and self.hd == 128) or (not fused_decode and ops.rope_write_adds_slices(
                T, self.hd, rot_dims, rt.dtype, write_kv, cos is not None))
            slices = self.qkv.forward(y, qkv, row_scale=row_scale, defer_slices=defer)
        attn = rt.buffer("attn", (T, self.q_dim))
        if fused_decode:
            # one token a sequence: norm, rotation, cache write and attention in one kernel
            mfma.attention_decode_fused(qkv, self.q_norm_w, self.k_norm_w, cos, sin, ctx.meta, kv, attn,
                                        self.nq, self.nkv, self.hd, self.eps, self.scale, self.window,
                                        qkv_slices=slices, scratch=rt.scratch)
            self.project_out(ctx, attn, x)
            return
        q = rt.buffer("q", (T, self.q_dim))
        ops.qk_norm_rope_write(qkv, self.q_norm_w, self.k_norm_w, cos, sin, rot_dims, ctx.meta, kv, q,
                               self.nq, self.nkv, self.hd, self.eps, write_kv=write_kv, qkv_slices=slices)
        self.attend(ctx, q, kv, attn)
        self.project_out(ctx, attn, x)

    def attend(self, ctx, q, kv, out):
        if q.dtype == torch.bfloat16:
            if mfma.attention_supported(q, kv, self.nq, self.nkv, self.hd):
                mfma.attention(q, ctx.meta, kv, out, self.nq, self.nkv, self.hd, self.scale, self.window,
                               scratch=ctx.rt.scratch)
                return
        ops.attention_plain(q, ctx.meta, kv, out, self.nq, self.nkv, self.hd, self.scale, self.window)
