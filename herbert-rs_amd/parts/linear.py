"""A weight matrix [out, in] and its product with activations.

In the float32 mode the plain kernel does all products. In the bfloat16 mode the MFMA kernels
do them where they take the shape, and then the matrix is kept in their packed order (the 1 KB
operand of 16 rows and 32 k contiguous, all operands of a k-step together), which streams from
HBM as a copy does;
the plain kernel (same storage types, float32 arithmetic) does the rest from row-major weights.
"""
import torch

from ..kernels import mfma, ops


class Linear:
    def __init__(self, weight, pack=True, scratch=None):
        """weight: [N, K] in the compute dtype on the GPU. scratch: the kernels' scratch memory of the
        owner (Runtime.scratch); None: the device's shared one."""
        self.scratch = scratch
        self.out_features, self.in_features = weight.shape
        self.packed = False
        if pack and weight.dtype == torch.bfloat16 and weight.is_cuda \
                and self.out_features % 16 == 0 and self.in_features % 32 == 0:
            weight = mfma.pack_weight(weight)
            self.packed = True
        self.weight = weight

    def forward(self, a, out, accumulate=False, leave=None, row_scale=None, defer_slices=False):
        """out[M, N] (+)= a[M, K] @ W^T. leave and row_scale hand an RMSNorm from one product to the
        next (see norm_handoff); they go to the MFMA kernel as kernels.mfma.gemm describes them.
        defer_slices: the caller's next kernel can add up slices of K; returns what kernels.mfma.gemm
        returns for it, (1, pointer to out, 0) if the product is whole."""
        if self.weight.dtype == torch.bfloat16 and a.dtype == torch.bfloat16:
            if self.packed or mfma.gemm_supported(a, self.weight, out):
                return mfma.gemm(a, self.weight, out, accumulate, packed=self.packed, leave=leave,
                                 row_scale=row_scale, defer_slices=defer_slices, scratch=self.scratch)
        if leave is not None or row_scale is not None:
            raise ValueError("this product cannot hand a norm on (ask norm_handoff first)")
        ops.gemm_plain(a, self.weight, out, accumulate)
        return (1, out.data_ptr(), 0) if defer_slices else None

    def norm_handoff(self, rows):
        """How this product, for that many rows, can prepare the RMSNorm of the rows it adds to: "half"
        (the next product finishes it), "whole" or None; see kernels.mfma.norm_handoff."""
        if self.weight.dtype != torch.bfloat16:
            return None
        return mfma.norm_handoff(rows, self.out_features, self.in_features)

    def finishes_norm(self, rows):
        """True if this product can take rows that are half normed (bf16(x * g) and sums of squares)."""
        if self.weight.dtype != torch.bfloat16 or self.in_features % 32:
            return False
        return rows <= mfma.NORM_HANDOFF_MAX_M

    @staticmethod
    def handed_rows(rows):
        """Rows of the sums of squares that go with a handed-on norm of that many rows."""
        return mfma.padded_rows(rows)

    def forward_swiglu(self, a, out, norm=None, row_scale=None):
        """out bf16 [M, N / 2] = silu(gate) * up for a weight whose rows are gate/up interleaved."""
        mfma.gemm_swiglu(a, self.weight, out, packed=self.packed, norm=norm, row_scale=row_scale,
                         scratch=self.scratch)

    def fuses_norm(self, x):
        """True if RMSNorm(x) @ W^T runs as one kernel for this input (few rows, bfloat16 weights)."""
        if self.weight.dtype != torch.bfloat16:
            return False
        return mfma.norm_fusable(x, self.weight)

    def forward_normed(self, x, norm_weight, eps, out):
        """out[M, N] = RMSNorm(x; norm_weight, eps) @ W^T in one kernel (see fuses_norm)."""
        mfma.gemm(x, self.weight, out, packed=self.packed, norm=(norm_weight, eps), scratch=self.scratch)
