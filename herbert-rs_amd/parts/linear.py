"""A weight matrix [out, in] and its product with activations.

In the float32 mode the plain kernel does all products. In the bfloat16 mode
the MFMA kernels do them where they take the shape and the plain kernel (same
storage types, float32 arithmetic) does the rest.
"""
import torch

from ..kernels import ops


class Linear:
    def __init__(self, weight):
        self.weight = weight           # [N, K], compute dtype, on the GPU
        self.out_features, self.in_features = weight.shape

    def forward(self, a, out, accumulate=False):
        """out[M, N] (+)= a[M, K] @ W^T."""
        if self.weight.dtype == torch.bfloat16 and a.dtype == torch.bfloat16:
            from ..kernels import mfma
            if mfma.gemm_supported(a, self.weight, out):
                mfma.gemm(a, self.weight, out, accumulate)
                return
        ops.gemm_plain(a, self.weight, out, accumulate)
