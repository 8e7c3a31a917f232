"""Host side of the bfloat16 MFMA kernels (matrix products and attention)."""


def gemm_supported(a, w, out):
    return False


def attention_supported(q, kv, nq, nkv, hd):
    return False
