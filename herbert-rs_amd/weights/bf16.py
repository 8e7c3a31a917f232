"""bfloat16 <-> float32 on the host, bit for bit as the reference converts.

crates/core/src/tensor.rs:7-9 (widen: the 16 bits become the upper half) and
:46-56 (narrow: round to nearest, ties to even).
"""
import torch


def f32_to_bf16_bits(x):
    """int32 tensor of the bfloat16 bit patterns of a float32 tensor."""
    bits = x.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    lsb = (bits >> 16) & 1
    round_bit = (bits >> 15) & 1
    sticky = bits & 0x7FFF
    up = (round_bit == 1) & ((sticky != 0) | (lsb == 1))
    return (((bits >> 16) + up.to(torch.int64)) & 0xFFFF).to(torch.int32)


def bf16_bits_to_f32(bits):
    """float32 tensor whose upper halves are the given bit patterns."""
    return ((bits.to(torch.int64) & 0xFFFF) << 16).to(torch.int32).view(torch.float32)
