"""Namespace with the functions of the reference's torch extension ``boolutil_cuda``
(extensions/booleanUtilities.cpp:61-66)."""
import torch

from . import booleanOperations as _ops

_BITS = {32: torch.int32, 64: torch.int64}


def _dtype(bits):
    if bits not in _BITS:
        # the reference also lists 8 and 16 (extensions/booleanUtilities.cpp:21-33); its CuPy kernels
        # never supported them (extensions/booleanOperations.py:25-28) and neither does this build
        raise RuntimeError("invalid bit size")
    return _BITS[bits]


def pack(input, bits):
    """extensions/booleanUtilities.cpp:36-40."""
    _ops._check(input, "input")
    return _ops.pack(input, _dtype(bits))


def unpack(input):
    """extensions/booleanUtilities.cpp:43-46."""
    _ops._check(input, "input")
    return _ops.unpack(input)


def sample_bits(p, n, bits, seed):
    """extensions/booleanUtilities.cpp:49-52."""
    _ops._check(p, "p")
    return _ops.sample_bits(p, n, _dtype(bits), seed)


def binary_weighted_sum(input, weights, z_bits):
    """extensions/booleanUtilities.cpp:54-59."""
    _ops._check(input, "input")
    _ops._check(weights, "weights")
    if input.device != weights.device:
        raise RuntimeError("Tensors are on different devices")
    return _ops.weighted_sum(input, weights, z_bits)


def pack8(input):
    """bool [R,C] -> int8 [R, ceil(C/8)] (extensions/booleanUtilities.cpp:15-18,
    extensions/booleanUtilitiesCuda.cu:31-50).  Expressed through the 32-bit pack: the little-endian
    bytes of the packed words are exactly the 8-bit packing."""
    _ops._check(input, "input")
    words = _ops.pack(input, torch.int32)
    nbytes = (input.size(1) + 7) // 8
    return words.view(torch.int8)[:, :nbytes].contiguous()
