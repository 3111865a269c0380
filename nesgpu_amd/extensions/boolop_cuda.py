"""Namespace with the functions of the reference's torch extension ``boolop_cuda``
(extensions/booleanOperations.cpp:86-90).  Inputs must be CUDA and contiguous, otherwise RuntimeError
(CHECK_INPUT, extensions/booleanOperations.cpp:13-15).  The two ``*_old`` direct-conv experiments of the
reference (:92-93) are dead code there and are not provided."""
import torch

from . import booleanOperations as _ops


def _require(cond, msg):
    if not cond:
        raise RuntimeError(msg)                       # TORCH_CHECK


def binary_bmm(A, B):
    """extensions/booleanOperations.cpp:34-41."""
    _ops._check(A, "A")
    _ops._check(B, "B")
    _require(A.size(0) == B.size(0), "Batch dim doesn't match")
    _require(A.size(2) == B.size(1), "Mult dim doesn't match")
    _require(A.device == B.device, "Tensors are on different devices")
    return _ops.bmm(A, B)


def batch_im2col(input, filterx, filtery, padx, pady, stridex, stridey):
    """extensions/booleanOperations.cpp:52-55."""
    _ops._check(input, "input")
    return _ops.batch_im2col(input, filterx, filtery, padx, pady, stridex, stridey)


def binary_batch_conv2d(input, filter, filterx, filtery, padx, pady, stridex, stridey):
    """extensions/booleanOperations.cpp:43-50; returns [D, h*w, O] like the reference
    (extensions/booleanOperationsCuda.cu:295-298 returns the bmm result without a view)."""
    _ops._check(input, "input")
    _ops._check(filter, "filter")
    _require(input.size(0) == filter.size(0), "Batch dim doesn't match")
    _require(input.device == filter.device, "Tensors are on different devices")
    _require(input.dtype == filter.dtype, "Tensors have different types")
    out = _ops.conv(input, filter, filterx, filtery, padx, pady, stridex, stridey)
    return out.view(out.size(0), -1, out.size(3))


def binary_seeded_bmv(A, B, seed):
    """Fused sample + XOR-popcount product (extensions/booleanOperations.cpp:58-63,
    extensions/booleanOperationsCuda.cu:172-202): A = probabilities fp16 [out, in], B = packed inputs
    [batch, Kw]; returns int32 [batch, out].  Weights are drawn from a Philox4x32-10 stream keyed by
    ``seed`` and never stored."""
    _ops._check(A, "A")
    _ops._check(B, "B")
    _require(A.device == B.device, "Tensors are on different devices")
    thr = _ops.thresholds_from_p(A)
    return _ops.seeded_bmv_philox(thr, B, A.size(0), A.size(1), seed)
