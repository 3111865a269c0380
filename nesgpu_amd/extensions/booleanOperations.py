"""Drop-in replacement for the reference's ``extensions/booleanOperations.py``.

Same function names, positional order, defaults and return shapes/dtypes as the reference module
(extensions/booleanOperations.py:82-252), but every op is one call into libnesbin.so -- hand-written
gfx950 kernels behind the C ABI of include/nesbin.h -- on the CURRENT torch stream (the reference
captures the stream once at import, extensions/booleanOperations.py:3-4).  Nothing is compiled or read
from disk at import, and there is no CPU path: tensors must live on the GPU.

Error behaviour follows the reference: shape/rank mistakes raise ``AssertionError``
(extensions/booleanOperations.py:108-111,132-138,176,204,219-220,233), an unsupported word dtype raises
``TypeError`` (what ``raise NotImplemented`` at :28,80 surfaces as), and -- from the torch-extension
half of the reference (extensions/booleanOperations.cpp:13-15) -- non-CUDA or non-contiguous inputs raise
``RuntimeError`` instead of being read through a wrong stride.

Additions that the reference lacks are grouped at the end (supplied-word / Philox sampling, the fused
sample+popcount product with a flip base, the fused conv->threshold->pack(->pool) op).
"""
import math

import torch

from .. import _lib

__all__ = [
    "batch_im2col", "bmm", "bmm_act", "conv", "conv_act", "pack", "int8pack", "sample_bits", "weighted_sum",
    "max_pool2d", "next_pow2_clip", "ceil_div", "unpack", "thresholds_from_p", "sample_bits_from_words",
    "flip_from_words", "sample_bits_philox", "flip_philox", "seeded_bmv_from_words", "seeded_bmv_philox",
    "philox_words", "conv_act_pack", "conv_popc_sums", "conv_bn_thresholds_from_input", "tap_pack_filter", "tap_packing_applies", "conv_engine", "conv_last_engine",
    "bmv_act_pack", "bmv_bn_act", "ExpandedRows", "expand_rows", "bmm_nt", "FlipRows", "flip_rows_from_weights",
    "bmv_flip", "bmv_flip_act_pack", "skip_table", "flip_rows_skip", "flip_rows_layered", "layer_tables", "flip_rows_to_weights",
    "center_fitness", "grad_regularize_", "bias_grad", "sample_bits_skip", "half_draws_apply", "bias_noise_scale_", "bmv_pm1",
]


def next_pow2_clip(v, cap):
    """Launch-shape helper kept for API parity (extensions/booleanOperations.py:57-67)."""
    if v > cap // 2:
        return cap
    p = 1
    while p < v:
        p *= 2
    return p


def ceil_div(a, b):
    return (a + b - 1) // b


# --------------------------------------------------------------------------------------------
def _suffix(dtype):
    if dtype == torch.int64:
        return "_i64", 64
    if dtype == torch.int32:
        return "_i32", 32
    # the reference executes `raise NotImplemented`, which Python turns into a TypeError
    raise TypeError("packed word dtype must be torch.int64 or torch.int32, got %r" % (dtype,))


def _check(t, name):
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s must be a torch.Tensor" % name)
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)       # booleanOperations.cpp:13
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)           # booleanOperations.cpp:14
    return t


def _same_device(a, b):
    if a.device != b.device:
        raise RuntimeError("Tensors are on different devices")       # booleanOperations.cpp:39


# The current stream's handle and the current device index straight from torch's C layer: the public wrappers build a
# Stream object / re-check initialisation on every call, which costs more than the rest of an op's host work together.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream(t):
    if _raw_stream is not None:
        return _raw_stream(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


class _Here:
    """No-op context: the tensor already lives on the current device (the usual case; saves the two device
    switches of torch.cuda.device on every op)."""

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_HERE = _Here()


def _on(t):
    """Context that makes ``t``'s device current for the launch."""
    cur = _raw_device() if _raw_device is not None else torch.cuda.current_device()
    return _HERE if t.device.index == cur else torch.cuda.device(t.device)


def _out_hw(inp, filterx, filtery, padx, pady, stridex, stridey):
    h = (inp.size(1) - filterx + 2 * padx) // stridex + 1
    w = (inp.size(2) - filtery + 2 * pady) // stridey + 1
    return h, w


# ---- reference API ----------------------------------------------------------------------------
def batch_im2col(input, filterx, filtery, padx, pady, stridex, stridey, REPEAT=128):
    """[B,H,W,Cw] -> [B, h*w, filterx*filtery*Cw] (extensions/booleanOperations.py:82-102).
    ``REPEAT`` was a launch-shape knob of the reference kernel; accepted and ignored."""
    _check(input, "input")
    assert len(input.shape) == 4
    suf, _ = _suffix(input.dtype)
    h, w = _out_hw(input, filterx, filtery, padx, pady, stridex, stridey)
    out = torch.empty((input.size(0), h * w, filterx * filtery * input.size(3)), dtype=input.dtype,
                      device=input.device)
    with _on(input):
        _lib.call("nb_im2col" + suf, out.data_ptr(), input.data_ptr(), input.size(0), input.size(1), input.size(2),
                  input.size(3), filterx, filtery, padx, pady, stridex, stridey, _stream(input))
    return out


def bmm(A, B):
    """C[z,x,y] = sum_k popcount(A[z,x,k] ^ B[z,k,y]), int32 (extensions/booleanOperations.py:107-129).
    ``A`` may be a :class:`FlipRows` (a population's weights as base + flip lists) with ``B`` [Z, Kw, 1]: the same
    sums from the sparse form."""
    if isinstance(A, FlipRows):
        assert len(B.shape) == 3 and B.size(0) == A.D and B.size(1) == A.Kw and B.size(2) == 1
        return bmv_flip(A, B.view(A.D, A.Kw)).unsqueeze(2)
    sa, sb = A.shape, B.shape
    assert len(sa) == 3
    assert len(sb) == 3
    assert sa[0] == sb[0]
    assert sa[2] == sb[1]
    _check(A, "A")
    _check(B, "B")
    _same_device(A, B)
    assert A.dtype == B.dtype
    suf, _ = _suffix(A.dtype)
    C = torch.empty((sa[0], sa[1], sb[2]), dtype=torch.int32, device=A.device)
    with _on(A):
        _lib.call("nb_bmm" + suf, C.data_ptr(), A.data_ptr(), B.data_ptr(), sa[0], sa[1], sa[2], sb[2], _stream(A))
    return C


def bmm_act(A, B, threshold):
    """bool = 2*popc > threshold[z,y] (extensions/booleanOperations.py:131-158)."""
    assert len(A.shape) == 3
    assert len(B.shape) == 3
    assert len(threshold.shape) == 2
    assert A.size(0) == B.size(0) == threshold.size(0)
    assert A.size(2) == B.size(1)
    assert threshold.size(1) == B.size(2)
    assert threshold.dtype == torch.int32
    _check(A, "A")
    _check(B, "B")
    _check(threshold, "threshold")
    _same_device(A, B)
    _same_device(A, threshold)
    assert A.dtype == B.dtype
    suf, _ = _suffix(A.dtype)
    C = torch.empty((A.size(0), A.size(1), B.size(2)), dtype=torch.bool, device=A.device)
    with _on(A):
        _lib.call("nb_bmm_act" + suf, C.data_ptr(), A.data_ptr(), B.data_ptr(), threshold.data_ptr(), A.size(0),
                  A.size(1), A.size(2), B.size(2), _stream(A))
    return C


def bmv_pm1(A, x, in_bits):
    """int32 [Z, M] = ``2 * bmm(A, x.view(Z, Kw, 1)).squeeze(2) - in_bits``: a linear layer's activations
    (modules/binary.py:97) in one kernel; A [Z, M, Kw] packed weights, x [Z, Kw] one packed input row per member."""
    assert len(A.shape) == 3 and len(x.shape) == 2
    assert A.size(0) == x.size(0) and A.size(2) == x.size(1)
    _check(A, "A")
    _check(x, "x")
    _same_device(A, x)
    assert A.dtype == x.dtype
    suf, bits = _suffix(A.dtype)
    assert 0 <= in_bits <= A.size(2) * bits
    out = torch.empty((A.size(0), A.size(1)), dtype=torch.int32, device=A.device)
    if out.numel() == 0:
        return out
    if A.size(2) == 0:
        return out.fill_(-int(in_bits))
    with _on(A):
        _lib.call("nb_bmv_pm1" + suf, out.data_ptr(), A.data_ptr(), x.data_ptr(), A.size(0), A.size(1), A.size(2),
                  int(in_bits), _stream(A))
    return out


def bmv_act_pack(A, x, threshold):
    """One input row per member, as the linear layers have it: A [Z,M,Kw] packed weights, x [Z,Kw] (or [Z,Kw,1])
    packed inputs, threshold [Z,M] int32 -> packed bits (2*popc(A[z,m] ^ x[z]) > threshold[z,m]) as [Z, ceil(M/bits)]
    words.  Not in the reference: it is ``pack(2 * bmm(A, x) > threshold)`` (the compare of
    modules/binary.py:97-106 and the next layer's pack) in one kernel, without the int32 and bool maps.  ``A`` may be
    a :class:`FlipRows`."""
    if isinstance(A, FlipRows):
        return bmv_flip_act_pack(A, x, threshold)
    _check(A, "A")
    _check(x, "x")
    _check(threshold, "threshold")
    _same_device(A, x)
    _same_device(A, threshold)
    assert len(A.shape) == 3
    assert A.dtype == x.dtype
    Z, M, Kw = A.shape
    assert x.numel() == Z * Kw and x.size(0) == Z                # "Batch dim doesn't match", booleanOperations.cpp:46
    assert tuple(threshold.shape) == (Z, M) and threshold.dtype == torch.int32
    suf, bits = _suffix(A.dtype)
    out = torch.empty((Z, ceil_div(M, bits)), dtype=A.dtype, device=A.device)
    with _on(A):
        _lib.call("nb_bmv_act_pack" + suf, out.data_ptr(), A.data_ptr(), x.data_ptr(), threshold.data_ptr(), Z, M, Kw,
                  _stream(A))
    return out


def bmv_bn_act(A, x, bias, bias_noise, in_bits, pack=False, workspace=None, round_fp16=False):
    """Linear layer with the population-mean threshold in one call (not in the reference as an op: it is the
    composition of modules/binary.py:97-102).  A [Z,M,Kw] packed weights, x [Z,Kw] (or [Z,Kw,1]) packed inputs, bias [M]
    and bias_noise [Z,M] fp16, ``in_bits`` the true bit count K of a row.  With act = 2*popc - K:
    thr[z,m] = fp16(fp16(bias + bias_noise) + fp16(float(sum_z act[z,m]) * (float(M) / float(Z*M)))) (torch's fp16
    mean: fp32 sum times the fp32 quotient of the element counts, the exact product rounded once), result = act > thr as bool [Z,M], or with
    ``pack`` packed along M into [Z, ceil(M/bits)] words.  ``workspace`` (uint8 CUDA tensor) is allocated when absent.
    ``round_fp16``: act is rounded to fp16 before the mean and the compare, as the reference's tensor expression does
    (``activation.type(torch.float16).mean(dim=0)``, then an int32 tensor compared with an fp16 one); it only matters
    for rows of more than 2048 bits, whose activations fp16 no longer holds exactly."""
    _check(A, "A")
    _check(x, "x")
    _check(bias, "bias")
    _check(bias_noise, "bias_noise")
    _same_device(A, x)
    _same_device(A, bias)
    _same_device(A, bias_noise)
    assert len(A.shape) == 3
    assert A.dtype == x.dtype
    Z, M, Kw = A.shape
    assert x.numel() == Z * Kw and x.size(0) == Z
    assert bias.dtype == torch.float16 and tuple(bias.shape) == (M,)
    assert bias_noise.dtype == torch.float16 and tuple(bias_noise.shape) == (Z, M)
    suf, bits = _suffix(A.dtype)
    assert 0 <= in_bits <= Kw * bits
    need = _lib.load().nb_bmv_bn_workspace_bytes(Z, M)
    if workspace is None:
        workspace = torch.empty((max(need, 1),), dtype=torch.uint8, device=A.device)
    else:
        _check(workspace, "workspace")
        _same_device(A, workspace)
        assert workspace.dtype == torch.uint8 and workspace.numel() >= need
    if pack:
        out = torch.empty((Z, ceil_div(M, bits)), dtype=A.dtype, device=A.device)
    else:
        out = torch.empty((Z, M), dtype=torch.bool, device=A.device)
    with _on(A):
        _lib.call("nb_bmv_bn_act" + suf, out.data_ptr(), A.data_ptr(), x.data_ptr(), bias.data_ptr(),
                  bias_noise.data_ptr(), Z, M, Kw, int(in_bits), (1 if pack else 0) | (2 if round_fp16 else 0),
                  workspace.data_ptr(),
                  workspace.numel(), _stream(A))
    return out


def conv_bn_thresholds(sums, bias, bias_noise, in_bits, pixels):
    """Thresholds of ``BinarizedConv2d(batch_norm=True)`` (modules/binary.py:147-155) from ``conv_popc_sums``: with
    act = 2*popc - in_bits, mean = fp16(float(sum over the pixels of act) * (float(D*O) / float(D*O*pixels))) (torch's
    fp16 mean over the pixels of a [D,h,w,O] map),
    thr = fp16(fp16(bias + bias_noise) + mean); returns int32 [D,O] = floor(thr) + in_bits (INT32_MAX for NaN), the
    threshold of ``conv_act`` / ``conv_act_pack`` (2*popc > threshold).  sums int32 [D,O], bias fp16 [O], bias_noise
    fp16 [D,O].  One kernel instead of a dozen elementwise tensor operations."""
    _check(sums, "sums")
    _check(bias, "bias")
    _check(bias_noise, "bias_noise")
    _same_device(sums, bias)
    _same_device(sums, bias_noise)
    assert sums.dtype == torch.int32 and len(sums.shape) == 2
    D, O = sums.shape
    assert bias.dtype == torch.float16 and tuple(bias.shape) == (O,)
    assert bias_noise.dtype == torch.float16 and tuple(bias_noise.shape) == (D, O)
    assert in_bits >= 0 and pixels >= 1
    out = torch.empty((D, O), dtype=torch.int32, device=sums.device)
    with _on(sums):
        _lib.call("nb_conv_bn_thresholds", out.data_ptr(), sums.data_ptr(), bias.data_ptr(), bias_noise.data_ptr(), D, O,
                  int(in_bits), int(pixels), _stream(sums))
    return out


def conv_bn_thresholds_from_input(input, filter, bias, bias_noise, filterx, filtery, padx, pady, stridex, stridey,
                                  in_bits=None, filter_tap_packed=False, channels=None):
    """``conv_bn_thresholds(conv_popc_sums(input, filter, ...), bias, bias_noise, channels * taps, h * w)`` in one call
    (one kernel where the pixel sums come from bit counts).  ``channels``: the layer's true input channels (default
    ``in_bits``, else every bit of the channel words)."""
    suf, _, input, filter, tap = _conv_args(input, filter, filterx, filtery, in_bits, filter_tap_packed)
    _check(bias, "bias")
    _check(bias_noise, "bias_noise")
    _same_device(input, bias)
    _same_device(input, bias_noise)
    D, O = input.size(0), filter.size(2)
    assert bias.dtype == torch.float16 and tuple(bias.shape) == (O,)
    assert bias_noise.dtype == torch.float16 and tuple(bias_noise.shape) == (D, O)
    if channels is None:
        channels = in_bits if in_bits is not None else input.size(3) * torch.iinfo(input.dtype).bits
    h, w = _out_hw(input, filterx, filtery, padx, pady, stridex, stridey)
    assert h * w >= 1
    out = torch.empty((D, O), dtype=torch.int32, device=input.device)
    with _on(input):
        _lib.call("nb_conv_bn_thresholds_from_input" + suf, out.data_ptr(), input.data_ptr(), filter.data_ptr(),
                  bias.data_ptr(), bias_noise.data_ptr(), D, input.size(1), input.size(2), input.size(3), O, filterx,
                  filtery, padx, pady, stridex, stridey, tap, int(channels) * filterx * filtery, _stream(input))
    return out


def conv_engine(engine=None):
    """Query / set the process-wide conv engine: 0 = automatic (matrix cores for populations of 128 or more, else
    XOR-popcount), 1 = XOR-popcount kernels only, 2 = matrix cores wherever a kernel covers the shape (FP4 codes for
    full channel words of 64, 128 or 256 channels, +-1 bytes otherwise), 3 = as 2 with +-1 bytes only.
    Returns the previous setting.  Results are identical either way."""
    return _lib.load().nb_conv_engine(-1 if engine is None else int(engine))


def conv_last_engine():
    """Engine that served this thread's latest conv launch: 1 = XOR-popcount, 2 = matrix cores on +-1 bytes (int8
    MFMA), 4 = matrix cores on FP4 codes, 5 = pixel sums from counts of the image's bits (no conv), 0 = none yet."""
    return _lib.load().nb_conv_last_engine()


def tap_packing_applies(in_bits, Cw, dtype):
    """True when a conv over inputs with ``in_bits`` true channels in ``Cw`` words per pixel can share one word
    between several filter taps (Cw == 1 and at least two taps fit a word)."""
    return in_bits is not None and Cw == 1 and 0 < 2 * int(in_bits) <= torch.iinfo(dtype).bits


def tap_pack_filter(filter, taps, in_bits):
    """[D, taps, O] per-member filters with one word per tap (only the low ``in_bits`` bits used) ->
    [D, ceil(taps/T), O] with T = bits // in_bits taps per word.  Feed the result to conv / conv_act /
    conv_act_pack with ``in_bits=...`` and ``filter_tap_packed=True``."""
    _check(filter, "filter")
    assert len(filter.shape) == 3 and filter.size(1) == taps
    suf, bits = _suffix(filter.dtype)
    assert 0 < 2 * in_bits <= bits
    T = bits // in_bits
    out = torch.empty((filter.size(0), ceil_div(taps, T), filter.size(2)), dtype=filter.dtype, device=filter.device)
    with _on(filter):
        _lib.call("nb_tap_pack_filter" + suf, out.data_ptr(), filter.data_ptr(), filter.size(0), taps, filter.size(2),
                  int(in_bits), _stream(filter))
    return out


def _pair_words(input, filter, taps):
    """32-bit words, an even number per pixel: the same bytes as 64-bit words.  The image is viewed as int64
    [D,H,W,Cw/2]; the filter [D, taps*Cw, O] has the two halves of a 64-bit word O words apart and is re-packed to
    int64 [D, taps*Cw/2, O] (one copy of the filters).  The kernels for 64-bit words then serve 32-bit tensors:
    half the instructions on the XOR-popcount path, and the matrix-core engines.  None if the tensors do not allow it."""
    Cw = input.size(3)
    if Cw == 0 or Cw % 2 or input.data_ptr() % 8 or filter.size(1) != taps * Cw:
        return None
    D, K, O = filter.shape
    f64 = filter.view(D, K // 2, 2, O).transpose(2, 3).contiguous().view(torch.int64).view(D, K // 2, O)
    return input.view(torch.int64), f64


def _conv_args(input, filter, filterx, filtery, in_bits=None, filter_tap_packed=False, out_words=None):
    """-> (suffix, bits, input to pass, filter to pass, tap_bits).  ``out_words``: for packed outputs, the words per
    pixel of the result in the input's word type (32-bit tensors are only handed to the 64-bit kernels when those
    write the same bytes)."""
    _check(input, "input")
    _check(filter, "filter")
    _same_device(input, filter)
    assert len(input.shape) == 4
    assert len(filter.shape) == 3
    assert input.size(0) == filter.size(0)                       # "Batch dim doesn't match", booleanOperations.cpp:46
    assert input.dtype == filter.dtype                           # booleanOperations.cpp:48
    suf, bits = _suffix(input.dtype)
    taps = filterx * filtery
    if tap_packing_applies(in_bits, input.size(3), input.dtype):
        T = bits // int(in_bits)
        if filter_tap_packed:
            assert filter.size(1) == ceil_div(taps, T)
        else:
            assert filter.size(1) == taps
            filter = tap_pack_filter(filter, taps, int(in_bits))
        return suf, bits, input, filter, int(in_bits)
    assert not filter_tap_packed, "filter_tap_packed needs in_bits with Cw == 1 and 2*in_bits <= word bits"
    assert filter.size(1) == taps * input.size(3)                # the bmm contraction assert (:111)
    if bits == 32 and (out_words is None or out_words % 2 == 0):
        paired = _pair_words(input, filter, taps)
        if paired is not None:
            return "_i64", 64, paired[0], paired[1], 0
    return suf, bits, input, filter, 0


def conv(input, filter, filterx, filtery, padx, pady, stridex, stridey, in_bits=None, filter_tap_packed=False):
    """bmm(batch_im2col(input), filter).view(D,h,w,O) without materialising the columns
    (extensions/booleanOperations.py:162-166).  filter is [D, filterx*filtery*Cw, O].

    ``in_bits`` (optional, not in the reference): the true channel count C of the packed input.  When the
    input has one word per pixel and 2*C <= word bits, several filter taps share a word (same sums, less
    work); the filter is re-packed on the fly unless ``filter_tap_packed`` says it already is."""
    suf, _, input, filter, tap = _conv_args(input, filter, filterx, filtery, in_bits, filter_tap_packed)
    h, w = _out_hw(input, filterx, filtery, padx, pady, stridex, stridey)
    out = torch.empty((input.size(0), h, w, filter.size(2)), dtype=torch.int32, device=input.device)
    with _on(input):
        _lib.call("nb_conv" + suf, out.data_ptr(), input.data_ptr(), filter.data_ptr(), input.size(0), input.size(1),
                  input.size(2), input.size(3), filter.size(2), filterx, filtery, padx, pady, stridex, stridey, tap,
                  _stream(input))
    return out


def conv_popc_sums(input, filter, filterx, filtery, padx, pady, stridex, stridey, in_bits=None,
                   filter_tap_packed=False):
    """conv(...).sum over the output pixels -> int32 [D, O], without the [D,h,w,O] maps reaching memory (not in the
    reference; it is the statistic behind the per-member mean of BinarizedConv2d(batch_norm=True),
    modules/binary.py:147-155).  With the automatic engine, 64-bit words, stride 1 and filters of at most 5 x 5 no
    conv runs at all: the sum over the pixels is taken first (counts of the image's bits per tap), then one small dot
    product per output channel; the same integers."""
    suf, _, input, filter, tap = _conv_args(input, filter, filterx, filtery, in_bits, filter_tap_packed)
    out = torch.empty((input.size(0), filter.size(2)), dtype=torch.int32, device=input.device)
    with _on(input):
        _lib.call("nb_conv_popc_sums" + suf, out.data_ptr(), input.data_ptr(), filter.data_ptr(), input.size(0),
                  input.size(1), input.size(2), input.size(3), filter.size(2), filterx, filtery, padx, pady, stridex,
                  stridey, tap, _stream(input))
    return out


def _bool_map_via_packed(input, filter, filterx, filtery, stridex, stridey, tap):
    """True where conv_act's bool map is better made by a packed-output kernel and unpack: whole output words, and
    either a shape the matrix-core kernels take (64-bit words, 3-row windows, stride 1, a population of 128 or
    more; not with the engine pinned to XOR-popcount) or a window of at most 32 bits."""
    bits = torch.iinfo(input.dtype).bits
    O = filter.size(2)
    if O == 0 or O % bits != 0 or input.size(0) * input.size(1) * input.size(2) == 0:
        return False
    if tap and filterx * filtery * tap <= 32:
        return True
    return (bits == 64 and filterx == 3 and stridex == 1 and stridey == 1 and input.size(0) >= 128
            and input.size(3) > 0 and conv_engine() != 1)


def conv_act(input, filter, threshold, filterx, filtery, padx, pady, stridex, stridey, in_bits=None,
             filter_tap_packed=False):
    """bmm_act(batch_im2col(input), filter, threshold).view(D,h,w,O) (extensions/booleanOperations.py:168-172)."""
    given, given_filter = input, filter
    suf, _, input, filter, tap = _conv_args(input, filter, filterx, filtery, in_bits, filter_tap_packed)
    _check(threshold, "threshold")
    _same_device(input, threshold)
    assert len(threshold.shape) == 2
    assert threshold.size(0) == input.size(0)
    assert threshold.size(1) == filter.size(2)
    assert threshold.dtype == torch.int32
    h, w = _out_hw(input, filterx, filtery, padx, pady, stridex, stridey)
    if _bool_map_via_packed(input, filter, filterx, filtery, stridex, stridey, tap):
        # the packed-output kernels (matrix cores, window-in-a-register) followed by unpack: same bools, and faster
        # than the XOR-popcount kernel that writes bool bytes itself, although the bits make one more trip
        if input.dtype != given.dtype:          # 32-bit words handed on as 64-bit ones: whole 64-bit output words
            packed = conv_act_pack(input, filter, threshold, filterx, filtery, padx, pady, stridex, stridey)
        else:
            packed = conv_act_pack(given, filter if tap else given_filter, threshold, filterx, filtery, padx, pady,
                                   stridex, stridey, in_bits=tap if tap else None, filter_tap_packed=bool(tap))
        return unpack(packed.view(-1, packed.size(3))).view(input.size(0), h, w, filter.size(2))
    out = torch.empty((input.size(0), h, w, filter.size(2)), dtype=torch.bool, device=input.device)
    with _on(input):
        _lib.call("nb_conv_act" + suf, out.data_ptr(), input.data_ptr(), filter.data_ptr(), threshold.data_ptr(),
                  input.size(0), input.size(1), input.size(2), input.size(3), filter.size(2), filterx, filtery, padx,
                  pady, stridex, stridey, tap, _stream(input))
    return out


def pack(input, dtype=torch.int32):
    """bool [R,C] -> words [R, ceil(C/bits)], LSB first (extensions/booleanOperations.py:175-187).
    The default word type is int32, as in the reference; the layers pass int64."""
    assert len(input.shape) == 2
    _check(input, "input")
    if input.dtype != torch.bool:
        raise TypeError("pack expects a torch.bool tensor, got %r" % (input.dtype,))
    suf, bits = _suffix(dtype)
    ret = torch.empty((input.size(0), ceil_div(input.shape[1], bits)), dtype=dtype, device=input.device)
    with _on(input):
        _lib.call("nb_pack" + suf, ret.data_ptr(), input.data_ptr(), input.size(0), input.size(1), _stream(input))
    return ret


def int8pack(input, dtype=torch.int32):
    """uint8 [R,C] -> words [R, ceil(C/(bits/8))], little-endian bytes (extensions/booleanOperations.py:189-201)."""
    assert len(input.shape) == 2
    _check(input, "input")
    if input.dtype not in (torch.uint8, torch.int8):
        raise TypeError("int8pack expects a uint8 tensor, got %r" % (input.dtype,))
    suf, bits = _suffix(dtype)
    ret = torch.empty((input.size(0), ceil_div(input.shape[1], bits // 8)), dtype=dtype, device=input.device)
    with _on(input):
        _lib.call("nb_int8pack" + suf, ret.data_ptr(), input.data_ptr(), input.size(0), input.size(1), _stream(input))
    return ret


def sample_bits(p, n, dtype, seed, conv_taps=None):
    """ret[m,r,z] bit i = Bernoulli(p[r, z*bits+i]), n independent members
    (extensions/booleanOperations.py:203-215, extensions/src/sample_bits.cu:47-57).

    Same law, layout and tail rule as the reference; the random stream is Philox4x32-10 keyed by
    ``seed`` instead of cuRAND XORWOW (whose exact bitstream no reference test pins).  ``conv_taps`` (not in the
    reference): see :func:`sample_bits_from_words`; returns ``(rows_layout, conv_layout)``."""
    assert len(p.shape) == 2
    return sample_bits_philox(thresholds_from_p(p), n, dtype, seed, conv_taps=conv_taps)


def weighted_sum(input, weights, zbits, fast=False):
    """ret[r,z] = fp16(sum_m weights[m] * bit(input[m,r,z/bits], z%bits)), fp32 accumulation
    (extensions/booleanOperations.py:218-229, extensions/src/weighted_sum.cu:28-46).  ``input`` may be a
    :class:`FlipRows` (see :func:`weighted_sum_flip`).

    ``fast=False`` adds in member order, as the reference's kernel does.  ``fast=True`` adds the members in blocks
    (tables of partial sums over 8 members): the fp32 roundings fall elsewhere, a few 1e-7 of sum|weights| away from
    the member-order result and far inside the reference's own tolerance for this op (booloptests.py:284-285), about
    three times as fast."""
    if isinstance(input, FlipRows):
        return weighted_sum_flip(input, weights, zbits)
    assert len(input.shape) == 3
    assert input.size(0) == weights.size(0)
    _check(input, "input")
    _check(weights, "weights")
    _same_device(input, weights)
    assert weights.dtype == torch.float16 and len(weights.shape) == 1
    suf, bits = _suffix(input.dtype)
    assert zbits <= input.size(2) * bits
    ret = torch.empty((input.size(1), zbits), dtype=torch.float16, device=input.device)
    with _on(input):
        _lib.call("nb_weighted_sum" + ("_fast" if fast else "") + suf, ret.data_ptr(), input.data_ptr(),
                  weights.data_ptr(), input.size(0),
                  input.size(1), input.size(2), zbits, _stream(input))
    return ret


def center_fitness(weights):
    """fp16 [n]: ``w = weights.type(torch.float16); w - w.mean()`` (modules/binary.py:68-69) in one kernel.  The mean
    is the exact one of the fp16 values rounded once to fp16 (torch's own adds in fp32 and can land one fp16 step
    away when the exact mean sits next to the middle between two fp16 numbers)."""
    assert len(weights.shape) == 1
    _check(weights, "weights")
    if weights.dtype not in (torch.float16, torch.float32):
        weights = weights.type(torch.float16)
    weights = weights.contiguous()
    out = torch.empty(weights.shape, dtype=torch.float16, device=weights.device)
    with _on(weights):
        _lib.call("nb_center_fitness_f16" if weights.dtype == torch.float16 else "nb_center_fitness_f32",
                  out.data_ptr(), weights.data_ptr(), weights.numel(), _stream(weights))
    return out


def grad_regularize_(grad, weight, l1=0.0, l2=0.0):
    """In place ``grad += l1 * sign(weight)`` (if l1), then ``grad += l2 * weight`` (if l2), with the roundings of
    those fp16 tensor expressions (modules/binary.py:73-76), in one kernel.  Returns ``grad``."""
    assert grad.dtype == torch.float16 and weight.dtype == torch.float16 and grad.shape == weight.shape
    _check(grad, "grad")
    _check(weight, "weight")
    _same_device(grad, weight)
    assert grad.is_contiguous() and weight.is_contiguous()
    with _on(grad):
        _lib.call("nb_grad_regularize", grad.data_ptr(), weight.data_ptr(), float(l1), float(l2), grad.numel(),
                  _stream(grad))
    return grad


def bias_noise_scale_(uniform):
    """In place ``(uniform - .5) * 6`` with the roundings of that fp16 tensor expression (modules/binary.py:63-64), one
    kernel; returns its argument."""
    assert uniform.dtype == torch.float16 and uniform.is_contiguous()
    _check(uniform, "uniform")
    with _on(uniform):
        _lib.call("nb_bias_noise_scale", uniform.data_ptr(), uniform.numel(), _stream(uniform))
    return uniform


def bias_grad(centered, bias_noise):
    """fp16 [out] = ``centered @ bias_noise`` (modules/binary.py:77) with fp32 accumulation in a fixed order; centered
    fp16 [n], bias_noise fp16 [n, out]."""
    assert centered.dtype == torch.float16 and bias_noise.dtype == torch.float16
    assert len(centered.shape) == 1 and len(bias_noise.shape) == 2 and bias_noise.size(0) == centered.size(0)
    _check(centered, "centered")
    _check(bias_noise, "bias_noise")
    _same_device(centered, bias_noise)
    centered, bias_noise = centered.contiguous(), bias_noise.contiguous()
    out = torch.empty((bias_noise.size(1),), dtype=torch.float16, device=centered.device)
    with _on(centered):
        _lib.call("nb_bias_grad", out.data_ptr(), centered.data_ptr(), bias_noise.data_ptr(), centered.size(0),
                  bias_noise.size(1), _stream(centered))
    return out


def max_pool2d(input, filterx, filtery, padx, pady, stridex, stridey, REPEAT=128):
    """[D,H,W,Cw] -> [D,h,w,Cw], bitwise OR over a 2x2 window (extensions/booleanOperations.py:232-252).
    As in the reference kernel the window is always 2x2 (extensions/src/max_pool2d.cu:21-23); filterx and
    filtery only enter the output size.  ``REPEAT`` is accepted and ignored."""
    assert len(input.shape) == 4
    _check(input, "input")
    suf, _ = _suffix(input.dtype)
    h, w = _out_hw(input, filterx, filtery, padx, pady, stridex, stridey)
    out = torch.empty((input.size(0), h, w, input.size(3)), dtype=input.dtype, device=input.device)
    with _on(input):
        _lib.call("nb_max_pool2d" + suf, out.data_ptr(), input.data_ptr(), input.size(0), input.size(1), input.size(2),
                  input.size(3), filterx, filtery, padx, pady, stridex, stridey, _stream(input))
    return out


# ---- additions ----------------------------------------------------------------------------------
def unpack(input):
    """words [R,Rw] -> bool [R, Rw*bits] (boolutil_cuda.unpack, extensions/booleanUtilitiesCuda.cu:77-90,182-195)."""
    assert len(input.shape) == 2
    _check(input, "input")
    suf, bits = _suffix(input.dtype)
    ret = torch.empty((input.size(0), input.size(1) * bits), dtype=torch.bool, device=input.device)
    with _on(input):
        _lib.call("nb_unpack" + suf, ret.data_ptr(), input.data_ptr(), input.size(0), input.size(1), _stream(input))
    return ret


def thresholds_from_p(p):
    """Probabilities -> uint32 thresholds T with P(word < T) = T / 2**32 ~= p:
    T = min(floor(p * 2**32), 2**32 - 1), computed exactly in float64.  p = 1.0 therefore fails only
    for the single word 0xFFFFFFFF, like ``p > u`` with u in (0, 1] in the reference
    (extensions/src/sample_bits.cu:54)."""
    p = p.detach()
    if p.dtype == torch.float16 and p.is_cuda and p.is_contiguous():     # the layers' case: one kernel
        out = torch.empty(p.shape, dtype=torch.uint32, device=p.device)
        with _on(p):
            _lib.call("nb_thresholds_from_p", out.data_ptr(), p.data_ptr(), p.numel(), _stream(p))
        return out
    t = torch.floor(p.to(torch.float64) * 4294967296.0).clamp_(0.0, 4294967295.0)
    return t.to(torch.int64).to(torch.uint32)


def _thr_args(threshold, R, C, device):
    """-> (tensor kept alive or None, pointer or None, scalar)"""
    if isinstance(threshold, torch.Tensor):
        _check(threshold, "threshold")
        assert tuple(threshold.shape) == (R, C)
        if threshold.dtype != torch.uint32:
            raise TypeError("threshold tensor must be torch.uint32 (see thresholds_from_p)")
        if threshold.device != device:
            raise RuntimeError("Tensors are on different devices")
        return threshold, threshold.data_ptr(), 0
    t = int(threshold)
    if not 0 <= t <= 0xFFFFFFFF:
        raise ValueError("scalar threshold must fit in uint32")
    return None, None, t


def _words_check(words):
    _check(words, "words")
    assert len(words.shape) == 3
    if words.dtype not in (torch.uint32, torch.int32):
        raise TypeError("random words must be torch.uint32 (or int32 holding the same bit patterns)")


def _base_check(base, R, Rw, dtype, device):
    if base is None:
        return None
    _check(base, "base")
    assert tuple(base.shape) == (R, Rw) and base.dtype == dtype
    if base.device != device:
        raise RuntimeError("Tensors are on different devices")
    return base.data_ptr()


def _conv_outputs(conv_taps, rows_too, n, R, Rw, dtype, device):
    """-> (conv-layout tensor [n, KK*Rw, O], row-layout tensor [n, R, Rw] or None, O)"""
    KK = int(conv_taps)
    assert KK >= 1 and R % KK == 0, "the rows must be (out channel, tap) pairs: R = O * taps"
    O = R // KK
    conv = torch.empty((n, KK * Rw, O), dtype=dtype, device=device)
    rows = torch.empty((n, R, Rw), dtype=dtype, device=device) if rows_too else None
    return conv, rows, O


def sample_bits_from_words(threshold, words, dtype, base=None, conv_taps=None, rows_too=True):
    """ret[m,r,z] bit i = words[m,r,z*bits+i] < threshold[r,z*bits+i]  (threshold: uint32 [R,C] tensor or a
    Python int); with ``base`` ([R,Rw] packed) the result is ``base ^ mask``.

    ``conv_taps`` = kx*ky (not in the reference): the rows are a conv layer's (out channel, tap) pairs and the same
    kernel also writes the filters where the conv multiplies them, [n, kx*ky*Rw, O] (modules/binary.py:134-137 in
    the same pass); returns ``(rows_layout, conv_layout)``, the first ``None`` when ``rows_too`` is False."""
    _words_check(words)
    suf, bits = _suffix(dtype)
    n, R, C = words.shape
    keep, tptr, ts = _thr_args(threshold, R, C, words.device)
    Rw = ceil_div(C, bits)
    bptr = _base_check(base, R, Rw, dtype, words.device)
    if conv_taps is not None:
        conv, rows, O = _conv_outputs(conv_taps, rows_too, n, R, Rw, dtype, words.device)
        with _on(words):
            _lib.call("nb_sample_conv_from_words" + suf, conv.data_ptr(), None if rows is None else rows.data_ptr(), bptr,
                      tptr, ts, words.data_ptr(), n, O, int(conv_taps), C, _stream(words))
        return rows, conv
    ret = torch.empty((n, R, Rw), dtype=dtype, device=words.device)
    with _on(words):
        _lib.call("nb_sample_from_words" + suf, ret.data_ptr(), bptr, tptr, ts, words.data_ptr(), n, R, C,
                  _stream(words))
    return ret


def flip_from_words(base_packed, words, threshold):
    """Per-member weights = base XOR Bernoulli flip mask: ret[m] = base ^ pack(words[m] < threshold)."""
    return sample_bits_from_words(threshold, words, base_packed.dtype, base=base_packed)


def half_draws_apply(C, dtype, first=0, threshold=None):
    """Whether :func:`sample_bits_philox` can draw this shape from 16-bit half-words: rows of whole words, a stream
    offset that is a multiple of 8, and (tensor thresholds) 16-byte aligned ones."""
    bits = torch.iinfo(dtype).bits
    ok = C > 0 and C % bits == 0 and int(first) % 8 == 0
    if isinstance(threshold, torch.Tensor):
        ok = ok and threshold.data_ptr() % 16 == 0
    return ok


def sample_bits_philox(threshold, n, dtype, seed, subsequence=0, first=0, base=None, shape=None, conv_taps=None,
                       rows_too=True, half_draws=False):
    """Like :func:`sample_bits_from_words` with the words generated in-kernel: word (m,r,c) is element
    ``first + (m*R+r)*C + c`` of the Philox4x32-10 stream (seed, subsequence) -- exactly what
    :func:`philox_words` returns, so both forms agree bit for bit.

    ``half_draws=True``: the same law from 16-bit draws, two columns per generated word, with a second stream
    (subsequence ^ 2**63) deciding ties exactly (about 1.4 times as fast: the generator's instructions bound these
    samplers); other bits than the default draws from the same seed; shapes as :func:`half_draws_apply` says."""
    suf, bits = _suffix(dtype)
    if isinstance(threshold, torch.Tensor):
        R, C = threshold.shape
        device = threshold.device
    else:
        R, C = shape
        device = base.device if base is not None else torch.device("cuda", torch.cuda.current_device())
    keep, tptr, ts = _thr_args(threshold, R, C, device)
    Rw = ceil_div(C, bits)
    bptr = _base_check(base, R, Rw, dtype, device)
    if half_draws and not half_draws_apply(C, dtype, first, threshold if isinstance(threshold, torch.Tensor) else None):
        raise ValueError("16-bit draws take rows of whole words and a stream offset that is a multiple of 8")
    kind = "philox16" if half_draws else "philox"
    if conv_taps is not None:
        conv, rows, O = _conv_outputs(conv_taps, rows_too, n, R, Rw, dtype, device)
        with torch.cuda.device(device):
            _lib.call("nb_sample_conv_" + kind + suf, conv.data_ptr(), None if rows is None else rows.data_ptr(), bptr,
                      tptr, ts, int(seed) & (2 ** 64 - 1), int(subsequence), int(first), n, O, int(conv_taps), C,
                      torch.cuda.current_stream(device).cuda_stream)
        return rows, conv
    ret = torch.empty((n, R, Rw), dtype=dtype, device=device)
    with torch.cuda.device(device):
        _lib.call("nb_sample_" + kind + suf, ret.data_ptr(), bptr, tptr, ts, int(seed) & (2 ** 64 - 1),
                  int(subsequence), int(first), n, R, C, torch.cuda.current_stream(device).cuda_stream)
    return ret


def flip_philox(base_packed, in_bits, n, threshold, seed, subsequence=0, first=0):
    """base XOR in-kernel Philox flip mask; ``in_bits`` is the true column count C of a row."""
    return sample_bits_philox(threshold, n, base_packed.dtype, seed, subsequence, first, base=base_packed,
                              shape=(base_packed.size(0), in_bits))


def seeded_bmv_from_words(threshold, x_packed, words, base=None):
    """C[m,r] = sum_k popcount(w(m,r,k) ^ x[m,k]) with w = base ^ (words < threshold) never materialised
    (the fused op of boolop_cuda.binary_seeded_bmv, extensions/booleanOperationsCuda.cu:172-202)."""
    _words_check(words)
    _check(x_packed, "x_packed")
    suf, bits = _suffix(x_packed.dtype)
    n, R, C = words.shape
    Rw = ceil_div(C, bits)
    assert tuple(x_packed.shape) == (n, Rw)
    _same_device(words, x_packed)
    keep, tptr, ts = _thr_args(threshold, R, C, words.device)
    bptr = _base_check(base, R, Rw, x_packed.dtype, words.device)
    out = torch.empty((n, R), dtype=torch.int32, device=words.device)
    with _on(words):
        _lib.call("nb_seeded_bmv_from_words" + suf, out.data_ptr(), bptr, tptr, ts, x_packed.data_ptr(),
                  words.data_ptr(), n, R, C, _stream(words))
    return out


def seeded_bmv_philox(threshold, x_packed, rows, in_bits, seed, subsequence=0, first=0, base=None, half_draws=False):
    """:func:`seeded_bmv_from_words` with in-kernel Philox words.  ``half_draws=True``: the 16-bit draws of
    :func:`sample_bits_philox` (``in_bits`` and ``first`` multiples of 8): the product over exactly the weights that
    ``sample_bits_philox(..., half_draws=True)`` writes."""
    _check(x_packed, "x_packed")
    suf, bits = _suffix(x_packed.dtype)
    n = x_packed.size(0)
    R, C = rows, in_bits
    Rw = ceil_div(C, bits)
    assert tuple(x_packed.shape) == (n, Rw)
    keep, tptr, ts = _thr_args(threshold, R, C, x_packed.device)
    bptr = _base_check(base, R, Rw, x_packed.dtype, x_packed.device)
    out = torch.empty((n, R), dtype=torch.int32, device=x_packed.device)
    with _on(x_packed):
        _lib.call("nb_seeded_bmv_philox" + ("16" if half_draws else "") + suf, out.data_ptr(), bptr, tptr, ts,
                  x_packed.data_ptr(), int(seed) & (2 ** 64 - 1), int(subsequence), int(first), n, R, C,
                  _stream(x_packed))
    return out


def philox_words(count, seed, subsequence=0, first=0, device=None):
    """uint32 [count]: elements first..first+count-1 of the Philox4x32-10 stream (seed, subsequence)."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    out = torch.empty((count,), dtype=torch.uint32, device=device)
    with torch.cuda.device(device):
        _lib.call("nb_philox_words", out.data_ptr(), int(seed) & (2 ** 64 - 1), int(subsequence), int(first), count,
                  torch.cuda.current_stream(device).cuda_stream)
    return out


def conv_act_pack(input, filter, threshold, filterx, filtery, padx, pady, stridex, stridey, pool=False, in_bits=None,
                  filter_tap_packed=False):
    """pack(conv_act(...)) along the channel axis -> [D,h,w,ceil(O/bits)]; with ``pool`` followed by the
    2x2/stride-2 OR-pool -> [D,h//2,w//2,ceil(O/bits)].  One kernel; the bool map never reaches memory.
    ``in_bits`` / ``filter_tap_packed`` as in :func:`conv`."""
    _, word_bits = _suffix(input.dtype)
    Ow = ceil_div(filter.size(2), word_bits)
    out_dtype = input.dtype
    suf, bits, input, filter, tap = _conv_args(input, filter, filterx, filtery, in_bits, filter_tap_packed, out_words=Ow)
    _check(threshold, "threshold")
    _same_device(input, threshold)
    assert tuple(threshold.shape) == (input.size(0), filter.size(2))
    assert threshold.dtype == torch.int32
    h, w = _out_hw(input, filterx, filtery, padx, pady, stridex, stridey)
    shape = (input.size(0), h // 2, w // 2, Ow) if pool else (input.size(0), h, w, Ow)
    out = torch.empty(shape, dtype=out_dtype, device=input.device)
    with _on(input):
        _lib.call("nb_conv_act_pack" + suf, out.data_ptr(), input.data_ptr(), filter.data_ptr(), threshold.data_ptr(),
                  input.size(0), input.size(1), input.size(2), input.size(3), filter.size(2), filterx, filtery, padx,
                  pady, stridex, stridey, 1 if pool else 0, tap, _stream(input))
    return out


# ---- sparse form of a population's linear layer: shared base + per-member flip lists ----------------------------
_GEMM_TILE = 128                     # row padding of the expanded operands of bmm_nt (the matrix-core tile)


class ExpandedRows:
    """Packed rows [rows, Kw] expanded to FP4 codes (+1.0 / -1.0, zero padding) for :func:`bmm_nt`:
    ``codes`` is uint8 [rows_padded, 32 * Kw_padded]."""

    def __init__(self, codes, rows, Kw, rows_padded, Kw_padded):
        self.codes, self.rows, self.Kw, self.rows_padded, self.Kw_padded = codes, rows, Kw, rows_padded, Kw_padded


def expand_rows(x):
    """int64 [rows, Kw] packed bits -> :class:`ExpandedRows` (one pass, 16 bytes out per 32 bits in)."""
    _check(x, "x")
    assert len(x.shape) == 2
    if x.dtype != torch.int64:
        raise TypeError("expand_rows takes 64-bit words")
    rows, Kw = x.shape
    rp = ceil_div(rows, _GEMM_TILE) * _GEMM_TILE
    kp = max(2, ceil_div(Kw, 2) * 2)
    codes = torch.empty((rp, 32 * kp), dtype=torch.uint8, device=x.device)
    with _on(x):
        _lib.call("nb_expand_fp4_i64", codes.data_ptr(), x.data_ptr(), rows, Kw, rp, kp, _stream(x))
    return ExpandedRows(codes, rows, Kw, rp, kp)


def bmm_nt(A, B):
    """C[m, n] = popcount(A[m, :] ^ B[n, :]), int32 [M, N]: the XOR-popcount product of two row sets that share K
    (both K-contiguous), on the matrix cores.  A, B: int64 [M, Kw] / [N, Kw] or :class:`ExpandedRows`.  Equals
    ``bmm(A[None], B.t()[None])[0]`` of the reference op (extensions/booleanOperations.py:107-129)."""
    ea = A if isinstance(A, ExpandedRows) else expand_rows(A)
    eb = B if isinstance(B, ExpandedRows) else expand_rows(B)
    assert ea.Kw == eb.Kw and ea.Kw_padded == eb.Kw_padded
    if ea.codes.device != eb.codes.device:
        raise RuntimeError("Tensors are on different devices")
    C = torch.empty((ea.rows, eb.rows), dtype=torch.int32, device=ea.codes.device)
    with _on(ea.codes):
        _lib.call("nb_bmm_nt_fp4", C.data_ptr(), ea.codes.data_ptr(), eb.codes.data_ptr(), ea.rows, eb.rows, ea.Kw,
                  ea.rows_padded, eb.rows_padded, ea.Kw_padded, _stream(ea.codes))
    return C


class FlipRows:
    """Per-member weights of a linear layer, W[d] = base ^ flips[d], kept as the shared base and per-member flip
    lists (layout in include/nesbin.h: every row owns ``cap`` 16-byte pieces at a fixed place, ``info[d, r]`` says how
    many flips and pieces it has).  Built by :func:`flip_rows_from_weights`, :func:`flip_rows_skip` or
    :func:`flip_rows_thin`; ``bmm`` / ``bmv_act_pack`` / ``weighted_sum`` accept it where they take materialised
    weights, and return what they return on those."""

    def __init__(self, base, D, R, Kw, in_bits, info, entries, cap, overflow):
        self.base, self.D, self.R, self.Kw, self.in_bits = base, D, R, Kw, in_bits
        self.info, self.entries, self.cap, self.overflow = info, entries, cap, overflow
        self.base_expanded = expand_rows(base)

    @property
    def cnt(self):
        """Flips per row, int32 [D, R]."""
        return (self.info.view(torch.int32) & 0xFFFF)

    def overflowed(self):
        """Rows whose lists did not fit ``cap`` pieces (a device read-back; such rows were cut short)."""
        return int(self.overflow.item())

    # what the reference's layer code asks of weight_noise (modules/binary.py:97)
    def size(self, dim=None):
        shape = (self.D, self.R, self.Kw)
        return shape if dim is None else shape[dim]

    @property
    def shape(self):
        return (self.D, self.R, self.Kw)

    @property
    def dtype(self):
        return torch.int64

    @property
    def device(self):
        return self.base.device

    def nbytes(self):
        """Bytes one forward reads of the member-specific data (the pieces the rows have, and info)."""
        pieces = int((self.info.view(torch.int32) >> 16).sum().item())
        return pieces * 16 + self.info.numel() * 4


def _flip_alloc(D, R, cap, dev):
    S = ceil_div(R, 64)
    entries = torch.empty((max(D * S * cap * 256, 4),), dtype=torch.uint32, device=dev)
    info = torch.empty((D, R), dtype=torch.uint32, device=dev)
    overflow = torch.zeros((1,), dtype=torch.int32, device=dev).view(torch.uint32)
    return entries, info, overflow


def flip_capacity(in_bits, p, sigmas=8.0):
    """16-byte pieces per row that hold the flips of a row of ``in_bits`` columns at flip probability ``p`` with
    ``sigmas`` standard deviations to spare (a row beyond it is cut short and counted in ``FlipRows.overflow``)."""
    mean = in_bits * p
    need = mean + sigmas * math.sqrt(max(mean * (1.0 - p), 1.0)) + 8
    return int(min(ceil_div(int(math.ceil(min(need, in_bits))), 8), 8191))


def flip_rows_from_weights(W, base, cap=None):
    """W int64 [D, R, Kw] (a population's materialised weights), base int64 [R, Kw] -> :class:`FlipRows` holding
    exactly the bits W ^ base.  ``cap`` (pieces per row) defaults to what the longest row needs (one read-back)."""
    _check(W, "W")
    _check(base, "base")
    _same_device(W, base)
    assert len(W.shape) == 3 and len(base.shape) == 2
    if W.dtype != torch.int64 or base.dtype != torch.int64:
        raise TypeError("flip lists take 64-bit words")
    D, R, Kw = W.shape
    assert tuple(base.shape) == (R, Kw)
    dev = W.device
    if cap is None:
        info = torch.empty((D, R), dtype=torch.uint32, device=dev)
        with _on(W):
            _lib.call("nb_flip_count_i64", info.data_ptr(), W.data_ptr(), base.data_ptr(), D, R, Kw, _stream(W))
        cap = int((info.view(torch.int32) >> 16).max().item()) if D * R else 0
    entries, info, overflow = _flip_alloc(D, R, int(cap), dev)
    with _on(W):
        _lib.call("nb_flip_fill_i64", entries.data_ptr(), info.data_ptr(), overflow.data_ptr(), W.data_ptr(),
                  base.data_ptr(), D, R, Kw, int(cap), _stream(W))
    return FlipRows(base, D, R, Kw, 64 * Kw, info, entries, int(cap), overflow)


def skip_table(threshold, cap=4096):
    """Gap table of the skip sampler for flip probability p = threshold / 2**32 (uint32 numpy array): entry k-1 =
    floor(2**32 * (1 - (1-p)**k)) for k = 1, 2, ... until it saturates at 2**32 - 1 (at most ``cap`` entries); entry
    0 is ``threshold`` itself; empty for p = 0 (no flips).  A random word with ``rank`` entries <= it moves a row's
    walk on by rank + 1 columns to the next flip, or, beyond the table, by its length without a flip."""
    import numpy as np
    t = int(threshold)
    if not 0 <= t <= 0xFFFFFFFF:
        raise ValueError("threshold must fit in uint32")
    p = t / 4294967296.0
    if p <= 0.0:
        return np.zeros(0, dtype=np.uint32)
    k = np.arange(1, cap + 1, dtype=np.float64)
    v = np.minimum(np.floor(-np.expm1(k * np.log1p(-p)) * 4294967296.0), 4294967295.0)
    v[0] = float(t)
    v = np.maximum.accumulate(v)
    full = v >= 4294967295.0
    n = int(np.argmax(full)) + 1 if full.any() else cap
    return v[:n].astype(np.uint32)


_skip_tables = {}


def skip_table_buffer(table, device):
    """A gap table (uint32 numpy array, see :func:`skip_table`) as the kernels take it, in device memory:
    [entries, bits of the float 1 / log2(1 - p), p * 2**32, 0, table...]."""
    import numpy as np
    words = int(_lib.load().nb_skip_table_words())
    buf = np.zeros(words, dtype=np.uint32)
    n = int(table.size)
    assert n <= words - 4
    buf[0] = n
    p = (float(table[0]) / 4294967296.0) if n else 0.0
    hint = np.float32(1.0 / math.log2(1.0 - p)) if 0.0 < p < 1.0 else np.float32(0.0)
    buf[1] = np.frombuffer(hint.tobytes(), dtype=np.uint32)[0]
    buf[2] = table[0] if n else 0
    buf[4:4 + n] = table
    return torch.from_numpy(buf.view(np.int32)).to(device).view(torch.uint32)


def _skip_table_for(threshold, device):
    """The device table for a host threshold, made once per (threshold, device)."""
    key = (int(threshold), str(device))
    buf = _skip_tables.get(key)
    if buf is None:
        if len(_skip_tables) > 64:
            _skip_tables.clear()
        buf = _skip_tables[key] = skip_table_buffer(skip_table(threshold), device)
    return buf


def flip_rows_skip(base, in_bits, n, threshold, seed, subsequence=0, first=0, cap=None, table=None):
    """:class:`FlipRows` for ``n`` members drawn by the skip sampler: every bit of a member's [R, in_bits] weights
    differs from ``base`` with probability threshold / 2**32, independently, as with :func:`flip_philox`, but the
    generator only draws the gaps between flips (about in_bits * p + 1 words per row instead of in_bits), and the
    materialised weights never exist.  Row q = m*R + r consumes the Philox words first + q*in_bits + i of the stream
    (seed, subsequence).  The stream differs from :func:`flip_philox`'s: the law is the same, the bits are not.
    One kernel and nothing read back; ``cap``: pieces per row (default :func:`flip_capacity` of the probability);
    ``table``: a device table from :func:`skip_table_buffer` (default: made from ``threshold`` and kept)."""
    _check(base, "base")
    assert len(base.shape) == 2
    if base.dtype != torch.int64:
        raise TypeError("flip lists take 64-bit words")
    R, Kw = base.shape
    C = int(in_bits)
    assert ceil_div(C, 64) == Kw
    dev = base.device
    t = int(threshold)
    if table is None:
        table = _skip_table_for(t, dev)
    if cap is None:
        cap = flip_capacity(C, t / 4294967296.0)
    entries, info, overflow = _flip_alloc(n, R, int(cap), dev)
    with _on(base):
        _lib.call("nb_flip_skip_i64", entries.data_ptr(), info.data_ptr(), overflow.data_ptr(), base.data_ptr(),
                  table.data_ptr(), int(seed) & (2 ** 64 - 1), int(subsequence), int(first), n, R, C, int(cap),
                  _stream(base))
    return FlipRows(base, n, R, Kw, C, info, entries, int(cap), overflow)


SKIP_DENSE_MAX_WORDS = 8      # rows the dense form of the skip sampler takes (words per row)


def sample_bits_skip(threshold, n, dtype, seed, subsequence=0, first=0, base=None, shape=None, conv_taps=None,
                     rows_too=True, table=None):
    """The skip sampler's draw as packed words, for rows of at most ``SKIP_DENSE_MAX_WORDS`` words: every bit of a
    member's [R, C] tensor is set (or, with ``base`` [R, Rw], differs from it) with probability threshold / 2**32,
    independently, like :func:`sample_bits_philox` with a scalar threshold; the generator draws only the gaps between
    the set bits (about C*p + 1 words per row).  The bits are those of :func:`flip_rows_skip` with the same seed
    (``flip_rows_to_weights`` of its lists), not those of the per-bit samplers.  ``conv_taps`` as in
    :func:`sample_bits_from_words`: returns ``(rows_layout, conv_layout)``."""
    suf, bits = _suffix(dtype)
    if base is not None:
        device = base.device
        R = base.size(0)
        C = int(shape[1]) if shape is not None else base.size(1) * bits
    else:
        R, C = shape
        device = torch.device("cuda", torch.cuda.current_device())
    Rw = ceil_div(C, bits)
    if Rw > SKIP_DENSE_MAX_WORDS:
        raise ValueError("sample_bits_skip takes rows of at most %d words; use flip_rows_skip" % SKIP_DENSE_MAX_WORDS)
    bptr = _base_check(base, R, Rw, dtype, device)
    if table is None:
        table = _skip_table_for(int(threshold), device)
    key = (int(seed) & (2 ** 64 - 1), int(subsequence), int(first))
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device).cuda_stream
        if conv_taps is not None:
            conv, rows, O = _conv_outputs(conv_taps, rows_too, n, R, Rw, dtype, device)
            _lib.call("nb_sample_conv_skip" + suf, conv.data_ptr(), None if rows is None else rows.data_ptr(), bptr,
                      table.data_ptr(), *key, n, O, int(conv_taps), C, stream)
            return rows, conv
        ret = torch.empty((n, R, Rw), dtype=dtype, device=device)
        _lib.call("nb_sample_skip" + suf, ret.data_ptr(), bptr, table.data_ptr(), *key, n, R, C, stream)
    return ret


class FlipLaw:
    """The sparse form of a layer's per-element law: ``law`` uint16 [R, C] (bit 15 = base bit, bits 14:0 = the fp16
    pattern of the flip probability min(P, 1 - P)), ``base`` int64 [R, Kw] packed base bits, ``table`` the skip
    sampler's device table for the largest flip probability of the layer (``table[2]`` = that threshold)."""

    def __init__(self, law, base, table, in_bits):
        self.law, self.base, self.table, self.in_bits = law, base, table, in_bits
        self._layers = None

    def layers(self):
        """The law sorted for :func:`flip_rows_layered`, made on first use and kept: (``pl`` uint32 [R, C] = column |
        law << 16, the columns class by class; ``cls`` uint32 [R, 17], where each class starts).  One kernel."""
        if self._layers is None:
            R, C = self.law.shape
            pl = torch.empty((R, C), dtype=torch.uint32, device=self.law.device)
            cls = torch.empty((R, 17), dtype=torch.uint32, device=self.law.device)
            with _on(self.law):
                _lib.call("nb_flip_law_layers", pl.data_ptr(), cls.data_ptr(), self.law.data_ptr(), R, C,
                          _stream(self.law))
            self._layers = (pl, cls)
        return self._layers

    def stats(self):
        """(mean flip probability of the layer, largest mean of a row, largest flip probability): two small kernels
        and ONE device read-back."""
        R, C = self.law.shape
        out = torch.empty((3,), dtype=torch.float64, device=self.law.device)
        rows = torch.empty((R,), dtype=torch.float32, device=self.law.device)
        with _on(self.law):
            _lib.call("nb_flip_law_stats", out.data_ptr(), rows.data_ptr(), self.law.data_ptr(), self.table.data_ptr(),
                      R, C, _stream(self.law))
        mean, row, peak = out.tolist()
        return mean, row, peak

    def max_flip_probability(self):
        """The largest flip probability of the layer (a device read-back)."""
        return float(self.table[2:3].view(torch.int32).to(torch.int64).item() & 0xFFFFFFFF) / 4294967296.0

    def mean_flip_probability(self):
        """The mean flip probability of the layer (a device read-back)."""
        return float((self.law.view(torch.int16) & 0x7FFF).view(torch.float16).float().mean().item())


def _law_workspace(device):
    return torch.empty((int(_lib.load().nb_law_workspace_bytes()),), dtype=torch.uint8, device=device)


def thresholds_from_weights(weight):
    """Latent fp16 weights -> uint32 sampler thresholds of P = sigmoid(5 w / (mean|w| + 1e-5)) (modules/binary.py:59-60):
    the tensor expression's roundings, in two small kernels (partial sums of |w|, the law) instead of nine."""
    w = weight.detach()
    _check(w, "weight")
    assert w.dtype == torch.float16
    out = torch.empty(w.shape, dtype=torch.uint32, device=w.device)
    ws = _law_workspace(w.device)
    with _on(w):
        _lib.call("nb_thresholds_from_weights", out.data_ptr(), w.data_ptr(), w.numel(), ws.data_ptr(), _stream(w))
    return out


def probabilities_from_weights(weight):
    """Latent fp16 weights -> fp16 probabilities P = sigmoid(5 w / (mean|w| + 1e-5)) (modules/binary.py:59-60)."""
    w = weight.detach()
    _check(w, "weight")
    assert w.dtype == torch.float16
    out = torch.empty(w.shape, dtype=torch.float16, device=w.device)
    ws = _law_workspace(w.device)
    with _on(w):
        _lib.call("nb_probabilities_from_weights", out.data_ptr(), w.data_ptr(), w.numel(), ws.data_ptr(), _stream(w))
    return out


def flip_law_from_weights(weight):
    """Latent fp16 weights [R, C] -> :class:`FlipLaw` of P = sigmoid(5 w / (mean|w| + 1e-5)): base bit = P >= 1/2,
    flip probability min(P, 1 - P), and the skip sampler's table for the layer's largest flip probability, all made
    on the device (three kernels, nothing read back)."""
    w = weight.detach()
    _check(w, "weight")
    assert w.dtype == torch.float16 and len(w.shape) == 2
    R, C = w.shape
    law = torch.empty((R, C), dtype=torch.uint16, device=w.device)
    base = torch.empty((R, ceil_div(C, 64)), dtype=torch.int64, device=w.device)
    table = torch.empty((int(_lib.load().nb_skip_table_words()),), dtype=torch.uint32, device=w.device)
    ws = _law_workspace(w.device)
    with _on(w):
        _lib.call("nb_flip_law_from_weights", law.data_ptr(), base.data_ptr(), table.data_ptr(), w.data_ptr(), R, C,
                  ws.data_ptr(), _stream(w))
    return FlipLaw(law, base, table, C)


def flip_rows_thin(law, n, seed, cap, subsequence=0, first=0):
    """:class:`FlipRows` for ``n`` members under a per-element law (:class:`FlipLaw`): the skip sampler walks at the
    layer's largest flip probability and a column it reaches flips with probability (its own) / (the largest), decided
    by the second word of a pair, so that every bit differs from the base with its own probability, independently.
    ``cap``: pieces per row (see :func:`flip_capacity`; rows beyond it are counted in ``overflow``)."""
    R, C = law.law.shape
    dev = law.law.device
    entries, info, overflow = _flip_alloc(n, R, int(cap), dev)
    with _on(law.law):
        _lib.call("nb_flip_skip_thin_i64", entries.data_ptr(), info.data_ptr(), overflow.data_ptr(), law.law.data_ptr(),
                  law.table.data_ptr(), int(seed) & (2 ** 64 - 1), int(subsequence), int(first), n, R, C, int(cap),
                  _stream(law.law))
    return FlipRows(law.base, n, R, law.base.size(1), C, info, entries, int(cap), overflow)


_layer_tables = {}


def layer_tables(device):
    """The 16 gap tables of :func:`flip_rows_layered` in device memory (constants: made once per device and kept)."""
    device = torch.device(device)
    key = (device.type, torch.cuda.current_device() if device.index is None else device.index)
    buf = _layer_tables.get(key)
    if buf is None:
        buf = torch.empty((int(_lib.load().nb_flip_layer_table_words()),), dtype=torch.uint32, device=device)
        with _on(buf):
            _lib.call("nb_flip_layer_tables", buf.data_ptr(), _stream(buf))
        _layer_tables[key] = buf
    return buf


def flip_rows_layered(law, n, seed, cap, subsequence=0, first=0):
    """:class:`FlipRows` for ``n`` members under a per-element law (:class:`FlipLaw`), for laws with a long tail: the
    columns of a row are walked class by class (classes by the binary size of the flip probability, 2**-(k+2) < y <=
    2**-(k+1)), each class at its own rate 2**-(k+1), so that a row costs about two word pairs per flip whatever the
    layer's largest probability is, where :func:`flip_rows_thin` pays for that largest one in every column.  Same
    law (every bit differs from the base with its own probability, independently), other masks.  For sparse laws:
    a row owns C words of the stream and uses two per step (about 1.5 steps per flip plus 16); a row that needs more
    than its C words reads on into the next row's."""
    R, C = law.law.shape
    dev = law.law.device
    pl, cls = law.layers()
    tables = layer_tables(dev)
    entries, info, overflow = _flip_alloc(n, R, int(cap), dev)
    with _on(law.law):
        _lib.call("nb_flip_skip_layered_i64", entries.data_ptr(), info.data_ptr(), overflow.data_ptr(), pl.data_ptr(),
                  cls.data_ptr(), tables.data_ptr(), int(seed) & (2 ** 64 - 1), int(subsequence), int(first), n, R, C,
                  int(cap), _stream(law.law))
    return FlipRows(law.base, n, R, law.base.size(1), C, info, entries, int(cap), overflow)


def flip_rows_to_weights(rows):
    """:class:`FlipRows` -> the materialised weights int64 [D, R, Kw] = base ^ flips (for the dense kernels, and for
    checking the two forms against each other)."""
    W = rows.base.unsqueeze(0).expand(rows.D, rows.R, rows.Kw).contiguous()
    with _on(W):
        _lib.call("nb_flip_to_dense_i64", W.data_ptr(), rows.entries.data_ptr(), rows.info.data_ptr(), rows.D, rows.R,
                  rows.Kw, rows.cap, _stream(W))
    return W


def _flip_args(rows, x, G):
    _check(x, "x")
    if x.dtype != torch.int64:
        raise TypeError("flip lists take 64-bit words")
    assert x.numel() == rows.D * rows.Kw and x.size(0) == rows.D
    if x.device != rows.entries.device:
        raise RuntimeError("Tensors are on different devices")
    if G is None:
        G = bmm_nt(x.view(rows.D, rows.Kw), rows.base_expanded)       # the shared product popcount(x_d ^ base_r)
    else:
        _check(G, "G")
        assert tuple(G.shape) == (rows.D, rows.R) and G.dtype == torch.int32
    return G


def bmv_flip(rows, x, G=None):
    """int32 [D, R]: sum_k popcount(W[d, r, k] ^ x[d, k]) for the weights held by ``rows`` (:class:`FlipRows`); what
    ``bmm(W, x.view(D, Kw, 1)).squeeze(2)`` gives on the materialised weights."""
    G = _flip_args(rows, x, G)
    out = torch.empty((rows.D, rows.R), dtype=torch.int32, device=x.device)
    with _on(x):
        _lib.call("nb_bmv_flip_i64", out.data_ptr(), G.data_ptr(), rows.entries.data_ptr(), rows.info.data_ptr(),
                  x.data_ptr(), rows.D, rows.R, rows.Kw, rows.cap, _stream(x))
    return out


def bmv_flip_act_pack(rows, x, threshold, G=None):
    """Packed bits (2 * sum > threshold[d, r]) as int64 [D, ceil(R/64)]: what ``bmv_act_pack(W, x, threshold)`` gives
    on the materialised weights."""
    G = _flip_args(rows, x, G)
    _check(threshold, "threshold")
    assert tuple(threshold.shape) == (rows.D, rows.R) and threshold.dtype == torch.int32
    out = torch.empty((rows.D, ceil_div(rows.R, 64)), dtype=torch.int64, device=x.device)
    with _on(x):
        _lib.call("nb_bmv_flip_act_pack_i64", out.data_ptr(), G.data_ptr(), rows.entries.data_ptr(),
                  rows.info.data_ptr(), x.data_ptr(), threshold.data_ptr(), rows.D, rows.R, rows.Kw, rows.cap,
                  _stream(x))
    return out


def weighted_sum_flip(rows, weights, zbits):
    """``weighted_sum`` over flip lists: fp16 [R, zbits] = sum_d weights[d] * bit_d with bit = base ^ flip; reads two
    bytes per flip instead of a bit per weight.  The additions are exact (integers after scaling by a power of two), so
    the result is the correctly rounded sum up to that scaling, whatever the order; ``weighted_sum`` on the
    materialised weights adds in fp32 in member order, and the two agree to fp32 rounding of the partial sums."""
    _check(weights, "weights")
    assert weights.dtype == torch.float16 and tuple(weights.shape) == (rows.D,)
    if weights.device != rows.entries.device:
        raise RuntimeError("Tensors are on different devices")
    assert zbits <= rows.Kw * 64
    out = torch.empty((rows.R, zbits), dtype=torch.float16, device=weights.device)
    with _on(weights):
        _lib.call("nb_flip_weighted_sum_i64", out.data_ptr(), rows.entries.data_ptr(), rows.info.data_ptr(),
                  rows.base.data_ptr(), weights.data_ptr(), rows.D, rows.R, int(zbits), rows.cap, _stream(weights))
    return out
