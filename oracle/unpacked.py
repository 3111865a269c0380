"""TEST INFRASTRUCTURE ONLY: a second, independent CPU statement of the same ops on UNPACKED
bits with numpy / torch-CPU library routines.  It shares no code with the C oracle and is what
the C oracle is pinned against: where the C oracle walks packed words with index arithmetic,
this file uses ``numpy.packbits``, integer matmul on +-1 values, ``torch.conv2d`` and
``torch.nn.functional.max_pool2d`` -- the formulations the reference's own check script uses
as ground truth (booloptests.py:94-95,101-102,150-160).
"""
import numpy as np


def _wbits(dtype):
    return np.dtype(dtype).itemsize * 8


def pack_bits(bits, dtype=np.int64):
    """bool [R, C] -> words [R, ceil(C/bits)], LSB-first, zero tail."""
    bits = np.asarray(bits).astype(np.uint8)
    wb = _wbits(dtype)
    R, C = bits.shape
    Rw = (C + wb - 1) // wb
    padded = np.zeros((R, Rw * wb), dtype=np.uint8)
    padded[:, :C] = bits != 0
    by = np.packbits(padded, axis=1, bitorder="little")          # [R, Rw*wb/8] bytes
    le = np.dtype(dtype).newbyteorder("<")
    return np.ascontiguousarray(by).view(le).astype(dtype).reshape(R, Rw)


def unpack_bits(words):
    """words [R, Rw] -> bool [R, Rw*bits]."""
    words = np.ascontiguousarray(words)
    le = words.astype(words.dtype.newbyteorder("<"))
    by = le.view(np.uint8).reshape(words.shape[0], -1)
    return np.unpackbits(by, axis=1, bitorder="little").astype(bool)


def popc_bmm_bits(a_bits, b_bits):
    """a_bits [Z,M,K] bool, b_bits [Z,K,N] bool -> number of positions where they differ.

    With x = 2a-1 and w = 1-2b (the reference's sign convention, booloptests.py:150,152)
    sum_k x*w = 2*popc(a^b) - K  (booloptests.py:160)."""
    x = 2 * a_bits.astype(np.int64) - 1
    w = 1 - 2 * b_bits.astype(np.int64)
    K = a_bits.shape[2]
    dot = np.einsum("zmk,zkn->zmn", x, w)
    assert np.all((dot + K) % 2 == 0)
    return ((dot + K) // 2).astype(np.int32)


def conv_popc_torch(in_bits, filt_bits, pad, stride):
    """Reference ground truth for conv (booloptests.py:150-155,160).

    in_bits   bool [D, H, W, C] (channels last)
    filt_bits bool [D, O, fx, fy, C]
    returns popc int32 [D, h, w, O] recovered from the +-1 grouped conv:
        2*popc - fx*fy*C == conv2d(pad(x, value=-1), -filter, groups=D)."""
    import torch
    D, H, W, C = in_bits.shape
    _, O, fx, fy, _ = filt_bits.shape
    x = torch.from_numpy(2.0 * (in_bits.astype(np.float64) - 0.5))
    x = x.permute(0, 3, 1, 2).contiguous().view(1, D * C, H, W)
    f = torch.from_numpy(-2.0 * (filt_bits.astype(np.float64) - 0.5))
    f = f.permute(0, 1, 4, 2, 3).contiguous().view(D * O, C, fx, fy)
    x = torch.nn.functional.pad(x, (pad,) * 4, value=-1.0)
    r = torch.conv2d(x, f, stride=(stride, stride), groups=D)
    r = r.view(D, O, r.shape[-2], r.shape[-1]).permute(0, 2, 3, 1)
    K = fx * fy * C
    popc2 = r + K
    out = (popc2 / 2).round().to(torch.int32).numpy()
    assert np.array_equal(out * 2 - K, r.numpy().astype(np.int64))
    return out


def im2col_bits(in_bits, fx, fy, px, py, sx, sy):
    """bool [B,H,W,C] -> bool [B, h*w, fx*fy*C] in (tap row i, tap col j, channel) order with
    zero fill, built by explicit padding and strided slicing (no index formula)."""
    B, H, W, C = in_bits.shape
    h = (H - fx + 2 * px) // sx + 1
    w = (W - fy + 2 * py) // sy + 1
    # pad generously on the far side so every strided slice is in range
    padded = np.zeros((B, H + 2 * px + fx, W + 2 * py + fy, C), dtype=bool)
    padded[:, px:px + H, py:py + W, :] = in_bits
    taps = []
    for i in range(fx):
        for j in range(fy):
            taps.append(padded[:, i:i + (h - 1) * sx + 1:sx, j:j + (w - 1) * sy + 1:sy, :])
    cols = np.stack(taps, axis=3)                                   # [B,h,w,fx*fy,C]
    return cols.reshape(B, h * w, fx * fy * C)


def max_pool_bits_torch(in_bits, k=2, pad=0, stride=2):
    """booloptests.py:94-95 -- F.max_pool2d on the bits as floats (pad value is -inf there,
    which for 0/1 data equals OR with zero fill)."""
    import torch
    x = torch.from_numpy(in_bits.astype(np.float32)).permute(0, 3, 1, 2)
    r = torch.nn.functional.max_pool2d(x, (k, k), (stride, stride), (pad, pad), (1, 1))
    return r.permute(0, 2, 3, 1).numpy() > 0.5


def or_pool2x2_bits(in_bits, fx, fy, px, py, sx, sy):
    """OR over the 2x2 window anchored at (xo*sx-px, yo*sy-py), zero outside; output size from
    the (fx, fy) formula -- the behaviour of extensions/src/max_pool2d.cu:14-32."""
    B, H, W, C = in_bits.shape
    h = (H - fx + 2 * px) // sx + 1
    w = (W - fy + 2 * py) // sy + 1
    big = np.zeros((B, px + max(H, (h - 1) * sx + 2) + 2, py + max(W, (w - 1) * sy + 2) + 2, C), dtype=bool)
    big[:, px:px + H, py:py + W, :] = in_bits
    out = np.zeros((B, h, w, C), dtype=bool)
    for i in range(2):
        for j in range(2):
            out |= big[:, i:i + (h - 1) * sx + 1:sx, j:j + (w - 1) * sy + 1:sy, :]
    return out
