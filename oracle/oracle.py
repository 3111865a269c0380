"""TEST INFRASTRUCTURE ONLY: numpy front-end of the C oracle (``libnesbin_oracle.so``).

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import
this module.  Every function takes and returns numpy arrays; packed words are ``int64`` or
``int32`` arrays holding the bit patterns (LSB-first, extensions/src/pack.cu:26).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force=False):
    """Compile the oracle with gcc (a few hundred ms)."""
    so = os.path.join(_HERE, "libnesbin_oracle.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libnesbin_oracle.so"])
    return so


def lib():
    global _LIB
    if _LIB is None:
        name = os.environ.get("NESBIN_ORACLE_LIB") or build()
        _LIB = ctypes.CDLL(name)
    return _LIB


def _suf(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.int64 or dtype == np.uint64:
        return "i64", 64, np.int64
    if dtype == np.int32 or dtype == np.uint32:
        return "i32", 32, np.int32
    raise TypeError("word dtype must be int64 or int32, got %r" % (dtype,))


def _p(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else ctypes.c_void_p(0)


def _c(a, dtype=None):
    a = np.ascontiguousarray(a) if dtype is None else np.ascontiguousarray(a, dtype=dtype)
    return a


def _i64(v):
    return ctypes.c_int64(int(v))


def out_hw(H, W, fx, fy, px, py, sx, sy):
    """Output size formula of booleanOperations.py:83-84."""
    return (H - fx + 2 * px) // sx + 1, (W - fy + 2 * py) // sy + 1


def pack(bits, dtype=np.int64):
    suf, wb, wt = _suf(dtype)
    bits = _c(bits).view(np.uint8)
    R, C = bits.shape
    out = np.empty((R, (C + wb - 1) // wb), dtype=wt)
    getattr(lib(), "nbo_pack_" + suf)(_p(out), _p(bits), _i64(R), _i64(C))
    return out


def unpack(words):
    suf, wb, _ = _suf(words.dtype)
    words = _c(words)
    R, Rw = words.shape
    out = np.empty((R, Rw * wb), dtype=np.uint8)
    getattr(lib(), "nbo_unpack_" + suf)(_p(out), _p(words), _i64(R), _i64(Rw))
    return out.view(np.bool_)


def int8pack(data, dtype=np.int64):
    suf, wb, wt = _suf(dtype)
    data = _c(data, np.uint8)
    R, C = data.shape
    per = wb // 8
    out = np.empty((R, (C + per - 1) // per), dtype=wt)
    getattr(lib(), "nbo_int8pack_" + suf)(_p(out), _p(data), _i64(R), _i64(C))
    return out


def batch_im2col(x, fx, fy, px, py, sx, sy):
    suf, _, wt = _suf(x.dtype)
    x = _c(x)
    B, H, W, Cw = x.shape
    h, w = out_hw(H, W, fx, fy, px, py, sx, sy)
    out = np.empty((B, h * w, fx * fy * Cw), dtype=wt)
    getattr(lib(), "nbo_im2col_" + suf)(_p(out), _p(x), _i64(B), _i64(H), _i64(W), _i64(Cw),
                                         fx, fy, px, py, sx, sy)
    return out


def bmm(A, B):
    suf, _, _ = _suf(A.dtype)
    A, B = _c(A), _c(B)
    assert A.dtype == B.dtype and A.ndim == 3 and B.ndim == 3
    Z, M, K = A.shape
    assert B.shape[0] == Z and B.shape[1] == K
    N = B.shape[2]
    out = np.empty((Z, M, N), dtype=np.int32)
    getattr(lib(), "nbo_bmm_" + suf)(_p(out), _p(A), _p(B), _i64(Z), _i64(M), _i64(K), _i64(N))
    return out


def bmm_act(A, B, thresh):
    suf, _, _ = _suf(A.dtype)
    A, B, thresh = _c(A), _c(B), _c(thresh, np.int32)
    Z, M, K = A.shape
    N = B.shape[2]
    assert thresh.shape == (Z, N)
    out = np.empty((Z, M, N), dtype=np.uint8)
    getattr(lib(), "nbo_bmm_act_" + suf)(_p(out), _p(A), _p(B), _p(thresh), _i64(Z), _i64(M), _i64(K), _i64(N))
    return out.view(np.bool_)


def conv(x, filt, fx, fy, px, py, sx, sy):
    suf, _, _ = _suf(x.dtype)
    x, filt = _c(x), _c(filt)
    D, H, W, Cw = x.shape
    O = filt.shape[2]
    assert filt.shape[:2] == (D, fx * fy * Cw) and filt.dtype == x.dtype
    h, w = out_hw(H, W, fx, fy, px, py, sx, sy)
    out = np.empty((D, h, w, O), dtype=np.int32)
    getattr(lib(), "nbo_conv_" + suf)(_p(out), _p(x), _p(filt), _i64(D), _i64(H), _i64(W), _i64(Cw), _i64(O),
                                       fx, fy, px, py, sx, sy)
    return out


def conv_act(x, filt, thresh, fx, fy, px, py, sx, sy):
    suf, _, _ = _suf(x.dtype)
    x, filt, thresh = _c(x), _c(filt), _c(thresh, np.int32)
    D, H, W, Cw = x.shape
    O = filt.shape[2]
    h, w = out_hw(H, W, fx, fy, px, py, sx, sy)
    out = np.empty((D, h, w, O), dtype=np.uint8)
    getattr(lib(), "nbo_conv_act_" + suf)(_p(out), _p(x), _p(filt), _p(thresh), _i64(D), _i64(H), _i64(W),
                                           _i64(Cw), _i64(O), fx, fy, px, py, sx, sy)
    return out.view(np.bool_)


def max_pool2d(x, fx, fy, px, py, sx, sy):
    suf, _, wt = _suf(x.dtype)
    x = _c(x)
    B, H, W, Cw = x.shape
    h, w = out_hw(H, W, fx, fy, px, py, sx, sy)
    out = np.empty((B, h, w, Cw), dtype=wt)
    getattr(lib(), "nbo_max_pool2d_" + suf)(_p(out), _p(x), _i64(B), _i64(H), _i64(W), _i64(Cw),
                                             fx, fy, px, py, sx, sy)
    return out


def _thr_args(thresh):
    if np.isscalar(thresh) or (isinstance(thresh, np.ndarray) and thresh.ndim == 0):
        return None, ctypes.c_uint32(int(thresh))
    return _c(thresh, np.uint32), ctypes.c_uint32(0)


def sample_from_words(thresh, words, dtype=np.int64, base=None):
    """bit = words[m,r,c] < thresh[r,c] (or a scalar); optional base [R,Rw] is XORed on."""
    suf, wb, wt = _suf(dtype)
    words = _c(words, np.uint32)
    n, R, C = words.shape
    tarr, tsc = _thr_args(thresh)
    if tarr is not None:
        assert tarr.shape == (R, C)
    if base is not None:
        base = _c(base)
        assert base.dtype == wt and base.shape == (R, (C + wb - 1) // wb)
    out = np.empty((n, R, (C + wb - 1) // wb), dtype=wt)
    getattr(lib(), "nbo_sample_from_words_" + suf)(_p(out), _p(base), _p(tarr), tsc, _p(words),
                                                    _i64(n), _i64(R), _i64(C))
    return out


def seeded_bmv_from_words(thresh, x, words, base=None):
    suf, wb, wt = _suf(x.dtype)
    x = _c(x)
    words = _c(words, np.uint32)
    n, R, C = words.shape
    assert x.shape == (n, (C + wb - 1) // wb)
    tarr, tsc = _thr_args(thresh)
    if base is not None:
        base = _c(base)
        assert base.dtype == wt
    out = np.empty((n, R), dtype=np.int32)
    getattr(lib(), "nbo_seeded_bmv_from_words_" + suf)(_p(out), _p(base), _p(tarr), tsc, _p(x), _p(words),
                                                        _i64(n), _i64(R), _i64(C))
    return out


def weighted_sum(words, w, zbits):
    suf, _, _ = _suf(words.dtype)
    words = _c(words)
    w = _c(w, np.float32)
    n, R, Rw = words.shape
    out = np.empty((R, zbits), dtype=np.float32)
    getattr(lib(), "nbo_weighted_sum_" + suf)(_p(out), _p(words), _p(w), _i64(n), _i64(R), _i64(Rw), _i64(zbits))
    return out


def philox4x32_10(ctr, key):
    ctr = _c(ctr, np.uint32)
    key = _c(key, np.uint32)
    out = np.empty(4, dtype=np.uint32)
    lib().nbo_philox4x32_10(_p(out), _p(ctr), _p(key))
    return out


def philox_words(seed, subseq, first, count):
    out = np.empty(int(count), dtype=np.uint32)
    lib().nbo_philox_words(_p(out), ctypes.c_uint64(int(seed)), ctypes.c_uint64(int(subseq)),
                           ctypes.c_uint64(int(first)), _i64(count))
    return out


def skip_cdf(T, cap=4096):
    """Gap table of the skip sampler for flip probability p = T / 2**32: entry k-1 = floor(2**32 * (1 - (1-p)**k)),
    k = 1, 2, ... until the table saturates at 2**32 - 1 (at most ``cap`` entries; a word beyond a table cut short
    moves the walk on without a flip); entry 0 is T itself.  The same
    formula as the product's ``skip_table`` (the table is INPUT DATA of the contract, not part of it)."""
    p = int(T) / 4294967296.0
    if p <= 0.0:
        return np.zeros(0, dtype=np.uint32)                 # the empty table stands for "no flips"
    k = np.arange(1, cap + 1, dtype=np.float64)
    v = np.floor(-np.expm1(k * np.log1p(-p)) * 4294967296.0) if p < 1.0 else np.full(cap, 4294967295.0)
    v = np.minimum(v, 4294967295.0)
    v[0] = float(min(int(T), 4294967295))
    v = np.maximum.accumulate(v)
    n = int(np.argmax(v >= 4294967295.0)) + 1 if (v >= 4294967295.0).any() else cap
    return v[:n].astype(np.uint32)


def sample_philox16(thresh, n, R, C, seed, subseq=0, first=0, dtype=np.int64, base=None):
    """Packed [n, R, ceil(C/bits)] draws from 16-bit half-words (see nbo_draws16): ``thresh`` uint32 [R, C] or a
    scalar; optional base [R, Rw] is XORed on."""
    suf, wb, wt = _suf(dtype)
    tarr, tsc = _thr_args(thresh)
    if tarr is not None:
        assert tarr.shape == (R, C)
    bits = np.empty((int(n) * int(R), int(C)), dtype=np.uint8)
    lib().nbo_draws16(_p(bits), _p(tarr), tsc, ctypes.c_uint64(int(seed)), ctypes.c_uint64(int(subseq)),
                      ctypes.c_uint64(int(first)), _i64(n * R), _i64(R), _i64(C))
    pad = (-int(C)) % wb
    words = np.packbits(np.pad(bits, ((0, 0), (0, pad))), axis=1, bitorder="little").view(wt).reshape(int(n), int(R), -1)
    if base is not None:
        words = words ^ _c(base)[None]
    return np.ascontiguousarray(words)


def skip_flips(cdf, seed, subseq, first, rows, C):
    """Flip masks [rows, ceil(C/64)] int64 by gap sampling (see nbo_skip_flips_i64)."""
    cdf = _c(cdf, np.uint32)
    out = np.empty((int(rows), (int(C) + 63) // 64), dtype=np.int64)
    lib().nbo_skip_flips_i64(_p(out), _p(cdf), _i64(cdf.shape[0]), ctypes.c_uint64(int(seed)),
                             ctypes.c_uint64(int(subseq)), ctypes.c_uint64(int(first)), _i64(rows), _i64(C))
    return out


def skip_flips_thin(law, cdf, tmax, seed, subseq, first, D):
    """Flip masks [D*R, ceil(C/64)] int64 under the per-element law ``law`` uint16 [R, C], by thinning (see
    nbo_skip_flips_thin_i64)."""
    law = _c(law, np.uint16)
    cdf = _c(cdf, np.uint32)
    R, C = law.shape
    out = np.empty((int(D) * R, (C + 63) // 64), dtype=np.int64)
    lib().nbo_skip_flips_thin_i64(_p(out), _p(law), _p(cdf), _i64(cdf.shape[0]), ctypes.c_uint32(int(tmax)),
                                  ctypes.c_uint64(int(seed)), ctypes.c_uint64(int(subseq)), ctypes.c_uint64(int(first)),
                                  _i64(D), _i64(R), _i64(C))
    return out


LAYERS, LAYER_TABLE = 16, 512


def law_thresholds(law):
    """Flip thresholds Tf = floor(y * 2**32) (at most 2**32 - 256) of a uint16 law array: y = the fp16 number of bits
    14:0."""
    y = (_c(law, np.uint16) & 0x7FFF).view(np.float16).astype(np.float32)
    return np.minimum(y * np.float32(4294967296.0), np.float32(4294967040.0)).astype(np.uint32)


def law_layers(law):
    """The per-element law uint16 [R, C] sorted for the class-by-class walk (see nbo_skip_flips_layered_i64):
    (pl uint32 [R, C], cls uint32 [R, 17]).  Class of a column: k with 2**(30-k) < Tf <= 2**(31-k), at most 15;
    Tf == 0: left out (the tail of pl holds 0xFFFF)."""
    law = _c(law, np.uint16)
    R, C = law.shape
    tf = law_thresholds(law).astype(np.int64)
    k = np.full((R, C), LAYERS, dtype=np.int64)
    nz = tf > 0
    # bit length of (tf - 1): clz32 = 32 - bit_length
    bl = np.zeros((R, C), dtype=np.int64)
    v = np.maximum(tf - 1, 0)
    for b in range(32):
        bl = np.where(v >> b, b + 1, bl)
    k[nz] = np.clip(32 - bl[nz] - 1, 0, LAYERS - 1)
    order = np.argsort(k, axis=1, kind="stable")
    ks = np.take_along_axis(k, order, axis=1)
    pl = (order.astype(np.uint32) | (np.take_along_axis(law, order, axis=1).astype(np.uint32) << 16))
    pl = np.where(ks == LAYERS, np.uint32(0xFFFF), pl).astype(np.uint32)
    cls = np.stack([(ks < c).sum(axis=1) for c in range(LAYERS + 1)], axis=1).astype(np.uint32)
    return np.ascontiguousarray(pl), np.ascontiguousarray(cls)


def layer_tables(cap=LAYER_TABLE):
    """The 16 gap tables of the class-by-class walk: (cdfs uint32 [16, cap], kts int32 [16]); class k's table is the
    first ``cap`` entries of skip_cdf(2**(31-k))."""
    cdfs = np.full((LAYERS, cap), 0xFFFFFFFF, dtype=np.uint32)
    kts = np.zeros(LAYERS, dtype=np.int32)
    for k in range(LAYERS):
        t = skip_cdf(1 << (31 - k), cap=cap)
        kts[k] = t.shape[0]
        cdfs[k, :t.shape[0]] = t
    return cdfs, kts


def skip_flips_layered(pl, cls, seed, subseq, first, D, tables=None):
    """Flip masks [D*R, ceil(C/64)] int64 under a per-element law sorted by law_layers (see
    nbo_skip_flips_layered_i64)."""
    pl, cls = _c(pl, np.uint32), _c(cls, np.uint32)
    R, C = pl.shape
    cdfs, kts = layer_tables() if tables is None else tables
    cdfs, kts = _c(cdfs, np.uint32), _c(kts, np.int32)
    out = np.empty((int(D) * R, (C + 63) // 64), dtype=np.int64)
    lib().nbo_skip_flips_layered_i64(_p(out), _p(pl), _p(cls), _p(cdfs), _p(kts), _i64(cdfs.shape[1]),
                                     ctypes.c_uint64(int(seed)), ctypes.c_uint64(int(subseq)),
                                     ctypes.c_uint64(int(first)), _i64(D), _i64(R), _i64(C))
    return out


def flip_law(P):
    """fp16 probabilities [R, C] -> (law uint16 [R, C], base bool [R, C], tmax): base = P >= 1/2, flip probability
    y = min(P, 1 - P) (exact in fp16), law = base << 15 | fp16 bits of y, tmax = the largest floor(y * 2**32)."""
    P = np.asarray(P, dtype=np.float16)
    p32 = P.astype(np.float32)
    base = p32 >= 0.5
    y = np.where(base, np.float32(1.0) - p32, p32).astype(np.float16)
    assert (y.astype(np.float32) == np.where(base, np.float32(1.0) - p32, p32)).all()
    law = (y.view(np.uint16) & 0x7FFF) | (base.astype(np.uint16) << 15)
    tf = np.minimum(y.astype(np.float64) * 4294967296.0, 4294967040.0).astype(np.uint64)
    return law.astype(np.uint16), base, int(tf.max()) if tf.size else 0


def max_threads():
    return int(lib().nbo_max_threads())


def set_threads(n):
    lib().nbo_set_threads(int(n))
