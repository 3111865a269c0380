"""Pins the C oracle (oracle/nesbin_oracle.c) against independent statements of the same
arithmetic: numpy.packbits, +-1 integer matmul, torch.conv2d / max_pool2d in the form the
reference's check script uses (booloptests.py:94-163), brute force and special cases.
CPU only."""
import itertools

import numpy as np
import pytest

from oracle import unpacked as U

WORD_DTYPES = [np.int64, np.int32]


def rng(seed):
    return np.random.default_rng(seed)


@pytest.mark.parametrize("dtype", WORD_DTYPES)
@pytest.mark.parametrize("R,C", [(1, 1), (3, 3), (5, 31), (4, 32), (7, 33), (2, 63), (9, 64), (3, 65),
                                 (6, 127), (5, 128), (2, 200), (1, 1024), (17, 576)])
def test_pack_matches_packbits_and_roundtrips(oracle, dtype, R, C):
    bits = rng(R * 1000 + C).integers(0, 2, size=(R, C)).astype(bool)
    got = oracle.pack(bits, dtype)
    assert got.dtype == dtype
    np.testing.assert_array_equal(got, U.pack_bits(bits, dtype))
    un = oracle.unpack(got)
    wb = np.dtype(dtype).itemsize * 8
    assert un.shape == (R, got.shape[1] * wb)
    np.testing.assert_array_equal(un[:, :C], bits)
    assert not un[:, C:].any()                      # zero tail (pack.cu:17)
    np.testing.assert_array_equal(un, U.unpack_bits(got))


def test_pack_bit_order_and_sign_bit(oracle):
    # bit i of word y is column y*bits+i (pack.cu:26); bit 63 makes the int64 negative
    bits = np.zeros((1, 128), dtype=bool)
    bits[0, 0] = True
    bits[0, 63] = True
    bits[0, 64 + 5] = True
    w = oracle.pack(bits, np.int64)
    assert w[0, 0] == np.int64(-(2 ** 63) + 1)
    assert w[0, 1] == 32
    w32 = oracle.pack(bits, np.int32)
    assert list(w32[0]) == [1, -(2 ** 31), 32, 0]


@pytest.mark.parametrize("dtype", WORD_DTYPES)
def test_int8pack_is_little_endian_view(oracle, dtype):
    per = np.dtype(dtype).itemsize
    for R, C in [(3, 1), (2, per), (4, per + 3), (5, 3 * per)]:
        data = rng(C).integers(0, 256, size=(R, C)).astype(np.uint8)
        Rw = (C + per - 1) // per
        padded = np.zeros((R, Rw * per), dtype=np.uint8)
        padded[:, :C] = data
        want = padded.view(np.dtype(dtype).newbyteorder("<")).astype(dtype)
        np.testing.assert_array_equal(oracle.int8pack(data, dtype), want)


@pytest.mark.parametrize("dtype", WORD_DTYPES)
@pytest.mark.parametrize("Z,M,K,N", [(1, 1, 1, 1), (3, 5, 7, 2), (2, 33, 70, 9), (4, 16, 64, 1), (2, 1, 130, 35),
                                     (5, 9, 200, 3)])
def test_bmm_matches_pm1_matmul(oracle, dtype, Z, M, K, N):
    g = rng(Z + 10 * M + 100 * K + N)
    a = g.integers(0, 2, size=(Z, M, K)).astype(bool)
    b = g.integers(0, 2, size=(Z, K, N)).astype(bool)
    A = U.pack_bits(a.reshape(Z * M, K), dtype).reshape(Z, M, -1)
    # B is [Z, Kw, N]: pack along K for every (z, n), then put N last
    Bp = U.pack_bits(b.transpose(0, 2, 1).reshape(Z * N, K), dtype).reshape(Z, N, -1).transpose(0, 2, 1)
    got = oracle.bmm(A, np.ascontiguousarray(Bp))
    want = U.popc_bmm_bits(a, b)
    np.testing.assert_array_equal(got, want)
    # brute force: number of differing positions
    brute = (a[:, :, :, None] != b[:, None, :, :]).sum(axis=2).astype(np.int32)
    np.testing.assert_array_equal(got, brute)


@pytest.mark.parametrize("dtype", WORD_DTYPES)
def test_bmm_special_cases(oracle, dtype):
    wb = np.dtype(dtype).itemsize * 8
    g = rng(7)
    K = 2 * wb + 5
    a = g.integers(0, 2, size=(3, 6, K)).astype(bool)
    A = U.pack_bits(a.reshape(18, K), dtype).reshape(3, 6, -1)
    Kw = A.shape[2]
    zeros = np.zeros((3, Kw, 4), dtype=dtype)
    # B == 0: popc counts the ones of A
    np.testing.assert_array_equal(oracle.bmm(A, zeros), np.repeat(a.sum(2)[:, :, None], 4, axis=2))
    # A == B: 0 ; B == ~A on the valid bits: K
    same = np.ascontiguousarray(A[:, 2:3, :].transpose(0, 2, 1))
    assert np.all(oracle.bmm(A[:, 2:3, :], same) == 0)
    inv = U.pack_bits(~a.reshape(18, K), dtype).reshape(3, 6, -1)
    invb = np.ascontiguousarray(inv[:, 2:3, :].transpose(0, 2, 1))
    assert np.all(oracle.bmm(A[:, 2:3, :], invb) == K)
    # all-ones words against zero: full word width per word (bit 63 / sign bit counted)
    ones = np.full((1, 1, 3), -1, dtype=dtype)
    assert oracle.bmm(ones, np.zeros((1, 3, 1), dtype=dtype))[0, 0, 0] == 3 * wb


@pytest.mark.parametrize("dtype", WORD_DTYPES)
def test_bmm_act_is_threshold_of_bmm(oracle, dtype):
    g = rng(11)
    Z, M, K, N = 3, 10, 150, 7
    A = g.integers(-2 ** 31, 2 ** 31, size=(Z, M, 3)).astype(dtype)
    B = g.integers(-2 ** 31, 2 ** 31, size=(Z, 3, N)).astype(dtype)
    popc = oracle.bmm(A, B)
    thr = (g.integers(0, 2 * popc.max() + 3, size=(Z, N)) - 1).astype(np.int32)
    got = oracle.bmm_act(A, B, thr)
    np.testing.assert_array_equal(got, 2 * popc > thr[:, None, :])     # booloptests.py:157-159
    assert got.any() and not got.all()


SWEEP = list(itertools.product([1, 3, 7], [0, 1, 2], [1, 2, 3]))      # booloptests.py:122-124


@pytest.mark.parametrize("dtype", WORD_DTYPES)
@pytest.mark.parametrize("C", [1, 3, 16, 64, 70])
def test_conv_sweep_matches_torch_grouped_conv(oracle, dtype, C):
    """The reference's own identity (booloptests.py:150-160) over its sweep of filter size x
    padding x stride, on a 10x10 input (booloptests.py:116)."""
    D, O, S = 3, 5, 10
    for fs, pad, stride in SWEEP:
        g = rng(fs * 100 + pad * 10 + stride + C)
        xb = g.integers(0, 2, size=(D, S, S, C)).astype(bool)
        fb = g.integers(0, 2, size=(D, O, fs, fs, C)).astype(bool)
        xp = U.pack_bits(xb.reshape(-1, C), dtype).reshape(D, S, S, -1)
        fp = U.pack_bits(fb.reshape(-1, C), dtype).reshape(D, O, fs, fs, -1)
        # modules/binary.py:136-137 / booloptests.py:62: [D,O,fx,fy,Cw] -> [D, fx*fy*Cw, O]
        fr = np.ascontiguousarray(fp.transpose(0, 2, 3, 4, 1).reshape(D, -1, O))
        got = oracle.conv(xp, fr, fs, fs, pad, pad, stride, stride)
        want = U.conv_popc_torch(xb, fb, pad, stride)
        np.testing.assert_array_equal(got, want, err_msg=str((fs, pad, stride)))
        K = fs * fs * C
        thr = (g.integers(0, K, size=(D, O)) - K // 2 + K).astype(np.int32)   # booloptests.py:130,133
        act = oracle.conv_act(xp, fr, thr, fs, fs, pad, pad, stride, stride)
        np.testing.assert_array_equal(act, 2 * want > thr[:, None, None, :])


@pytest.mark.parametrize("dtype", WORD_DTYPES)
def test_im2col_matches_slicing_and_1x1_conv_is_bmm(oracle, dtype):
    g = rng(5)
    B, H, W, C = 2, 6, 9, 70
    xb = g.integers(0, 2, size=(B, H, W, C)).astype(bool)
    xp = U.pack_bits(xb.reshape(-1, C), dtype).reshape(B, H, W, -1)
    Cw = xp.shape[3]
    wb = np.dtype(dtype).itemsize * 8
    for fx, fy, px, py, sx, sy in [(3, 3, 1, 1, 1, 1), (1, 1, 0, 0, 1, 1), (2, 3, 0, 2, 2, 1), (3, 2, 2, 0, 1, 3),
                                   (5, 5, 2, 2, 2, 2)]:
        got = oracle.batch_im2col(xp, fx, fy, px, py, sx, sy)
        cols_bits = U.im2col_bits(xb, fx, fy, px, py, sx, sy)             # [B, hw, taps*C]
        hw = cols_bits.shape[1]
        # pack per tap so that the word layout is (tap, channel word)
        per_tap = cols_bits.reshape(B * hw * fx * fy, C)
        want = U.pack_bits(per_tap, dtype).reshape(B, hw, fx * fy * Cw)
        np.testing.assert_array_equal(got, want)
    # 1x1 / no pad / stride 1: im2col is the identity reshape, conv is bmm
    filt = g.integers(-2 ** 31, 2 ** 31, size=(B, Cw, 4)).astype(dtype)
    filt &= np.array(-1, dtype=dtype)  # any bits: padding bits of the input are zero anyway
    np.testing.assert_array_equal(oracle.batch_im2col(xp, 1, 1, 0, 0, 1, 1), xp.reshape(B, H * W, Cw))
    np.testing.assert_array_equal(oracle.conv(xp, filt, 1, 1, 0, 0, 1, 1).reshape(B, H * W, 4),
                                  oracle.bmm(xp.reshape(B, H * W, Cw), filt))
    assert wb in (32, 64)


@pytest.mark.parametrize("dtype", WORD_DTYPES)
def test_max_pool_matches_torch_and_or_window(oracle, dtype):
    g = rng(3)
    for C in [1, 16, 64, 100]:
        for S in [10, 7]:
            xb = g.integers(0, 2, size=(3, S, S, C)).astype(bool)
            xp = U.pack_bits(xb.reshape(-1, C), dtype).reshape(3, S, S, -1)
            # booloptests.py:138-141: 2x2 stride 2 no padding against F.max_pool2d
            got = oracle.max_pool2d(xp, 2, 2, 0, 0, 2, 2)
            want_bits = U.max_pool_bits_torch(xb)
            want = U.pack_bits(want_bits.reshape(-1, C), dtype).reshape(got.shape)
            np.testing.assert_array_equal(got, want)
            for fx, fy, px, py, sx, sy in [(2, 2, 1, 1, 2, 2), (2, 2, 0, 1, 1, 2), (3, 3, 1, 1, 2, 2), (2, 2, 0, 0, 1, 1),
                                           (2, 2, 1, 0, 3, 3)]:
                got = oracle.max_pool2d(xp, fx, fy, px, py, sx, sy)
                wb_ = U.or_pool2x2_bits(xb, fx, fy, px, py, sx, sy)
                want = U.pack_bits(wb_.reshape(-1, C), dtype).reshape(got.shape)
                np.testing.assert_array_equal(got, want, err_msg=str((C, S, fx, fy, px, py, sx, sy)))
    # padded torch pooling agrees where the 2x2 window is what the caller asked for
    xb = g.integers(0, 2, size=(2, 8, 8, 5)).astype(bool)
    xp = U.pack_bits(xb.reshape(-1, 5), dtype).reshape(2, 8, 8, -1)
    got = oracle.max_pool2d(xp, 2, 2, 1, 1, 2, 2)
    want = U.pack_bits(U.max_pool_bits_torch(xb, 2, 1, 2).reshape(-1, 5), dtype).reshape(got.shape)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("dtype", WORD_DTYPES)
@pytest.mark.parametrize("n,R,C", [(3, 4, 64), (2, 3, 1), (5, 2, 63), (2, 5, 65), (3, 2, 200), (1, 1, 256)])
def test_sample_from_words_closed_form(oracle, dtype, n, R, C):
    g = rng(n * 7 + R * 3 + C)
    words = g.integers(0, 2 ** 32, size=(n, R, C), dtype=np.uint64).astype(np.uint32)
    thr = g.integers(0, 2 ** 32, size=(R, C), dtype=np.uint64).astype(np.uint32)
    got = oracle.sample_from_words(thr, words, dtype)
    want = U.pack_bits((words < thr[None]).reshape(n * R, C), dtype).reshape(n, R, -1)
    np.testing.assert_array_equal(got, want)
    # scalar threshold + base (flip form): weights = base ^ mask
    T = 214748364                                              # floor(0.05 * 2**32)
    base_bits = g.integers(0, 2, size=(R, C)).astype(bool)
    base = U.pack_bits(base_bits, dtype)
    got = oracle.sample_from_words(T, words, dtype, base=base)
    want = U.pack_bits(((words < T) ^ base_bits[None]).reshape(n * R, C), dtype).reshape(n, R, -1)
    np.testing.assert_array_equal(got, want)
    # edge thresholds: 0 never fires; 2**32-1 fires unless the word is 0xFFFFFFFF
    assert not oracle.sample_from_words(0, words, dtype).any()
    allw = np.full((1, 1, C), 0xFFFFFFFF, dtype=np.uint32)
    assert not oracle.sample_from_words(0xFFFFFFFF, allw, dtype).any()


def test_sample_rate_is_p(oracle):
    g = rng(0)
    words = g.integers(0, 2 ** 32, size=(64, 16, 256), dtype=np.uint64).astype(np.uint32)
    for p in [0.01, 0.02, 0.05, 0.5]:
        T = int(p * 2 ** 32)
        m = oracle.sample_from_words(T, words, np.int64)
        rate = U.unpack_bits(m.reshape(-1, 4)).mean()
        assert abs(rate - p) < 4 * np.sqrt(p * (1 - p) / words.size) + 1e-4


@pytest.mark.parametrize("dtype", WORD_DTYPES)
@pytest.mark.parametrize("n,R,C", [(3, 4, 64), (4, 7, 100), (2, 3, 31), (2, 2, 300)])
def test_seeded_bmv_equals_materialised(oracle, dtype, n, R, C):
    g = rng(C)
    words = g.integers(0, 2 ** 32, size=(n, R, C), dtype=np.uint64).astype(np.uint32)
    xb = g.integers(0, 2, size=(n, C)).astype(bool)
    x = U.pack_bits(xb, dtype)
    base = U.pack_bits(g.integers(0, 2, size=(R, C)).astype(bool), dtype)
    T = int(0.05 * 2 ** 32)
    thr = g.integers(0, 2 ** 32, size=(R, C), dtype=np.uint64).astype(np.uint32)
    for kw in [dict(thresh=T, base=base), dict(thresh=thr, base=None), dict(thresh=thr, base=base)]:
        W = oracle.sample_from_words(kw["thresh"], words, dtype, base=kw["base"])
        want = oracle.bmm(W, x.reshape(n, -1, 1))[:, :, 0]
        got = oracle.seeded_bmv_from_words(kw["thresh"], x, words, base=kw["base"])
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("dtype", WORD_DTYPES)
def test_weighted_sum_matches_einsum(oracle, dtype):
    g = rng(2)
    n, R, C = 37, 5, 100
    bits = g.integers(0, 2, size=(n, R, C)).astype(bool)
    words = U.pack_bits(bits.reshape(n * R, C), dtype).reshape(n, R, -1)
    w = g.standard_normal(n).astype(np.float32)
    got = oracle.weighted_sum(words, w, C)
    want = np.einsum("n,nrc->rc", w.astype(np.float64), bits.astype(np.float64))
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)


def test_skip_flips_against_searchsorted_and_the_geometric_law(oracle):
    """Gap sampling of flip masks (the skip sampler's contract): the C restatement against an independent numpy
    evaluation (searchsorted + cumsum over the Philox words, which the known-answer vectors pin), then what the law
    fixes: flip rate p, geometric gap frequencies, no correlation between neighbouring columns."""
    T = int(0.03 * 2 ** 32)
    cdf = oracle.skip_cdf(T)
    assert cdf[0] == T and cdf[-1] == 2 ** 32 - 1 and (np.diff(cdf.astype(np.int64)) >= 0).all()
    p = T / 2.0 ** 32
    np.testing.assert_allclose(cdf[:50] / 2.0 ** 32, 1 - (1 - p) ** np.arange(1, 51), atol=2 ** -31)
    for rows, C, first in [(7, 200, 0), (3, 64, 5), (5, 1, 2), (4, 1000, 4 * 0xFFFFFFFF)]:
        seed, sub = 0xABCDEF0123, 9
        got = oracle.skip_flips(cdf, seed, sub, first, rows, C)
        bits = np.unpackbits(got.view(np.uint8), axis=1, bitorder="little")[:, :((C + 63) // 64) * 64]
        assert not bits[:, C:].any()
        for q in range(rows):
            words = oracle.philox_words(seed, sub, first + q * C, C)
            rank = np.searchsorted(cdf, words, side="right").astype(np.int64)
            pos = np.cumsum(np.where(rank < len(cdf), rank + 1, len(cdf))) - 1
            want = np.zeros(bits.shape[1], np.uint8)
            want[pos[(pos < C) & (rank < len(cdf))]] = 1
            np.testing.assert_array_equal(bits[q], want, err_msg="rows=%d C=%d row %d" % (rows, C, q))
    rows, C = 400, 4096
    bits = np.unpackbits(oracle.skip_flips(cdf, 1, 2, 0, rows, C).view(np.uint8), axis=1, bitorder="little")
    assert abs(bits.mean() - p) < 4 * np.sqrt(p * (1 - p) / bits.size)
    assert abs(bits[:, 0].mean() - p) < 5 * np.sqrt(p / rows)                    # the first gap starts before column 0
    cols = [np.flatnonzero(r) for r in bits]
    gaps = np.concatenate([np.diff(c) for c in cols])
    for k in range(1, 6):
        expect = (1 - p) ** (k - 1) * p
        assert abs((gaps == k).mean() - expect) < 5 * np.sqrt(expect / gaps.size), k
    a, b = bits[:, :-1].astype(np.float64), bits[:, 1:].astype(np.float64)
    assert abs((a * b).mean() - p * p) < 5 * p / np.sqrt(a.size)                 # neighbours independent
    # a table cut short of saturation (tiny p): words beyond it move on without a flip, the rate stays p
    T2 = 2 ** 32 // 5000
    short = oracle.skip_cdf(T2, cap=64)
    assert len(short) == 64 and short[-1] < 2 ** 32 - 1
    got = oracle.skip_flips(short, 5, 1, 0, 300, 3000)
    b2 = np.unpackbits(got.view(np.uint8), axis=1, bitorder="little")[:, :3000]
    assert abs(b2.mean() - 1 / 5000) < 5 * np.sqrt(1 / 5000 / b2.size)
    words = oracle.philox_words(5, 1, 7 * 3000, 3000)
    rank = np.searchsorted(short, words, side="right").astype(np.int64)
    pos = np.cumsum(np.where(rank < 64, rank + 1, 64)) - 1
    want = np.zeros(3000, np.uint8)
    want[pos[(pos < 3000) & (rank < 64)]] = 1
    np.testing.assert_array_equal(b2[7], want)
    # p = 1: every column flips (one word in 2**32 would skip one); p = 0: none
    ones = oracle.skip_flips(oracle.skip_cdf(2 ** 32 - 1), 3, 0, 0, 4, 130)
    assert np.unpackbits(ones.view(np.uint8), axis=1, bitorder="little")[:, :130].all()
    assert not oracle.skip_flips(oracle.skip_cdf(0), 3, 0, 0, 4, 130).any()


def test_skip_flips_thin_against_a_numpy_walk_and_the_per_column_law(oracle):
    """Thinned gap sampling (per-element flip probabilities): the C restatement against an independent evaluation
    (searchsorted + cumsum over the pinned Philox words, the acceptance in Python integers), then what the law fixes:
    every column flips at its own rate, neighbouring columns are uncorrelated, and a law whose probabilities all equal
    the largest one accepts everything, i.e. reduces to the plain walk over the pairs' first words."""
    g = np.random.default_rng(77)
    R, C, D = 3, 500, 4
    # probabilities on both sides of 1/2, most of them near 0 or 1: flip probabilities of a few percent
    P = np.where(g.random((R, C)) < 0.5, g.random((R, C)) * 0.06, 1.0 - g.random((R, C)) * 0.06).astype(np.float16)
    law, base, tmax = oracle.flip_law(P)
    assert ((law >> 15).astype(bool) == (P.astype(np.float32) >= 0.5)).all()
    y = (law & 0x7FFF).view(np.float16).astype(np.float64)
    np.testing.assert_array_equal(y, np.minimum(P.astype(np.float64), 1.0 - P.astype(np.float64)))
    tf = np.floor(y * 2.0 ** 32).astype(np.uint64)
    assert tmax == int(tf.max())
    cdf = oracle.skip_cdf(tmax)
    seed, sub = 0x1234567, 3
    for first in (0, 6, 1):
        got = oracle.skip_flips_thin(law, cdf, tmax, seed, sub, first, D)
        bits = np.unpackbits(got.view(np.uint8), axis=1, bitorder="little")
        assert not bits[:, C:].any()
        for q in range(D * R):
            words = oracle.philox_words(seed, sub, first + q * C, 2 * C + 2)
            gap, acc = words[0::2], words[1::2]
            rank = np.searchsorted(cdf, gap, side="right").astype(np.int64)
            pos = np.cumsum(np.where(rank < len(cdf), rank + 1, len(cdf))) - 1
            want = np.zeros(bits.shape[1], np.uint8)
            for i in np.flatnonzero((pos < C) & (rank < len(cdf))):
                if int(acc[i]) * tmax < (int(tf[q % R, pos[i]]) << 32):
                    want[pos[i]] = 1
            np.testing.assert_array_equal(bits[q], want, err_msg="first=%d row %d" % (first, q))
    # rates: many members of one row whose probabilities come in two levels
    R2, C2, D2 = 1, 256, 6000
    y2 = np.where(np.arange(C2) % 2 == 0, 0.05, 0.0125).astype(np.float16)
    law2, _, tmax2 = oracle.flip_law(y2[None, :])
    bits = np.unpackbits(oracle.skip_flips_thin(law2, oracle.skip_cdf(tmax2), tmax2, 9, 0, 0, D2).view(np.uint8),
                         axis=1, bitorder="little")[:, :C2].astype(np.float64)
    p2 = y2.astype(np.float64)
    rate = bits.mean(axis=0)
    assert (np.abs(rate - p2) < 5 * np.sqrt(p2 * (1 - p2) / D2)).all()
    assert abs(rate[0::2].mean() - p2[0]) < 4 * np.sqrt(p2[0] / (D2 * C2 / 2))
    assert abs(rate[1::2].mean() - p2[1]) < 4 * np.sqrt(p2[1] / (D2 * C2 / 2))
    a, b = bits[:, :-1], bits[:, 1:]
    assert abs((a * b).mean() - p2[0] * p2[1]) < 5 * np.sqrt(p2[0] * p2[1] / a.size)      # neighbours independent
    # all probabilities equal to the largest: every column the walk reaches flips
    y3 = np.full((2, 300), 0.03, dtype=np.float16)
    law3, _, tmax3 = oracle.flip_law(y3)
    cdf3 = oracle.skip_cdf(tmax3)
    got = np.unpackbits(oracle.skip_flips_thin(law3, cdf3, tmax3, 5, 2, 0, 3).view(np.uint8), axis=1, bitorder="little")
    for q in range(6):
        gap = oracle.philox_words(5, 2, q * 300, 600)[0::2]
        rank = np.searchsorted(cdf3, gap, side="right").astype(np.int64)
        pos = np.cumsum(np.where(rank < len(cdf3), rank + 1, len(cdf3))) - 1
        want = np.zeros(got.shape[1], np.uint8)
        want[pos[(pos < 300) & (rank < len(cdf3))]] = 1
        np.testing.assert_array_equal(got[q], want)


def _fp16_law(y):
    """uint16 law (base bit 0) of flip probabilities y <= 1/2."""
    return np.ascontiguousarray(np.asarray(y, dtype=np.float16)).view(np.uint16) & np.uint16(0x7FFF)


def test_skip_flips_layered_against_thinning_a_numpy_walk_and_the_per_column_law(oracle):
    """The class-by-class walk.  (1) The sort: classes from the thresholds' binary size, by Python integers.  (2) A row
    whose columns share one class k is the thinned walk (pinned above) with class k's table and tmax = 2^(31-k): same
    words, same columns.  (3) Mixed rows against an evaluation in numpy, one searchsorted + cumsum per class over the
    pinned Philox words, each class starting at the pair after the one that ended the class before.  (4) What the law
    fixes: every column flips at its own rate across five orders of magnitude, neighbours uncorrelated."""
    g = np.random.default_rng(5)
    cdfs, kts = oracle.layer_tables()
    assert cdfs.shape == (16, 512) and kts[0] < 40 and (kts[5:] == 512).all()
    # (1) the sort
    y = np.concatenate([[0.0, 0.5, 0.25, 0.25 + 2 ** -12, 2.0 ** -16, 2.0 ** -17, 2.0 ** -24, 6e-8, 0.3, 0.0],
                        g.random(54) * 0.5 * 10.0 ** -g.integers(0, 6, 54)])
    law = _fp16_law(y)[None, :]
    pl, cls = oracle.law_layers(law)
    tf = [int(min(float(np.float16(v)) * 2.0 ** 32, 4294967040.0)) for v in y]
    def klass(t):
        for k in range(15):
            if (1 << (30 - k)) < t <= (1 << (31 - k)):
                return k
        return 15 if t > 0 else 16
    ks = [klass(t) for t in tf]
    assert klass(1 << 31) == 0 and klass((1 << 30) + 1) == 0 and klass(1 << 30) == 1 and klass(1) == 15
    want = sorted(range(len(y)), key=lambda c: (ks[c], c))
    n_live = sum(k < 16 for k in ks)
    assert [int(e & 0xFFFF) for e in pl[0, :n_live]] == want[:n_live]
    assert all(int(pl[0, i] >> 16) == int(law[0, want[i]]) for i in range(n_live))
    assert (pl[0, n_live:] == 0xFFFF).all()
    assert [int(c) for c in cls[0]] == [sum(k < c for k in ks) for c in range(17)]
    # (2) one class per row: the thinned walk with the class's table
    C, D = 333, 3
    for k in (0, 1, 3, 6, 11, 15):
        lo = 2.0 ** -(k + 2) * (1 + 2.0 ** -9) if k < 15 else 2.0 ** -24   # the boundary itself is class k + 1
        yk = (lo + (2.0 ** -(k + 1) - lo) * g.random((2, C))).astype(np.float16)
        yk[0, :5] = 2.0 ** -(k + 1)                                      # the class's upper end: always accepted
        lawk = _fp16_law(yk)
        plk, clsk = oracle.law_layers(lawk)
        assert (clsk[:, k] == 0).all() and (clsk[:, k + 1] == C).all(), k
        for first in (0, 3):
            got = oracle.skip_flips_layered(plk, clsk, 11, 2, first, D)
            thin = oracle.skip_flips_thin(lawk, cdfs[k, :kts[k]], 1 << (31 - k), 11, 2, first, D)
            np.testing.assert_array_equal(got, thin, err_msg="class %d first %d" % (k, first))
    # (3) mixed rows
    R, C, D = 3, 700, 3
    y = (g.random((R, C)) * 0.5 * 10.0 ** -g.integers(0, 5, (R, C))).astype(np.float16)
    y[1, ::7] = 0.0
    law = _fp16_law(y)
    pl, cls = oracle.law_layers(law)
    tfs = oracle.law_thresholds(law).astype(np.uint64)
    seed, sub = 0xABCDE, 1
    for first in (0, 2, 5):
        got = np.unpackbits(oracle.skip_flips_layered(pl, cls, seed, sub, first, D).view(np.uint8), axis=1,
                            bitorder="little")
        assert not got[:, C:].any()
        for q in range(D * R):
            r = q % R
            words = oracle.philox_words(seed, sub, first + q * C, 2 * C + 64)
            want = np.zeros(got.shape[1], np.uint8)
            at = 0                                                        # pairs used so far
            for k in range(16):
                s0, s1 = int(cls[r, k]), int(cls[r, k + 1])
                if s1 == s0:
                    continue
                gap, acc = words[2 * at::2], words[2 * at + 1::2]
                cdf = cdfs[k, :kts[k]]
                rank = np.searchsorted(cdf, gap, side="right").astype(np.int64)
                pos = np.cumsum(np.where(rank < len(cdf), rank + 1, len(cdf))) - 1
                used = int(np.argmax(pos >= s1 - s0)) + 1                 # the pair that leaves the class is used up
                for i in range(used - 1):
                    if rank[i] < len(cdf):
                        col = int(pl[r, s0 + pos[i]] & 0xFFFF)
                        if int(acc[i]) < (int(tfs[r, col]) << (k + 1)):
                            want[col] = 1
                at += used
            np.testing.assert_array_equal(got[q], want, err_msg="first=%d row %d" % (first, q))
    # (4) rates
    C2, D2 = 256, 20000
    levels = np.array([0.4, 0.11, 0.03, 0.004, 0.0003, 0.26, 0.0625, 0.001], dtype=np.float16)
    y2 = levels[np.arange(C2) % 8]
    pl2, cls2 = oracle.law_layers(_fp16_law(y2)[None, :])
    bits = np.unpackbits(oracle.skip_flips_layered(pl2, cls2, 9, 0, 0, D2).view(np.uint8), axis=1,
                         bitorder="little")[:, :C2].astype(np.float64)
    p2 = y2.astype(np.float64)
    rate = bits.mean(axis=0)
    assert (np.abs(rate - p2) < 5 * np.sqrt(p2 * (1 - p2) / D2)).all()
    for j in range(8):
        pj = float(levels[j])
        assert abs(rate[j::8].mean() - pj) < 4.5 * np.sqrt(pj * (1 - pj) / (D2 * C2 / 8)), j
    a, b = bits[:, 0::8], bits[:, 5::8]                                   # columns of the same class (0.4 and 0.26)
    pa, pb = float(levels[0]), float(levels[5])
    assert abs((a * b).mean() - pa * pb) < 5 * np.sqrt(pa * pb / a.size)
    a, b = bits[:, 1::8], bits[:, 2::8]                                   # of neighbouring classes
    pa, pb = float(levels[1]), float(levels[2])
    assert abs((a * b).mean() - pa * pb) < 5 * np.sqrt(pa * pb / a.size)


def test_draws16_against_a_numpy_evaluation_ties_and_rates(oracle):
    """Bernoulli draws from 16-bit half-words: the C restatement against an evaluation in numpy from the pinned
    Philox words (first stream: half-words; second stream, subsequence ^ 2**63: the tie-breaking low halves), with
    thresholds chosen so that a third of the columns tie; then what the law fixes: P(bit) = T / 2**32 also where T
    has a non-zero low half, and the two halves of one word give uncorrelated bits."""
    seed, sub = 0xC0FFEE, 7
    n, R, C = 3, 5, 96
    for first in (0, 8, 5):
        g = first + np.arange(n * R * C, dtype=np.uint64)
        w1 = oracle.philox_words(seed, sub, first // 2, (n * R * C + 3) // 2 + 2)
        e = (g >> np.uint64(1)) - np.uint64(first // 2)
        w = w1[e.astype(np.int64)]
        h = np.where(g & np.uint64(1), w >> np.uint32(16), w & np.uint32(0xFFFF)).astype(np.uint32).reshape(n, R, C)
        low = (oracle.philox_words(seed, sub ^ (1 << 63), first, n * R * C) & np.uint32(0xFFFF)).reshape(n, R, C)
        rng = np.random.default_rng(first)
        T = rng.integers(0, 2 ** 32, size=(R, C), dtype=np.uint64).astype(np.uint32)
        # every third column: the high half of the threshold equals member 1's half-word there, so that member ties
        tie_cols = (np.arange(C) % 3 == 0)
        T[:, tie_cols] = (h[1][:, tie_cols] << np.uint32(16)) | (T[:, tie_cols] & np.uint32(0xFFFF))
        thi, tlo = T >> np.uint32(16), T & np.uint32(0xFFFF)
        want = (h < thi[None]) | ((h == thi[None]) & (low < tlo[None]))
        assert ((h == thi[None]).sum()) >= R * tie_cols.sum()
        got = oracle.sample_philox16(T, n, R, C, seed, sub, first, np.int64)
        bits = np.unpackbits(got.view(np.uint8), axis=2, bitorder="little")[:, :, :C].astype(bool)
        np.testing.assert_array_equal(bits, want, err_msg="first=%d" % first)
        assert not np.unpackbits(got.view(np.uint8), axis=2, bitorder="little")[:, :, C:].any()
        got32 = oracle.sample_philox16(T, n, R, C, seed, sub, first, np.int32)
        np.testing.assert_array_equal(np.unpackbits(got32.view(np.uint8), axis=2, bitorder="little")[:, :, :C].astype(bool), want)
    # rates: thresholds below 2**16 (only ties can set the bit), around 2**-10, and 1/3, over 200 000 draws a column
    Tr = np.array([[40000, 3 << 20 | 12345, 0x55555555, 0]], dtype=np.uint32)
    n2 = 200000
    b = oracle.sample_philox16(Tr, n2, 1, 4, 99, 0, 0, np.int64)
    cols = np.unpackbits(b.view(np.uint8), axis=2, bitorder="little")[:, 0, :4].astype(np.float64)
    p = Tr[0].astype(np.float64) / 2.0 ** 32
    assert (np.abs(cols.mean(axis=0) - p) <= 5 * np.sqrt(p * (1 - p) / n2) + 1e-12).all()
    assert cols[:, 3].sum() == 0
    # the two halves of a word: columns 0 and 1 of rows of two columns at p = 1/2
    b2 = oracle.sample_philox16(1 << 31, n2, 1, 2, 5, 1, 0, np.int64)
    c2 = np.unpackbits(b2.view(np.uint8), axis=2, bitorder="little")[:, 0, :2].astype(np.float64)
    assert abs((c2[:, 0] * c2[:, 1]).mean() - 0.25) < 5 * np.sqrt(0.25 * 0.75 / n2)
    # base is XORed on
    base = np.array([[0x0F0F]], dtype=np.int64)
    np.testing.assert_array_equal(oracle.sample_philox16(1 << 31, 4, 1, 16, 5, 1, 0, np.int64, base=base),
                                  oracle.sample_philox16(1 << 31, 4, 1, 16, 5, 1, 0, np.int64) ^ base[None])
