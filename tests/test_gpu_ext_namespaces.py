"""GPU tests of the two torch-extension namespaces of the reference, ``boolop_cuda``
(extensions/booleanOperations.cpp:86-90) and ``boolutil_cuda`` (extensions/booleanUtilities.cpp:61-66), as this
package provides them: every function against the CPU oracle or the closed form numpy has for it."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

NDT = {32: np.int32, 64: np.int64}
TDT = {32: torch.int32, 64: torch.int64}


@pytest.fixture(scope="module")
def boolop():
    assert torch.cuda.is_available()
    from nesgpu_amd.extensions import boolop_cuda
    return boolop_cuda


@pytest.fixture(scope="module")
def boolutil():
    assert torch.cuda.is_available()
    from nesgpu_amd.extensions import boolutil_cuda
    return boolutil_cuda


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.cpu().numpy()


def rand_words(g, shape, dtype):
    return g.integers(-2 ** 63, 2 ** 63, size=shape, dtype=np.int64).astype(dtype)


def test_the_reference_import_names_resolve(boolop, boolutil):
    import sys
    import nesgpu_amd
    nesgpu_amd.install_as_reference_modules()
    assert sys.modules["boolop_cuda"] is boolop and sys.modules["boolutil_cuda"] is boolutil
    for name in ("binary_bmm", "batch_im2col", "binary_batch_conv2d", "binary_seeded_bmv"):
        assert callable(getattr(boolop, name))                         # booleanOperations.cpp:86-90
    for name in ("pack8", "pack", "unpack", "sample_bits", "binary_weighted_sum"):
        assert callable(getattr(boolutil, name))                       # booleanUtilities.cpp:61-66


@pytest.mark.parametrize("bits", [64, 32])
def test_binary_bmm(boolop, oracle, bits):
    g = np.random.default_rng(bits)
    # multiples of 16 (all the reference's own kernel handles, booleanOperationsCuda.cu:49-50) and ragged shapes
    for Z, M, Kw, N in [(3, 32, 16, 16), (2, 48, 5, 64), (4, 7, 3, 9), (2, 100, 9, 1)]:
        A, B = rand_words(g, (Z, M, Kw), NDT[bits]), rand_words(g, (Z, Kw, N), NDT[bits])
        got = boolop.binary_bmm(dev(A), dev(B))
        assert got.dtype == torch.int32 and tuple(got.shape) == (Z, M, N)
        np.testing.assert_array_equal(host(got), oracle.bmm(A, B))
    A = torch.zeros(2, 4, 3, dtype=TDT[bits], device="cuda")
    with pytest.raises(RuntimeError, match="Batch dim"):
        boolop.binary_bmm(A, torch.zeros(3, 3, 2, dtype=TDT[bits], device="cuda"))
    with pytest.raises(RuntimeError, match="Mult dim"):
        boolop.binary_bmm(A, torch.zeros(2, 4, 2, dtype=TDT[bits], device="cuda"))
    with pytest.raises(RuntimeError, match="contiguous"):
        boolop.binary_bmm(A.transpose(1, 2), torch.zeros(2, 4, 2, dtype=TDT[bits], device="cuda"))
    with pytest.raises(RuntimeError, match="CUDA"):
        boolop.binary_bmm(A.cpu(), A.cpu())


@pytest.mark.parametrize("bits", [64, 32])
def test_batch_im2col_and_binary_batch_conv2d(boolop, oracle, bits):
    """binary_batch_conv2d returns the bmm result WITHOUT the view to [D,h,w,O]: [D, h*w, O]
    (extensions/booleanOperationsCuda.cu:295-298)."""
    g = np.random.default_rng(7 + bits)
    for D, H, W, Cw, O, geom in [(3, 10, 10, 1, 64, (3, 3, 1, 1, 1, 1)), (2, 9, 13, 2, 20, (3, 2, 1, 0, 1, 2)),
                                 (4, 8, 8, 1, 16, (1, 1, 0, 0, 1, 1)), (2, 11, 7, 1, 5, (7, 7, 2, 2, 3, 3))]:
        x = rand_words(g, (D, H, W, Cw), NDT[bits])
        f = rand_words(g, (D, geom[0] * geom[1] * Cw, O), NDT[bits])
        cols = boolop.batch_im2col(dev(x), *geom)
        want_cols = oracle.batch_im2col(x, *geom)
        np.testing.assert_array_equal(host(cols), want_cols)
        out = boolop.binary_batch_conv2d(dev(x), dev(f), *geom)
        h, w = oracle.out_hw(H, W, *geom)
        assert tuple(out.shape) == (D, h * w, O) and out.dtype == torch.int32 and out.is_contiguous()
        np.testing.assert_array_equal(host(out), oracle.conv(x, f, *geom).reshape(D, h * w, O))
        np.testing.assert_array_equal(host(out), oracle.bmm(want_cols, f))     # im2col then bmm, as the reference does
    x = torch.zeros(2, 4, 4, 1, dtype=TDT[bits], device="cuda")
    with pytest.raises(RuntimeError, match="Batch dim"):
        boolop.binary_batch_conv2d(x, torch.zeros(3, 9, 4, dtype=TDT[bits], device="cuda"), 3, 3, 1, 1, 1, 1)
    other = torch.int32 if bits == 64 else torch.int64
    with pytest.raises(RuntimeError, match="different types"):
        boolop.binary_batch_conv2d(x, torch.zeros(2, 9, 4, dtype=other, device="cuda"), 3, 3, 1, 1, 1, 1)


@pytest.mark.parametrize("bits", [64, 32])
def test_binary_seeded_bmv(boolop, oracle, bits):
    """binary_seeded_bmv(P, B, seed): weights w[m,r,c] = (word(m,r,c) < floor(P[r,c] * 2**32)) drawn from the Philox
    stream (seed, subsequence 0) and never stored; the result must equal the oracle's fused product on the same
    words regenerated on the host, and bmm(sample_bits(P, ...), B) on the GPU."""
    from nesgpu_amd.extensions import booleanOperations as ops
    g = np.random.default_rng(11 + bits)
    for batch, out_f, in_f in [(4, 16, 64), (3, 33, 100), (8, 64, 1024), (2, 5, 7)]:
        seed = 1000 + in_f
        P = g.random((out_f, in_f)).astype(np.float16)
        P[0, 0], P[-1, -1] = 0.0, 1.0
        nd = NDT[bits]
        Bb = g.integers(0, 2, size=(batch, in_f)).astype(bool)
        B = oracle.pack(Bb, nd)
        got = boolop.binary_seeded_bmv(dev(P), dev(B), seed)
        assert tuple(got.shape) == (batch, out_f) and got.dtype == torch.int32
        thr = np.minimum(np.floor(P.astype(np.float64) * 4294967296.0), 4294967295.0).astype(np.uint32)
        words = oracle.philox_words(seed, 0, 0, batch * out_f * in_f).reshape(batch, out_f, in_f)
        np.testing.assert_array_equal(host(got), oracle.seeded_bmv_from_words(thr, B, words))
        Wm = ops.sample_bits(dev(P), batch, TDT[bits], seed)
        np.testing.assert_array_equal(host(Wm), oracle.sample_from_words(thr, words, nd))
        assert torch.equal(ops.bmm(Wm, dev(B).view(batch, -1, 1)).squeeze(2), got)


@pytest.mark.parametrize("bits", [64, 32])
def test_pack_unpack(boolutil, oracle, bits):
    g = np.random.default_rng(3 + bits)
    for R, C in [(1, 1), (7, 63), (5, 64), (33, 65), (100, 200), (1000, 16), (9, 1024)]:
        b = g.integers(0, 2, size=(R, C)).astype(bool)
        got = boolutil.pack(dev(b), bits)
        assert got.dtype == TDT[bits]
        want = oracle.pack(b, NDT[bits])
        np.testing.assert_array_equal(host(got), want)
        # closed form: little-endian bit order over columns zero-padded to whole words
        pad = (-C) % bits
        ref = np.packbits(np.pad(b, ((0, 0), (0, pad))), axis=1, bitorder="little").view("<i%d" % (bits // 8))
        np.testing.assert_array_equal(host(got), ref)
        un = boolutil.unpack(got)
        assert un.dtype == torch.bool and tuple(un.shape) == (R, want.shape[1] * bits)
        np.testing.assert_array_equal(host(un)[:, :C], b)
        assert not host(un)[:, C:].any()
    with pytest.raises(RuntimeError, match="invalid bit size"):
        boolutil.pack(torch.zeros(2, 2, dtype=torch.bool, device="cuda"), 12)


def test_pack8(boolutil):
    """pack8: bool [R,C] -> int8 [R, ceil(C/8)], bit i of byte y = element 8*y+i, short last byte zero-filled
    (extensions/booleanUtilitiesCuda.cu:31-50)."""
    g = np.random.default_rng(8)
    for R, C in [(1, 1), (3, 7), (4, 8), (5, 9), (17, 31), (64, 32), (9, 33), (300, 100), (2, 784), (1025, 3)]:
        b = g.integers(0, 2, size=(R, C)).astype(bool)
        got = boolutil.pack8(dev(b))
        assert got.dtype == torch.int8 and tuple(got.shape) == (R, (C + 7) // 8) and got.is_contiguous()
        np.testing.assert_array_equal(host(got).view(np.uint8), np.packbits(b, axis=1, bitorder="little"))
    ones = torch.ones(2, 8, dtype=torch.bool, device="cuda")
    assert host(boolutil.pack8(ones)).tolist() == [[-1], [-1]]              # bit 7 set: a negative int8


@pytest.mark.parametrize("bits", [64, 32])
def test_sample_bits(boolutil, oracle, bits):
    """sample_bits(p, n, bits, seed): [n, R, ceil(C/bits)], tail bits zero; the stream is Philox (seed, subsequence 0),
    so the host can regenerate it."""
    g = np.random.default_rng(5 + bits)
    for n, R, C in [(3, 4, 64), (5, 7, 100), (2, 9, 1024), (17, 4, 256), (2, 27, 3)]:
        P = g.random((R, C)).astype(np.float16)
        got = boolutil.sample_bits(dev(P), n, bits, 77)
        assert got.dtype == TDT[bits] and tuple(got.shape) == (n, R, (C + bits - 1) // bits)
        thr = np.minimum(np.floor(P.astype(np.float64) * 4294967296.0), 4294967295.0).astype(np.uint32)
        words = oracle.philox_words(77, 0, 0, n * R * C).reshape(n, R, C)
        np.testing.assert_array_equal(host(got), oracle.sample_from_words(thr, words, NDT[bits]))
    p = torch.full((8, 256), 0.3, dtype=torch.float16, device="cuda")
    rate = host(boolutil.unpack(boolutil.sample_bits(p, 256, bits, 5).view(-1, 256 // bits))).mean()
    assert abs(rate - 0.3) < 3e-3


@pytest.mark.parametrize("bits", [64, 32])
def test_binary_weighted_sum(boolutil, oracle, bits):
    g = np.random.default_rng(13 + bits)
    for n, R, C in [(37, 5, 100), (128, 16, 64), (70, 3, 330)]:
        words = rand_words(g, (n, R, (C + bits - 1) // bits), NDT[bits])
        w = g.standard_normal(n).astype(np.float16)
        got = boolutil.binary_weighted_sum(dev(words), dev(w), C)
        assert got.dtype == torch.float16 and tuple(got.shape) == (R, C)
        want = oracle.weighted_sum(words, w.astype(np.float32), C)
        np.testing.assert_array_equal(host(got).astype(np.float32), want.astype(np.float16).astype(np.float32))
