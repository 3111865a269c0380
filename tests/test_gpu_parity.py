"""GPU parity tests: the HIP kernels, called through the Python op layer (ctypes -> C ABI of
include/nesbin.h), against the committed golden fixtures and the CPU oracle on the same seeded inputs.
Integer / bit results must match exactly."""
import itertools

import os

import numpy as np
import pytest
import torch

from golden_util import (BMM_CASES, CONV_CASES, PACK_WIDTHS, POOL_CASES, SMP_CASES, TAGS, load_ops, load_philox,
                         torch_mean_fp16)

pytestmark = pytest.mark.gpu

G = load_ops()
TDT = {"i64": torch.int64, "i32": torch.int32}
NDT = {torch.int64: np.int64, torch.int32: np.int32}


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from nesgpu_amd.extensions import booleanOperations
    return booleanOperations


@pytest.fixture(params=[2, 3], ids=["fp4-where-it-exists", "int8-only"])
def mc_engine(request):
    """The two matrix-core settings: 2 = FP4 kernel where it exists, 3 = int8 kernel only."""
    return request.param


def _fp4_shape(C, O, fy):
    """Shapes the FP4 flavour of the matrix-core kernel takes: 3 x fy windows on full channel words (1, 2 or 4 words
    per pixel, no tap packing: more than 32 channels), more than one 128-position chunk per filter row, and the
    output-channel counts the kernel tiles (16, 32, or 64 and more; not 32 with four words per pixel)."""
    Cw = (C + 63) // 64
    if C <= 32 or Cw not in (1, 2, 4) or O % 16:
        return False
    cpr = (fy + 1) // 2 if Cw == 1 else fy * (Cw // 2)           # 128-position chunks per filter row
    return cpr in (2, 3, 6) and (O >= 64 or O == 16 or (O == 32 and cpr != 6))


@pytest.fixture(params=[1, 2, 3], ids=["popcount", "matrixcore", "matrixcore-int8"])
def engine(request, ops):
    """Runs a conv test once per engine: 1 = XOR-popcount kernels only, 2 = matrix cores wherever a kernel covers the
    shape (FP4 codes for full channel words of 64, 128 or 256 channels, +-1 bytes otherwise; the XOR-popcount kernels
    take the rest), 3 = the same with +-1 bytes only."""
    prev = ops.conv_engine(request.param)
    yield request.param
    ops.conv_engine(prev)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.cpu().numpy()


def rng(seed):
    return np.random.default_rng(seed)


def rand_words(g, shape, dtype):
    return g.integers(-2 ** 63, 2 ** 63, size=shape, dtype=np.int64).astype(dtype)


# ---------------------------------------------------------------------------------------------- golden
@pytest.mark.parametrize("tag", TAGS)
def test_golden_pack_unpack(ops, tag):
    for C in PACK_WIDTHS:
        bits = G[f"pack_{tag}_C{C}_in"]
        got = ops.pack(dev(bits), TDT[tag])
        np.testing.assert_array_equal(host(got), G[f"pack_{tag}_C{C}_out"])
        un = host(ops.unpack(got))
        np.testing.assert_array_equal(un[:, :C], bits)
        assert not un[:, C:].any()


@pytest.mark.parametrize("tag", TAGS)
@pytest.mark.parametrize("case", BMM_CASES)
def test_golden_bmm(ops, tag, case):
    A, B = dev(G[f"bmm_{tag}_{case}_A"]), dev(G[f"bmm_{tag}_{case}_B"])
    np.testing.assert_array_equal(host(ops.bmm(A, B)), G[f"bmm_{tag}_{case}_C"])
    act = ops.bmm_act(A, B, dev(G[f"bmm_{tag}_{case}_thr"]))
    assert act.dtype == torch.bool
    np.testing.assert_array_equal(host(act), G[f"bmm_{tag}_{case}_act"])


@pytest.mark.parametrize("tag", TAGS)
@pytest.mark.parametrize("case", CONV_CASES)
def test_golden_conv(ops, engine, tag, case):
    x, f = dev(G[f"conv_{tag}_{case}_x"]), dev(G[f"conv_{tag}_{case}_f"])
    thr = dev(G[f"conv_{tag}_{case}_thr"])
    geom = [int(v) for v in G[f"conv_{tag}_{case}_geom"]]
    np.testing.assert_array_equal(host(ops.batch_im2col(x, *geom)), G[f"conv_{tag}_{case}_cols"])
    popc = ops.conv(x, f, *geom)
    assert popc.dtype == torch.int32
    np.testing.assert_array_equal(host(popc), G[f"conv_{tag}_{case}_popc"])
    np.testing.assert_array_equal(host(ops.conv_act(x, f, thr, *geom)), G[f"conv_{tag}_{case}_act"])


@pytest.mark.parametrize("tag", TAGS)
@pytest.mark.parametrize("case", POOL_CASES)
def test_golden_pool(ops, tag, case):
    geom = [int(v) for v in G[f"pool_{tag}_{case}_geom"]]
    got = ops.max_pool2d(dev(G[f"pool_{tag}_{case}_x"]), *geom)
    np.testing.assert_array_equal(host(got), G[f"pool_{tag}_{case}_out"])


@pytest.mark.parametrize("tag", TAGS)
@pytest.mark.parametrize("case", SMP_CASES)
def test_golden_sampling(ops, tag, case):
    p = f"smp_{tag}_{case}_"
    words, thr, base, x = dev(G[p + "words"]), dev(G[p + "thr"]), dev(G[p + "base"]), dev(G[p + "x"])
    T = 214748364
    np.testing.assert_array_equal(host(ops.sample_bits_from_words(thr, words, TDT[tag])), G[p + "sample"])
    np.testing.assert_array_equal(host(ops.flip_from_words(base, words, T)), G[p + "flip"])
    np.testing.assert_array_equal(host(ops.seeded_bmv_from_words(thr, x, words)), G[p + "bmv_sample"])
    np.testing.assert_array_equal(host(ops.seeded_bmv_from_words(T, x, words, base=base)), G[p + "bmv_flip"])


def test_golden_philox(ops):
    P = load_philox()
    for case in P["rocrand"]:
        got = ops.philox_words(len(case["words"]), case["seed"], case["subsequence"], case["offset"])
        assert [int(v) for v in host(got)] == case["words"]


# ---------------------------------------------------------------------------------------------- vs oracle
@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("R,C", [(1, 16), (5, 64), (300, 128), (1000, 16), (77, 48), (33, 256), (9, 8192), (4097, 3),
                                 (64, 80), (2, 1), (513, 576),
                                 # rows of whole 8-byte chunks that are not whole 16-byte chunks
                                 (1000, 24), (333, 8), (77, 40), (65, 72), (9, 200), (3, 1048)])
def test_pack_unpack_vs_oracle(ops, oracle, dtype, R, C):
    bits = rng(R + C).integers(0, 2, size=(R, C)).astype(bool)
    want = oracle.pack(bits, NDT[dtype])
    got = ops.pack(dev(bits), dtype)
    np.testing.assert_array_equal(host(got), want)
    np.testing.assert_array_equal(host(ops.unpack(got)), oracle.unpack(want))


def test_pack_counts_any_nonzero_byte_as_one(ops):
    raw = rng(1).integers(0, 256, size=(8, 64)).astype(np.uint8)
    t = dev(raw).view(torch.bool)
    got = host(ops.pack(t, torch.int64))
    want = np.packbits(raw != 0, axis=1, bitorder="little").view("<i8")
    np.testing.assert_array_equal(got, want)
    raw = rng(2).integers(0, 256, size=(9, 24)).astype(np.uint8)          # rows of three 8-byte chunks
    raw[raw > 200] = 0
    got = host(ops.pack(dev(raw).view(torch.bool), torch.int64))
    want = np.packbits(np.pad(raw != 0, ((0, 0), (0, 40))), axis=1, bitorder="little").view("<i8")
    np.testing.assert_array_equal(got, want)


def test_pack_misaligned_rows_take_the_generic_path(ops, oracle):
    bits = rng(3).integers(0, 2, size=(41, 64)).astype(bool)
    big = dev(np.concatenate([np.zeros(3, dtype=bool), bits.ravel()]))
    view = big[3:].view(41, 64)                         # data pointer not 16-byte aligned
    np.testing.assert_array_equal(host(ops.pack(view, torch.int64)), oracle.pack(bits, np.int64))


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_int8pack_vs_oracle(ops, oracle, dtype):
    for R, C in [(3, 1), (50, 8), (7, 13), (100, 784)]:
        data = rng(C).integers(0, 256, size=(R, C)).astype(np.uint8)
        np.testing.assert_array_equal(host(ops.int8pack(dev(data), dtype)), oracle.int8pack(data, NDT[dtype]))


LINEAR_SHAPES = [(8, 256, 4), (5, 10, 16), (3, 1000, 128), (7, 33, 9), (4, 64, 1), (2, 3, 200), (9, 1, 2), (1, 5, 31),
                 (6, 130, 6),
                 # four-rows-per-group kernel: 16, 32 and 64 lanes per row, rows that are not a multiple of the lane count
                 (5, 12, 32), (2, 8, 200), (3, 4, 66), (2, 20, 34), (1, 4, 512), (300, 8, 64),
                 # row-per-lane kernel for rows of 16, 32 or 64 bytes: members that do not fill a run of 64 rows, a ragged
                 # last workgroup, one row
                 (1000, 3, 8), (7, 300, 2), (3, 1025, 4), (1, 1, 8), (600, 5, 4), (2, 2048, 16)]


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("Z,M,Kw", LINEAR_SHAPES)
def test_bmm_matrix_vector_form_vs_oracle(ops, oracle, dtype, Z, M, Kw):
    g = rng(Z * 31 + M * 7 + Kw)
    A = rand_words(g, (Z, M, Kw), NDT[dtype])
    x = rand_words(g, (Z, Kw, 1), NDT[dtype])
    np.testing.assert_array_equal(host(ops.bmm(dev(A), dev(x))), oracle.bmm(A, x))


def test_bmm_matrix_vector_unaligned_operands(ops, oracle):
    g = rng(17)
    A = rand_words(g, (3, 20, 4), np.int64)
    x = rand_words(g, (3, 4, 1), np.int64)
    bigA = dev(np.concatenate([np.zeros(1, np.int64), A.ravel()]))[1:].view(3, 20, 4)      # 8- but not 16-byte aligned
    np.testing.assert_array_equal(host(ops.bmm(bigA, dev(x))), oracle.bmm(A, x))


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_bmm_random_shapes_vs_oracle(ops, oracle, dtype):
    """Sixty seeded random (Z, M, Kw, N): matrix-vector forms of every row length class (the row-group kernel and the
    16/32/64-lane four-row kernel with one to four row steps in flight) and general products."""
    g = rng(4242)
    for ci in range(60):
        Z, M = int(g.integers(1, 7)), int(g.integers(1, 70))
        Kw = int(g.choice([1, 2, 3, 4, 7, 16, 31, 32, 33, 64, 96, 128, 130, 256, 512]))
        N = 1 if ci % 3 else int(g.integers(2, 40))
        if ci % 6 == 1:
            M = 4 * int(g.integers(1, 30))                # the four-row kernel needs M % 4 == 0
        print("case", ci, (Z, M, Kw, N), flush=True)
        A = rand_words(g, (Z, M, Kw), NDT[dtype])
        B = rand_words(g, (Z, Kw, N), NDT[dtype])
        np.testing.assert_array_equal(host(ops.bmm(dev(A), dev(B))), oracle.bmm(A, B))


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_bmv_act_pack_random_shapes_vs_oracle(ops, oracle, dtype):
    """The fused matrix-vector -> threshold -> pack op against pack(2 * bmm > threshold) of the oracle: rows of every
    length class of the four-row kernel (members of whole words, several workgroups, ragged last workgroup) and the
    general kernel (ragged members, short rows), thresholds around the sums plus always / never."""
    nd = NDT[dtype]
    bits = np.dtype(nd).itemsize * 8
    g = rng(777)
    vec = 16 // np.dtype(nd).itemsize                      # words per 16 bytes
    for ci in range(48):
        Z = int(g.integers(1, 6))
        if ci % 2 == 0:                                    # shapes the four-row kernel takes
            M = bits * int(g.integers(1, 9))
            Kw = vec * int(g.choice([16, 17, 32, 48, 64, 96, 128, 256, 272]))
        else:
            M = int(g.integers(1, 200))
            Kw = int(g.choice([0, 1, 3, 16, 31, 64, 130]))
        print("case", ci, (Z, M, Kw), flush=True)
        A = rand_words(g, (Z, M, Kw), nd)
        x = rand_words(g, (Z, Kw, 1), nd)
        sums = oracle.bmm(A, x)[:, :, 0]
        K = Kw * bits
        thr = (2 * sums + g.integers(-3, 4, size=sums.shape)).astype(np.int32)
        thr[0, 0] = -1
        thr[-1, -1] = 2 * K + 1
        want = oracle.pack(2 * sums.astype(np.int64) > thr, nd)
        got = ops.bmv_act_pack(dev(A), dev(x), dev(thr))
        assert tuple(got.shape) == want.shape
        np.testing.assert_array_equal(host(got), want, err_msg="case %d: Z=%d M=%d Kw=%d" % (ci, Z, M, Kw))
        np.testing.assert_array_equal(host(ops.bmv_act_pack(dev(A), dev(x[:, :, 0]), dev(thr))), want)


GENERAL_SHAPES = [(2, 300, 9, 64), (3, 65, 4, 16), (2, 257, 18, 5), (2, 40, 40, 33), (1, 1, 1, 2), (2, 513, 3, 128),
                  (3, 7, 17, 17), (2, 100, 0, 4)]


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("Z,M,Kw,N", GENERAL_SHAPES)
def test_bmm_general_and_act_vs_oracle(ops, oracle, dtype, Z, M, Kw, N):
    g = rng(Z + M + Kw + N)
    A = rand_words(g, (Z, M, Kw), NDT[dtype])
    B = rand_words(g, (Z, Kw, N), NDT[dtype])
    want = oracle.bmm(A, B)
    np.testing.assert_array_equal(host(ops.bmm(dev(A), dev(B))), want)
    hi = max(int(want.max()), 1)
    thr = (g.integers(0, 2 * hi + 2, size=(Z, N)) - 1).astype(np.int32)
    np.testing.assert_array_equal(host(ops.bmm_act(dev(A), dev(B), dev(thr))), oracle.bmm_act(A, B, thr))


def test_bmm_special_cases(ops):
    g = rng(4)
    A = rand_words(g, (2, 70, 5), np.int64)
    At = np.ascontiguousarray(A.transpose(0, 2, 1))
    got = host(ops.bmm(dev(A), dev(At)))
    assert (got[:, np.arange(70), np.arange(70)] == 0).all()                  # a ^ a
    got = host(ops.bmm(dev(A), dev(~At)))
    assert (got[:, np.arange(70), np.arange(70)] == 5 * 64).all()             # a ^ ~a, sign bits included
    zeros = np.zeros((2, 5, 3), np.int64)
    ones = np.unpackbits(A.view(np.uint8), axis=2).sum(axis=2)
    np.testing.assert_array_equal(host(ops.bmm(dev(A), dev(zeros))), np.repeat(ones[:, :, None], 3, 2))


SWEEP = list(itertools.product([1, 3, 7], [0, 1, 2], [1, 2, 3]))                # booloptests.py:122-124


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("C,O", [(1, 64), (16, 16), (64, 5), (70, 33), (130, 8)])
def test_conv_reference_sweep_vs_oracle(ops, oracle, engine, dtype, C, O):
    """The reference's check_result sweep (filter x padding x stride on a 10x10 input, booloptests.py:113-124)."""
    D, S = 5, 10
    bits = torch.iinfo(dtype).bits
    Cw = (C + bits - 1) // bits
    for fs, pad, st in SWEEP:
        g = rng(fs * 100 + pad * 10 + st + C)
        xb = g.integers(0, 2, size=(D * S * S, C)).astype(bool)
        x = oracle.pack(xb, NDT[dtype]).reshape(D, S, S, Cw)
        fb = g.integers(0, 2, size=(D * O * fs * fs, C)).astype(bool)
        f5 = oracle.pack(fb, NDT[dtype]).reshape(D, O, fs, fs, Cw)
        f = np.ascontiguousarray(f5.transpose(0, 2, 3, 4, 1).reshape(D, -1, O))
        K = fs * fs * C
        thr = (g.integers(0, K, size=(D, O)) - K // 2 + K).astype(np.int32)
        geom = (fs, fs, pad, pad, st, st)
        xd, fd, td = dev(x), dev(f), dev(thr)
        want = oracle.conv(x, f, *geom)
        np.testing.assert_array_equal(host(ops.conv(xd, fd, *geom)), want, err_msg=str(geom))
        np.testing.assert_array_equal(host(ops.conv_act(xd, fd, td, *geom)), 2 * want > thr[:, None, None, :])
        np.testing.assert_array_equal(host(ops.batch_im2col(xd, *geom)), oracle.batch_im2col(x, *geom))
        # fused conv -> threshold -> pack (-> pool) against the op chain of the oracle
        act = oracle.conv_act(x, f, thr, *geom)
        h, w = act.shape[1:3]
        packed = oracle.pack(act.reshape(-1, O), NDT[dtype]).reshape(D, h, w, -1)
        np.testing.assert_array_equal(host(ops.conv_act_pack(xd, fd, td, *geom)), packed)
        if h >= 2 and w >= 2:
            pooled = oracle.max_pool2d(packed, 2, 2, 0, 0, 2, 2)
            np.testing.assert_array_equal(host(ops.conv_act_pack(xd, fd, td, *geom, pool=True)), pooled)


def test_conv_rectangular_window_and_image(ops, oracle, engine):
    g = rng(8)
    D, H, W, Cw, O = 3, 9, 13, 2, 20
    x = rand_words(g, (D, H, W, Cw), np.int64)
    for fx, fy, px, py, sx, sy in [(3, 2, 1, 0, 1, 2), (1, 5, 0, 2, 2, 1), (4, 4, 3, 3, 3, 2)]:
        f = rand_words(g, (D, fx * fy * Cw, O), np.int64)
        want = oracle.conv(x, f, fx, fy, px, py, sx, sy)
        np.testing.assert_array_equal(host(ops.conv(dev(x), dev(f), fx, fy, px, py, sx, sy)), want)


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_max_pool_vs_oracle(ops, oracle, dtype):
    g = rng(12)
    for B, H, W, Cw in [(3, 10, 10, 1), (2, 7, 9, 3), (5, 64, 64, 1), (1, 2, 2, 1), (2, 33, 5, 2), (4, 16, 12, 4),
                        (2, 9, 8, 1), (3, 6, 6, 2), (300, 8, 8, 1), (2, 4, 6, 1)]:
        x = rand_words(g, (B, H, W, Cw), NDT[dtype])
        for geom in [(2, 2, 0, 0, 2, 2), (2, 2, 1, 1, 2, 2), (3, 3, 1, 1, 2, 2), (2, 2, 0, 0, 1, 1), (2, 2, 0, 1, 3, 2)]:
            if H - geom[0] + 2 * geom[2] < 0 or W - geom[1] + 2 * geom[3] < 0:
                continue
            np.testing.assert_array_equal(host(ops.max_pool2d(dev(x), *geom)), oracle.max_pool2d(x, *geom),
                                          err_msg=str((B, H, W, Cw, geom)))


SAMPLE_SHAPES = [(3, 4, 64), (2, 3, 1), (5, 2, 63), (2, 5, 65), (3, 2, 200), (4, 7, 256), (2, 576, 64), (3, 10, 1024),
                 (2, 9, 16), (3, 5, 128), (2, 3, 100), (2, 5, 256), (2, 7, 512), (2, 3, 768), (2, 3, 2048), (3, 33, 1024),
                 # more members than one member group of the wide kernel; a long row; a 3-column row (first conv layer)
                 (17, 4, 8192), (2, 27, 3), (19, 6, 256), (9, 1024, 8), (6, 576, 24), (3, 40, 12)]


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("n,R,C", SAMPLE_SHAPES)
def test_sampling_from_words_vs_oracle(ops, oracle, dtype, n, R, C):
    g = rng(n * 7 + R * 3 + C)
    words = g.integers(0, 2 ** 32, size=(n, R, C), dtype=np.uint64).astype(np.uint32)
    thr = g.integers(0, 2 ** 32, size=(R, C), dtype=np.uint64).astype(np.uint32)
    T = int(0.05 * 2 ** 32)
    nd = NDT[dtype]
    wb = np.dtype(nd).itemsize * 8
    base = rand_words(g, (R, (C + wb - 1) // wb), nd)
    if C % wb:
        base[:, -1] &= nd((1 << (C % wb)) - 1)
    x = rand_words(g, (n, (C + wb - 1) // wb), nd)
    if C % wb:
        x[:, -1] &= nd((1 << (C % wb)) - 1)          # tail bits are zero by contract (pack.cu:17)
    wd, td, bd, xd = dev(words), dev(thr), dev(base), dev(x)
    np.testing.assert_array_equal(host(ops.sample_bits_from_words(td, wd, dtype)), oracle.sample_from_words(thr, words, nd))
    np.testing.assert_array_equal(host(ops.flip_from_words(bd, wd, T)), oracle.sample_from_words(T, words, nd, base=base))
    np.testing.assert_array_equal(host(ops.sample_bits_from_words(td, wd, dtype, base=bd)),
                                  oracle.sample_from_words(thr, words, nd, base=base))
    for kw in (dict(base=None, thr=thr), dict(base=base, thr=T), dict(base=base, thr=thr)):
        want = oracle.seeded_bmv_from_words(kw["thr"], x, words, base=kw["base"])
        tarr = td if isinstance(kw["thr"], np.ndarray) else kw["thr"]
        got = ops.seeded_bmv_from_words(tarr, xd, wd, base=None if kw["base"] is None else bd)
        np.testing.assert_array_equal(host(got), want)
        # fused == materialise + bmm on the GPU as well
        Wm = ops.sample_bits_from_words(tarr, wd, dtype, base=None if kw["base"] is None else bd)
        np.testing.assert_array_equal(host(ops.bmm(Wm, xd.view(n, -1, 1)))[:, :, 0], want)


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("n,R,C,first", [(3, 4, 64, 0), (2, 5, 100, 0), (2, 3, 256, 8), (2, 3, 64, 5), (3, 2, 63, 2),
                                         (2, 7, 1024, 4 * 0xFFFFFFFE),
                                         (20, 700, 4096, 0),   # enough words for eight members per lane
                                         # rows shorter than a word: whole generator blocks (24, 16, 4 columns), blocks
                                         # that straddle rows (a stream that starts inside a block; 3 and 30 columns)
                                         (5, 70, 24, 0), (3, 9, 16, 12), (2, 5, 24, 6), (4, 27, 3, 0), (130, 3, 4, 0),
                                         (3, 11, 30, 0)])
def test_philox_mode_equals_supplied_words_mode(ops, oracle, dtype, n, R, C, first):
    """Generator mode is defined as: the words nb_philox_words writes, fed to the supplied-words kernels."""
    seed, sub = 0x1234ABCD5678EF01, 3
    g = rng(C + first % 97)
    nd = NDT[dtype]
    wb = np.dtype(nd).itemsize * 8
    words_gpu = ops.philox_words(n * R * C, seed, sub, first)
    words_cpu = oracle.philox_words(seed, sub, first, n * R * C)
    np.testing.assert_array_equal(host(words_gpu), words_cpu)
    words = words_gpu.view(n, R, C)
    thr = dev(g.integers(0, 2 ** 32, size=(R, C), dtype=np.uint64).astype(np.uint32))
    base = rand_words(g, (R, (C + wb - 1) // wb), nd)
    if C % wb:
        base[:, -1] &= nd((1 << (C % wb)) - 1)
    bd = dev(base)
    xh = rand_words(g, (n, (C + wb - 1) // wb), nd)
    if C % wb:
        xh[:, -1] &= nd((1 << (C % wb)) - 1)
    x = dev(xh)
    T = int(0.02 * 2 ** 32)
    a = ops.sample_bits_philox(thr, n, dtype, seed, sub, first)
    assert torch.equal(a, ops.sample_bits_from_words(thr, words, dtype))
    a = ops.flip_philox(bd, C, n, T, seed, sub, first)
    assert torch.equal(a, ops.flip_from_words(bd, words, T))
    a = ops.seeded_bmv_philox(T, x, R, C, seed, sub, first, base=bd)
    assert torch.equal(a, ops.seeded_bmv_from_words(T, x, words, base=bd))
    a = ops.seeded_bmv_philox(thr, x, R, C, seed, sub, first)
    assert torch.equal(a, ops.seeded_bmv_from_words(thr, x, words))


def test_thresholds_from_p_kernel_equals_the_float64_expression(ops):
    """Every fp16 bit pattern (finite, subnormal, negative, above one, infinities, NaNs) through the one-kernel
    thresholds against floor(p * 2**32) clamped in float64 on the host."""
    bits = np.arange(65536, dtype=np.uint16)
    p = bits.view(np.float16)
    got = host(ops.thresholds_from_p(dev(p).view(torch.float16))).astype(np.int64) & 0xFFFFFFFF
    with np.errstate(invalid="ignore", over="ignore"):
        want = np.floor(p.astype(np.float64) * 4294967296.0)
    want = np.where(np.isnan(want), 0.0, np.clip(want, 0.0, 4294967295.0)).astype(np.int64)
    np.testing.assert_array_equal(got, want)
    assert int(got[np.float16(0.5).view(np.uint16)]) == 2 ** 31 and int(got[np.float16(1.0).view(np.uint16)]) == 2 ** 32 - 1


def test_sample_bits_law_and_layout(ops):
    """sample_bits(p, n, dtype, seed): shape [n,R,ceil(C/bits)], zero tail bits, rate ~= p, seed-reproducible."""
    p = torch.tensor([[0.0] * 100, [1.0] * 100, [0.25] * 100, [0.5] * 100], dtype=torch.float16, device="cuda")
    a = ops.sample_bits(p, 512, torch.int64, 999)
    assert a.shape == (512, 4, 2) and a.dtype == torch.int64
    assert torch.equal(a, ops.sample_bits(p, 512, torch.int64, 999))
    assert not torch.equal(a, ops.sample_bits(p, 512, torch.int64, 1000))
    bits = host(ops.unpack(a.view(-1, 2))).reshape(512, 4, 128)
    assert not bits[:, :, 100:].any()
    assert not bits[:, 0].any() and bits[:, 1, :100].all()
    assert abs(bits[:, 2, :100].mean() - 0.25) < 0.01 and abs(bits[:, 3, :100].mean() - 0.5) < 0.01


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_sampler_from_half_word_draws_vs_oracle(ops, oracle, dtype):
    """sample_bits_philox(half_draws=True) == the oracle's restatement of the 16-bit draws: scalar and per-element
    thresholds (small probabilities: non-zero low halves), base, conv layout, few and many members (two and eight per
    lane), stream offsets, and thresholds built from the stream itself so that one member ties in every third column
    (the second stream decides those)."""
    nd = NDT[dtype]
    wb = np.dtype(nd).itemsize * 8
    g = rng(41)
    for n, R, C, first in [(3, 5, 2 * wb, 0), (9, 4, wb, 8), (40, 130, 3 * wb, 16), (2, 1, wb, 0), (600, 64, 4 * wb, 0)]:
        seed, sub = 1234 + n, 3
        Rw = C // wb
        base = rand_words(g, (R, Rw), nd)
        # per-element thresholds: probabilities from 1e-6 to 1, and every third column tied for member 1
        P = 10.0 ** (-6 * g.random((R, C)))
        T = np.minimum(np.floor(P * 2.0 ** 32), 2.0 ** 32 - 1).astype(np.uint32)
        gi = first + R * C + np.arange(R * C, dtype=np.uint64)                       # member 1's flat indices
        w1 = oracle.philox_words(seed, sub, int(gi[0]) // 2, R * C // 2 + 2)
        w = w1[((gi >> np.uint64(1)) - np.uint64(int(gi[0]) // 2)).astype(np.int64)]
        h = np.where(gi & np.uint64(1), w >> np.uint32(16), w & np.uint32(0xFFFF)).astype(np.uint32).reshape(R, C)
        tie = np.arange(C) % 3 == 0
        T[:, tie] = (h[:, tie] << np.uint32(16)) | (T[:, tie] & np.uint32(0xFFFF))
        Td = torch.from_numpy(T.view(np.int32)).cuda().view(torch.uint32)
        want = oracle.sample_philox16(T, n, R, C, seed, sub, first, nd, base=base)
        got = ops.sample_bits_philox(Td, n, dtype, seed, sub, first, base=dev(base), half_draws=True)
        np.testing.assert_array_equal(host(got), want, err_msg=str((n, R, C, first)))
        want_s = oracle.sample_philox16(0x03000001, n, R, C, seed, sub, first, nd)
        got_s = ops.sample_bits_philox(0x03000001, n, dtype, seed, sub, first, shape=(R, C), half_draws=True)
        np.testing.assert_array_equal(host(got_s), want_s)
        if R % 5 == 0:
            KK, O = 5, R // 5
            rows, conv = ops.sample_bits_philox(Td, n, dtype, seed, sub, first, base=dev(base), conv_taps=KK, half_draws=True)
            np.testing.assert_array_equal(host(rows), want)
            np.testing.assert_array_equal(host(conv), want.reshape(n, O, KK, Rw).transpose(0, 2, 3, 1).reshape(n, KK * Rw, O))
    assert ops.half_draws_apply(64, torch.int64) and not ops.half_draws_apply(24, torch.int64)
    assert not ops.half_draws_apply(64, torch.int64, first=4)
    with pytest.raises(ValueError, match="whole words"):
        ops.sample_bits_philox(1 << 30, 2, dtype, 1, shape=(3, wb + 8), half_draws=True)
    with pytest.raises(RuntimeError, match="16-bit draws"):
        out = torch.empty((2, 3, 1), dtype=dtype, device="cuda")
        ops._lib.call("nb_sample_philox16" + ("_i64" if wb == 64 else "_i32"), out.data_ptr(), None, None, 1 << 30, 1, 0, 4, 2, 3, wb, None)


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_fused_product_over_half_word_draws_vs_oracle(ops, oracle, dtype):
    """seeded_bmv_philox(half_draws=True) == bmm of the weights the oracle's 16-bit draws give, also for rows that are
    whole bytes but not whole words, with ties forced for one member, and == bmm on what the sampler itself writes."""
    nd = NDT[dtype]
    wb = np.dtype(nd).itemsize * 8
    g = rng(43)
    for n, R, C, first in [(3, 5, 2 * wb, 0), (5, 9, 1024, 8), (2, 7, wb + 8, 0), (4, 130, 520, 16), (1, 1, 8, 0), (70, 3, 4096, 0)]:
        seed, sub = 77 + n, 2
        Rw = (C + wb - 1) // wb
        base = rand_words(g, (R, Rw), nd)
        x = rand_words(g, (n, Rw), nd)
        if C % wb:                                       # tail bits are zero on every operand
            keep = np.array((1 << (C % wb)) - 1).astype(np.uint64).astype(np.dtype("u%d" % (wb // 8))).view(nd)
            base[:, -1] &= keep
            x[:, -1] &= keep
        P = 10.0 ** (-4 * g.random((R, C)))
        T = np.minimum(np.floor(P * 2.0 ** 32), 2.0 ** 32 - 1).astype(np.uint32)
        if n > 1:                                        # member 1 ties in every third column
            gi = first + R * C + np.arange(R * C, dtype=np.uint64)
            w1 = oracle.philox_words(seed, sub, int(gi[0]) // 2, R * C // 2 + 2)
            w = w1[((gi >> np.uint64(1)) - np.uint64(int(gi[0]) // 2)).astype(np.int64)]
            h = np.where(gi & np.uint64(1), w >> np.uint32(16), w & np.uint32(0xFFFF)).astype(np.uint32).reshape(R, C)
            tie = np.arange(C) % 3 == 0
            T[:, tie] = (h[:, tie] << np.uint32(16)) | (T[:, tie] & np.uint32(0xFFFF))
        Td = torch.from_numpy(T.view(np.int32)).cuda().view(torch.uint32)
        W = oracle.sample_philox16(T, n, R, C, seed, sub, first, nd, base=base)
        want = oracle.bmm(W, x.reshape(n, Rw, 1))[:, :, 0]
        got = ops.seeded_bmv_philox(Td, dev(x), R, C, seed, sub, first, base=dev(base), half_draws=True)
        np.testing.assert_array_equal(host(got), want, err_msg=str((n, R, C, first)))
        Ws = oracle.sample_philox16(0x10000001, n, R, C, seed, sub, first, nd)
        got_s = ops.seeded_bmv_philox(0x10000001, dev(x), R, C, seed, sub, first, half_draws=True)
        np.testing.assert_array_equal(host(got_s), oracle.bmm(Ws, x.reshape(n, Rw, 1))[:, :, 0])
        if C % wb == 0:
            Wg = ops.sample_bits_philox(Td, n, dtype, seed, sub, first, base=dev(base), half_draws=True)
            assert torch.equal(ops.bmm(Wg, dev(x).view(n, Rw, 1)).squeeze(2), got)
    with pytest.raises(RuntimeError, match="16-bit draws"):
        ops.seeded_bmv_philox(5, dev(rand_words(g, (2, 1), nd)), 3, 12, 1, half_draws=True)


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_weighted_sum_vs_oracle(ops, oracle, dtype):
    g = rng(21)
    # the second line: rows that are whole 32-byte pieces (a wave per piece), also with fewer output bits than the
    # row holds, fewer members than a wave has lanes, and a member count that is not a multiple of 64; the third:
    # rows of 32 bytes or more that are not whole pieces (a conv layer's nine words); the fourth: outputs large enough for
    # the wave-per-piece kernel (1024 pieces or more), whole pieces and ragged
    for n, R, C in [(37, 5, 100), (128, 16, 64), (64, 3, 256), (200, 7, 90), (130, 3, 330), (1, 1, 1),
                    (64, 5, 512), (70, 3, 1000), (130, 2, 1536), (100, 9, 2048), (3, 6, 1024), (257, 1, 520 + 504),
                    (70, 4, 576), (65, 2, 2600), (9, 3, 300),
                    (66, 400, 576), (10, 1100, 256), (5, 130, 2300),
                    # rows without a tail bit (a conv layer's one- and two-word taps): summed as one long row
                    (130, 5000, 64), (40, 4500, 128), (33, 4099, 64), (70, 600, 64),
                    # outputs of 1024 to 2047 16-byte pieces: a wave per two columns (whole pieces, rows of 9 words, ragged)
                    (70, 2304, 64), (50, 300, 576), (37, 260, 520),
                    # no members: zeros
                    (0, 3, 100), (0, 2, 4096)]:
        nd = NDT[dtype]
        wb = np.dtype(nd).itemsize * 8
        words = rand_words(g, (n, R, (C + wb - 1) // wb), nd)
        w = g.standard_normal(n).astype(np.float16)
        got = host(ops.weighted_sum(dev(words), dev(w), C)).astype(np.float32)
        want = oracle.weighted_sum(words, w.astype(np.float32), C)
        # same fp32 additions in the same order, then one rounding to fp16
        np.testing.assert_array_equal(got, want.astype(np.float16).astype(np.float32))


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_bmv_pm1_is_the_linear_layers_activation(ops, oracle, dtype):
    """bmv_pm1(A, x, K) == 2 * bmm(A, x) - K (modules/binary.py:97), on every matrix-vector kernel: rows of 16 / 32 /
    64 bytes, long rows of whole 16-byte vectors, odd rows, unaligned word counts."""
    nd = NDT[dtype]
    wb = np.dtype(nd).itemsize * 8
    g = rng(5)
    for Z, M, Kw in [(5, 7, 64 // (wb // 8) // 4 or 1), (3, 256, 2), (4, 64, 4), (2, 8, 8), (3, 12, 32 * 64 // wb),
                     (2, 16, 512 * 64 // wb), (3, 5, 3), (2, 9, 37), (1, 1, 1), (6, 1000, 16)]:
        A = rand_words(g, (Z, M, Kw), nd)
        x = rand_words(g, (Z, Kw), nd)
        K = Kw * wb - 5 if Kw * wb > 5 else Kw * wb
        want = 2 * oracle.bmm(A, x.reshape(Z, Kw, 1))[:, :, 0].astype(np.int64) - K
        got = ops.bmv_pm1(dev(A), dev(x), K)
        assert got.dtype == torch.int32 and tuple(got.shape) == (Z, M)
        np.testing.assert_array_equal(host(got).astype(np.int64), want, err_msg=str((Z, M, Kw)))
        # the plain product is untouched by the map
        np.testing.assert_array_equal(host(ops.bmm(dev(A), dev(x).view(Z, Kw, 1)))[:, :, 0], oracle.bmm(A, x.reshape(Z, Kw, 1))[:, :, 0])
    with pytest.raises(RuntimeError, match="does not fit"):
        ops._lib.call("nb_bmv_pm1" + ("_i64" if wb == 64 else "_i32"), 8, 8, 8, 1, 1, 1, wb + 1, None)


def _fp16_interval(exact, slack):
    """The fp16 values a correctly rounded result may take when `exact` is known to within `slack`."""
    with np.errstate(over="ignore"):
        return (exact - slack).astype(np.float16).astype(np.float64), (exact + slack).astype(np.float16).astype(np.float64)


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_weighted_sum_fast_mode_within_fp16_rounding_of_the_exact_sum(ops, dtype):
    """fast=True adds the members in blocks through tables of partial sums; the check is the float64 sum over the
    unpacked bits: the result must be the fp16 rounding of a value within 1e-6 * sum|w| of it (fp32 roundings of
    the partial sums), whatever the order.  Shapes: every member split (few / many columns), member counts around
    the chunk of 64 and the block of 32, ragged rows, rows with unused words, one member, no members."""
    g = rng(77)
    nd = NDT[dtype]
    wb = np.dtype(nd).itemsize * 8
    for n, R, C in [(1024, 64, 1024), (1000, 7, 200), (64, 3, 256), (65, 2, 330), (33, 5, 100), (32, 4, 64),
                    (31, 1, 31), (1, 1, 1), (200, 9, 576), (130, 700, 64), (257, 1, 1024), (2100, 3, 96),
                    (96, 1300, 128), (70, 16, 2048), (40, 4200, 64), (512, 300, 1152), (0, 3, 100), (5, 2, 40)]:
        for extra in (0, 1, 2):  # rows with a word that holds no output bit; 2: the other kernel for small outputs
            words = rand_words(g, (n, R, (C + wb - 1) // wb + (extra & 1)), nd)
            w = (g.standard_normal(n) * (3.0 if n % 2 else 0.05)).astype(np.float16)
            if extra == 2:      # force / forbid the kernel whose waves split into two member halves
                os.environ["NESBIN_WSUM_HALVES"] = "0" if n >= 961 else "1"
                os.environ["NESBIN_WSUM_SPLIT"] = "4" if n % 2 else "3"
            try:
                got = host(ops.weighted_sum(dev(words), dev(w), C, fast=True)).astype(np.float64)
            finally:
                os.environ.pop("NESBIN_WSUM_HALVES", None)
                os.environ.pop("NESBIN_WSUM_SPLIT", None)
            bits = np.unpackbits(np.ascontiguousarray(words).view(np.uint8), axis=-1, bitorder="little")[:, :, :C]
            exact = np.einsum("m,mrc->rc", w.astype(np.float64), bits.astype(np.float64))
            lo, hi = _fp16_interval(exact, 1e-6 * float(np.abs(w.astype(np.float64)).sum()) + 1e-30)
            assert got.shape == (R, C)
            bad = (got < lo) | (got > hi)
            assert not bad.any(), (n, R, C, extra, int(bad.sum()), got[bad][:4], exact[bad][:4])
    # the same call twice: the same bits (the order of the additions is fixed)
    words = dev(rand_words(g, (1024, 256, 1024 // wb), nd))
    w = dev(g.standard_normal(1024).astype(np.float16))
    a = ops.weighted_sum(words, w, 1024, fast=True)
    assert torch.equal(a, ops.weighted_sum(words, w, 1024, fast=True))
    # and against the member-order kernel: equal up to the last fp16 digit
    b = ops.weighted_sum(words, w, 1024)
    assert (a.float() - b.float()).abs().max().item() <= 2.0 ** -5


def test_ops_run_on_the_current_stream(ops, oracle):
    g = rng(2)
    A = rand_words(g, (4, 100, 9), np.int64)
    B = rand_words(g, (4, 9, 16), np.int64)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        Ad, Bd = dev(A), dev(B)
        out = ops.bmm(Ad, Bd)
    s.synchronize()
    np.testing.assert_array_equal(host(out), oracle.bmm(A, B))


def test_errors_match_the_reference_conventions(ops):
    a = torch.zeros(2, 3, 4, dtype=torch.int64, device="cuda")
    with pytest.raises(AssertionError):
        ops.bmm(a, torch.zeros(3, 4, 1, dtype=torch.int64, device="cuda"))
    with pytest.raises(RuntimeError, match="contiguous"):
        ops.bmm(a.transpose(1, 2), torch.zeros(2, 3, 1, dtype=torch.int64, device="cuda"))
    with pytest.raises(TypeError):
        ops.bmm(a.to(torch.int16), torch.zeros(2, 4, 1, dtype=torch.int16, device="cuda"))
    with pytest.raises(RuntimeError):
        ops.conv(torch.zeros(1, 2, 2, 1, dtype=torch.int64, device="cuda"),
                 torch.zeros(1, 25, 4, dtype=torch.int64, device="cuda"), 5, 5, 0, 0, 1, 1)
    assert ops.bmm(torch.zeros(0, 3, 4, dtype=torch.int64, device="cuda"),
                   torch.zeros(0, 4, 2, dtype=torch.int64, device="cuda")).shape == (0, 3, 2)


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("C,O,k,pad,stride", [(16, 16, 3, 1, 1), (3, 64, 3, 1, 1), (1, 5, 7, 2, 3), (8, 33, 5, 2, 2),
                                              (32, 20, 3, 0, 1), (16, 70, 1, 0, 1), (5, 16, 3, 2, 1), (2, 4, 9, 4, 1)])
def test_conv_tap_packing_gives_the_same_sums(ops, oracle, engine, dtype, C, O, k, pad, stride):
    """in_bits=C lets several filter taps share a word; every output must equal the one-word-per-tap path."""
    nd = NDT[dtype]
    bits = torch.iinfo(dtype).bits
    D, S = 4, 11
    g = rng(C * 100 + O + k)
    xb = g.integers(0, 2, size=(D * S * S, C)).astype(bool)
    x = oracle.pack(xb, nd).reshape(D, S, S, 1)
    fb = g.integers(0, 2, size=(D * O * k * k, C)).astype(bool)
    f = np.ascontiguousarray(oracle.pack(fb, nd).reshape(D, O, k, k, 1).transpose(0, 2, 3, 4, 1).reshape(D, -1, O))
    K = k * k * C
    thr = (g.integers(0, K + 1, size=(D, O)) - K // 2 + K).astype(np.int32)
    geom = (k, k, pad, pad, stride, stride)
    xd, fd, td = dev(x), dev(f), dev(thr)
    want = oracle.conv(x, f, *geom)
    eligible = 2 * C <= bits
    assert ops.tap_packing_applies(C, 1, dtype) == eligible
    got = ops.conv(xd, fd, *geom, in_bits=C)
    np.testing.assert_array_equal(host(got), want)
    if eligible:
        fp = ops.tap_pack_filter(fd, k * k, C)
        T = bits // C
        assert tuple(fp.shape) == (D, (k * k + T - 1) // T, O)
        # closed form of the packed filter: OR of tap words shifted by C*t
        fw = f.astype(np.uint64 if bits == 64 else np.uint32)
        ref = np.zeros(fp.shape, dtype=fw.dtype)
        for tap in range(k * k):
            ref[:, tap // T, :] |= fw[:, tap, :] << fw.dtype.type(C * (tap % T))
        np.testing.assert_array_equal(host(fp).view(ref.dtype), ref)
        kw = dict(in_bits=C, filter_tap_packed=True)
        np.testing.assert_array_equal(host(ops.conv(xd, fp, *geom, **kw)), want)
        np.testing.assert_array_equal(host(ops.conv_act(xd, fp, td, *geom, **kw)), 2 * want > thr[:, None, None, :])
        act = oracle.conv_act(x, f, thr, *geom)
        h, w = act.shape[1:3]
        packed = oracle.pack(act.reshape(-1, O), nd).reshape(D, h, w, -1)
        np.testing.assert_array_equal(host(ops.conv_act_pack(xd, fp, td, *geom, **kw)), packed)
        assert torch.equal(ops.conv_act_pack(xd, fd, td, *geom, in_bits=C), ops.conv_act_pack(xd, fd, td, *geom))
        if h >= 2 and w >= 2:
            np.testing.assert_array_equal(host(ops.conv_act_pack(xd, fp, td, *geom, pool=True, **kw)),
                                          oracle.max_pool2d(packed, 2, 2, 0, 0, 2, 2))


# (C, O, k, pad, H, W, tap-packed filter, kernel expected): one case per instantiation of the matrix-core kernel
# (K chunks per filter row x channel tiles per wave), ragged widths, channel counts that are not a multiple of 64,
# images that need several bands of rows, and shapes it must decline.
MATRIX_CORE_CASES = [
    (3, 64, 3, 1, 9, 20, True, True),      # 16-byte pixels, 64 channels = two 32-channel tiles
    (3, 16, 3, 1, 12, 12, True, True),     # 16-byte pixels, one 16-channel tile
    (4, 16, 3, 0, 7, 33, False, True),     # in_bits known, filter packed on the fly
    (16, 16, 3, 1, 20, 18, True, True),
    (16, 32, 3, 1, 10, 16, True, True),    # one 32-channel tile, full-word stores with a zero upper half
    (16, 80, 3, 2, 6, 17, False, True),    # O = 80: second task has 16 live channels
    (24, 64, 3, 1, 9, 17, True, True),     # 32-byte pixels, two tap columns per chunk
    (32, 16, 3, 1, 11, 8, True, True),
    (64, 64, 3, 1, 12, 21, False, True),   # 64-byte pixels, one chunk per tap
    (64, 144, 3, 1, 8, 8, False, True),    # three tasks per image, last one 16 channels wide
    (64, 16, 3, 1, 9, 31, False, True),
    (50, 64, 3, 0, 9, 9, False, True),     # tail bits of the channel word are zero
    (128, 96, 3, 1, 5, 16, False, True),   # two channel words per pixel, 16-channel tiles, four per task
    (128, 64, 3, 1, 12, 12, False, True),
    (64, 64, 3, 1, 44, 40, False, True),   # several bands of rows, the last one shorter
    (64, 64, 3, 0, 43, 21, False, True),   # odd output height and width: the pooled map drops the last row / column
    (16, 16, 3, 1, 70, 66, True, True),    # bands limited by the words a producer thread holds in flight
    (64, 64, 1, 0, 6, 40, False, False),   # 1x1 filter: XOR-popcount kernels
    (128, 32, 3, 1, 10, 12, False, False), # 128 input channels need 64 or more output channels
    (8, 16, 5, 2, 9, 9, True, False),      # 5x5 filter
    (64, 24, 3, 1, 8, 8, False, False),    # O % 16 != 0
    (64, 48, 3, 1, 8, 8, False, False),    # three 16-channel tiles
    (448, 64, 3, 1, 6, 6, False, False),   # more than six chunks per filter row
]


@pytest.mark.parametrize("C,O,H,W,served", [(64, 64, 12, 20, "wide"), (128, 64, 9, 9, "wide"), (16, 16, 20, 18, "narrow"),
                                            (16, 64, 11, 17, "narrow"), (8, 32, 16, 16, "narrow"), (64, 16, 8, 8, "odd"),
                                            (96, 64, 8, 8, "odd")])
def test_conv_matrix_core_engines_take_32_bit_words(ops, oracle, mc_engine, C, O, H, W, served):
    """int32 tensors (the word type of the reference's own check, booloptests.py:121) on the matrix-core engines:
    an even number of 32-bit words per pixel is handed on as 64-bit words (filters re-packed), narrow tap-packed layers
    are read as they are by the wave-per-strip kernel; odd word counts and packed outputs of an odd number of 32-bit
    words stay on the XOR-popcount kernels.  All against the oracle run on the int32 tensors."""
    D, k = 3, 3
    g = rng(C * 100 + O + H)
    Cw = (C + 31) // 32
    x = oracle.pack(g.integers(0, 2, size=(D * H * W, C)).astype(bool), np.int32).reshape(D, H, W, Cw)
    f = np.ascontiguousarray(oracle.pack(g.integers(0, 2, size=(D * O * 9, C)).astype(bool), np.int32)
                             .reshape(D, O, 3, 3, Cw).transpose(0, 2, 3, 4, 1).reshape(D, -1, O))
    K = 9 * C
    thr = (g.integers(0, K + 1, size=(D, O)) - K // 2 + K).astype(np.int32)
    thr[0, 0], thr[0, 1] = -5, 2 * K + 3
    geom = (3, 3, 1, 1, 1, 1)
    xd, fd, td = dev(x), dev(f), dev(thr)
    kw = dict(in_bits=C) if 2 * C <= 32 else {}
    want = oracle.conv(x, f, *geom)
    act = oracle.conv_act(x, f, thr, *geom)
    packed = oracle.pack(act.reshape(-1, O), np.int32).reshape(D, H, W, -1)
    prev = ops.conv_engine(mc_engine)
    try:
        got = ops.conv(xd, fd, *geom, **kw)
        assert got.dtype == torch.int32
        np.testing.assert_array_equal(host(got), want)
        if served == "wide":
            assert ops.conv_last_engine() in (2, 4)
        gotp = ops.conv_act_pack(xd, fd, td, *geom, **kw)
        assert gotp.dtype == torch.int32 and tuple(gotp.shape) == packed.shape
        np.testing.assert_array_equal(host(gotp), packed)
        if served in ("wide", "narrow"):
            assert ops.conv_last_engine() in (2, 4), ops.conv_last_engine()
        elif C == 64:
            assert ops.conv_last_engine() == 1            # one 32-bit output word per pixel: not what the 64-bit kernels write
        gotq = ops.conv_act_pack(xd, fd, td, *geom, pool=True, **kw)
        np.testing.assert_array_equal(host(gotq), oracle.max_pool2d(packed, 2, 2, 0, 0, 2, 2))
        np.testing.assert_array_equal(host(ops.conv_act(xd, fd, td, *geom, **kw)), act)
        np.testing.assert_array_equal(host(ops.conv_popc_sums(xd, fd, *geom, **kw)), want.sum(axis=(1, 2)))
    finally:
        ops.conv_engine(prev)


@pytest.mark.parametrize("C,O,k,pad,H,W,tap,covered", MATRIX_CORE_CASES)
def test_conv_matrix_core_engine_vs_oracle(ops, oracle, mc_engine, C, O, k, pad, H, W, tap, covered):
    """The matrix-core engines on shapes chosen per kernel variant: int32 sums, packed and pooled outputs against the
    oracle, and the engine that actually served the call (1 popcount, 2 int8, 4 FP4)."""
    D = 3
    g = rng(C * 1000 + O * 10 + k + H + W)
    Cw = (C + 63) // 64
    xb = g.integers(0, 2, size=(D * H * W, C)).astype(bool)
    x = oracle.pack(xb, np.int64).reshape(D, H, W, Cw)
    fb = g.integers(0, 2, size=(D * O * k * k, C)).astype(bool)
    f = np.ascontiguousarray(oracle.pack(fb, np.int64).reshape(D, O, k, k, Cw).transpose(0, 2, 3, 4, 1)
                             .reshape(D, -1, O))
    K = k * k * C
    thr = (g.integers(0, K + 1, size=(D, O)) - K // 2 + K).astype(np.int32)
    thr[0, 0], thr[0, 1] = -5, 2 * K + 3                                   # always / never above the threshold
    geom = (k, k, pad, pad, 1, 1)
    xd, fd, td = dev(x), dev(f), dev(thr)
    kw = {}
    if C < 64:
        kw = dict(in_bits=C)
    if tap:
        fd = ops.tap_pack_filter(fd, k * k, C)
        kw["filter_tap_packed"] = True
    want = oracle.conv(x, f, *geom)
    act = oracle.conv_act(x, f, thr, *geom)
    h, w = act.shape[1:3]
    packed = oracle.pack(act.reshape(-1, O), np.int64).reshape(D, h, w, -1)
    served = 4 if mc_engine == 2 and k == 3 and _fp4_shape(C, O, k) else (2 if covered else 1)
    # int32 maps of one-word pixels with up to 64 output channels stay on the int8 flavour of the staged-image kernel
    # (write bound) unless the wave-per-strip kernel takes them (3x3 windows)
    served_i32 = (2 if covered else 1) if Cw == 1 and O <= 64 and k != 3 else served
    prev = ops.conv_engine(mc_engine)
    try:
        got = ops.conv(xd, fd, *geom, **kw)
        assert ops.conv_last_engine() == served_i32
        np.testing.assert_array_equal(host(got), want)
        got = ops.conv_act_pack(xd, fd, td, *geom, **kw)
        assert ops.conv_last_engine() == served
        np.testing.assert_array_equal(host(got), packed)
        got = ops.conv_act_pack(xd, fd, td, *geom, pool=True, **kw)
        np.testing.assert_array_equal(host(got), oracle.max_pool2d(packed, 2, 2, 0, 0, 2, 2))
        np.testing.assert_array_equal(host(ops.conv_act(xd, fd, td, *geom, **kw)), act)
        # bool output: the popcount kernels for three members, except a window of at most 32 bits with whole output
        # words, which goes through the packed-output kernel and unpack
        assert ops.conv_last_engine() == (served if tap and k * k * C <= 32 and O % 64 == 0 else 1)
        ops.conv_engine(1)
        ops.conv(xd, fd, *geom, **kw)
        assert ops.conv_last_engine() == 1
    finally:
        ops.conv_engine(prev)


# (C, O, fy, px, py, H, W, D): the wave-per-strip matrix-core kernel for narrow layers (at most 16 channels in, at
# most 64 out, packed output).  Output channel counts below 16, channel counts that leave zero positions in a pixel's 16,
# one to three filter columns, paddings 0-2, images of one to three rows (the short sub-band path), odd heights (the
# pooled map drops the last row), several sub-bands with 13 to 20 rows (every remainder of the four-row loop),
# several strips with a ragged last one, and a population large enough for whole-image sub-bands.
NARROW_CASES = [
    (16, 16, 3, 1, 1, 20, 18, 3),
    (16, 5, 3, 1, 1, 19, 33, 2),
    (7, 16, 3, 1, 1, 67, 20, 2),
    (13, 9, 2, 0, 1, 73, 17, 1),
    (1, 1, 3, 2, 2, 9, 9, 4),
    (16, 16, 1, 1, 0, 35, 70, 2),
    (12, 3, 3, 0, 0, 3, 40, 3),
    (16, 16, 3, 1, 1, 1, 16, 5),
    (16, 16, 3, 1, 1, 2, 5, 5),
    (5, 16, 3, 2, 1, 3, 3, 2),
    (16, 11, 3, 1, 1, 50, 48, 1),
    (9, 16, 3, 1, 2, 38, 31, 3),
    (16, 16, 3, 1, 1, 21, 16, 300),
    (16, 32, 3, 1, 1, 20, 18, 3),              # two channel tiles per wave
    (12, 17, 3, 1, 1, 19, 33, 2),
    (16, 64, 3, 1, 1, 35, 40, 2),              # four tiles: a whole output word
    (9, 33, 2, 0, 1, 67, 20, 2),
    (16, 48, 3, 1, 1, 3, 40, 3),               # four tiles, one of them dead; the short sub-band path
    (8, 64, 3, 1, 1, 38, 31, 130),
]


@pytest.mark.parametrize("C,O,fy,px,py,H,W,D", NARROW_CASES)
def test_conv_narrow_matrix_core_kernel_vs_oracle(ops, oracle, C, O, fy, px, py, H, W, D):
    """Packed and pooled outputs of narrow layers against the oracle, thresholds spread around the sums (and one
    always / one never above), filter tap-packed by the caller and on the fly, and identical to the XOR-popcount
    kernels' answer."""
    g = rng(C * 1000 + O * 10 + fy + H + W)
    x = oracle.pack(g.integers(0, 2, size=(D * H * W, C)).astype(bool), np.int64).reshape(D, H, W, 1)
    fb = g.integers(0, 2, size=(D * O * 3 * fy, C)).astype(bool)
    f = np.ascontiguousarray(oracle.pack(fb, np.int64).reshape(D, O, 3, fy, 1).transpose(0, 2, 3, 4, 1).reshape(D, -1, O))
    K = 3 * fy * C
    thr = (g.integers(0, K + 3, size=(D, O)) - K // 2 + K - 1).astype(np.int32)
    thr[0, 0] = -7
    if O > 1:
        thr[0, 1] = 2 * K + 5
    geom = (3, fy, px, py, 1, 1)
    act = oracle.conv_act(x, f, thr, *geom)
    h, w = act.shape[1:3]
    packed = oracle.pack(act.reshape(-1, O), np.int64).reshape(D, h, w, -1)
    xd, fd, td = dev(x), dev(f), dev(thr)
    ft = ops.tap_pack_filter(fd, 3 * fy, C)
    prev = ops.conv_engine(3)
    try:
        got = ops.conv_act_pack(xd, ft, td, *geom, in_bits=C, filter_tap_packed=True)
        assert ops.conv_last_engine() == 2
        np.testing.assert_array_equal(host(got), packed)
        assert torch.equal(ops.conv_act_pack(xd, fd, td, *geom, in_bits=C), got)
        if h >= 2 and w >= 2:
            pooled = ops.conv_act_pack(xd, ft, td, *geom, pool=True, in_bits=C, filter_tap_packed=True)
            assert ops.conv_last_engine() == 2
            np.testing.assert_array_equal(host(pooled), oracle.max_pool2d(packed, 2, 2, 0, 0, 2, 2))
        ops.conv_engine(1)
        assert torch.equal(ops.conv_act_pack(xd, ft, td, *geom, in_bits=C, filter_tap_packed=True), got)
        assert ops.conv_last_engine() == 1
    finally:
        ops.conv_engine(prev)


# The strip kernels for one word per pixel: tap-packed layers of 17 to 32 channels (+-1 bytes; every taps-per-word
# count and channel counts that leave dead byte positions in the upper half) and full channel words (FP4), with 16,
# 32, 64 and more output channels, images of one to three rows (the short sub-band path), every remainder of the
# four-row loop, ragged strips, unequal paddings, and a population large enough for whole-image sub-bands.
WIDE_STRIP_CASES = [
    (17, 16, 1, 1, 19, 18, 3),
    (21, 32, 1, 1, 20, 33, 2),
    (22, 64, 1, 1, 21, 20, 2),
    (24, 64, 1, 1, 32, 32, 3),
    (31, 128, 0, 1, 22, 17, 2),
    (32, 80, 1, 0, 35, 40, 2),
    (29, 64, 2, 2, 9, 9, 4),
    (24, 64, 1, 1, 1, 16, 5),
    (32, 16, 1, 1, 2, 5, 5),
    (20, 32, 1, 1, 3, 40, 3),
    (27, 64, 1, 1, 67, 31, 1),
    (24, 64, 1, 1, 12, 12, 300),
    (33, 64, 1, 1, 21, 20, 2),
    (64, 32, 1, 2, 38, 31, 2),
    (50, 16, 2, 1, 3, 40, 3),
    (64, 64, 1, 1, 2, 20, 3),                  # the short path of the FP4 flavour
    (64, 16, 1, 1, 129, 5, 1),                 # eight sub-bands of 18 rows, the last one 3 rows: short path after others
    (24, 16, 1, 1, 129, 7, 1),
]


@pytest.mark.parametrize("C,O,px,py,H,W,D", WIDE_STRIP_CASES)
def test_conv_wide_strip_kernels_vs_oracle(ops, oracle, C, O, px, py, H, W, D):
    """Packed and pooled outputs, pixel sums and int32 maps of 3x3 layers with one word per pixel against the oracle,
    thresholds spread around the sums (one always, one never above), on the engine that the shape should get, and identical to
    the XOR-popcount kernels' answer."""
    g = rng(C * 1000 + O * 10 + H + W)
    x = oracle.pack(g.integers(0, 2, size=(D * H * W, C)).astype(bool), np.int64).reshape(D, H, W, 1)
    fb = g.integers(0, 2, size=(D * O * 9, C)).astype(bool)
    f = np.ascontiguousarray(oracle.pack(fb, np.int64).reshape(D, O, 3, 3, 1).transpose(0, 2, 3, 4, 1).reshape(D, -1, O))
    K = 9 * C
    thr = (g.integers(0, K + 3, size=(D, O)) - K // 2 + K - 1).astype(np.int32)
    thr[0, 0], thr[0, 1] = -7, 2 * K + 5
    geom = (3, 3, px, py, 1, 1)
    want = oracle.conv(x, f, *geom)
    act = oracle.conv_act(x, f, thr, *geom)
    h, w = act.shape[1:3]
    packed = oracle.pack(act.reshape(-1, O), np.int64).reshape(D, h, w, -1)
    xd, fd, td = dev(x), dev(f), dev(thr)
    kw = dict(in_bits=C) if C < 64 else {}
    served = 2 if C <= 32 else 4
    if C <= 32:
        fd = ops.tap_pack_filter(fd, 9, C)
        kw["filter_tap_packed"] = True
    prev = ops.conv_engine(2)
    try:
        got = ops.conv_act_pack(xd, fd, td, *geom, **kw)
        assert ops.conv_last_engine() == served
        np.testing.assert_array_equal(host(got), packed)
        if h >= 2 and w >= 2:
            pooled = ops.conv_act_pack(xd, fd, td, *geom, pool=True, **kw)
            assert ops.conv_last_engine() == served
            np.testing.assert_array_equal(host(pooled), oracle.max_pool2d(packed, 2, 2, 0, 0, 2, 2))
        sums = ops.conv_popc_sums(xd, fd, *geom, **kw)
        assert ops.conv_last_engine() == served
        np.testing.assert_array_equal(host(sums), want.reshape(D, -1, O).sum(axis=1))
        maps = ops.conv(xd, fd, *geom, **kw)                                  # int32 maps: whole pixels through an LDS tile
        assert ops.conv_last_engine() == served
        np.testing.assert_array_equal(host(maps), want)
        ops.conv_engine(1)
        assert torch.equal(ops.conv_act_pack(xd, fd, td, *geom, **kw), got)
        assert ops.conv_last_engine() == 1
    finally:
        ops.conv_engine(prev)


def _random_matrix_core_cases(n, seed):
    g = np.random.default_rng(seed)
    cases = []
    while len(cases) < n:
        C = int(g.choice([1, 3, 5, 8, 13, 16, 17, 24, 31, 32, 33, 50, 64, 65, 100, 128]))
        O = int(g.choice([16, 32, 64, 80, 96, 128, 144]))
        fy = int(g.integers(1, 4))
        px, py = int(g.integers(0, 3)), int(g.integers(0, 3))
        H, W = int(g.integers(3, 41)), int(g.integers(3, 71))
        if W + 2 * py < fy:
            continue
        cases.append((C, O, fy, px, py, H, W, int(g.integers(1, 6)), bool(g.integers(0, 2))))
    return cases


def test_conv_matrix_core_random_shapes(ops, oracle, mc_engine):
    """Forty-eight seeded random shapes (channels, output channels, 3 x fy windows, unequal paddings, ragged image
    sizes, 1-5 members, filters tap-packed or not) with engine 2 asked for: all four outputs against the oracle, and
    the matrix-core kernel serves exactly the shapes it is built for."""
    prev = ops.conv_engine(mc_engine)
    try:
        for ci, (C, O, fy, px, py, H, W, D, tap) in enumerate(_random_matrix_core_cases(48, 20240607)):
            print("case", ci, (C, O, fy, px, py, H, W, D, tap), flush=True)
            g = rng(7000 + ci)
            Cw = (C + 63) // 64
            x = oracle.pack(g.integers(0, 2, size=(D * H * W, C)).astype(bool), np.int64).reshape(D, H, W, Cw)
            fb = g.integers(0, 2, size=(D * O * 3 * fy, C)).astype(bool)
            f = np.ascontiguousarray(oracle.pack(fb, np.int64).reshape(D, O, 3, fy, Cw).transpose(0, 2, 3, 4, 1)
                                     .reshape(D, -1, O))
            K = 3 * fy * C
            thr = (g.integers(0, K + 1, size=(D, O)) - K // 2 + K).astype(np.int32)
            geom = (3, fy, px, py, 1, 1)
            xd, fd, td = dev(x), dev(f), dev(thr)
            kw = {}
            if C < 64:
                kw = dict(in_bits=C)
                if tap and C <= 32:
                    fd = ops.tap_pack_filter(fd, 3 * fy, C)
                    kw["filter_tap_packed"] = True
            want = oracle.conv(x, f, *geom)
            act = oracle.conv_act(x, f, thr, *geom)
            h, w = act.shape[1:3]
            packed = oracle.pack(act.reshape(-1, O), np.int64).reshape(D, h, w, -1)
            # chunks per filter row: the kernel exists for 1, 2, 3 and 6; 6 needs 16 or at least 64 output channels
            cpr = (1 if C <= 16 else (fy + 1) // 2) if C <= 32 else fy * Cw
            covered = cpr in (1, 2, 3, 6) and (O >= 64 or O == 16 or (O == 32 and cpr != 6))
            np.testing.assert_array_equal(host(ops.conv(xd, fd, *geom, **kw)), want)
            if mc_engine == 3:
                assert ops.conv_last_engine() != 4
            np.testing.assert_array_equal(host(ops.conv_act_pack(xd, fd, td, *geom, **kw)), packed)
            fp4 = mc_engine == 2 and _fp4_shape(C, O, fy)
            if fp4 and not (Cw == 4 and fy == 3):        # six chunks: also depends on the band fitting the LDS
                assert ops.conv_last_engine() == 4
            elif not fp4 and cpr != 6:                   # likewise with 6 chunks of +-1 bytes
                assert ops.conv_last_engine() == (2 if covered else 1)
            if h >= 2 and w >= 2:
                got = ops.conv_act_pack(xd, fd, td, *geom, pool=True, **kw)
                np.testing.assert_array_equal(host(got), oracle.max_pool2d(packed, 2, 2, 0, 0, 2, 2))
            np.testing.assert_array_equal(host(ops.conv_popc_sums(xd, fd, *geom, **kw)),
                                          want.reshape(D, -1, O).sum(axis=1))
    finally:
        ops.conv_engine(prev)


@pytest.mark.parametrize("C,O,S,mode", [(16, 16, 8, "pool"), (64, 64, 8, "pool"), (64, 128, 6, "pack"),
                                         (64, 64, 8, "sums"), (3, 64, 10, "pack")])
def test_conv_matrix_core_many_members(ops, oracle, mc_engine, C, O, S, mode):
    """More members than workgroups or wave slots: every workgroup of the persistent kernel walks several members
    (fragments and image buffers change hands many times), the strip kernels run in several rounds; every member
    against the oracle."""
    D = 1300
    g = rng(C + O + S)
    Cw = (C + 63) // 64
    x = oracle.pack(g.integers(0, 2, size=(D * S * S, C)).astype(bool), np.int64).reshape(D, S, S, Cw)
    fb = g.integers(0, 2, size=(D * O * 9, C)).astype(bool)
    f = np.ascontiguousarray(oracle.pack(fb, np.int64).reshape(D, O, 3, 3, Cw).transpose(0, 2, 3, 4, 1).reshape(D, -1, O))
    K = 9 * C
    thr = (g.integers(0, K + 1, size=(D, O)) - K // 2 + K).astype(np.int32)
    geom = (3, 3, 1, 1, 1, 1)
    xd, fd, td = dev(x), dev(f), dev(thr)
    kw = dict(in_bits=C) if C < 64 else {}
    served = 4 if mc_engine == 2 and _fp4_shape(C, O, 3) else 2
    prev = ops.conv_engine(mc_engine)
    try:
        if mode == "sums":
            got = ops.conv(xd, fd, *geom, **kw)
            assert ops.conv_last_engine() == served
            np.testing.assert_array_equal(host(got), oracle.conv(x, f, *geom))
        else:
            act = oracle.conv_act(x, f, thr, *geom)
            packed = oracle.pack(act.reshape(-1, O), np.int64).reshape(D, S, S, -1)
            got = ops.conv_act_pack(xd, fd, td, *geom, pool=(mode == "pool"), **kw)
            assert ops.conv_last_engine() == served
            np.testing.assert_array_equal(host(got), oracle.max_pool2d(packed, 2, 2, 0, 0, 2, 2) if mode == "pool" else packed)
    finally:
        ops.conv_engine(prev)


def test_conv_window_random_shapes(ops, oracle):
    """Randomly drawn small-window geometries (1-5 channels, windows up to 5x5 with at most 32 window bits, strides,
    paddings, ragged channel counts, both word widths): packed and bool outputs against the oracle."""
    g0 = rng(4242)
    done = 0
    for ci in range(260):
        nd = np.int64 if g0.integers(0, 2) else np.int32
        bits = np.dtype(nd).itemsize * 8
        C, fx, fy = int(g0.integers(1, 6)), int(g0.integers(1, 6)), int(g0.integers(1, 6))
        sx, sy = int(g0.choice([1, 1, 1, 2])), int(g0.choice([1, 1, 1, 2]))
        px, py = int(g0.integers(0, 4)), int(g0.integers(0, 4))
        H, W, D = int(g0.integers(1, 40)), int(g0.integers(1, 90)), int(g0.integers(1, 6))
        O = int(g0.choice([1, 7, 16, 31, 32, 33, 64, 64, 64, 100, 128]))
        if fx * fy * C > 32 or fx * fy > bits // C or H + 2 * px < fx or W + 2 * py < fy:
            continue
        g = rng(100 + ci)
        x = oracle.pack(g.integers(0, 2, size=(D * H * W, C)).astype(bool), nd).reshape(D, H, W, 1)
        fb = g.integers(0, 2, size=(D * O * fx * fy, C)).astype(bool)
        f = np.ascontiguousarray(oracle.pack(fb, nd).reshape(D, O, fx, fy, 1).transpose(0, 2, 3, 4, 1)
                                 .reshape(D, -1, O))
        K = fx * fy * C
        thr = (g.integers(0, K + 3, size=(D, O)) - K // 2 + K - 1).astype(np.int32)
        geom = (fx, fy, px, py, sx, sy)
        act = oracle.conv_act(x, f, thr, *geom)
        h, w = act.shape[1:3]
        want = oracle.pack(act.reshape(-1, O), nd).reshape(D, h, w, -1)
        xd, fd, td = dev(x), dev(f), dev(thr)
        case = "case %d: %s C=%d O=%d window %dx%d pad %d,%d stride %d,%d image %dx%d D=%d" % (
            ci, np.dtype(nd).name, C, O, fx, fy, px, py, sx, sy, H, W, D)
        np.testing.assert_array_equal(host(ops.conv_act_pack(xd, fd, td, *geom, in_bits=C)), want, err_msg=case)
        assert ops.conv_last_engine() == 1, case
        np.testing.assert_array_equal(host(ops.conv_act(xd, fd, td, *geom, in_bits=C)), act, err_msg=case)
        done += 1
    assert done > 100


@pytest.mark.parametrize("C,O,D,H,W,engine_served", [
    (64, 64, 130, 6, 7, 4),      # full channel word, a population the matrix cores take: FP4 pack kernel + unpack
    (100, 128, 128, 5, 5, 4),    # two channel words with zero tail bits
    (64, 64, 128, 4, 5, 4),
    (3, 64, 5, 9, 9, 1),         # 27-bit window: window-in-a-register kernel + unpack, any population
    (64, 64, 5, 6, 6, 1),        # small population: the XOR-popcount kernel writes the bools itself
    (64, 48, 130, 6, 6, 1),      # O is not a whole number of words: likewise
])
def test_conv_act_bool_map_via_packed_kernels(ops, oracle, C, O, D, H, W, engine_served):
    """conv_act's bool map comes from a packed-output kernel plus unpack where that is the faster way; same bools
    as the oracle either way, and the same as with the engine pinned to the XOR-popcount kernels."""
    g = rng(C + O + D)
    Cw = (C + 63) // 64
    x = oracle.pack(g.integers(0, 2, size=(D * H * W, C)).astype(bool), np.int64).reshape(D, H, W, Cw)
    fb = g.integers(0, 2, size=(D * O * 9, C)).astype(bool)
    f = np.ascontiguousarray(oracle.pack(fb, np.int64).reshape(D, O, 3, 3, Cw).transpose(0, 2, 3, 4, 1).reshape(D, -1, O))
    K = 9 * C
    thr = (g.integers(0, K + 1, size=(D, O)) - K // 2 + K).astype(np.int32)
    geom = (3, 3, 1, 1, 1, 1)
    want = oracle.conv_act(x, f, thr, *geom)
    xd, fd, td = dev(x), dev(f), dev(thr)
    kw = dict(in_bits=C) if C < 32 else {}
    prev = ops.conv_engine(0)
    try:
        got = ops.conv_act(xd, fd, td, *geom, **kw)
        assert got.dtype == torch.bool and got.is_contiguous() and tuple(got.shape) == want.shape
        assert ops.conv_last_engine() == engine_served
        np.testing.assert_array_equal(host(got), want)
        ops.conv_engine(1)
        np.testing.assert_array_equal(host(ops.conv_act(xd, fd, td, *geom, **kw)), want)
        assert ops.conv_last_engine() == 1
    finally:
        ops.conv_engine(prev)


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("C,O,fx,fy,px,py,sx,sy,H,W,D", [
    (3, 64, 3, 3, 1, 1, 1, 1, 32, 32, 5),      # the first layer of an RGB network
    (3, 128, 3, 3, 1, 1, 1, 1, 9, 21, 3),      # two output words per pixel
    (3, 40, 3, 3, 0, 2, 1, 1, 7, 300, 2),      # O not a multiple of 32, more pixels than one workgroup per row
    (2, 100, 3, 3, 2, 0, 2, 1, 11, 13, 4),     # strides, 18-bit window
    (1, 16, 5, 5, 2, 2, 1, 2, 12, 12, 3),      # 25-bit window
    (1, 33, 3, 1, 1, 0, 1, 1, 6, 6, 2),
    (3, 64, 3, 3, 1, 1, 1, 1, 5, 5, 300),      # many members
    (1, 32, 5, 5, 2, 2, 1, 1, 10, 11, 2),      # stride 1 with one to five window rows / columns: the row gather
    (2, 48, 2, 4, 0, 3, 1, 1, 9, 10, 2),
    (4, 32, 1, 5, 0, 1, 1, 1, 4, 7, 3),
    (1, 64, 4, 2, 3, 1, 1, 1, 5, 6, 2),
    (5, 24, 2, 3, 1, 2, 1, 1, 3, 3, 7),        # output wider than the input
    # rows so wide that the LDS copy of a workgroup's input rows would pass 48 KB: the stride-1 gather straight from
    # memory (a workgroup's 256 pixel quads lie inside one output row, or straddle two)
    (1, 33, 3, 3, 1, 1, 1, 1, 3, 3300, 1),
    (3, 40, 3, 3, 1, 0, 1, 1, 4, 3100, 2),
    (2, 64, 2, 5, 0, 2, 1, 1, 2, 4099, 1),
])
def test_conv_window_in_a_register_vs_oracle(ops, oracle, dtype, C, O, fx, fy, px, py, sx, sy, H, W, D):
    """Windows of at most 32 bits with packed output take the window-in-a-register kernel (engines 0 and 1):
    against the oracle, with the filter tap-packed by the caller or on the fly, and identical to the matrix-core
    answer where that engine has a kernel."""
    nd = NDT[dtype]
    bits = np.dtype(nd).itemsize * 8
    g = rng(C * 100 + O + fx + H)
    x = oracle.pack(g.integers(0, 2, size=(D * H * W, C)).astype(bool), nd).reshape(D, H, W, 1)
    fb = g.integers(0, 2, size=(D * O * fx * fy, C)).astype(bool)
    f = np.ascontiguousarray(oracle.pack(fb, nd).reshape(D, O, fx, fy, 1).transpose(0, 2, 3, 4, 1).reshape(D, -1, O))
    K = fx * fy * C
    thr = (g.integers(0, K + 3, size=(D, O)) - K // 2 + K - 1).astype(np.int32)
    thr[0, 0], thr[0, 1] = -7, 2 * K + 5                                     # always / never above the threshold
    geom = (fx, fy, px, py, sx, sy)
    act = oracle.conv_act(x, f, thr, *geom)
    h, w = act.shape[1:3]
    want = oracle.pack(act.reshape(-1, O), nd).reshape(D, h, w, -1)
    xd, fd, td = dev(x), dev(f), dev(thr)
    prev = ops.conv_engine(0)
    try:
        for eng in (0, 1):
            ops.conv_engine(eng)
            np.testing.assert_array_equal(host(ops.conv_act_pack(xd, fd, td, *geom, in_bits=C)), want)
            assert ops.conv_last_engine() == 1
            ft = ops.tap_pack_filter(fd, fx * fy, C)
            got = ops.conv_act_pack(xd, ft, td, *geom, in_bits=C, filter_tap_packed=True)
            np.testing.assert_array_equal(host(got), want)
        if bits == 64 and fx == 3 and sx == 1 and sy == 1 and O % 16 == 0:
            ops.conv_engine(2)
            np.testing.assert_array_equal(host(ops.conv_act_pack(xd, fd, td, *geom, in_bits=C)), want)
            assert ops.conv_last_engine() == 2
    finally:
        ops.conv_engine(prev)


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("C,O,k,pad,stride,H,W,D", [(16, 16, 3, 1, 1, 9, 20, 5), (64, 64, 3, 1, 1, 12, 21, 3),
                                                     (3, 64, 3, 1, 1, 10, 10, 4), (64, 144, 3, 0, 1, 8, 8, 3),
                                                     (128, 64, 3, 1, 1, 6, 18, 2), (20, 7, 5, 2, 2, 11, 9, 3),
                                                     (70, 33, 1, 0, 1, 4, 40, 2), (64, 64, 3, 1, 1, 36, 34, 2),
                                                     (16, 16, 3, 1, 1, 8, 8, 300)])
def test_conv_popc_sums_vs_oracle(ops, oracle, engine, dtype, C, O, k, pad, stride, H, W, D):
    """Sums of the popcount maps over the pixels, per member and channel, against the oracle's conv summed in numpy;
    both engines, shapes the matrix-core kernel covers (several strips, bands, ragged widths) and shapes it does not."""
    nd = NDT[dtype]
    bits = torch.iinfo(dtype).bits
    g = rng(C + O + k + H + W)
    Cw = (C + bits - 1) // bits
    x = oracle.pack(g.integers(0, 2, size=(D * H * W, C)).astype(bool), nd).reshape(D, H, W, Cw)
    fb = g.integers(0, 2, size=(D * O * k * k, C)).astype(bool)
    f = np.ascontiguousarray(oracle.pack(fb, nd).reshape(D, O, k, k, Cw).transpose(0, 2, 3, 4, 1).reshape(D, -1, O))
    geom = (k, k, pad, pad, stride, stride)
    want = oracle.conv(x, f, *geom).sum(axis=(1, 2), dtype=np.int64).astype(np.int32)
    got = ops.conv_popc_sums(dev(x), dev(f), *geom)
    assert got.dtype == torch.int32 and tuple(got.shape) == (D, O)
    np.testing.assert_array_equal(host(got), want)
    if ops.tap_packing_applies(C, Cw, dtype):
        np.testing.assert_array_equal(host(ops.conv_popc_sums(dev(x), dev(f), *geom, in_bits=C)), want)
    np.testing.assert_array_equal(host(ops.conv_popc_sums(dev(x), dev(f), *geom)), want)   # zeroed again on every call


COUNT_SUM_CASES = [
    # C, O, fx, fy, px, py, H, W, D, tap-packed filter
    (64, 64, 3, 3, 1, 1, 32, 32, 5, False),
    (24, 64, 3, 3, 1, 1, 20, 33, 3, True),
    (3, 16, 3, 3, 1, 1, 9, 9, 4, True),
    (200, 48, 5, 5, 2, 2, 19, 20, 2, False),       # four channel words, the 5 x 5 instance
    (64, 64, 3, 3, 0, 0, 9, 10, 5, False),         # no padding: two border rows / columns at either end
    (70, 33, 1, 1, 0, 0, 4, 40, 2, False),         # 1 x 1: no borders at all
    (16, 16, 3, 2, 2, 0, 7, 5, 3, True),           # unequal paddings, two filter columns
    (64, 16, 3, 3, 1, 1, 70, 66, 2, False),        # more pixels than one LDS chunk holds
    (128, 256, 3, 3, 1, 1, 8, 8, 3, False),
    (64, 2100, 3, 3, 1, 1, 6, 6, 2, False),        # more channels than one LDS sum array holds
    (8, 16, 5, 3, 2, 1, 3, 3, 2, True),            # no row that every tap sees
    (64, 32, 3, 3, 2, 2, 5, 6, 3, False),          # padding of 2 with a 3 x 3 filter: output larger than the image
    (33, 16, 2, 4, 0, 1, 12, 9, 2, False),
]


@pytest.mark.parametrize("C,O,fx,fy,px,py,H,W,D,tap", COUNT_SUM_CASES)
def test_conv_popc_sums_from_bit_counts(ops, oracle, C, O, fx, fy, px, py, H, W, D, tap):
    """The automatic engine takes the pixel sums of stride-1 layers from counts of the image's bits per tap (no conv):
    against the oracle's conv summed in numpy, and identical to the conv kernels' sums."""
    g = rng(C * 100 + O + fx + fy + H + W)
    Cw = (C + 63) // 64
    x = oracle.pack(g.integers(0, 2, size=(D * H * W, C)).astype(bool), np.int64).reshape(D, H, W, Cw)
    fb = g.integers(0, 2, size=(D * O * fx * fy, C)).astype(bool)
    f = np.ascontiguousarray(oracle.pack(fb, np.int64).reshape(D, O, fx, fy, Cw).transpose(0, 2, 3, 4, 1)
                             .reshape(D, -1, O))
    geom = (fx, fy, px, py, 1, 1)
    want = oracle.conv(x, f, *geom).sum(axis=(1, 2), dtype=np.int64).astype(np.int32)
    xd, fd = dev(x), dev(f)
    kw = {}
    if tap:
        fd = ops.tap_pack_filter(fd, fx * fy, C)
        kw = dict(in_bits=C, filter_tap_packed=True)
    prev = ops.conv_engine(0)
    try:
        got = ops.conv_popc_sums(xd, fd, *geom, **kw)
        assert ops.conv_last_engine() == 5
        np.testing.assert_array_equal(host(got), want)
        ops.conv_engine(1)
        assert torch.equal(ops.conv_popc_sums(xd, fd, *geom, **kw), got)
        assert ops.conv_last_engine() == 1
        ops.conv_engine(0)
        strided = ops.conv_popc_sums(xd, fd, fx, fy, px, py, 2, 1, **kw)       # a stride: the conv kernels' business
        assert ops.conv_last_engine() != 5
        np.testing.assert_array_equal(host(strided), oracle.conv(x, f, fx, fy, px, py, 2, 1).sum(axis=(1, 2)))
    finally:
        ops.conv_engine(prev)


def test_conv_engine_selector_round_trip(ops):
    prev = ops.conv_engine()
    assert prev in (0, 1, 2, 3)
    assert ops.conv_engine(2) == prev and ops.conv_engine(3) == 2 and ops.conv_engine(1) == 3
    assert ops.conv_engine(7) == 1 and ops.conv_engine() == 1                 # values out of range change nothing
    ops.conv_engine(prev)


def _bn_expected(popc, bias, noise, K):
    """numpy restatement of the population-mean threshold: exact integer sums, one rounding to float32, torch's
    multiplication by float32(M) / float32(Z * M), one rounding to fp16; fp16 additions in the reference's order
    (modules/binary.py:99-101); exact comparison."""
    Z, M = popc.shape
    act = 2 * popc.astype(np.int64) - K
    mean = torch_mean_fp16(act.sum(axis=0), M, Z * M)
    with np.errstate(invalid="ignore", over="ignore"):
        thr = (bias[None, :] + noise).astype(np.float16)
        thr = (thr + mean[None, :]).astype(np.float16)
    return act.astype(np.float64) > thr.astype(np.float64)


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_bmv_bn_act_vs_oracle(ops, oracle, dtype):
    """Linear layer with the population-mean threshold in one call: the oracle's bmm for the sums, numpy for the
    fp16 threshold arithmetic; bool and packed output, ragged member / output counts, rows of every kernel class,
    thresholds that sit on the sums, infinities and NaNs in the noise."""
    nd = NDT[dtype]
    bits = np.dtype(nd).itemsize * 8
    g = rng(31337)
    vec = 16 // np.dtype(nd).itemsize
    for ci, (Z, M, Kw) in enumerate([(16, 64, 4), (7, 10, 2), (33, 130, 16), (5, 64, vec * 16), (12, 256, vec * 32),
                                     (3, 1, 1), (100, 33, 3), (9, 128, 0), (64, 1000, 8), (1000, 24, 5),
                                     (112, 56, 9)]):
        K = Kw * bits - (ci % 3) * (Kw > 0)                       # the true bit count may stop inside the last word
        A = rand_words(g, (Z, M, Kw), nd)
        x = rand_words(g, (Z, Kw), nd)
        if Kw and K < Kw * bits:                                   # tail bits are zero on both operands (pack.cu:17)
            keep = nd(-1) if bits - (Kw * bits - K) == bits else nd((1 << (bits - (Kw * bits - K))) - 1)
            A[:, :, -1] &= keep
            x[:, -1] &= keep
        popc = oracle.bmm(A, x.reshape(Z, Kw, 1))[:, :, 0] if Kw else np.zeros((Z, M), np.int32)
        bias = (g.standard_normal(M) * 4).astype(np.float16)
        noise = ((g.random((Z, M)) - 0.5) * 6).astype(np.float16)
        # make some thresholds land exactly on an activation: noise = act - mean - bias, then the compare is a tie
        act = 2 * popc.astype(np.int64) - K
        mean = torch_mean_fp16(act.sum(axis=0), M, Z * M)
        tie = g.random((Z, M)) < 0.2
        noise[tie] = (act - mean[None, :].astype(np.float64) - bias[None, :].astype(np.float64)).astype(np.float16)[tie]
        noise[0, 0] = np.float16(np.inf)
        if Z > 1:
            noise[1, 0] = np.float16(-np.inf)
        if M > 1:
            noise[0, 1] = np.float16(np.nan)
        want = _bn_expected(popc, bias, noise, K)
        Ad, xd, bd, nz = dev(A), dev(x), dev(bias), dev(noise)
        got = ops.bmv_bn_act(Ad, xd, bd, nz, K)
        assert got.dtype == torch.bool and tuple(got.shape) == (Z, M)
        np.testing.assert_array_equal(host(got), want, err_msg="case %d" % ci)
        ws = torch.empty(int(ops._lib.load().nb_bmv_bn_workspace_bytes(Z, M)) + 256, dtype=torch.uint8, device="cuda")
        ws.fill_(0xA5)                                             # stale contents must not matter
        gotp = ops.bmv_bn_act(Ad, xd.view(Z, Kw, 1), bd, nz, K, pack=True, workspace=ws)
        assert gotp.dtype == dtype and tuple(gotp.shape) == (Z, (M + bits - 1) // bits)
        np.testing.assert_array_equal(host(gotp), oracle.pack(want, nd), err_msg="case %d packed" % ci)
        # against torch's own expression of the reference wherever its fp32 sums are exact (activations within
        # fp16's integers, totals below 2**24): any population size, also those whose reciprocal is not exact
        if K <= 2048 and Z * K < 2 ** 24:
            act_t = dev(act.astype(np.int32))
            thresh = bd + nz
            thresh += act_t.type(torch.float16).mean(dim=0, keepdim=True)
            assert torch.equal(got, act_t > thresh)
    with pytest.raises(RuntimeError, match="workspace"):
        ops._lib.call("nb_bmv_bn_act_i64", 256, 256, 256, 256, 256, 4, 64, 1, 64, 0, 256, 16, None)


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("n,O,k,C", [(3, 16, 3, 16), (2, 64, 3, 64), (5, 8, 3, 3), (2, 33, 5, 70), (17, 64, 3, 128),
                                     (2, 4, 1, 256), (9, 128, 3, 64)])
def test_sampler_writes_the_conv_layout_in_the_same_pass(ops, oracle, dtype, n, O, k, C):
    """sample_bits*(conv_taps=k*k): the rows layout [n, O*k*k, Cw] equals the plain sampler's (and the oracle's), and
    the conv layout equals its view -> permute(0,2,3,4,1) -> reshape(n, k*k*Cw, O) (modules/binary.py:134-137);
    supplied words and generator mode, thresholds per element and a scalar flip probability with a base."""
    nd = NDT[dtype]
    wb = np.dtype(nd).itemsize * 8
    KK, R, Cw = k * k, O * k * k, (C + wb - 1) // wb
    g = rng(n + O + k + C)
    words = g.integers(0, 2 ** 32, size=(n, R, C), dtype=np.uint64).astype(np.uint32)
    thr = g.integers(0, 2 ** 32, size=(R, C), dtype=np.uint64).astype(np.uint32)
    base = rand_words(g, (R, Cw), nd)
    if C % wb:
        base[:, -1] &= nd((1 << (C % wb)) - 1)
    T = int(0.02 * 2 ** 32)

    def permuted(rows):                                                   # numpy restatement of the layer's permute
        return np.ascontiguousarray(rows.reshape(n, O, k, k, Cw).transpose(0, 2, 3, 4, 1).reshape(n, KK * Cw, O))

    want = oracle.sample_from_words(thr, words, nd)
    rows, conv = ops.sample_bits_from_words(dev(thr), dev(words), dtype, conv_taps=KK)
    np.testing.assert_array_equal(host(rows), want)
    assert tuple(conv.shape) == (n, KK * Cw, O) and conv.is_contiguous()
    np.testing.assert_array_equal(host(conv), permuted(want))
    want = oracle.sample_from_words(T, words, nd, base=base)
    rows, conv = ops.sample_bits_from_words(T, dev(words), dtype, base=dev(base), conv_taps=KK, rows_too=False)
    assert rows is None
    np.testing.assert_array_equal(host(conv), permuted(want))
    # generator mode: the same stream as the plain sampler
    plain = ops.sample_bits_philox(dev(thr), n, dtype, 99, 5)
    rows, conv = ops.sample_bits_philox(dev(thr), n, dtype, 99, 5, conv_taps=KK)
    assert torch.equal(rows, plain)
    np.testing.assert_array_equal(host(conv), permuted(host(plain)))
