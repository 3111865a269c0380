"""Sparse form of a population's linear layer (shared base + per-member flip lists) against the CPU oracle's bmm on
the materialised weights: the shared product on the matrix cores, the structure of the flip lists, and the corrected
sums / thresholded packed bits.  Everything is integer work: bit-exact."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available()
    from nesgpu_amd.extensions import booleanOperations
    return booleanOperations


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.cpu().numpy()


def rand_words(g, shape):
    return g.integers(-2 ** 63, 2 ** 63, size=shape, dtype=np.int64)


def sparse_mask(g, shape_bits, p):
    """packed int64 mask [.., ceil(C/64)] with Bernoulli(p) bits in the first C columns"""
    *lead, C = shape_bits
    bits = g.random((int(np.prod(lead)), C)) < p
    pad = (-C) % 64
    words = np.packbits(np.pad(bits, ((0, 0), (0, pad))), axis=1, bitorder="little").view("<i8")
    return words.reshape(*lead, -1)


@pytest.mark.parametrize("M,N,Kw", [(1, 1, 1), (5, 7, 3), (128, 128, 2), (130, 257, 5), (300, 64, 128), (64, 1000, 16),
                                    (33, 129, 511), (256, 384, 64)])
def test_bmm_nt_vs_oracle(ops, oracle, M, N, Kw):
    """popcount(A_m ^ B_n) on the matrix cores (FP4 codes) == the oracle's bmm with B transposed, sign bits and all."""
    g = np.random.default_rng(M * 7 + N * 3 + Kw)
    A, B = rand_words(g, (M, Kw)), rand_words(g, (N, Kw))
    if M > 2:
        A[0] = 0
        A[1] = -1                                               # all ones
        A[2] = B[0]                                             # equal rows: 0
    want = oracle.bmm(A[None], np.ascontiguousarray(B.T)[None])[0]
    got = ops.bmm_nt(dev(A), dev(B))
    assert got.dtype == torch.int32 and tuple(got.shape) == (M, N)
    np.testing.assert_array_equal(host(got), want)
    eb = ops.expand_rows(dev(B))                                # an operand expanded once and used again
    np.testing.assert_array_equal(host(ops.bmm_nt(dev(A), eb)), want)
    if M > 2:
        assert int(got[2, 0]) == 0


def test_expand_rows_codes(ops):
    """bit 1 -> E2M1 code 0x2 (+1.0), bit 0 -> 0xA (-1.0), bit j of a byte -> nibble j; padding rows / words -> 0."""
    x = np.array([[0x01, -1], [0x8000000000000000 - 2 ** 64, 0xF0]], dtype=np.int64)
    e = ops.expand_rows(dev(x))
    assert e.rows_padded == 128 and e.Kw_padded == 2 and tuple(e.codes.shape) == (128, 64)
    c = host(e.codes)
    bits = np.unpackbits(x.view(np.uint8), axis=1, bitorder="little")              # [2, 128]
    nib = np.stack([c[:2] & 15, c[:2] >> 4], axis=2).reshape(2, 128)                 # low nibble first
    np.testing.assert_array_equal(nib, np.where(bits == 1, 0x2, 0xA))
    assert not c[2:].any()


def decode_flip_rows(rows):
    """FlipRows -> boolean flip mask [D, R, 64 * Kw] and the base bit every entry claims, read back entry by entry."""
    D, R, Kw = rows.D, rows.R, rows.Kw
    S = (R + 63) // 64
    ent = host(rows.entries).astype(np.uint32)
    off, ln, perm = host(rows.slice_off), host(rows.slice_len), host(rows.perm).astype(np.int64)
    mask = np.zeros((D, R, 64 * Kw), dtype=bool)
    bflag = np.zeros((D, R, 64 * Kw), dtype=bool)
    sentinel = (4 * Kw) << 5
    for d in range(D):
        for s in range(S):
            L = int(ln[d, s])                                                            # 16-byte pieces per lane
            assert off[d, s] % 4 == 0
            blk = ent[off[d, s]: off[d, s] + L * 256].reshape(L, 64, 4).transpose(0, 2, 1).reshape(4 * L, 64)
            halves = np.stack([blk & 0xFFFF, blk >> 16], axis=1).reshape(8 * L, 64)     # flips in order, per lane
            for lane in range(64):
                p = s * 64 + lane
                col_prev, ended = -1, False
                for e in halves[:, lane]:
                    e = int(e)
                    if e == sentinel:
                        ended = True
                        continue
                    assert not ended and p < R, "a flip after the sentinel / in a lane without a row"
                    piece, bit = e >> 5, e & 31
                    assert piece < 4 * Kw
                    b = bool(piece & 1)
                    col = (piece >> 1) * 32 + bit
                    assert col > col_prev                                                # column order
                    col_prev = col
                    mask[d, perm[d, p], col] = True
                    bflag[d, perm[d, p], col] = b
    return mask, bflag


@pytest.mark.parametrize("D,R,C,p", [(3, 64, 64, 0.1), (2, 100, 200, 0.05), (2, 1024, 256, 0.02), (3, 1100, 128, 0.3),
                                     (1, 2100, 64, 0.01), (4, 7, 960, 0.0), (2, 130, 70, 1.0)])
def test_flip_rows_hold_exactly_the_flipped_bits(ops, D, R, C, p):
    g = np.random.default_rng(D + R + C)
    Kw = (C + 63) // 64
    base = sparse_mask(g, (R, C), 0.5)
    flips = sparse_mask(g, (D, R, C), p)
    W = base[None] ^ flips
    rows = ops.flip_rows_from_weights(dev(W), dev(base))
    cnt = host(rows.cnt).astype(np.int64)
    want_bits = np.unpackbits(flips.view(np.uint8), axis=2, bitorder="little").astype(bool)   # [D, R, 64 Kw]
    np.testing.assert_array_equal(cnt, want_bits.sum(axis=2))
    perm = host(rows.perm).astype(np.int64)
    for d in range(D):
        assert sorted(perm[d].tolist()) == list(range(R))                                      # a permutation ...
        assert (perm[d] // 1024 == np.arange(R) // 1024).all()                                 # ... inside blocks of 1024
        for b0 in range(0, R, 1024):
            assert (np.diff(cnt[d, perm[d, b0:b0 + 1024]]) >= 0).all()                         # ordered by flip count
    S = (R + 63) // 64
    cs = np.pad(np.take_along_axis(cnt, perm, axis=1), ((0, 0), (0, S * 64 - R))).reshape(D, S, 64)
    np.testing.assert_array_equal(host(rows.slice_len), (cs.max(axis=2) + 7) // 8)
    mask, bflag = decode_flip_rows(rows)
    np.testing.assert_array_equal(mask, want_bits)
    base_bits = np.unpackbits(base.view(np.uint8), axis=1, bitorder="little").astype(bool)
    np.testing.assert_array_equal(bflag, mask & base_bits[None])


@pytest.mark.parametrize("D,R,C,p", [(5, 64, 64, 0.1), (3, 100, 200, 0.05), (4, 1024, 8192, 0.01), (2, 1100, 128, 0.3),
                                     (300, 128, 256, 0.02), (2, 2100, 64, 0.01), (4, 7, 960, 0.0), (2, 130, 70, 1.0),
                                     (3, 1, 1, 0.5), (2, 1024, 32704, 0.002)])
def test_bmv_flip_vs_oracle(ops, oracle, D, R, C, p):
    """Sums and thresholded packed bits from base + flip lists == the oracle's bmm on the materialised weights."""
    g = np.random.default_rng(D * 5 + R + C)
    Kw = (C + 63) // 64
    base = sparse_mask(g, (R, C), 0.5)
    W = base[None] ^ sparse_mask(g, (D, R, C), p)
    x = sparse_mask(g, (D, C), 0.5)
    want = oracle.bmm(W, x.reshape(D, Kw, 1))[:, :, 0]
    Wd, xd = dev(W), dev(x)
    rows = ops.flip_rows_from_weights(Wd, dev(base))
    got = ops.bmv_flip(rows, xd)
    assert got.dtype == torch.int32 and tuple(got.shape) == (D, R)
    np.testing.assert_array_equal(host(got), want)
    assert torch.equal(got, ops.bmm(Wd, xd.view(D, Kw, 1)).squeeze(2))                 # and the dense GPU kernel
    thr = (2 * want + g.integers(-3, 4, size=want.shape)).astype(np.int32)
    thr[0, 0], thr[-1, -1] = -1, 2 * 64 * Kw + 1                                        # always / never
    bits = 2 * want.astype(np.int64) > thr
    gotp = ops.bmv_flip_act_pack(rows, xd.view(D, Kw, 1), dev(thr))
    assert gotp.dtype == torch.int64 and tuple(gotp.shape) == (D, (R + 63) // 64)
    np.testing.assert_array_equal(host(gotp), oracle.pack(bits, np.int64))
    # a precomputed shared product may be passed in
    G = ops.bmm_nt(xd, rows.base_expanded)
    np.testing.assert_array_equal(host(G), oracle.bmm(x[None], np.ascontiguousarray(base.T)[None])[0])
    assert torch.equal(ops.bmv_flip(rows, xd, G=G), got)


@pytest.mark.parametrize("D,R,hi", [(1, 1, 5), (3, 63, 3), (2, 64, 100), (5, 100, 2), (3, 1024, 40), (2, 1100, 7),
                                    (2, 2053, 65535), (70, 130, 9)])
def test_flip_layout_orders_blocks_of_rows_by_count(ops, D, R, hi):
    """Row order and slice lengths against numpy: a stable sort by count inside every block of 1024 rows, pieces per
    lane from the longest row of each run of 64; running offsets in dwords."""
    g = np.random.default_rng(D * 1000 + R)
    cnt = g.integers(0, hi + 1, size=(D, R)).astype(np.uint16)
    perm, slice_len, slice_off, total = ops._flip_rows_layout(dev(cnt.view(np.int16)).view(torch.uint16), D, R)
    S = (R + 63) // 64
    want_perm = np.concatenate([b0 + np.argsort(cnt[:, b0:b0 + 1024].astype(np.int64), axis=1, kind="stable")
                                for b0 in range(0, R, 1024)], axis=1)
    np.testing.assert_array_equal(host(perm.view(torch.int16)).view(np.uint16), want_perm.astype(np.uint16))
    sorted_cnt = np.take_along_axis(cnt.astype(np.int64), want_perm, axis=1)
    padded = np.zeros((D, S * 64), dtype=np.int64)
    padded[:, :R] = sorted_cnt
    want_len = (padded.reshape(D, S, 64).max(axis=2) + 7) // 8
    np.testing.assert_array_equal(host(slice_len), want_len.astype(np.int32))
    lens = want_len.reshape(-1) * 256
    np.testing.assert_array_equal(host(slice_off).reshape(-1), np.cumsum(lens) - lens)
    assert total == int(lens.sum())
    assert slice_off.dtype == torch.int64 and slice_len.dtype == torch.int32 and perm.dtype == torch.uint16


def test_flip_shapes_are_checked(ops):
    with pytest.raises(RuntimeError, match="at most 511"):
        ops._lib.call("nb_flip_count_i64", 256, 256, 256, 1, 4, 512, None)
    with pytest.raises(RuntimeError, match="whole tiles"):
        ops._lib.call("nb_bmm_nt_fp4", 256, 256, 256, 130, 4, 2, 128, 128, 2, None)


@pytest.mark.parametrize("D,R,C,p,first", [(3, 64, 64, 0.1, 0), (2, 100, 200, 0.05, 8), (4, 1024, 8192, 0.01, 0),
                                           (2, 1100, 128, 0.3, 3), (300, 128, 256, 0.02, 0), (2, 70, 3000, 0.0002, 5),
                                           (2, 10, 64, 0.0, 0), (2, 130, 70, 1.0, 0), (3, 1, 1, 0.5, 1),
                                           # rows on block boundaries of the stream with a table cut short (words
                                           # beyond it: no flip), p = 1 there, and more rows than one pass of lanes
                                           (2, 70, 3000, 0.0002, 4), (3, 130, 72, 1.0, 0), (2, 64, 4, 0.5, 12),
                                           (600, 1024, 64, 0.1, 0)])
def test_skip_sampler_vs_oracle(ops, oracle, D, R, C, p, first):
    """Flip lists drawn by the skip sampler == the oracle's restatement of the same walk (materialised through
    flip_rows_to_weights), and the products from those lists == the oracle's bmm on the oracle's weights."""
    g = np.random.default_rng(D + R + C)
    Kw = (C + 63) // 64
    T = min(int(p * 2 ** 32), 2 ** 32 - 1)
    seed, sub = 0x5EED0000 + C, 21
    base = sparse_mask(g, (R, C), 0.5)
    table = ops.skip_table(T)
    np.testing.assert_array_equal(table, oracle.skip_cdf(T))
    want_W = base[None] ^ oracle.skip_flips(table, seed, sub, first, D * R, C).reshape(D, R, Kw)
    rows = ops.flip_rows_skip(dev(base), C, D, T, seed, subsequence=sub, first=first)
    flips = np.unpackbits((want_W ^ base[None]).view(np.uint8), axis=2, bitorder="little")
    np.testing.assert_array_equal(host(rows.cnt).astype(np.int64), flips.sum(axis=2))
    W = ops.flip_rows_to_weights(rows)
    np.testing.assert_array_equal(host(W), want_W)
    x = sparse_mask(g, (D, C), 0.5)
    want = oracle.bmm(want_W, x.reshape(D, Kw, 1))[:, :, 0]
    np.testing.assert_array_equal(host(ops.bmv_flip(rows, dev(x))), want)
    assert torch.equal(ops.bmm(W, dev(x).view(D, Kw, 1)).squeeze(2), ops.bmv_flip(rows, dev(x)))
    if D * R * C <= 500000:                                     # the lists themselves, entry by entry
        mask, bflag = decode_flip_rows(rows)
        np.testing.assert_array_equal(mask[:, :, :C], flips[:, :, :C].astype(bool))
        base_bits = np.unpackbits(base.view(np.uint8), axis=1, bitorder="little").astype(bool)
        np.testing.assert_array_equal(bflag, mask & base_bits[None])
    # lists built from the materialised weights hold the same flips
    again = ops.flip_rows_from_weights(W, dev(base))
    assert torch.equal(again.cnt, rows.cnt) and torch.equal(ops.flip_rows_to_weights(again), W)


def test_skip_sampler_rate_at_the_size_of_a_wide_layer(ops):
    """8192 columns, p = 0.01, 64 members x 1024 rows: flip rate, row-count spread and column uniformity."""
    T = 42949672
    base = torch.zeros((1024, 128), dtype=torch.int64, device="cuda")
    rows = ops.flip_rows_skip(base, 8192, 64, T, 7)
    cnt = rows.cnt.view(torch.int16).to(torch.float64)
    n = cnt.numel() * 8192
    p = T / 2 ** 32
    assert abs(float(cnt.sum()) / n - p) < 4 * (p / n) ** 0.5
    assert abs(float(cnt.std()) - (8192 * p * (1 - p)) ** 0.5) < 0.1
    W = ops.flip_rows_to_weights(rows)
    per_col = ops.unpack(W.view(-1, 128)).view(64 * 1024, 8192).float().mean(dim=0)
    assert float((per_col - p).abs().max()) < 6 * (p / (64 * 1024)) ** 0.5
