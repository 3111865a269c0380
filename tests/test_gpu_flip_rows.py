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


def decode_flip_rows(rows, ordered=True):
    """FlipRows -> boolean flip mask [D, R, 64 * Kw] and the base bit every entry claims, read back entry by entry.
    ``ordered``: the entries of a row come in column order (else: every column at most once)."""
    D, R, Kw, cap = rows.D, rows.R, rows.Kw, rows.cap
    S = (R + 63) // 64
    ent = host(rows.entries).astype(np.uint32)
    info = host(rows.info.view(torch.int32)).astype(np.int64)
    mask = np.zeros((D, R, 64 * Kw), dtype=bool)
    bflag = np.zeros((D, R, 64 * Kw), dtype=bool)
    sentinel = (4 * Kw) << 5
    for d in range(D):
        for r in range(R):
            n, pieces = int(info[d, r] & 0xFFFF), int(info[d, r] >> 16)
            assert pieces <= cap and (n + 7) // 8 <= pieces
            col_prev, seen = -1, 0
            for j in range(pieces):
                at = (((d * S + r // 64) * cap + j) * 64 + r % 64) * 4
                for dw in ent[at: at + 4]:
                    for e in (int(dw) & 0xFFFF, int(dw) >> 16):
                        if e == sentinel:
                            continue
                        piece, bit = e >> 5, e & 31
                        assert piece < 4 * Kw
                        col = (piece >> 1) * 32 + bit
                        assert col > col_prev if ordered else not mask[d, r, col]
                        col_prev = col
                        seen += 1
                        mask[d, r, col] = True
                        bflag[d, r, col] = bool(piece & 1)
            assert seen == n
    return mask, bflag


@pytest.mark.parametrize("D,R,C,p", [(3, 64, 64, 0.1), (2, 100, 200, 0.05), (2, 1024, 256, 0.02), (3, 1100, 128, 0.3),
                                     (1, 2100, 64, 0.01), (4, 7, 960, 0.0), (2, 130, 70, 1.0)])
def test_flip_rows_hold_exactly_the_flipped_bits(ops, D, R, C, p):
    g = np.random.default_rng(D + R + C)
    base = sparse_mask(g, (R, C), 0.5)
    flips = sparse_mask(g, (D, R, C), p)
    W = base[None] ^ flips
    rows = ops.flip_rows_from_weights(dev(W), dev(base))
    want_bits = np.unpackbits(flips.view(np.uint8), axis=2, bitorder="little").astype(bool)   # [D, R, 64 Kw]
    np.testing.assert_array_equal(host(rows.cnt).astype(np.int64), want_bits.sum(axis=2))
    assert rows.cap == (int(want_bits.sum(axis=2).max()) + 7) // 8 and rows.overflowed() == 0
    mask, bflag = decode_flip_rows(rows)
    np.testing.assert_array_equal(mask, want_bits)
    base_bits = np.unpackbits(base.view(np.uint8), axis=1, bitorder="little").astype(bool)
    np.testing.assert_array_equal(bflag, mask & base_bits[None])
    # a capacity with room to spare holds the same lists; one that is too small is reported
    roomy = ops.flip_rows_from_weights(dev(W), dev(base), cap=rows.cap + 3)
    assert torch.equal(ops.flip_rows_to_weights(roomy), dev(W)) and roomy.overflowed() == 0
    if rows.cap > 1:
        tight = ops.flip_rows_from_weights(dev(W), dev(base), cap=rows.cap - 1)
        assert tight.overflowed() == int(((want_bits.sum(axis=2) + 7) // 8 > rows.cap - 1).sum())


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


def test_flip_shapes_are_checked(ops):
    with pytest.raises(RuntimeError, match="at most 511"):
        ops._lib.call("nb_flip_count_i64", 256, 256, 256, 1, 4, 512, None)
    with pytest.raises(RuntimeError, match="at most 8191"):
        ops._lib.call("nb_bmv_flip_i64", 256, 256, 256, 256, 256, 1, 4, 2, 9000, None)
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
    assert rows.overflowed() == 0
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


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("n,O,KK,C,p,first", [(5, 64, 9, 64, 0.01, 0), (3, 128, 9, 64, 0.05, 4), (4, 16, 9, 16, 0.1, 3),
                                              (2, 64, 9, 3, 0.02, 0), (3, 24, 1, 512, 0.01, 0), (2, 300, 1, 200, 0.3, 8),
                                              (2, 7, 25, 130, 0.002, 1), (3, 70, 9, 256, 0.0, 0), (2, 33, 4, 100, 1.0, 0),
                                              (9, 512, 9, 64, 0.01, 0), (1, 1, 1, 1, 0.5, 0)])
def test_skip_sampler_as_packed_words_vs_oracle(ops, oracle, dtype, n, O, KK, C, p, first):
    """sample_bits_skip (short rows, packed words) == base ^ the oracle's skip walk, in the row layout and in the conv
    layout; for 64-bit words also == the lists of flip_rows_skip with the same seed, expanded."""
    bits = 64 if dtype == torch.int64 else 32
    R = O * KK
    Rw = (C + bits - 1) // bits
    if Rw > 8:
        pytest.skip("rows of more than 8 words take the lists")
    g = np.random.default_rng(n + O + C)
    T = min(int(p * 2 ** 32), 2 ** 32 - 1)
    seed, sub = 0xABCD + C, 5
    base64 = sparse_mask(g, (R, C), 0.5)                                       # int64 [R, ceil(C/64)], tail bits zero
    mask64 = oracle.skip_flips(ops.skip_table(T), seed, sub, first, n * R, C).reshape(n, R, -1)
    want64 = base64[None] ^ mask64
    if bits == 64:
        base, want = base64, want64
    else:                                                                       # the same bits as 32-bit words
        base = np.ascontiguousarray(base64.view(np.int32)[:, :Rw])
        want = np.ascontiguousarray(want64.view(np.int32).reshape(n, R, -1)[:, :, :Rw])
    got = ops.sample_bits_skip(T, n, dtype, seed, subsequence=sub, first=first, base=dev(base), shape=(R, C))
    np.testing.assert_array_equal(host(got), want)
    rows, conv = ops.sample_bits_skip(T, n, dtype, seed, subsequence=sub, first=first, base=dev(base), shape=(R, C),
                                      conv_taps=KK)
    np.testing.assert_array_equal(host(rows), want)
    # [n, KK*Rw, O]: word k of row (o, t) at [m][t*Rw + k][o]
    want_conv = want.reshape(n, O, KK, Rw).transpose(0, 2, 3, 1).reshape(n, KK * Rw, O)
    np.testing.assert_array_equal(host(conv), want_conv)
    only_conv = ops.sample_bits_skip(T, n, dtype, seed, subsequence=sub, first=first, base=dev(base), shape=(R, C),
                                     conv_taps=KK, rows_too=False)
    assert only_conv[0] is None and torch.equal(only_conv[1], conv)
    nobase = ops.sample_bits_skip(T, n, dtype, seed, subsequence=sub, first=first, shape=(R, C))
    np.testing.assert_array_equal(host(nobase) ^ base[None], want)
    if bits == 64:
        lists = ops.flip_rows_skip(dev(base), C, n, T, seed, subsequence=sub, first=first)
        if lists.overflowed() == 0:
            assert torch.equal(ops.flip_rows_to_weights(lists), got)


def test_skip_sampler_as_packed_words_rejects_long_rows(ops):
    base = torch.zeros((4, 9), dtype=torch.int64, device="cuda")
    with pytest.raises(ValueError, match="at most 8 words"):
        ops.sample_bits_skip(1 << 24, 2, torch.int64, 1, base=base, shape=(4, 576))
    with pytest.raises(RuntimeError, match="more than 8 words"):
        ops._lib.call("nb_sample_skip_i64", base.data_ptr(), base.data_ptr(), ops.skip_table_buffer(ops.skip_table(1 << 24), "cuda").data_ptr(),
                      1, 0, 0, 1, 4, 576, None)


def test_skip_sampler_rate_at_the_size_of_a_wide_layer(ops):
    """8192 columns, p = 0.01, 64 members x 1024 rows: flip rate, row-count spread and column uniformity."""
    T = 42949672
    base = torch.zeros((1024, 128), dtype=torch.int64, device="cuda")
    rows = ops.flip_rows_skip(base, 8192, 64, T, 7)
    cnt = rows.cnt.to(torch.float64)
    n = cnt.numel() * 8192
    p = T / 2 ** 32
    assert abs(float(cnt.sum()) / n - p) < 4 * (p / n) ** 0.5
    assert abs(float(cnt.std()) - (8192 * p * (1 - p)) ** 0.5) < 0.1
    W = ops.flip_rows_to_weights(rows)
    per_col = ops.unpack(W.view(-1, 128)).view(64 * 1024, 8192).float().mean(dim=0)
    assert float((per_col - p).abs().max()) < 6 * (p / (64 * 1024)) ** 0.5


def test_skip_sampler_reports_rows_beyond_the_capacity(ops, oracle):
    """A capacity below what some rows need: those rows are cut to capacity * 8 flips and counted, the others are
    what they are with room to spare."""
    g = np.random.default_rng(4)
    R, C, D, T = 70, 512, 9, int(0.05 * 2 ** 32)
    base = dev(sparse_mask(g, (R, C), 0.5))
    full = ops.flip_rows_skip(base, C, D, T, 11)
    need = (full.cnt + 7) // 8
    cap = int(need.max().item()) - 1
    cut = ops.flip_rows_skip(base, C, D, T, 11, cap=cap)
    assert cut.overflowed() == int((need > cap).sum().item()) > 0
    fine = (need <= cap)
    assert torch.equal(cut.cnt[fine], full.cnt[fine]) and bool((cut.cnt[~fine] == 8 * cap).all())
    Wc, Wf = ops.flip_rows_to_weights(cut), ops.flip_rows_to_weights(full)
    assert torch.equal(Wc[fine], Wf[fine])


@pytest.mark.parametrize("D,R,C,first,spread", [(3, 64, 64, 0, 0.2), (2, 100, 200, 8, 0.05), (3, 1024, 2048, 0, 0.02),
                                                (2, 70, 300, 3, 0.1), (40, 130, 72, 0, 0.3), (2, 9, 8192, 4, 0.01),
                                                (3, 5, 77, 1, 0.05), (2, 16, 16384, 0, 0.004)])
def test_thinning_sampler_vs_oracle(ops, oracle, D, R, C, first, spread):
    """Flip lists under a per-element law == the oracle's restatement of the thinned walk, given the same law and the
    same table (the one the library made on the device); sums from the lists == the oracle's bmm."""
    g = np.random.default_rng(D + R + C)
    Kw = (C + 63) // 64
    P = np.where(g.random((R, C)) < 0.5, g.random((R, C)) * spread, 1.0 - g.random((R, C)) * spread).astype(np.float16)
    law_np, base_bits, tmax = oracle.flip_law(P)
    base = oracle.pack(base_bits, np.int64)
    # the table: made on the device from the largest threshold
    tbl = torch.zeros((int(ops._lib.load().nb_skip_table_words()),), dtype=torch.int32, device="cuda")
    thr = torch.tensor([tmax - 2 ** 32 if tmax >= 2 ** 31 else tmax], dtype=torch.int32, device="cuda")
    ops._lib.call("nb_skip_table", tbl.data_ptr(), thr.data_ptr(), None)
    th = host(tbl).view(np.uint32)
    Kt = int(th[0])
    cdf = th[4:4 + Kt].copy()
    assert int(th[2]) == tmax and (np.diff(cdf.astype(np.int64)) >= 0).all()
    ref = ops.skip_table(tmax)
    assert Kt == len(ref) and np.abs(cdf.astype(np.int64) - ref.astype(np.int64)).max() <= 1   # another libm: +-1
    law = ops.FlipLaw(dev(law_np.view(np.int16)).view(torch.uint16), dev(base), tbl.view(torch.uint32), C)
    seed, sub = 0xFEED + C, 5
    want_flips = oracle.skip_flips_thin(law_np, cdf, tmax, seed, sub, first, D).reshape(D, R, Kw)
    cap = ops.flip_capacity(C, min(2 * spread, 0.5))
    rows = ops.flip_rows_thin(law, D, seed, cap, subsequence=sub, first=first)
    assert rows.overflowed() == 0
    W = ops.flip_rows_to_weights(rows)
    np.testing.assert_array_equal(host(W), base[None] ^ want_flips)
    np.testing.assert_array_equal(host(rows.cnt).astype(np.int64),
                                  np.unpackbits(want_flips.view(np.uint8), axis=2, bitorder="little").sum(axis=2))
    x = sparse_mask(g, (D, C), 0.5)
    want = oracle.bmm(base[None] ^ want_flips, x.reshape(D, Kw, 1))[:, :, 0]
    np.testing.assert_array_equal(host(ops.bmm(rows, dev(x).view(D, Kw, 1)))[:, :, 0], want)
    if D * R * C <= 500000:
        mask, bflag = decode_flip_rows(rows)
        fb = np.unpackbits(want_flips.view(np.uint8), axis=2, bitorder="little").astype(bool)
        np.testing.assert_array_equal(mask, fb)
        bb = np.unpackbits(base.view(np.uint8), axis=1, bitorder="little").astype(bool)
        np.testing.assert_array_equal(bflag, mask & bb[None])


def test_law_statistics_in_one_read_back(ops, oracle):
    """FlipLaw.stats(): mean / largest row mean / largest flip probability of the law the library made from latent
    weights, against numpy on the law read back."""
    g = torch.Generator(device="cuda")
    g.manual_seed(12)
    for R, C in ((16, 2048), (70, 333), (1, 64), (1024, 8192)):
        w = (torch.randn((R, C), device="cuda", generator=g) * (0.2 + torch.rand((R, 1), device="cuda", generator=g))).half()
        law = ops.flip_law_from_weights(w)
        y = (host(law.law.view(torch.int16)).view(np.uint16) & 0x7FFF).view(np.float16).astype(np.float64)
        mean, row, peak = law.stats()
        assert abs(mean - y.mean()) <= 1e-6 * y.mean() + 1e-12
        assert abs(row - y.mean(axis=1).max()) <= 1e-5 * row
        assert peak == float(np.floor(y.max() * 2.0 ** 32)) / 2.0 ** 32 == law.max_flip_probability()


def long_tailed_law(g, R, C, mean):
    """fp16 probabilities whose flip probabilities span five orders of magnitude, a few of them near 1/2."""
    y = mean * 0.3 * 10.0 ** (g.random((R, C)) * 1.0)
    y = np.where(g.random((R, C)) < 0.02, g.random((R, C)) * 0.5, y)
    y = np.where(g.random((R, C)) < 0.3, y * 10.0 ** -(3 * g.random((R, C))), y)
    y = np.minimum(y, 0.5)
    return np.where(g.random((R, C)) < 0.5, y, 1.0 - y).astype(np.float16)


@pytest.mark.parametrize("D,R,C,first,mean", [(3, 64, 64, 0, 0.1), (2, 100, 200, 8, 0.05), (3, 1024, 2048, 0, 0.01),
                                              (2, 70, 300, 3, 0.05), (40, 130, 72, 0, 0.1), (2, 9, 8192, 4, 0.005),
                                              (3, 5, 77, 1, 0.05), (2, 16, 16384, 0, 0.004), (2, 3, 32704, 0, 0.002),
                                              (600, 2, 1024, 0, 0.02)])
def test_layered_sampler_vs_oracle(ops, oracle, D, R, C, first, mean):
    """Flip lists under a per-element law drawn class by class == the oracle's restatement of that walk: the sort of
    the law (made on the device) against the oracle's stable sort, the 16 tables against the host formula, then the
    lists, bit for bit, and the sums from them."""
    g = np.random.default_rng(D + R + C)
    Kw = (C + 63) // 64
    P = long_tailed_law(g, R, C, mean)
    if R > 2:
        P[1, : C // 2] = 1.0                                               # columns that never flip
        P[2, :] = 0.0                                                      # a row that never flips
    law_np, base_bits, tmax = oracle.flip_law(P)
    base = oracle.pack(base_bits, np.int64)
    law = ops.FlipLaw(dev(law_np.view(np.int16)).view(torch.uint16), dev(base), None, C)
    pl, cls = law.layers()
    want_pl, want_cls = oracle.law_layers(law_np)
    np.testing.assert_array_equal(host(cls.view(torch.int32)).view(np.uint32), want_cls)
    live = np.arange(C)[None, :] < want_cls[:, 16:17]
    np.testing.assert_array_equal(np.where(live, host(pl.view(torch.int32)).view(np.uint32), 0xFFFF), want_pl)
    words = int(ops._lib.load().nb_skip_table_words())
    tb = host(ops.layer_tables("cuda").view(torch.int32)).view(np.uint32).reshape(16, words)
    cdfs, kts = oracle.layer_tables()
    for k in range(16):
        assert int(tb[k, 2]) == 1 << (31 - k) and min(int(tb[k, 0]), 512) == kts[k]
        assert np.abs(tb[k, 4:4 + kts[k]].astype(np.int64) - cdfs[k, :kts[k]].astype(np.int64)).max() <= 1   # another libm
        cdfs[k, :kts[k]] = tb[k, 4:4 + kts[k]]                             # the table is input data of the contract
    seed, sub = 0xFEED + C, 5
    want_flips = oracle.skip_flips_layered(want_pl, want_cls, seed, sub, first, D, tables=(cdfs, kts)).reshape(D, R, Kw)
    y = (law_np & 0x7FFF).view(np.float16).astype(np.float64)
    cap = ops.flip_capacity(C, float(y.mean(axis=1).max()))
    rows = ops.flip_rows_layered(law, D, seed, cap, subsequence=sub, first=first)
    assert rows.overflowed() == 0
    W = ops.flip_rows_to_weights(rows)
    np.testing.assert_array_equal(host(W), base[None] ^ want_flips)
    np.testing.assert_array_equal(host(rows.cnt).astype(np.int64),
                                  np.unpackbits(want_flips.view(np.uint8), axis=2, bitorder="little").sum(axis=2))
    x = sparse_mask(g, (D, C), 0.5)
    want = oracle.bmm(base[None] ^ want_flips, x.reshape(D, Kw, 1))[:, :, 0]
    np.testing.assert_array_equal(host(ops.bmm(rows, dev(x).view(D, Kw, 1)))[:, :, 0], want)
    if D * R * C <= 500000:
        mask, bflag = decode_flip_rows(rows, ordered=False)
        fb = np.unpackbits(want_flips.view(np.uint8), axis=2, bitorder="little").astype(bool)
        np.testing.assert_array_equal(mask, fb)
        bb = np.unpackbits(base.view(np.uint8), axis=1, bitorder="little").astype(bool)
        np.testing.assert_array_equal(bflag, mask & bb[None])


@pytest.mark.parametrize("walk", ["layered", "thin"])
def test_per_element_walks_report_rows_beyond_the_capacity(ops, oracle, walk):
    """The per-element walks with a capacity below what some rows need: those rows are cut to capacity * 8 flips and
    counted, the others are what they are with room to spare; and shapes at the edges (one row, one member, no
    column that can flip) come out as empty or short lists."""
    g = np.random.default_rng(8)
    R, C, D = 70, 512, 9
    P = long_tailed_law(g, R, C, 0.05)
    law_np, base_bits, tmax = oracle.flip_law(P)
    law = ops.flip_law_from_weights(torch.zeros((R, C), dtype=torch.float16, device="cuda"))   # for its table's place
    law.law.copy_(dev(law_np.view(np.int16)).view(torch.uint16))
    law.base.copy_(dev(oracle.pack(base_bits, np.int64)))
    thr = torch.tensor([tmax], dtype=torch.int64, device="cuda").to(torch.int32)
    ops._lib.call("nb_skip_table", law.table.data_ptr(), thr.data_ptr(), None)
    draw = ops.flip_rows_layered if walk == "layered" else ops.flip_rows_thin
    full = draw(law, D, 11, 64)
    assert full.overflowed() == 0
    need = (full.cnt + 7) // 8
    cap = int(need.max().item()) - 1
    cut = draw(law, D, 11, cap)
    assert cut.overflowed() == int((need > cap).sum().item()) > 0
    fine = (need <= cap)
    assert torch.equal(cut.cnt[fine], full.cnt[fine]) and bool((cut.cnt[~fine] == 8 * cap).all())
    Wc, Wf = ops.flip_rows_to_weights(cut), ops.flip_rows_to_weights(full)
    assert torch.equal(Wc[fine], Wf[fine])
    # nothing can flip: empty lists, the base itself
    never = ops.FlipLaw(torch.zeros((3, 128), dtype=torch.uint16, device="cuda"),
                        dev(sparse_mask(g, (3, 128), 0.5)), law.table, 128)
    if walk == "layered":
        rows = ops.flip_rows_layered(never, 5, 1, 2)
        assert int(rows.cnt.sum().item()) == 0 and rows.overflowed() == 0
        assert torch.equal(ops.flip_rows_to_weights(rows), never.base[None].expand(5, 3, 2))


def test_layered_sampler_flip_rates_at_size(ops, oracle):
    """4096 members of a 64 x 8192 layer: every column's flip count against its own probability (binomial tails),
    and the lists stay inside the capacity chosen from the largest row mean."""
    g = np.random.default_rng(3)
    D, R, C = 4096, 64, 8192
    P = long_tailed_law(g, R, C, 0.007)
    law_np, base_bits, tmax = oracle.flip_law(P)
    base = oracle.pack(base_bits, np.int64)
    law = ops.FlipLaw(dev(law_np.view(np.int16)).view(torch.uint16), dev(base), None, C)
    y = (law_np & 0x7FFF).view(np.float16).astype(np.float64)
    cap = ops.flip_capacity(C, float(y.mean(axis=1).max()))
    rows = ops.flip_rows_layered(law, D, 99, cap)
    assert rows.overflowed() == 0
    flips = ops.flip_rows_to_weights(rows) ^ dev(base)[None]
    count = np.stack([host(((flips >> b) & 1).sum(dim=0)) for b in range(64)], axis=2).reshape(R, C).astype(np.float64)
    pq = oracle.law_thresholds(law_np).astype(np.float64) / 2.0 ** 32
    from scipy.stats import binom
    tail = np.minimum(binom.cdf(count, D, pq), binom.sf(count - 1, D, pq))       # exact: the small means are not normal
    assert tail.min() > 1e-10, (float(tail.min()), np.unravel_index(tail.argmin(), tail.shape))
    assert abs(count.sum() - D * pq.sum()) <= 5 * np.sqrt(D * pq.sum())


@pytest.mark.parametrize("D,R,C,p", [(64, 8, 64, 0.1), (300, 70, 200, 0.05), (1024, 16, 8192, 0.01), (5, 1, 1, 0.5),
                                     (33, 130, 960, 0.0), (17, 9, 32704, 0.001)])
def test_weighted_sum_over_flip_lists(ops, oracle, D, R, C, p):
    """weighted_sum on the lists against the float64 sum over the unpacked bits (exact up to the scaling of the
    weights to integers and the final rounding to fp16), and against the dense kernel on the materialised weights."""
    g = np.random.default_rng(D + R + C)
    Kw = (C + 63) // 64
    base = sparse_mask(g, (R, C), 0.5)
    W = base[None] ^ sparse_mask(g, (D, R, C), p)
    rows = ops.flip_rows_from_weights(dev(W), dev(base))
    w = (g.standard_normal(D) * (1 + 10 * (D % 3))).astype(np.float16)
    got = ops.weighted_sum(rows, dev(w), C)
    assert got.dtype == torch.float16 and tuple(got.shape) == (R, C)
    bits = np.unpackbits(W.view(np.uint8), axis=2, bitorder="little")[:, :, :C].astype(np.float64)
    want = np.einsum("d,drc->rc", w.astype(np.float64), bits)
    scale = np.abs(w.astype(np.float64)).sum() + 1.0
    err = np.abs(host(got).astype(np.float64) - want)
    # half an fp16 ulp of the result + the integer scaling (2**-29 of sum |w| per term, at most D terms)
    tol = np.maximum(np.abs(want), 2.0 ** -14) * 2.0 ** -11 + D * scale * 2.0 ** -28
    assert (err <= tol).all(), float((err / tol).max())
    dense = ops.weighted_sum(dev(W), dev(w), C)
    np.testing.assert_allclose(host(got).astype(np.float64), host(dense).astype(np.float64), rtol=2e-3,
                               atol=2e-3 * float(np.abs(w.astype(np.float64)).sum()) / max(D, 1) ** 0.5 + 1e-6)
    # the same call twice: integer additions commute, so the result does not depend on the order of arrival
    assert torch.equal(got, ops.weighted_sum(rows, dev(w), C))


@pytest.mark.parametrize("R,C,scale", [(64, 64, 1.0), (10, 1000, 0.01), (1024, 1024, 3.0), (7, 3, 100.0), (33, 130, 0.0)])
def test_law_kernels_against_the_tensor_expression(ops, R, C, scale):
    """probabilities / thresholds / sparse law of a layer against modules/binary.py:59-60 evaluated by torch:
    P = sigmoid((w / (mean|w| + 1e-5) * 5).float()).half().  The elementwise steps round where the tensor expression
    rounds; torch's fp16 mean adds in fp32 in its own order, the kernel's mean is the exact one rounded once, so the
    denominators may differ by an fp16 ulp when the mean falls next to a rounding boundary: the test asks for equal
    denominators and, given those, bit-equal probabilities."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(R * 1000 + C)
    w = (torch.randn(R, C, device="cuda", generator=gen) * scale).to(torch.float16)
    denom = w.abs().mean() + 1e-5
    P_t = torch.sigmoid((w / denom * 5).float()).half()
    P = ops.probabilities_from_weights(w)
    exact = (w.abs().double().sum() / w.numel()).item()
    assert float(w.abs().mean()) == float(torch.tensor(exact, dtype=torch.float64).to(torch.float16)), \
        "the test's weights put torch's mean on the other side of a rounding boundary: pick another seed"
    assert torch.equal(P, P_t)
    T = ops.thresholds_from_weights(w)
    assert torch.equal(T.view(torch.int32), ops.thresholds_from_p(P_t).view(torch.int32))
    law = ops.flip_law_from_weights(w)
    Pf = P_t.float()
    one = Pf >= 0.5
    y = torch.where(one, 1.0 - Pf, Pf).half()
    want_law = (y.view(torch.int16) & 0x7FFF) | torch.where(one, torch.tensor(-32768, dtype=torch.int16, device="cuda"),
                                                            torch.tensor(0, dtype=torch.int16, device="cuda"))
    assert torch.equal(law.law.view(torch.int16), want_law)
    assert torch.equal(law.base, ops.pack(one, torch.int64))
    tmax = int(torch.floor(y.double() * 2.0 ** 32).max().item())
    th = host(law.table.view(torch.int32)).view(np.uint32)
    assert int(th[2]) == tmax
    ref = ops.skip_table(tmax)
    assert int(th[0]) == len(ref) and (len(ref) == 0 or np.abs(th[4:4 + len(ref)].astype(np.int64) - ref.astype(np.int64)).max() <= 1)
    assert abs(law.max_flip_probability() - tmax / 2.0 ** 32) < 1e-12
