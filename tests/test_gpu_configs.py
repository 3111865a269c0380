"""The five benchmark configurations at their FULL sizes on the GPU.

Each is checked two ways: (1) a size-independent identity over the whole population computed by a second,
independent GPU path (fused == materialise-then-bmm, implicit conv == bmm(im2col), fused epilogue == op
chain), and (2) bit-exact agreement with the CPU oracle on a few members, whose random words are regenerated
on the host from the same Philox stream (oracle/nesbin_oracle.c: nbo_philox_words)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

MEMBERS = (0, 1, 511, 1023)


@pytest.fixture(scope="module")
def wk():
    assert torch.cuda.is_available()
    from nesgpu_amd import workloads
    return workloads


@pytest.fixture(scope="module")
def ops():
    from nesgpu_amd.extensions import booleanOperations
    return booleanOperations


def host_member_weights(oracle, base, in_bits, rows, T, seed, subseq, m):
    """base ^ flips of member m, regenerated on the host."""
    words = oracle.philox_words(seed, subseq, m * rows * in_bits, rows * in_bits).reshape(1, rows, in_bits)
    return oracle.sample_from_words(T, words, np.int64, base=base)[0]


def test_config1_linear_256_materialised(wk, ops, oracle):
    w = wk.linear_flip_materialised()
    out = w.step()
    assert tuple(out.shape) == (1024, 256, 1) and out.dtype == torch.int32
    base, x, W = (w.tensors[k].cpu().numpy() for k in ("base", "x", "W"))
    # whole population against the oracle (small enough)
    words = oracle.philox_words(0, 1, 0, 1024 * 256 * 256).reshape(1024, 256, 256)
    Wn = oracle.sample_from_words(wk.T_P01, words, np.int64, base=base)
    np.testing.assert_array_equal(W, Wn)
    popc = oracle.bmm(Wn, x.reshape(1024, 4, 1))
    np.testing.assert_array_equal(out.cpu().numpy(), popc)
    flips = oracle.unpack((Wn ^ base[None]).reshape(-1, 4)).mean()
    assert abs(flips - 0.01) < 2e-4                                         # Bernoulli(p = 0.01)
    # the configuration's stated output K - 2*popcount(x XOR w) is the XNOR reading of the same sum
    xb = oracle.unpack(x)[:, :256]
    wb = oracle.unpack(Wn[7])[:, :256]
    dot = ((2 * xb[7].astype(int) - 1) * (2 * wb.astype(int) - 1)).sum(1)
    np.testing.assert_array_equal(256 - 2 * popc[7, :, 0], dot)


def test_config2_linear_1024_fused_from_words(wk, ops, oracle):
    w = wk.linear_flip_fused()
    out = w.step()
    assert tuple(out.shape) == (1024, 1024) and out.dtype == torch.int32
    base, x, words = w.tensors["base"], w.tensors["x"], w.tensors["words"]
    # identity over the whole population: fused == materialise + bmm (two different kernels)
    ref = torch.empty_like(out)
    for lo in range(0, 1024, 256):
        Wm = ops.flip_from_words(base, words[lo:lo + 256], wk.T_P05)
        ref[lo:lo + 256] = ops.bmm(Wm, x[lo:lo + 256].view(256, -1, 1)).squeeze(2)
    assert torch.equal(out, ref)
    # generator mode reproduces the same numbers without reading any words
    assert torch.equal(ops.seeded_bmv_philox(wk.T_P05, x, 1024, 1024, 0, subsequence=2, base=base), out)
    # oracle on a few members
    bh, xh = base.cpu().numpy(), x.cpu().numpy()
    for m in MEMBERS:
        wm = oracle.philox_words(0, 2, m * 1024 * 1024, 1024 * 1024).reshape(1, 1024, 1024)
        want = oracle.seeded_bmv_from_words(wk.T_P05, xh[m:m + 1], wm, base=bh)
        np.testing.assert_array_equal(out[m].cpu().numpy(), want[0])
    rate = (ops.unpack((ops.flip_from_words(base, words[:8], wk.T_P05) ^ base).view(-1, 16)).float().mean().item())
    assert abs(rate - 0.05) < 5e-4


def test_config2_generator_mode_with_half_word_draws(wk, ops, oracle):
    """Configuration 2 with 16-bit draws: the fused product equals bmm on what the sampler writes from the same
    stream, over the whole population; members regenerated on the host; the flip rate."""
    w = wk.linear_flip_generated(half_draws=True)
    out = w.step()
    assert tuple(out.shape) == (1024, 1024) and out.dtype == torch.int32
    base, x = w.tensors["base"], w.tensors["x"]
    W = ops.sample_bits_philox(wk.T_P05, 1024, torch.int64, 0, 2, base=base, shape=(1024, 1024), half_draws=True)
    assert torch.equal(ops.bmm(W, x.view(1024, -1, 1)).squeeze(2), out)
    bh, xh = base.cpu().numpy(), x.cpu().numpy()
    for m in MEMBERS:
        Wm = oracle.sample_philox16(wk.T_P05, 1, 1024, 1024, 0, 2, m * 1024 * 1024, np.int64, base=bh)
        np.testing.assert_array_equal(W[m].cpu().numpy(), Wm[0])
        np.testing.assert_array_equal(out[m].cpu().numpy(), oracle.bmm(Wm, xh[m:m + 1].reshape(1, -1, 1))[0, :, 0])
    rate = ops.unpack((W[:64] ^ base).view(-1, 16)).float().mean().item()
    assert abs(rate - 0.05) < 2e-4
    assert not torch.equal(out, wk.linear_flip_generated().step())          # other bits than the 32-bit draws


def test_config3_conv_64_int32(wk, ops, oracle):
    w = wk.conv_int32()
    out = w.step()
    assert tuple(out.shape) == (1024, 32, 32, 64) and out.dtype == torch.int32
    x, filt, base = w.tensors["x"], w.tensors["filt"], w.tensors["base"]
    for lo in range(0, 1024, 256):                                          # implicit conv == bmm(im2col)
        cols = ops.batch_im2col(x[lo:lo + 256], 3, 3, 1, 1, 1, 1)
        assert torch.equal(ops.bmm(cols, filt[lo:lo + 256]).view(256, 32, 32, 64), out[lo:lo + 256])
    bh = base.cpu().numpy()
    for m in MEMBERS:
        Wn = host_member_weights(oracle, bh, 64, 576, wk.T_P02, 0, 3, m)                 # [576, 1]
        f = np.ascontiguousarray(Wn.reshape(1, 64, 3, 3, 1).transpose(0, 2, 3, 4, 1).reshape(1, 9, 64))
        np.testing.assert_array_equal(filt[m].cpu().numpy(), f[0])
        want = oracle.conv(x[m:m + 1].cpu().numpy(), f, 3, 3, 1, 1, 1, 1)
        np.testing.assert_array_equal(out[m].cpu().numpy(), want[0])
    # padding is the zero word = every padded bit -1: a corner pixel only sees 4 real taps
    xm, fm = x[0].cpu().numpy().view(np.uint64), filt[0].cpu().numpy().view(np.uint64)
    taps = [(1, 1, 0, 0), (1, 2, 0, 1), (2, 1, 1, 0), (2, 2, 1, 1)]                     # (i, j, y, x)
    for o in (0, 63):
        s = sum(bin(int(xm[y, xx, 0] ^ fm[i * 3 + j, o])).count("1") for i, j, y, xx in taps)
        s += sum(bin(int(fm[i * 3 + j, o])).count("1") for i in range(3) for j in range(3)
                 if (i, j) not in [(t[0], t[1]) for t in taps])
        assert int(out[0, 0, 0, o]) == s


def test_config4_conv_16_sign_pool(wk, ops, oracle):
    w = wk.conv_sign_pool()
    out = w.step()
    assert tuple(out.shape) == (1024, 32, 32, 1) and out.dtype == torch.int64
    x, filt, thr = w.tensors["x"], w.tensors["filt"], w.tensors["thr"]
    for lo in range(0, 1024, 256):                                          # fused == conv_act -> pack -> max_pool2d
        act = ops.conv_act(x[lo:lo + 256], filt[lo:lo + 256], thr[lo:lo + 256], 3, 3, 1, 1, 1, 1)
        sign = 2 * ops.conv(x[lo:lo + 256], filt[lo:lo + 256], 3, 3, 1, 1, 1, 1) - 144 > 0
        assert torch.equal(act, sign)                                       # threshold K <=> sign of 2*popc - K
        packed = ops.pack(act.view(-1, 16), torch.int64).view(256, 64, 64, 1)
        assert torch.equal(ops.max_pool2d(packed, 2, 2, 0, 0, 2, 2), out[lo:lo + 256])
    assert int((out >> 16).abs().max()) == 0                               # only 16 channel bits per word
    for m in MEMBERS:
        xm, fm = x[m:m + 1].cpu().numpy(), filt[m:m + 1].cpu().numpy()
        act = oracle.conv_act(xm, fm, np.full((1, 16), 144, np.int32), 3, 3, 1, 1, 1, 1)
        want = oracle.max_pool2d(oracle.pack(act.reshape(-1, 16), np.int64).reshape(1, 64, 64, 1), 2, 2, 0, 0, 2, 2)
        np.testing.assert_array_equal(out[m].cpu().numpy(), want[0])


def test_config5_cifar_net(wk, ops, oracle):
    D = 4096
    w = wk.cifar_net(D=D)
    out = w.step()
    assert tuple(out.shape) == (D, 10) and out.dtype == torch.int32
    assert torch.equal(w.step(), out)                                      # deterministic
    t = dict(w.tensors)
    # the 8192 -> 1024 layer runs from the shared base + flip lists (drawn by the skip sampler; the 4 GiB of weights
    # are materialised here only to check): the logits must be those of the dense kernels on the materialised
    # weights, every member; and so must the layer itself on the net's real features and on random inputs with
    # thresholds around the sums
    assert w.meta["fc"].startswith("base + flip lists")
    t["W4"] = w.meta["W4"]()
    assert tuple(t["W4"].shape) == (D, 1024, 128)
    rows4 = w.meta["rows4"]
    rate = float(rows4.cnt.view(torch.int16).double().sum()) / (D * 1024 * 8192)
    assert abs(rate - 0.01) < 2e-5                                          # Bernoulli(p = 0.01) per weight bit
    assert torch.equal(ops.flip_rows_from_weights(t["W4"], t["b4"]).cnt, rows4.cnt)      # counted on the dense form
    assert torch.equal(w.meta["step_dense"](), out)
    feats = w.meta["features"]()
    assert torch.equal(ops.bmv_flip_act_pack(rows4, feats, w.meta["thr4"]), ops.bmv_act_pack(t["W4"], feats, w.meta["thr4"]))
    assert torch.equal(ops.bmv_flip(rows4, feats), ops.bmm(t["W4"], feats).squeeze(2))
    del feats
    # the fused linear-layer kernel against the unfused composition, every member, thresholds around the sums
    a4 = torch.randint(-2 ** 62, 2 ** 62, (D, 128, 1), dtype=torch.int64, device="cuda")
    sums = ops.bmm(t["W4"], a4).squeeze(2)
    thr4 = (2 * sums + torch.randint(-2, 3, sums.shape, device="cuda")).to(torch.int32)
    assert torch.equal(ops.bmv_act_pack(t["W4"], a4, thr4), ops.pack(2 * sums > thr4, torch.int64))
    assert torch.equal(ops.bmv_flip_act_pack(rows4, a4, thr4), ops.pack(2 * sums > thr4, torch.int64))
    assert torch.equal(ops.bmv_flip(rows4, a4), sums)
    del a4, sums, thr4
    # the first layer on all members: window-per-register kernel (automatic choice) == int8 matrix-core kernel
    thr1 = torch.full((D, 64), 27, dtype=torch.int32, device="cuda")
    prev = ops.conv_engine(0)
    try:
        l1 = ops.conv_act_pack(t["x"], t["f1"], thr1, 3, 3, 1, 1, 1, 1, in_bits=3)
        assert ops.conv_last_engine() == 1
        ops.conv_engine(3)
        assert torch.equal(ops.conv_act_pack(t["x"], t["f1"], thr1, 3, 3, 1, 1, 1, 1, in_bits=3), l1)
        assert ops.conv_last_engine() == 2
    finally:
        ops.conv_engine(prev)
    # the two 64-channel layers on all members, pooled packed output with thresholds spread around the sums and the
    # maps' pixel sums: the wave-per-strip FP4 kernel (automatic choice) == the staged-image int8 kernel == the
    # XOR-popcount kernels
    g5 = torch.Generator(device="cuda")
    g5.manual_seed(5)
    for name, S, O in (("f2", 32, 64), ("f3", 16, 128)):
        xin = torch.randint(-2 ** 62, 2 ** 62, (D, S, S, 1), dtype=torch.int64, device="cuda", generator=g5)
        thr = (576 + torch.randint(-40, 41, (D, O), device="cuda", generator=g5)).to(torch.int32)
        got, sums = {}, {}
        # (engine asked for, engine that serves the packed map, engine that serves the pixel sums: the automatic choice
        # takes those from bit counts, without a conv)
        for eng, served, served_sums in ((0, 4, 5), (2, 4, 4), (3, 2, 2), (1, 1, 1)):
            ops.conv_engine(eng)
            got[eng] = ops.conv_act_pack(xin, t[name], thr, 3, 3, 1, 1, 1, 1, pool=True)
            assert ops.conv_last_engine() == served
            sums[eng] = ops.conv_popc_sums(xin, t[name], 3, 3, 1, 1, 1, 1)
            assert ops.conv_last_engine() == served_sums
        ops.conv_engine(prev)
        assert torch.equal(got[0], got[3]) and torch.equal(got[0], got[1]) and torch.equal(got[0], got[2]), name
        assert torch.equal(sums[0], sums[3]) and torch.equal(sums[0], sums[1]) and torch.equal(sums[0], sums[2]), name
        assert 0.2 < float(ops.unpack(got[0].view(-1, got[0].shape[-1])).float().mean()) < 0.8      # not degenerate
        del xin, thr, got, sums
    del l1, thr1
    # the members' weights regenerated on the host from the Philox stream (subsequences 10..14 in layer order) must
    # be what the GPU sampler wrote: all filters, eight rows of the 8192 -> 1024 layer, all of the last layer
    T, seed = w.meta["T"], w.meta["seed"]
    b4h, b5h = t["b4"].cpu().numpy(), t["b5"].cpu().numpy()
    for m in (0, 2047, 4095):
        for li, (name, C, O) in enumerate((("f1", 3, 64), ("f2", 64, 64), ("f3", 64, 128))):
            bh = t["b%d" % (li + 1)].cpu().numpy()
            if C >= 32:      # 64-channel taps: the skip sampler's walk over the member's O*9 rows
                Wn = bh ^ oracle.skip_flips(oracle.skip_cdf(T), seed, 10 + li, m * O * 9 * C, O * 9, C)
            else:
                Wn = host_member_weights(oracle, bh, C, O * 9, T, seed, 10 + li, m)
            f = np.ascontiguousarray(Wn.reshape(1, O, 3, 3, 1).transpose(0, 2, 3, 4, 1).reshape(9, O))
            np.testing.assert_array_equal(t[name][m].cpu().numpy(), f, err_msg="%s member %d" % (name, m))
        W4m = t["W4"][m].cpu().numpy()
        table = oracle.skip_cdf(T)
        for r in (0, 1, 255, 256, 511, 777, 1022, 1023):                   # the skip sampler's walk, row by row
            want = b4h[r] ^ oracle.skip_flips(table, seed, 13, (m * 1024 + r) * 8192, 1, 8192)[0]
            np.testing.assert_array_equal(W4m[r], want, err_msg="W4 member %d row %d" % (m, r))
        np.testing.assert_array_equal(t["W5"][m].cpu().numpy(), host_member_weights(oracle, b5h, 1024, 10, T, seed, 14, m))
    for m in (0, 2047, 4095):
        a = t["x"][m:m + 1].cpu().numpy()                                  # [1,32,32,1]
        for name, C, O, pool in (("f1", 3, 64, False), ("f2", 64, 64, True), ("f3", 64, 128, True)):
            f = t[name][m:m + 1].cpu().numpy()
            act = oracle.conv_act(a, f, np.full((1, O), 9 * C, np.int32), 3, 3, 1, 1, 1, 1)
            a = oracle.pack(act.reshape(-1, O), np.int64).reshape(1, act.shape[1], act.shape[2], -1)
            if pool:
                a = oracle.max_pool2d(a, 2, 2, 0, 0, 2, 2)
        a = a.reshape(1, 128, 1)
        p4 = oracle.bmm(t["W4"][m:m + 1].cpu().numpy(), a)[:, :, 0]        # [1,1024]
        a5 = oracle.pack(2 * p4 > 8192, np.int64).reshape(1, 16, 1)
        want = oracle.bmm(t["W5"][m:m + 1].cpu().numpy(), a5)[:, :, 0]
        np.testing.assert_array_equal(out[m].cpu().numpy(), want[0])
