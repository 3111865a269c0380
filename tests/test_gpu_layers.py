"""GPU tests of the layer API (nesgpu_amd.modules.binary) against the CPU oracle: the layers are driven with
caller-supplied random words so that every sampled weight bit is reproducible on the host."""
import numpy as np
import pytest
import torch

from golden_util import torch_mean_fp16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def binary():
    assert torch.cuda.is_available()
    from nesgpu_amd.modules import binary as b
    return b


def rng(seed):
    return np.random.default_rng(seed)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host_thresholds(layer):
    """uint32 thresholds the layer samples with, recomputed on the host from the fp16 probabilities
    (T = min(floor(P * 2**32), 2**32 - 1))."""
    P = layer.probabilities().cpu().numpy().astype(np.float64)
    return np.minimum(np.floor(P * 4294967296.0), 4294967295.0).astype(np.uint32)


def randomise(layer, g):
    with torch.no_grad():
        layer.weight.copy_(dev(g.standard_normal(tuple(layer.weight.shape)).astype(np.float16)))
        if layer.bias is not None:
            layer.bias.copy_(dev((g.standard_normal(tuple(layer.bias.shape)) * 4).astype(np.float16)))


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("in_f,out_f", [(256, 64), (100, 10), (1024, 33)])
def test_linear_forward(binary, oracle, dtype, in_f, out_f):
    D = 16
    g = rng(in_f + out_f)
    nd = np.int64 if dtype == torch.int64 else np.int32
    for threshold, batch_norm in [(False, False), (True, False), (True, True)]:
        layer = binary.BinarizedLinear(in_f, out_f, D, threshold=threshold, batch_norm=batch_norm, dtype=dtype)
        randomise(layer, g)
        words = g.integers(0, 2 ** 32, size=(D, out_f, in_f), dtype=np.uint64).astype(np.uint32)
        layer.set_seed(11)
        layer.set_noise(words=dev(words))
        T = host_thresholds(layer)
        Wn = oracle.sample_from_words(T, words, nd)
        np.testing.assert_array_equal(layer.weight_noise.cpu().numpy(), Wn)           # modules/binary.py:62
        xb = g.integers(0, 2, size=(D, in_f)).astype(bool)
        layer.perturbed_flag = True
        out = layer(dev(xb))
        popc = oracle.bmm(Wn, oracle.pack(xb, nd).reshape(D, -1, 1))[:, :, 0]
        act = 2 * popc - in_f                                                          # modules/binary.py:97
        # same +-1 reading as the reference's check: x = 2b-1, w = 1-2b
        want_dot = ((2 * xb.astype(np.int64) - 1)[:, None, :] *
                    (1 - 2 * oracle.unpack(Wn.reshape(D * out_f, -1))[:, :in_f].reshape(D, out_f, in_f).astype(np.int64))
                    ).sum(2)
        np.testing.assert_array_equal(act, want_dot)
        if not threshold:
            assert out.dtype == torch.int32
            np.testing.assert_array_equal(out.cpu().numpy(), act)
            continue
        assert out.dtype == torch.bool and tuple(out.shape) == (D, out_f)
        assert tuple(layer.bias_noise.shape) == (D, out_f) and layer.bias_noise.dtype == torch.float16
        assert float(layer.bias_noise.abs().max()) <= 3.0                              # (rand - .5) * 6
        act_t = torch.from_numpy(act.astype(np.int32)).cuda()
        thresh = layer.bias + layer.bias_noise
        if batch_norm:
            thresh = thresh + act_t.type(torch.float16).mean(dim=0, keepdim=True)      # modules/binary.py:101
        assert torch.equal(out, act_t > thresh)
        # packed input is accepted as is (modules/binary.py:95)
        assert torch.equal(layer(dev(oracle.pack(xb, nd))), out)
        if not batch_norm:
            # pack_output=True: the same bits, packed, from the fused kernel
            layer.pack_output = True
            packed = layer(dev(xb))
            layer.pack_output = False
            assert packed.dtype == dtype
            np.testing.assert_array_equal(packed.cpu().numpy(), oracle.pack(out.cpu().numpy(), nd))


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("C,O,k,pad,stride", [(16, 16, 3, 1, 1), (64, 70, 3, 1, 1), (3, 8, 5, 2, 2), (100, 4, 1, 0, 1)])
def test_conv_forward(binary, oracle, dtype, C, O, k, pad, stride):
    D, S = 6, 12
    g = rng(C * 3 + O + k)
    nd = np.int64 if dtype == torch.int64 else np.int32
    K = C * k * k
    xb = g.integers(0, 2, size=(D, S, S, C)).astype(bool)
    xp = oracle.pack(xb.reshape(-1, C), nd).reshape(D, S, S, -1)
    geom = (k, k, pad, pad, stride, stride)
    for threshold, batch_norm in [(False, False), (True, False), (True, True)]:
        layer = binary.BinarizedConv2d(C, O, D, k, stride=stride, padding=pad, threshold=threshold,
                                       batch_norm=batch_norm, dtype=dtype)
        randomise(layer, g)
        words = g.integers(0, 2 ** 32, size=(D, O * k * k, C), dtype=np.uint64).astype(np.uint32)
        layer.set_seed(5)
        layer.set_noise(words=dev(words))
        Wn = oracle.sample_from_words(host_thresholds(layer), words, nd)             # [D, O*k*k, Cw]
        filt = np.ascontiguousarray(Wn.reshape(D, O, k, k, -1).transpose(0, 2, 3, 4, 1).reshape(D, -1, O))
        np.testing.assert_array_equal(layer.weight_noise_reshaped.cpu().numpy(), filt)   # modules/binary.py:136-137
        popc = oracle.conv(xp, filt, *geom)
        act = 2 * popc - K                                                              # modules/binary.py:145,158
        layer.perturbed_flag = True
        out = layer(dev(xb))
        if not threshold:
            np.testing.assert_array_equal(out.cpu().numpy(), act)
            continue
        assert out.dtype == torch.bool and tuple(out.shape) == act.shape
        if batch_norm:
            # :147-155 with the mean taken from exact integer sums, as torch's fp16 mean forms it
            mean = torch_mean_fp16(act.sum(axis=(1, 2), dtype=np.int64), D * O, act.size)
            bn = (layer.bias + layer.bias_noise).detach().cpu().numpy()                           # fp16 [D, O]
            thresh = (bn + mean).astype(np.float16)
            np.testing.assert_array_equal(out.cpu().numpy(), act.astype(np.float16) > thresh[:, None, None, :])
            # ... which is what torch's own fp16 mean gives as well (the reference's expression)
            act_t = torch.from_numpy(act.astype(np.int32)).cuda()
            tref = layer.bias + layer.bias_noise + act_t.type(torch.float16).mean(dim=[1, 2])   # :151
            assert torch.equal(out, act_t > tref.unsqueeze(1).unsqueeze(1))
            layer.pack_output = True                                                               # fused packed form
            np.testing.assert_array_equal(layer(dev(xp)).cpu().numpy(),
                                          oracle.pack(out.cpu().numpy().reshape(-1, O), nd).reshape(*out.shape[:3], -1))
            layer.pack_output = False
        else:
            thr = (layer.bias + layer.bias_noise).type(torch.int32).cpu().numpy() + K          # :156
            np.testing.assert_array_equal(out.cpu().numpy(), oracle.conv_act(xp, filt, thr, *geom))
            assert torch.equal(layer(dev(xp)), out)                                            # packed input
            # fused packed / pooled outputs of the same layer
            layer.pack_output = True
            packed = layer(dev(xp))
            want = oracle.pack(out.cpu().numpy().reshape(-1, O), nd).reshape(*out.shape[:3], -1)
            np.testing.assert_array_equal(packed.cpu().numpy(), want)
            if out.shape[1] >= 2:
                layer.pool_output = True
                np.testing.assert_array_equal(layer(dev(xp)).cpu().numpy(), oracle.max_pool2d(want, 2, 2, 0, 0, 2, 2))
                pool = binary.BinarizedMaxPool2d(dtype=dtype)
                assert torch.equal(pool(out), layer(dev(xp)))                                   # bool input gets packed


def test_maxpool_module(binary, oracle):
    g = rng(9)
    xb = g.integers(0, 2, size=(4, 10, 10, 70)).astype(bool)
    pool = binary.BinarizedMaxPool2d()
    want = oracle.max_pool2d(oracle.pack(xb.reshape(-1, 70), np.int64).reshape(4, 10, 10, 2), 2, 2, 0, 0, 2, 2)
    np.testing.assert_array_equal(pool(dev(xb)).cpu().numpy(), want)
    np.testing.assert_array_equal(pool(dev(oracle.pack(xb.reshape(-1, 70), np.int64).reshape(4, 10, 10, 2))).cpu().numpy(),
                                  want)


def test_perturbed_model_step(binary):
    """set_seed -> set_noise -> forward -> update on a small conv/pool/linear stack through PerturbedModel
    (the NES step of cifar10test.py:150-179 restricted to the binary layers)."""
    D = 32
    model = torch.nn.Sequential(
        binary.BinarizedConv2d(16, 64, D, 3, padding=1, batch_norm=True),
        binary.BinarizedMaxPool2d(),
        binary.BinarizedConv2d(64, 64, D, 3, padding=1, batch_norm=False),
        binary.BinarizedMaxPool2d(),
        torch.nn.Flatten(),
        binary.BinarizedLinear(64 * 2 * 2, 10, D, threshold=False),
    )
    pm = binary.PerturbedModel(model, D)
    assert len(pm.perturbed_layers) == 3
    g = rng(0)
    for layer in pm.perturbed_layers:
        randomise(layer, g)
    pm.set_seed(123)
    bg = torch.Generator(device="cuda")
    bg.manual_seed(9)
    pm.set_noise(bias_generator=bg)
    x = dev(g.integers(0, 2, size=(D, 8, 8, 16)).astype(bool))
    out = pm.forward(x)
    assert tuple(out.shape) == (D, 10) and out.dtype == torch.int32
    assert all(not l.perturbed_flag for l in pm.perturbed_layers)
    assert int(out.abs().max()) <= 256 and (out % 2 == 0).all()               # 2*popc - K with K even
    # same seed (and the same state of the bias generator) -> same noise -> same output; another seed -> different
    # weights
    w0 = [l.weight_noise.clone() for l in pm.perturbed_layers]
    b0 = [l.bias_noise.clone() for l in pm.perturbed_layers]
    bg.manual_seed(9)
    pm.set_noise(bias_generator=bg)
    assert all(torch.equal(a, l.weight_noise) for a, l in zip(w0, pm.perturbed_layers))
    assert all(torch.equal(a, l.bias_noise) for a, l in zip(b0, pm.perturbed_layers))
    assert torch.equal(pm.forward(x), out)
    # without a generator the bias noise comes from torch's global one, as in the reference (modules/binary.py:63-64):
    # a second set_noise() under the same seed keeps the weights but draws fresh bias noise, and two layers of the
    # same shape under one shared seed do not share it
    pm.set_noise()
    assert all(torch.equal(a, l.weight_noise) for a, l in zip(w0, pm.perturbed_layers))
    b1 = [l.bias_noise.clone() for l in pm.perturbed_layers]
    pm.set_noise()
    assert all(not torch.equal(a, l.bias_noise) for a, l in zip(b1, pm.perturbed_layers))
    c0, c1 = pm.perturbed_layers[0], pm.perturbed_layers[1]
    assert c0.bias_noise.shape == c1.bias_noise.shape and not torch.equal(c0.bias_noise, c1.bias_noise)
    assert all(float(l.bias_noise.abs().max()) <= 3.0 for l in pm.perturbed_layers)
    pm.set_seed(124)
    pm.set_noise()
    assert not torch.equal(w0[0], pm.perturbed_layers[0].weight_noise)
    # update: gradients with the parameter shapes (modules/binary.py:67-77)
    fitness = dev(g.standard_normal(D).astype(np.float32))
    pm.update(fitness)
    for l in pm.perturbed_layers:
        assert l.weight.grad.shape == l.weight.shape and l.weight.grad.dtype == torch.float16
        assert torch.isfinite(l.weight.grad.float()).all()
        if l.threshold:
            assert l.bias.grad.shape == l.bias.shape
    # the weight gradient is the fitness-weighted sum of the sampled bits
    lin = pm.perturbed_layers[2]
    from nesgpu_amd.extensions import booleanOperations as ops
    bits = ops.unpack(lin.weight_noise.view(-1, lin.weight_noise.size(2)))[:, :lin.in_features].view(D, 10, -1)
    f16 = fitness.type(torch.float16)
    f16 = f16 - f16.mean()
    want = torch.einsum("d,doi->oi", f16.float(), bits.float()) + 1e-3 * lin.weight.float()
    assert torch.allclose(lin.weight.grad.float(), want, rtol=1e-2, atol=2e-2)     # tolerance of booloptests.py:284
    # the default adds the members in blocks; exact=True is the member-order op, bit for bit
    fast = lin.weight.grad.clone()
    pm.update(fitness, exact=True)
    member_order = ops.weighted_sum(lin.weight_noise, f16.contiguous(), lin.in_degree) + 1e-3 * lin.weight
    assert torch.equal(lin.weight.grad, member_order)
    assert (fast.float() - lin.weight.grad.float()).abs().max().item() <= 2.0 ** -6
    pm.free_memory()
    assert all(l.weight_noise is None for l in pm.perturbed_layers)


def test_reference_import_names_resolve(binary):
    import sys
    import nesgpu_amd
    saved = {k: sys.modules.get(k) for k in ("extensions", "extensions.booleanOperations", "modules", "modules.binary")}
    try:
        for k in saved:
            sys.modules.pop(k, None)
        nesgpu_amd.install_as_reference_modules()
        from extensions import booleanOperations as ref_ops       # the reference's import lines
        from modules import binary as ref_binary
        assert ref_ops.bmm is nesgpu_amd.extensions.booleanOperations.bmm
        assert ref_binary.BinarizedLinear is binary.BinarizedLinear
    finally:
        for k, v in saved.items():
            if v is None:
                sys.modules.pop(k, None)
            else:
                sys.modules[k] = v


def test_conv_bn_thresholds_equal_the_layer_arithmetic():
    from nesgpu_amd.extensions import booleanOperations as ops
    """conv_bn_thresholds against the tensor expression it replaces (modules/binary.py:147-155 on exact pixel sums):
    mean = the exact product float32(sum of activations) * (float32(D * O) / float32(D * O * pixels)) rounded once to
    fp16, as torch's fp16 mean over the pixels of a [D, h, w, O] map; thr = fp16(fp16(bias + noise) + mean),
    threshold = floor(thr) + K; random sums over the whole range, biases that round in fp16, and the non-finite cases
    decided like `activation > thr` (never for NaN and +inf, always for -inf)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(11)
    for D, O, K, pixels in [(64, 64, 576, 1024), (7, 5, 144, 4096), (300, 16, 27, 49), (3, 130, 2048, 1),
                            (50, 24, 216, 112), (9, 64, 576, 56)]:
        sums = torch.randint(0, K * pixels + 1, (D, O), dtype=torch.int32, device="cuda", generator=g)
        bias = (torch.randn(O, device="cuda", generator=g) * 30).to(torch.float16)
        noise = (torch.rand(D, O, device="cuda", generator=g) - 0.5).to(torch.float16)
        got = ops.conv_bn_thresholds(sums, bias, noise, K, pixels)
        s64 = sums.to(torch.int64)
        tot = 2 * s64 - K * pixels
        mean = torch.from_numpy(torch_mean_fp16(tot.cpu().numpy(), D * O, D * O * pixels)).cuda()
        want = torch.floor((bias + noise + mean).to(torch.float32)).to(torch.int32) + K
        assert got.dtype == torch.int32 and torch.equal(got, want)
        # torch's own fp16 mean of a map with these pixel sums (an activation per pixel: the sum spread evenly, the
        # remainder on the first pixels), wherever its fp32 sums are exact
        if K <= 2048 and K * pixels < 2 ** 24:
            q, r = torch.div(tot, pixels, rounding_mode="floor"), torch.remainder(tot, pixels)
            amap = q[:, None, :] + (torch.arange(pixels, device="cuda")[None, :, None] < r[:, None, :]).to(torch.int64)
            assert torch.equal(amap.to(torch.float16).view(D, pixels, 1, O).mean(dim=[1, 2]), mean)
    sums = torch.full((1, 4), 100, dtype=torch.int32, device="cuda")
    bias = torch.tensor([float("nan"), float("inf"), float("-inf"), 60000.0], dtype=torch.float16, device="cuda")
    noise = torch.tensor([[0.0, 0.0, 0.0, 60000.0]], dtype=torch.float16, device="cuda")       # 60000 + 60000 = inf
    got = ops.conv_bn_thresholds(sums, bias, noise, 144, 64).cpu().tolist()[0]
    assert got[0] == 2 ** 31 - 1 and got[1] == 2 ** 31 - 1 and got[3] == 2 ** 31 - 1             # never above
    assert got[2] < -2 ** 30                                                                      # always above


@pytest.mark.parametrize("C,O,k,pad,stride,H,W,D", [(64, 64, 3, 1, 1, 12, 21, 5), (24, 32, 3, 1, 1, 9, 9, 4),
                                                     (130, 48, 3, 0, 1, 7, 8, 3), (8, 16, 5, 2, 2, 11, 9, 3),
                                                     (64, 16, 1, 0, 1, 4, 5, 2), (64, 64, 3, 1, 1, 70, 66, 2)])
@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_conv_bn_thresholds_from_input_equal_the_two_steps(C, O, k, pad, stride, H, W, D, dtype):
    """The one-call thresholds (one kernel where the pixel sums come from bit counts, sums turned into thresholds in
    place elsewhere) == conv_bn_thresholds(conv_popc_sums(...)) under every engine, tap-packed filters included."""
    from nesgpu_amd.extensions import booleanOperations as ops
    g = torch.Generator(device="cuda")
    g.manual_seed(C + O + H)
    bits = torch.iinfo(dtype).bits
    Cw = (C + bits - 1) // bits
    lim = 2 ** (bits - 2)
    x = torch.randint(-lim, lim, (D, H, W, Cw), dtype=dtype, device="cuda", generator=g)
    f = torch.randint(-lim, lim, (D, k * k * Cw, O), dtype=dtype, device="cuda", generator=g)
    if C % bits:
        x[..., -1] &= (1 << (C % bits)) - 1
        f.view(D, k * k, Cw, O)[:, :, -1] &= (1 << (C % bits)) - 1
    bias = (torch.randn(O, device="cuda", generator=g) * 10).to(torch.float16)
    noise = ((torch.rand(D, O, device="cuda", generator=g) - 0.5) * 6).to(torch.float16)
    geom = (k, k, pad, pad, stride, stride)
    h, w = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    kw = dict(in_bits=C) if ops.tap_packing_applies(C, Cw, dtype) else {}
    prev = ops.conv_engine(0)
    try:
        for eng in (0, 1, 2):
            ops.conv_engine(eng)
            want = ops.conv_bn_thresholds(ops.conv_popc_sums(x, f, *geom, **kw), bias, noise, C * k * k, h * w)
            got = ops.conv_bn_thresholds_from_input(x, f, bias, noise, *geom, channels=C, **kw)
            if eng == 0 and stride == 1 and bits == 64:
                assert ops.conv_last_engine() == 5
            assert got.dtype == torch.int32 and torch.equal(got, want), eng
    finally:
        ops.conv_engine(prev)


@pytest.mark.parametrize("C,O,k", [(16, 16, 3), (8, 32, 3), (3, 8, 5), (24, 64, 3)])
def test_pixel_sums_ignore_input_bits_above_the_channels(C, O, k):
    """Tap-packed layers: an input word with bits set above the layer's channel count gives the same pixel sums (and
    so the same batch-norm thresholds) under every engine, namely those of the input with these bits cleared."""
    from nesgpu_amd.extensions import booleanOperations as ops
    g = torch.Generator(device="cuda")
    g.manual_seed(C * 7 + O)
    D, H, W = 130, 9, 11
    x = torch.randint(-2 ** 62, 2 ** 62, (D, H, W, 1), dtype=torch.int64, device="cuda", generator=g)   # stray bits
    clean = x & ((1 << C) - 1)
    f = torch.randint(0, 2 ** C, (D, k * k, O), dtype=torch.int64, device="cuda", generator=g)
    assert ops.tap_packing_applies(C, 1, torch.int64)
    geom = (k, k, k // 2, k // 2, 1, 1)
    prev = ops.conv_engine(0)
    try:
        ops.conv_engine(1)
        want = ops.conv_popc_sums(clean, f, *geom, in_bits=C)
        for eng in (0, 1, 2):
            ops.conv_engine(eng)
            assert torch.equal(ops.conv_popc_sums(x, f, *geom, in_bits=C), want), eng
    finally:
        ops.conv_engine(prev)


@pytest.mark.parametrize("K,M,Z", [(16384, 10, 1024), (4096, 33, 256), (8192, 7, 64), (3000, 5, 128), (65504, 3, 256),
                                   (4096, 33, 1000), (3000, 5, 100), (2100, 9, 7)])
def test_linear_bn_beyond_2048_inputs_equals_the_tensor_expression(K, M, Z):
    """BinarizedLinear(batch_norm=True) with rows longer than fp16's exact integers: the one-call kernel with
    fp16-rounded activations against the reference's tensor expression (modules/binary.py:97-102) evaluated by torch,
    bit for bit; weights with few ones / many ones so that the activations spread over the whole range."""
    from nesgpu_amd.modules import binary
    from nesgpu_amd.extensions import booleanOperations as ops
    g = torch.Generator(device="cuda")
    g.manual_seed(K + M)
    lin = binary.BinarizedLinear(K, M, Z, batch_norm=True)
    with torch.no_grad():
        lin.weight.copy_((torch.randn(M, K, device="cuda", generator=g) * 2).to(torch.float16))
        lin.bias.copy_((torch.randn(M, device="cuda", generator=g) * 40).to(torch.float16))
    lin.set_seed(5)
    lin.set_noise()
    lin.perturbed_flag = True
    Kw = (K + 63) // 64
    x = torch.randint(-2 ** 62, 2 ** 62, (Z, Kw), dtype=torch.int64, device="cuda", generator=g)
    if K % 64:
        x[:, -1] &= (1 << (K % 64)) - 1
    # half of the members see the complement of their weights' majority: large positive and negative activations
    x[::2] = ~x[::2] if K % 64 == 0 else x[::2]
    with torch.no_grad():
        got = lin(x)
        popc = ops.bmm(lin.weight_noise, x.view(Z, -1, 1))
        activation = 2 * popc.squeeze(dim=2) - K
        thresh = (lin.bias + lin.bias_noise)
        thresh = thresh + activation.type(torch.float16).mean(dim=0, keepdim=True)
        want = activation > thresh
    assert got.dtype == torch.bool and torch.equal(got, want)
    assert 0.02 < float(want.float().mean()) < 0.98


def _saturated(shape, g, lo=0.9, hi=1.6):
    """Latent weights of one magnitude scale and random signs: flip probabilities sigmoid(-5 |w| / mean|w|) of about
    a percent, the regime in which a wide layer keeps its members as base + flip lists."""
    w = (lo + (hi - lo) * torch.rand(shape, device="cuda", generator=g)) * (torch.randint(0, 2, shape, device="cuda", generator=g) * 2 - 1)
    return w.to(torch.float16)


@pytest.mark.parametrize("mode", ["law", "law_layered", "flip_probability"])
@pytest.mark.parametrize("threshold,batch_norm,pack_output", [(True, False, True), (True, False, False),
                                                              (False, False, False), (True, True, False)])
def test_wide_linear_layer_in_sparse_form(binary, oracle, mode, threshold, batch_norm, pack_output):
    """BinarizedLinear keeps a wide layer's members as base + flip lists when their flip probabilities are small
    (sparse="auto"): the lists are the oracle's restatement of the sampler's walk on the layer's own law, forward
    equals the oracle's bmm on those weights, and update equals weighted_sum on them."""
    from nesgpu_amd.extensions import booleanOperations as ops
    K, M, D = 4096, 70, 24
    g = torch.Generator(device="cuda")
    g.manual_seed(5 + len(mode))
    kw = dict(flip_probability=0.01) if mode == "flip_probability" else {}
    lin = binary.BinarizedLinear(K, M, D, threshold=threshold, batch_norm=batch_norm, pack_output=pack_output, **kw)
    with torch.no_grad():
        lin.weight.copy_(_saturated((M, K), g))
        if threshold:
            lin.bias.copy_((torch.randn(M, device="cuda", generator=g) * 20).to(torch.float16))
    if mode.startswith("law"):
        assert lin.sparse_walk == "auto" and lin._sparse_walk_now() == "layered"   # largest probability: 4 x the mean
        lin.sparse_walk = "layered" if mode == "law_layered" else "thin"
    lin.set_seed(77)
    lin.set_noise()
    rows = lin.weight_noise
    assert isinstance(rows, ops.FlipRows) and rows.overflowed() == 0
    # the members' weights, regenerated on the host
    if mode.startswith("law"):
        P = lin.probabilities().cpu().numpy()
        law_np, base_bits, tmax = oracle.flip_law(P)
        plan = lin._sparse_plan()
        np.testing.assert_array_equal(plan["law"].law.view(torch.int16).cpu().numpy().view(np.uint16), law_np)
        th = plan["law"].table.view(torch.int32).cpu().numpy().view(np.uint32)
        assert int(th[2]) == tmax
        if mode == "law":
            flips = oracle.skip_flips_thin(law_np, th[4:4 + int(th[0])].copy(), tmax, 77, 0, 0, D)
        else:
            words = int(ops._lib.load().nb_skip_table_words())
            tb = ops.layer_tables("cuda").view(torch.int32).cpu().numpy().view(np.uint32).reshape(16, words)
            cdfs, kts = oracle.layer_tables()
            for k in range(16):
                cdfs[k, :kts[k]] = tb[k, 4:4 + kts[k]]                           # the tables are input data
            flips = oracle.skip_flips_layered(*oracle.law_layers(law_np), 77, 0, 0, D, tables=(cdfs, kts))
        base = oracle.pack(base_bits, np.int64)
    else:
        base = oracle.pack(lin.weight.detach().cpu().numpy() >= 0, np.int64)
        flips = oracle.skip_flips(ops.skip_table(int(0.01 * 2 ** 32)), 77, 0, 0, D * M, K)
    W = base[None] ^ flips.reshape(D, M, K // 64)
    np.testing.assert_array_equal(ops.flip_rows_to_weights(rows).cpu().numpy(), W)
    rate = np.unpackbits(flips.view(np.uint8), axis=1, bitorder="little").mean()
    assert 0.002 < rate < 0.03
    x = torch.randint(-2 ** 62, 2 ** 62, (D, K // 64), dtype=torch.int64, device="cuda", generator=g)
    lin.perturbed_flag = True
    with torch.no_grad():
        out = lin(x)
    act = 2 * oracle.bmm(W, x.cpu().numpy().reshape(D, -1, 1))[:, :, 0].astype(np.int64) - K
    if not threshold:
        np.testing.assert_array_equal(out.cpu().numpy(), act)
    else:
        thr = (lin.bias + lin.bias_noise).detach()
        act_t = torch.from_numpy(act.astype(np.int32)).cuda()
        if batch_norm:
            thr = thr + act_t.type(torch.float16).mean(dim=0, keepdim=True)
        want = act_t > thr                                                      # modules/binary.py:97-103
        if pack_output:
            assert torch.equal(out, ops.pack(want, torch.int64))
        else:
            assert torch.equal(out, want)
    # update: the gradient estimate from the lists against the dense op on the materialised weights
    fit = torch.randn(D, device="cuda", generator=g)
    lin.update(fit)
    wts = (fit.half() - fit.half().mean())
    dense = ops.weighted_sum(torch.from_numpy(W).cuda(), wts.contiguous(), K).float() + 1e-3 * lin.weight.float()
    torch.testing.assert_close(lin.weight.grad.float(), dense, rtol=2e-3, atol=2e-2)
    lin.free_memory()
    assert lin.weight_noise is None and not lin._cache


def test_sparse_form_is_chosen_by_the_flip_probabilities(binary):
    from nesgpu_amd.extensions import booleanOperations as ops
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    lin = binary.BinarizedLinear(2048, 16, 8)
    lin.sparse_recheck = 1                                   # look at the law at every version of the weights
    lin.set_seed(1)
    lin.set_noise()                                          # zero latent weights: every probability 1/2
    assert isinstance(lin.weight_noise, torch.Tensor) and tuple(lin.weight_noise.shape) == (8, 16, 32)
    with torch.no_grad():
        lin.weight.copy_(_saturated((16, 2048), g))
    lin.set_noise()
    assert isinstance(lin.weight_noise, ops.FlipRows)
    assert lin._sparse_walk_now() == "layered"               # probabilities between 0.2 % and 3 %
    with torch.no_grad():
        lin.weight.copy_(torch.sign(lin.weight))             # one magnitude: one probability, one walk at it
    lin.set_noise()
    assert isinstance(lin.weight_noise, ops.FlipRows) and lin._sparse_walk_now() == "thin"
    with torch.no_grad():
        lin.weight[3, 5] = 0.0                               # one undecided weight: a class of its own
    lin.set_noise()
    assert isinstance(lin.weight_noise, ops.FlipRows) and lin._sparse_walk_now() == "layered"
    with torch.no_grad():
        lin.weight[:, ::4] *= 0.125                          # a quarter of the weights near 1/2: too many flips
    lin.set_noise()
    assert isinstance(lin.weight_noise, torch.Tensor)
    # a clearly dense law stands for sparse_recheck versions of the weights before it is looked at again
    slow = binary.BinarizedLinear(2048, 16, 8)
    assert slow.sparse_recheck == 8
    slow.set_seed(1)
    slow.set_noise()
    assert isinstance(slow.weight_noise, torch.Tensor) and "sparse_plan" in slow._cache
    for version in range(1, 9):
        with torch.no_grad():
            slow.weight.copy_(_saturated((16, 2048), g))
        slow.set_noise()
        slow.set_noise()                                     # the same version again: counted once
        assert isinstance(slow.weight_noise, ops.FlipRows) == (version == 8), version
    narrow = binary.BinarizedLinear(1024, 16, 8)
    with torch.no_grad():
        narrow.weight.copy_(_saturated((16, 1024), g))
    narrow.set_seed(1)
    narrow.set_noise()
    assert isinstance(narrow.weight_noise, torch.Tensor)     # short rows stay dense
    with pytest.raises(NotImplementedError):
        binary.BinarizedLinear(1024, 16, 8, dtype=torch.int32, sparse=True).set_noise()
    off = binary.BinarizedLinear(2048, 16, 8, sparse=False, flip_probability=0.01)
    off.set_seed(2)
    off.set_noise()
    assert isinstance(off.weight_noise, torch.Tensor)
    flips = ops.unpack((off.weight_noise ^ off.sign_base()[None]).view(-1, 32)).float().mean().item()
    assert abs(flips - 0.01) < 0.002


def test_wide_layer_workload_under_the_per_weight_law(binary, oracle):
    """The bench's wide-layer workload at a small size: both walks give lists, the materialised form a tensor, and
    each form's forward is the oracle's product on that form's own weights."""
    from nesgpu_amd import workloads
    from nesgpu_amd.extensions import booleanOperations as ops
    D, K, M = 8, 2048, 16
    for kw in (dict(sparse=True, walk="layered"), dict(sparse=True, walk="thin"), dict(sparse=False)):
        lin, set_noise, forward, update = workloads.wide_linear_law_step(D=D, in_features=K, out_features=M, **kw)
        sparse = isinstance(lin.weight_noise, ops.FlipRows)
        assert sparse == bool(kw["sparse"])
        W = (ops.flip_rows_to_weights(lin.weight_noise) if sparse else lin.weight_noise).cpu().numpy()
        out = forward()
        # the input the workload drew is not handed out: take the product on a fresh one
        x = torch.randint(-2 ** 62, 2 ** 62, (D, K // 64), dtype=torch.int64, device="cuda")
        with torch.no_grad():
            got = lin(x)
        act = 2 * oracle.bmm(W, x.cpu().numpy().reshape(D, -1, 1))[:, :, 0].astype(np.int64) - K
        want = torch.from_numpy(act.astype(np.int32)).cuda() > (lin.bias + lin.bias_noise).detach()
        assert torch.equal(got, ops.pack(want, torch.int64)) and got.shape == out.shape
        update()
        assert lin.weight.grad is not None and torch.isfinite(lin.weight.grad.float()).all()


def test_update_helper_kernels_against_the_tensor_expressions(binary):
    """center_fitness, grad_regularize_ and bias_grad against the lines of modules/binary.py:67-77 they replace:
    the elementwise ones bit for bit (given the same mean), the two reductions against float64."""
    from nesgpu_amd.extensions import booleanOperations as ops
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    for n, dtype in [(1024, torch.float32), (1000, torch.float16), (1, torch.float32), (4096, torch.float64), (70, torch.float32)]:
        fit = (torch.randn(n, device="cuda", generator=g, dtype=torch.float32) * 3 + 0.7).to(dtype)
        got = ops.center_fitness(fit)
        w16 = fit.type(torch.float16)
        # the definition: exact mean of the fp16 values, rounded once
        mean = torch.tensor(float(w16.double().sum().item() / n), dtype=torch.float64).to(torch.float16).cuda()
        assert torch.equal(got, w16 - mean), (n, dtype)
        # torch's own mean: the same, or one fp16 step of the mean away
        theirs = w16 - w16.mean()
        step = float(torch.finfo(torch.float16).eps) * max(abs(float(mean)), 2.0 ** -14)
        # (one step of the mean, plus one of the difference where the two roundings fall apart)
        assert (got.float() - theirs.float()).abs().max().item() <= step + 2.0 ** -10 * float((w16.abs().max() + mean.abs()))
    for shape in [(10, 300), (64, 576), (1, 1), (257, 33)]:
        w = torch.randn(shape, device="cuda", generator=g).half()
        w[0, 0] = 0.0
        grad0 = torch.randn(shape, device="cuda", generator=g).half()
        for l1, l2 in [(0, 1e-3), (0.01, 0), (0.02, 0.3), (0, 0)]:
            want = grad0.clone()
            if l1:
                want += l1 * torch.sign(w)
            if l2:
                want += l2 * w
            got = ops.grad_regularize_(grad0.clone(), w, l1, l2)
            assert torch.equal(got, want), (shape, l1, l2)
    for shape in [(1024, 64), (7, 3), (1, 1)]:
        u = torch.rand(shape, device="cuda", generator=g, dtype=torch.float16)
        assert torch.equal(ops.bias_noise_scale_(u.clone()), (u - .5) * 6)           # modules/binary.py:63-64
    for n, O in [(1024, 64), (1000, 10), (16, 256), (3, 1), (2048, 130)]:
        c = torch.randn(n, device="cuda", generator=g).half()
        noise = ((torch.rand((n, O), device="cuda", generator=g) - 0.5) * 6).half()
        got = ops.bias_grad(c, noise).double()
        exact = c.double() @ noise.double()
        slack = 1e-6 * float((c.double().abs().unsqueeze(1) * noise.double().abs()).sum(0).max())
        lo, hi = (exact - slack).half().double(), (exact + slack).half().double()
        assert ((got >= lo) & (got <= hi)).all(), (n, O)
        assert torch.allclose(got.float(), (c @ noise).float(), rtol=2e-3, atol=2e-2)
        assert torch.equal(ops.bias_grad(c, noise).double(), got)
