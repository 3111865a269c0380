"""One NES step of a SmallNet-shaped binary network (models/cifar10models.py:76-104: conv 24->64, pool, conv 64->256,
pool, flatten, linear 16384->classes, batch_norm everywhere) through PerturbedModel, as cifar10test.py:150-179 drives
it (set_seed -> set_noise -> forward -> update), on synthetic uint8 images expanded to bit planes by ExtractBits; the
forward is replayed on the host with the CPU oracle for every member.  Then the checkpoint contract of
culetest.py:117-119 / README.md:107: free_memory(), save, load, same seed -> same population -> same outputs."""
import numpy as np
import pytest
import torch

from golden_util import torch_mean_fp16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def binary():
    assert torch.cuda.is_available()
    from nesgpu_amd.modules import binary
    return binary


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def small_net(binary, directions, classes, in_channels=24):
    """The layer stack of SmallNet (models/cifar10models.py:83-99) with a binary last layer."""
    layers, cin = [], in_channels
    for out_channels in [64, "M", 256, "M"]:
        if out_channels == "M":
            layers += [binary.BinarizedMaxPool2d()]
        else:
            layers += [binary.BinarizedConv2d(cin, out_channels, directions, 3, batch_norm=True, padding=1)]
            cin = out_channels
    layers += [torch.nn.Flatten()]
    layers += [binary.BinarizedLinear(cin * 8 ** 2, classes, directions, batch_norm=True)]
    return torch.nn.Sequential(*layers)


def randomise(model, seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    with torch.no_grad():
        for p in model.parameters():
            scale = 4.0 if p.dim() == 1 else 1.0
            p.copy_((torch.randn(p.shape, generator=g) * scale).to(torch.float16).to(p.device))


def thresholds(layer):
    """floor(P * 2**32) of the layer's probabilities, computed on the host from its fp16 probabilities."""
    P = layer.probabilities().cpu().numpy().astype(np.float64)
    return np.minimum(np.floor(P * 4294967296.0), 4294967295.0).astype(np.uint32)


def f16(t):
    return t.detach().cpu().numpy().astype(np.float16)


def host_weights(oracle, layer, D, R, C):
    """The members' weights as set_noise draws them, regenerated on the host from the Philox stream (seed of the
    layer, subsequence 0): 16-bit draws where the rows are whole words, one 32-bit draw per bit elsewhere."""
    if layer._half_draws():
        return oracle.sample_philox16(thresholds(layer), D, R, C, layer.seed, 0, 0, np.int64)
    words = oracle.philox_words(layer.seed, 0, 0, D * R * C).reshape(D, R, C)
    return oracle.sample_from_words(thresholds(layer), words, np.int64)


def host_forward(oracle, layers, images_bits, D):
    """The forward of modules/binary.py replayed with the oracle's ops: weights regenerated from the Philox stream
    (seed of the layer, subsequence 0), fp16 threshold arithmetic in numpy in the reference's order."""
    conv1, conv2, lin = layers
    a = images_bits                                                                   # [D,32,32,24] bool
    for conv in (conv1, conv2):
        C, O = conv.in_channels, conv.out_channels
        K = 9 * C
        Wn = host_weights(oracle, conv, D, O * 9, C)                                  # [D, O*9, Cw]
        np.testing.assert_array_equal(conv.weight_noise.cpu().numpy(), Wn)
        Cw = Wn.shape[2]
        filt = np.ascontiguousarray(Wn.reshape(D, O, 3, 3, Cw).transpose(0, 2, 3, 4, 1).reshape(D, 9 * Cw, O))
        H = a.shape[1]
        x = oracle.pack(a.reshape(-1, C), np.int64).reshape(D, H, H, Cw) if a.dtype == np.bool_ else a
        act = 2 * oracle.conv(x, filt, 3, 3, 1, 1, 1, 1).astype(np.int64) - K        # modules/binary.py:145
        mean = torch_mean_fp16(act.sum(axis=(1, 2)), D * O, act.size)                   # :151, exact sums
        thr = (f16(conv.bias)[None] + f16(conv.bias_noise)).astype(np.float16)
        thr = (thr + mean).astype(np.float16)
        bits = act > thr[:, None, None, :].astype(np.float64)                         # :155
        a = oracle.max_pool2d(oracle.pack(bits.reshape(-1, O), np.int64).reshape(D, H, H, -1), 2, 2, 0, 0, 2, 2)
    feats = a.reshape(D, -1)                                                          # nn.Flatten: (h, w, word) order
    Kin = lin.in_features
    Wn = host_weights(oracle, lin, D, lin.out_features, Kin)
    np.testing.assert_array_equal(lin.weight_noise.cpu().numpy(), Wn)
    act = 2 * oracle.bmm(Wn, feats.reshape(D, -1, 1))[:, :, 0].astype(np.int64) - Kin  # :97
    # :99-102 literally: the int32 activations go through fp16 (16384 input bits: beyond fp16's exact integers)
    act16 = torch.from_numpy(act.astype(np.int32)).type(torch.float16)
    thr = torch.from_numpy(f16(lin.bias))[None] + torch.from_numpy(f16(lin.bias_noise))
    thr = thr + act16.mean(dim=0, keepdim=True)
    return feats, (act16 > thr).numpy()


def test_smallnet_shaped_nes_step_and_checkpoint(binary, oracle, tmp_path):
    D, classes = 8, 10
    model = small_net(binary, D, classes)
    randomise(model, 1)
    pm = binary.PerturbedModel(model, D)
    assert [type(l).__name__ for l in pm.perturbed_layers] == ["BinarizedConv2d", "BinarizedConv2d", "BinarizedLinear"]
    g = np.random.default_rng(5)
    images = g.integers(0, 256, size=(D, 32, 32, 3)).astype(np.uint8)
    planes = binary.ExtractBits(torch.uint8)(dev(images))                             # [D,32,32,24] bool
    assert planes.dtype == torch.bool and tuple(planes.shape) == (D, 32, 32, 24)
    np.testing.assert_array_equal(planes.cpu().numpy().reshape(D, 32, 32, 3, 8),
                                  np.unpackbits(images[..., None], axis=4, bitorder="little").astype(bool))
    bg = torch.Generator(device="cuda")
    with torch.no_grad():
        pm.set_seed(2024)
        pm.set_noise_scale(0.1)
        bg.manual_seed(77)
        pm.set_noise(bias_generator=bg)
        pred = pm.forward(planes)
    assert pred.dtype == torch.bool and tuple(pred.shape) == (D, classes)
    feats, want = host_forward(oracle, pm.perturbed_layers, planes.cpu().numpy(), D)
    np.testing.assert_array_equal(pred.cpu().numpy(), want)
    # the packed activations that reach the linear layer, too (conv -> mean threshold -> pool chain of every member)
    pm._flags(True)
    try:
        got_feats = model[:5](planes)
    finally:
        pm._flags(False)
    np.testing.assert_array_equal(got_feats.cpu().numpy(), feats)
    # update with per-member fitness (cifar10test.py:163-166): gradients of the parameters' shapes
    with torch.no_grad():
        reward = dev(g.standard_normal(D).astype(np.float32))
        pm.update((reward - reward.mean()) * 0.5 / 0.1)
    for layer in pm.perturbed_layers:
        assert layer.weight.grad.shape == layer.weight.shape and layer.weight.grad.dtype == torch.float16
        assert layer.bias.grad.shape == layer.bias.shape
        assert torch.isfinite(layer.weight.grad.float()).all()
    # checkpoint: free the per-member tensors, save, load into a fresh model, same seed -> same population
    pm.free_memory()
    assert all(l.weight_noise is None and l.bias_noise is None for l in pm.perturbed_layers)
    assert pm.perturbed_layers[0].weight_noise_reshaped is None
    path = tmp_path / "epoch_0.pt"
    torch.save(model.state_dict(), path)
    model2 = small_net(binary, D, classes)
    model2.load_state_dict(torch.load(path, weights_only=True))
    pm2 = binary.PerturbedModel(model2, D)
    with torch.no_grad():
        pm2.set_seed(2024)
        bg.manual_seed(77)
        pm2.set_noise(bias_generator=bg)
        assert torch.equal(pm2.forward(planes), pred)
    # the reference pickles the whole module after free_memory() (culetest.py:117-119); that works here as well
    pm2.free_memory()
    whole = tmp_path / "epoch_0.pkl"
    torch.save(model2, whole)
    model3 = torch.load(whole, weights_only=False)               # a file this test wrote itself
    pm3 = binary.PerturbedModel(model3, D)
    with torch.no_grad():
        pm3.set_seed(2024)
        bg.manual_seed(77)
        pm3.set_noise(bias_generator=bg)
        assert torch.equal(pm3.forward(planes), pred)
    assert sum(p.numel() for p in model3.parameters()) == sum(p.numel() for p in model.parameters())


@pytest.mark.parametrize("dtype,np_dtype", [(torch.uint8, np.uint8), (torch.int8, np.int8), (torch.int32, np.int32),
                                            (torch.int64, np.int64)])
def test_extract_bits_on_the_gpu(binary, oracle, dtype, np_dtype):
    """ExtractBits feeds bit-plane inputs to the first layer (models/mnistmodels.py:92: 784 * 8 input bits): bits LSB
    first along the last axis; for signed types the sign position follows the reference's `> 0` (never set) unless
    sign_bit=True.  The extracted planes packed by the library equal the raw little-endian bytes."""
    g = np.random.default_rng(3)
    info = np.iinfo(np_dtype)
    v = g.integers(info.min, int(info.max) + 1, size=(5, 7), dtype=np.int64).astype(np_dtype)
    bits = info.bits
    full = np.unpackbits(v.view(np.uint8).reshape(5, 7, bits // 8), axis=2, bitorder="little").astype(bool)
    got = binary.ExtractBits(dtype)(dev(v))
    assert got.dtype == torch.bool and tuple(got.shape) == (5, 7 * bits)
    want = full.copy()
    if info.min < 0:
        want[:, :, bits - 1] = False
    np.testing.assert_array_equal(got.cpu().numpy(), want.reshape(5, -1))
    every = binary.ExtractBits(dtype, sign_bit=True)(dev(v))
    np.testing.assert_array_equal(every.cpu().numpy(), full.reshape(5, -1))
    from nesgpu_amd.extensions import booleanOperations as ops
    packed = ops.pack(every, torch.int64).cpu().numpy()
    raw = np.zeros((5, packed.shape[1] * 8), np.uint8)
    raw[:, :7 * bits // 8] = v.view(np.uint8).reshape(5, -1)
    np.testing.assert_array_equal(packed.view(np.uint8).reshape(5, -1), raw)
    if dtype == torch.uint8:                                     # the same words int8pack makes from the bytes
        np.testing.assert_array_equal(ops.int8pack(dev(v), torch.int64).cpu().numpy(), packed)


def test_fuse_packed_outputs_changes_nothing_but_the_kernels(binary):
    """fuse_packed_outputs on the SmallNet-shaped stack: the two convs take their pools in (pool_output), nothing else
    is eligible (the last layer has 16384 inputs per output); same predictions as the unfused stack from the same
    seeds.  On a stack of small layers every boundary is fused: conv -> pool, conv -> Flatten -> linear (64 channels =
    whole words), linear -> linear; same outputs again."""
    D = 8
    g = np.random.default_rng(9)
    planes = binary.ExtractBits(torch.uint8)(dev(g.integers(0, 256, size=(D, 32, 32, 3)).astype(np.uint8)))
    bg = torch.Generator(device="cuda")

    def run(model):
        pm = binary.PerturbedModel(model, D)
        with torch.no_grad():
            pm.set_seed(31)
            pm.set_noise_scale(0.1)
            bg.manual_seed(5)
            pm.set_noise(bias_generator=bg)
            return pm.forward(planes)

    model = small_net(binary, D, 10)
    randomise(model, 3)
    want = run(model)
    assert binary.fuse_packed_outputs(model) == 2
    assert [type(l).__name__ for l in model] == ["BinarizedConv2d", "Identity", "BinarizedConv2d", "Identity", "Flatten",
                                                 "BinarizedLinear"]
    assert model[0].pool_output and model[2].pool_output and not model[5].pack_output
    assert torch.equal(run(model), want)
    assert binary.fuse_packed_outputs(model) == 0                               # idempotent

    small = torch.nn.Sequential(
        binary.BinarizedConv2d(24, 16, D, 3, batch_norm=True, padding=1), binary.BinarizedMaxPool2d(),
        binary.BinarizedConv2d(16, 64, D, 3, batch_norm=False, padding=1), torch.nn.Flatten(),
        binary.BinarizedLinear(16 * 16 * 64, 96, D),
        binary.BinarizedLinear(96, 10, D, batch_norm=True))
    randomise(small, 4)
    want = run(small)
    n = binary.fuse_packed_outputs(small)
    assert small[0].pool_output and small[2].pack_output and small[5].threshold
    assert not small[4].pack_output                                            # 16384 inputs per output: left alone
    assert n == 2
    assert torch.equal(run(small), want)


@pytest.mark.parametrize("kind", ["smallnet", "plain"])
def test_captured_forward_follows_the_eager_one(binary, kind):
    """binary.capture: the forward replayed from a HIP graph gives what the eager forward gives, for new inputs, for
    new noise drawn through the helper (several draws: replays after the first must see the new values, with eager
    work and synchronisations in between), and after the parameters have moved (thresholds that depend on the bias)."""
    D = 16
    g = torch.Generator(device="cuda")
    g.manual_seed(9)
    if kind == "smallnet":
        model = small_net(binary, D, 10)
        binary.fuse_packed_outputs(model)
        x = torch.randint(0, 2, (D, 32, 32, 24), device="cuda", generator=g).bool()
    else:
        # thresholds from bias + bias_noise (no batch norm), a flip-list layer, an int32 output
        model = torch.nn.Sequential(
            binary.BinarizedConv2d(16, 64, D, 3, padding=1, batch_norm=False, flip_probability=0.02),
            binary.BinarizedMaxPool2d(), torch.nn.Flatten(),
            binary.BinarizedLinear(64 * 8 * 8, 64, D, flip_probability=0.01, sparse=True),
            binary.BinarizedLinear(64, 10, D, threshold=False))
        binary.fuse_packed_outputs(model, max_fan_in=None)
        x = torch.randint(0, 2, (D, 16, 16, 16), device="cuda", generator=g).bool()
    randomise(model, 3)
    pm = binary.PerturbedModel(model, D)
    pm.set_seed(11)
    pm.set_noise()
    cap = binary.capture(pm, x)
    with torch.no_grad():
        assert torch.equal(cap(), pm.forward(x))
        for it in range(3):
            x2 = torch.randint(0, 2, tuple(x.shape), device="cuda", generator=g).bool()
            pm.set_seed(100 + it)
            if it == 2:
                for p in model.parameters():                       # an optimiser step between two draws
                    p.add_(torch.randn(p.shape, device="cuda", generator=g).to(p.dtype))
            cap.set_noise()
            got = cap(x2).clone()
            torch.cuda.synchronize()
            want = pm.forward(x2)                                    # eager, on the same (static) noise tensors
            assert torch.equal(got, want), it
            assert torch.equal(cap(x2), want)
            # the noise the graph used is the noise a fresh eager draw with the same seeds gives
            ref_model = pm.model
            before = [l.weight_noise for l in pm.perturbed_layers]
            gen_state = torch.cuda.get_rng_state()
            pm.set_noise()
            torch.cuda.set_rng_state(gen_state)
            for l, b in zip(pm.perturbed_layers, before):
                if isinstance(b, torch.Tensor):
                    assert torch.equal(l.weight_noise, b)
                else:
                    assert torch.equal(l.weight_noise.entries[:8], b.entries[:8]) and torch.equal(l.weight_noise.info, b.info)
            cap.set_noise()                                         # back onto the graph's tensors
            assert ref_model is pm.model
            # update replayed from its own graph against the eager update on the same noise and fitness
            fit = torch.randn(D, device="cuda", generator=g)
            cap.update(fit)
            got_grads = [(l.weight.grad.clone(), l.bias.grad.clone() if l.threshold else None)
                         for l in pm.perturbed_layers]
            torch.cuda.synchronize()
            pm.update(fit)
            for l, (gw, gb) in zip(pm.perturbed_layers, got_grads):
                assert torch.equal(l.weight.grad, gw), (it, type(l).__name__)
                if gb is not None:
                    assert torch.equal(l.bias.grad, gb), (it, type(l).__name__)


def test_captured_forward_over_several_batches(binary):
    """binary.capture(batches=K): one replay evaluates K input batches on the same noise; every output equals the
    eager forward of its batch, also after new noise and new inputs."""
    D, K = 32, 5
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    model = torch.nn.Sequential(binary.BinarizedLinear(256, 256, D, threshold=False, flip_probability=0.01))
    randomise(model, 4)
    pm = binary.PerturbedModel(model, D)
    pm.set_seed(1)
    pm.set_noise()
    xs = torch.randint(0, 2, (K, D, 256), device="cuda", generator=g).bool()
    cap = binary.capture(pm, xs, batches=K)
    with torch.no_grad():
        for it in range(3):
            outs = [o.clone() for o in cap(xs)]
            torch.cuda.synchronize()
            assert len(outs) == K
            for b in range(K):
                assert torch.equal(outs[b], pm.forward(xs[b])), (it, b)
            xs = torch.randint(0, 2, (K, D, 256), device="cuda", generator=g).bool()
            pm.set_seed(10 + it)
            cap.set_noise()
