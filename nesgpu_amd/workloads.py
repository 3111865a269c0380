"""The five benchmark configurations as seeded synthetic workloads on one GPU.

Every builder returns a :class:`Workload` whose ``step()`` launches the population forward of that
configuration (inputs already resident in HBM) and returns its output tensor.  Small operands (inputs,
base weights) come from ``torch.Generator().manual_seed(seed)`` on the CPU; the per-bit random words come
from the library's Philox4x32-10 stream (seed, subsequence) so that a CPU checker can regenerate exactly the
same words for any subset of members without moving gigabytes over PCIe.

Bit convention: +1 <-> bit 1.  Ops return raw popcount sums ``popc``; the reference layer applies
``2*popc - K`` (modules/binary.py:97,145).
"""
from dataclasses import dataclass, field
from typing import Callable, Dict

import torch

from .extensions import booleanOperations as ops

# floor(p * 2**32) for the flip probabilities the configurations name
T_P01 = 42949672
T_P02 = 85899345
T_P05 = 214748364

HBM_PEAK = 8.0e12                     # B/s, MI355X datasheet
VALU_POPC_PEAK = 6.29e14              # bit-MAC/s: 256 CU x 64 lanes x 2.4 GHz / (4 lane-ops per 64 bits) x 64
MFMA_INT8_PEAK = 2.5e15               # byte-MAC/s: dense int8 5.0 POP/s, one +-1 byte MAC per bit-MAC
MFMA_FP4_PEAK = 5.05e15               # MAC/s: dense FP4 10.1 PFLOP/s, one +-1 FP4 MAC per bit-MAC


@dataclass
class Workload:
    name: str
    population: int
    bit_macs: int                      # valid bit-MACs per step (word padding never counted)
    algo_bytes: int                    # algorithmic HBM bytes per step of the dominant kernel
    bound: str                         # "hbm" or "valu"
    step: Callable[[], torch.Tensor]
    tensors: Dict[str, torch.Tensor] = field(default_factory=dict)
    meta: Dict[str, object] = field(default_factory=dict)


def _gen(seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def _bits(g, shape):
    return torch.randint(0, 2, shape, generator=g, dtype=torch.uint8).bool()


def linear_flip_materialised(D=1024, out_f=256, in_f=256, T=T_P01, seed=0, dtype=torch.int64, device="cuda"):
    """Config 1: per-member weights = base ^ flips are materialised once (outside the step); the step is the
    batched matrix-vector XOR-popcount product, one input row per member."""
    g = _gen(seed)
    base_bits = _bits(g, (out_f, in_f))
    x_bits = _bits(g, (D, in_f))
    base = ops.pack(base_bits.to(device), dtype)
    x = ops.pack(x_bits.to(device), dtype)
    W = ops.flip_philox(base, in_f, D, T, seed, subsequence=1)
    xv = x.view(D, -1, 1)
    Kw = W.size(2)
    w = Workload(
        name="linear %dx%d D=%d N=1 p-flip materialised weights" % (out_f, in_f, D),
        population=D, bit_macs=D * out_f * in_f,
        algo_bytes=W.numel() * W.element_size() + x.numel() * x.element_size() + D * out_f * 4,
        bound="hbm", step=lambda: ops.bmm(W, xv),
        tensors=dict(base=base, x=x, W=W), meta=dict(T=T, seed=seed, subsequence=1, in_f=in_f, out_f=out_f, Kw=Kw))
    return w


def linear_flip_fused(D=1024, out_f=1024, in_f=1024, T=T_P05, seed=0, dtype=torch.int64, device="cuda"):
    """Config 2: flip masks are sampled from SUPPLIED uint32 words (threshold compare) inside the XOR-popcount
    product; the words are the only large operand (4 bytes per weight bit)."""
    g = _gen(seed)
    base_bits = _bits(g, (out_f, in_f))
    x_bits = _bits(g, (D, in_f))
    base = ops.pack(base_bits.to(device), dtype)
    x = ops.pack(x_bits.to(device), dtype)
    words = ops.philox_words(D * out_f * in_f, seed, subsequence=2, device=device).view(D, out_f, in_f)
    w = Workload(
        name="linear %dx%d D=%d N=1 p=0.05 flips from supplied uint32 words, fused" % (out_f, in_f, D),
        population=D, bit_macs=D * out_f * in_f,
        algo_bytes=words.numel() * 4 + base.numel() * base.element_size() + x.numel() * x.element_size()
        + D * out_f * 4,
        bound="hbm", step=lambda: ops.seeded_bmv_from_words(T, x, words, base=base),
        tensors=dict(base=base, x=x, words=words), meta=dict(T=T, seed=seed, subsequence=2, in_f=in_f, out_f=out_f))
    return w


def linear_flip_generated(D=1024, out_f=1024, in_f=1024, T=T_P05, seed=0, dtype=torch.int64, device="cuda",
                          half_draws=False):
    """Config 2 in generator mode: the same product with the random words produced inside the kernel by
    Philox4x32-10 (seed, subsequence 2) instead of being read: no 4 GiB operand, the generator's arithmetic is the
    limit.  Bit for bit the same output as :func:`linear_flip_fused` (same stream).  ``half_draws``: 16 bits of the
    stream per weight bit (same law, other bits: the output then equals the product over
    ``sample_bits_philox(..., half_draws=True)``'s weights)."""
    g = _gen(seed)
    base_bits = _bits(g, (out_f, in_f))
    x_bits = _bits(g, (D, in_f))
    base = ops.pack(base_bits.to(device), dtype)
    x = ops.pack(x_bits.to(device), dtype)
    return Workload(
        name="linear %dx%d D=%d N=1 p=0.05 flips from in-kernel Philox %s, fused"
             % (out_f, in_f, D, "half-words (16-bit draws)" if half_draws else "words"),
        population=D, bit_macs=D * out_f * in_f,
        algo_bytes=base.numel() * base.element_size() + x.numel() * x.element_size() + D * out_f * 4,
        bound="generator", step=lambda: ops.seeded_bmv_philox(T, x, out_f, in_f, seed, subsequence=2, base=base,
                                                              half_draws=half_draws),
        tensors=dict(base=base, x=x), meta=dict(T=T, seed=seed, subsequence=2, in_f=in_f, out_f=out_f))


def _conv_filters(base_bits, D, O, k, C, T, seed, subseq, dtype, device):
    """base_bits [O*k*k, C] (rows ordered (out, kx, ky), modules/binary.py:125) -> per-member filters
    [D, k*k*Cw, O] (modules/binary.py:136-137)."""
    base = ops.pack(base_bits.to(device), dtype)                                  # [O*k*k, Cw]
    # one sampler pass writes the rows layout [D, O*k*k, Cw] and the conv layout [D, k*k*Cw, O]
    Wn, filt = ops.sample_bits_philox(T, D, dtype, seed, subseq, base=base, shape=(O * k * k, C), conv_taps=k * k)
    return base, Wn, filt


def _tap(filt, k, C):
    """(filter to pass, extra conv kwargs): the tap-packed filter when C is narrow enough, as
    BinarizedConv2d.set_noise prepares it."""
    if ops.tap_packing_applies(C, 1, filt.dtype) and filt.size(1) == k * k:
        return ops.tap_pack_filter(filt, k * k, C), dict(in_bits=C, filter_tap_packed=True)
    return filt, {}


def conv_int32(D=1024, C=64, O=64, S=32, k=3, pad=1, T=T_P02, seed=0, dtype=torch.int64, device="cuda"):
    """Config 3: batched binary conv, int32 popcount maps out."""
    g = _gen(seed)
    x_bits = _bits(g, (D, S, S, C))
    base_bits = _bits(g, (O * k * k, C))
    x = ops.pack(x_bits.view(-1, C).to(device), dtype).view(D, S, S, -1)
    base, Wn, filt = _conv_filters(base_bits, D, O, k, C, T, seed, 3, dtype, device)
    h = S + 2 * pad - k + 1
    w = Workload(
        name="conv %d->%d %dx%d pad %d on %dx%d D=%d int32 out" % (C, O, k, k, pad, S, S, D),
        population=D, bit_macs=D * h * h * O * k * k * C,
        algo_bytes=x.numel() * x.element_size() + filt.numel() * filt.element_size() + D * h * h * O * 4,
        bound="valu", step=lambda: ops.conv(x, filt, k, k, pad, pad, 1, 1),
        tensors=dict(x=x, base=base, Wn=Wn, filt=filt), meta=dict(T=T, seed=seed, subsequence=3, C=C, O=O, k=k,
                                                                   pad=pad))
    return w


def conv_sign_pool(D=1024, C=16, O=16, S=64, k=3, pad=1, T=T_P02, seed=0, dtype=torch.int64, device="cuda"):
    """Config 4: conv -> sign (2*popc - K > 0) -> pack along channels -> 2x2/s2 OR-pool, one fused kernel."""
    g = _gen(seed)
    x_bits = _bits(g, (D, S, S, C))
    base_bits = _bits(g, (O * k * k, C))
    x = ops.pack(x_bits.view(-1, C).to(device), dtype).view(D, S, S, -1)
    base, Wn, filt = _conv_filters(base_bits, D, O, k, C, T, seed, 4, dtype, device)
    K = k * k * C
    thr = torch.full((D, O), K, dtype=torch.int32, device=device)                # 2*popc > K  <=>  2*popc - K > 0
    ftap, kw = _tap(filt, k, C)
    h = S + 2 * pad - k + 1
    out_words = D * (h // 2) * (h // 2) * ((O + 63) // 64)
    w = Workload(
        name="conv %d->%d %dx%d pad %d on %dx%d D=%d -> sign -> 2x2 OR-pool, packed out" % (C, O, k, k, pad, S, S, D),
        population=D, bit_macs=D * h * h * O * K,
        algo_bytes=x.numel() * x.element_size() + filt.numel() * filt.element_size() + out_words * 8,
        bound="valu", step=lambda: ops.conv_act_pack(x, ftap, thr, k, k, pad, pad, 1, 1, pool=True, **kw),
        tensors=dict(x=x, base=base, Wn=Wn, filt=filt, thr=thr, filt_tap=ftap), meta=dict(T=T, seed=seed, subsequence=4, C=C, O=O,
                                                                             k=k, pad=pad))
    return w


def cifar_net(D=4096, T=T_P01, seed=0, dtype=torch.int64, device="cuda", classes=10, sparse_fc=True):
    """Config 5: conv3->64, conv64->64, pool, conv64->128, pool, linear 8192->1024, linear 1024->10 on 3x32x32
    inputs binarised at their per-channel mean; sign threshold 0 between layers; int32 logits (raw popc).

    ``sparse_fc`` (64-bit words): the 8192->1024 layer keeps its per-member weights as the shared base plus flip
    lists drawn by the skip sampler (Philox stream (seed, subsequence 13); only the gaps between flips are drawn, the
    4 GiB of materialised weights never exist) and runs as one product for the whole population on the matrix cores
    plus 2 bytes per flipped weight.  ``meta["W4"]()`` materialises the same weights for the dense kernels
    (``meta["step_dense"]``), which give the same bits.  With ``sparse_fc=False`` the layer's weights come from the
    per-bit compare sampler (same law, another stream) and are streamed."""
    g = _gen(seed)
    z = torch.randn((D, 3, 32, 32), generator=g)
    x_bits = (z > z.mean(dim=(0, 2, 3), keepdim=True)).permute(0, 2, 3, 1).contiguous()      # [D,32,32,3]
    x = ops.pack(x_bits.view(-1, 3).to(device), dtype).view(D, 32, 32, 1)
    shapes = ((3, 64, 32), (64, 64, 32), (64, 128, 16))
    conv_bases = [ops.pack(_bits(g, (O * 9, C)).to(device), dtype) for (C, O, S) in shapes]
    b4 = ops.pack(_bits(g, (1024, 8192)).to(device), dtype)
    b5 = ops.pack(_bits(g, (classes, 1024)).to(device), dtype)
    sparse = bool(sparse_fc) and dtype == torch.int64
    macs = sum(D * S * S * O * 9 * C for (C, O, S) in shapes) + D * 1024 * 8192 + D * classes * 1024
    thr4 = torch.full((D, 1024), 8192, dtype=torch.int32, device=device)
    state = {}

    def resample():
        """Draw every member's weights of every layer again (what a training step's set_noise does)."""
        layers = []
        for i, (C, O, S) in enumerate(shapes):
            # 64-channel taps: only the gaps between flips are drawn; the 3-channel first layer keeps the per-bit sampler
            draw = ops.sample_bits_skip if C >= 32 else ops.sample_bits_philox
            _, filt = draw(T, D, dtype, seed, 10 + i, base=conv_bases[i], shape=(O * 9, C), conv_taps=9, rows_too=False)
            thr = torch.full((D, O), 9 * C, dtype=torch.int32, device=device)
            layers.append((filt, thr) + _tap(filt, 3, C))
        state["layers"] = layers
        if sparse:
            state["rows4"], state["W4"] = ops.flip_rows_skip(b4, 8192, D, T, seed, subsequence=13), None
        else:
            state["rows4"], state["W4"] = None, ops.flip_philox(b4, 8192, D, T, seed, subsequence=13)  # 4 GiB at 4096
        state["W5"] = ops.flip_philox(b5, 1024, D, T, seed, subsequence=14)

    resample()

    def W4():
        if state["W4"] is None:
            state["W4"] = ops.flip_rows_to_weights(state["rows4"])
        return state["W4"]

    def features():
        a = x
        for i, pool in enumerate((False, True, True)):                   # [D,32,32,1] [D,16,16,1] [D,8,8,2]
            _, thr, f, kw = state["layers"][i]
            a = ops.conv_act_pack(a, f, thr, 3, 3, 1, 1, 1, 1, pool=pool, **kw)
        return a.view(D, -1, 1)                                                                 # [D,128,1]

    def step_dense():
        a = ops.bmv_act_pack(W4(), features(), thr4).view(D, -1, 1)       # pack(2 * bmm(W4, a) > 8192): [D,16,1]
        return ops.bmm(state["W5"], a).squeeze(2)                                               # [D,classes] popc

    def step_sparse():
        a = ops.bmv_flip_act_pack(state["rows4"], features(), thr4).view(D, -1, 1)   # the same bits from the lists
        return ops.bmm(state["W5"], a).squeeze(2)

    def stages():
        """The step's launches one by one, for timing each alone: (name, callable, bound, bit-MACs or bytes).
        bound: "valu" (XOR-popcount issue), "fp4" (FP4 matrix cores) or "hbm"."""
        acts = [x]
        for i, pool in enumerate((False, True, True)):
            _, thr, f, kw = state["layers"][i]
            acts.append(ops.conv_act_pack(acts[-1], f, thr, 3, 3, 1, 1, 1, 1, pool=pool, **kw))
        feats = acts[3].view(D, -1)
        out = []
        for i, pool in enumerate((False, True, True)):
            C, O, S = shapes[i]
            _, thr, f, kw = state["layers"][i]
            a_in = acts[i]
            out.append(("conv %d->%d on %dx%d%s" % (C, O, S, S, ", pooled" if pool else ""),
                        (lambda a_in=a_in, f=f, thr=thr, pool=pool, kw=kw:
                         ops.conv_act_pack(a_in, f, thr, 3, 3, 1, 1, 1, 1, pool=pool, **kw)),
                        "valu" if C == 3 else "fp4", D * S * S * O * 9 * C))
        if sparse:
            rows = state["rows4"]
            ex = ops.expand_rows(feats)
            G = ops.bmm_nt(ex, rows.base_expanded)
            out.append(("input bits -> FP4 codes", lambda: ops.expand_rows(feats), "hbm",
                        feats.numel() * 8 + ex.codes.numel()))
            out.append(("shared product 4096 x 1024 x 8192", lambda: ops.bmm_nt(ex, rows.base_expanded), "fp4",
                        D * 1024 * 8192))
            out.append(("corrections from the flip lists, threshold, pack",
                        lambda: ops.bmv_flip_act_pack(rows, feats, thr4, G=G), "hbm",
                        rows.nbytes() + G.numel() * 4 + thr4.numel() * 4 + feats.numel() * 8))
        else:
            W = W4()
            out.append(("linear 8192->1024 on materialised weights", lambda: ops.bmv_act_pack(W, feats, thr4), "hbm",
                        W.numel() * 8))
        a5 = ops.bmv_act_pack(W4(), feats, thr4).view(D, -1, 1) if not sparse else \
            ops.bmv_flip_act_pack(state["rows4"], feats, thr4).view(D, -1, 1)
        out.append(("linear 1024->%d" % classes, lambda: ops.bmm(state["W5"], a5), "hbm",
                    state["W5"].numel() * 8 + D * classes * 4))
        return out

    w = Workload(
        name="CIFAR-shaped binary net D=%d (conv3-64, conv64-64, pool, conv64-128, pool, fc8192-1024, fc1024-%d)"
             % (D, classes),
        population=D, bit_macs=macs,
        algo_bytes=state["rows4"].nbytes() if sparse else D * 1024 * 128 * 8, bound="valu",
        step=step_sparse if sparse else step_dense,
        tensors=dict(x=x, f1=state["layers"][0][0], f2=state["layers"][1][0], f3=state["layers"][2][0],
                     W5=state["W5"], b1=conv_bases[0], b2=conv_bases[1], b3=conv_bases[2], b4=b4, b5=b5),
        meta=dict(T=T, seed=seed, first_subsequence=10, step_dense=step_dense, features=features,
                  rows4=state["rows4"], W4=W4, thr4=thr4, resample=resample, stages=stages,
                  fc="base + flip lists (skip sampler)" if sparse else "materialised weights"))
    return w


def cifar_net_layers(D=4096, p=0.01, seed=0, device="cuda", classes=10):
    """Config 5 through the layer API: the same network as :func:`cifar_net` built from BinarizedConv2d /
    BinarizedMaxPool2d / BinarizedLinear with ``flip_probability=p`` (weights = sign of the latent weight XOR a
    Bernoulli(p) flip mask), wrapped in a PerturbedModel; packed and pooled outputs between the layers
    (``fuse_packed_outputs``); the wide layer picks the base + flip list form itself.  Thresholds are the layers' own
    ``bias + bias_noise`` (zero bias, noise in [-3, 3)) instead of the fixed 0 of the ops-level workload: the same
    kernels and the same work.  Returns (model, step, set_noise): ``step()`` is one population forward giving int32
    logits ``2 * popc - 1024``."""
    from .modules import binary
    from .modules.base import PerturbedModel
    kw = dict(batch_norm=False, padding=1, device=device, flip_probability=p)
    net = torch.nn.Sequential(
        binary.BinarizedConv2d(3, 64, D, 3, **kw), binary.BinarizedConv2d(64, 64, D, 3, **kw),
        binary.BinarizedMaxPool2d(), binary.BinarizedConv2d(64, 128, D, 3, **kw), binary.BinarizedMaxPool2d(),
        torch.nn.Flatten(), binary.BinarizedLinear(8192, 1024, D, device=device, flip_probability=p),
        binary.BinarizedLinear(1024, classes, D, threshold=False, device=device, flip_probability=p))
    binary.fuse_packed_outputs(net, max_fan_in=None)
    g = _gen(seed)
    with torch.no_grad():
        for m in net.modules():
            if isinstance(m, binary.Binarized):
                m.weight.copy_((torch.randint(0, 2, m.weight.shape, generator=g) * 2 - 1).to(torch.float16))
    model = PerturbedModel(net, D)
    for i, m in enumerate(model.perturbed_layers):
        m.set_seed(seed + 100 + i)
    z = torch.randn((D, 3, 32, 32), generator=g)
    x_bits = (z > z.mean(dim=(0, 2, 3), keepdim=True)).permute(0, 2, 3, 1).contiguous()
    x = ops.pack(x_bits.view(-1, 3).to(device), torch.int64).view(D, 32, 32, 1)

    def set_noise():
        model.set_noise()

    def step():
        with torch.no_grad():
            return model.forward(x)

    set_noise()
    return model, step, set_noise


def small_net_step(D=1024, classes=10, in_channels=24, seed=0, device="cuda", fuse=True):
    """One NES step of a SmallNet-shaped binary network through the layer API (the reference's
    models/cifar10models.py:76-104 driven as in cifar10test.py:150-179): conv 24->64, pool, conv 64->256, pool,
    flatten, linear 16384->classes, batch_norm everywhere, on 32x32 images of 3 x 8 bit planes.  Returns
    (set_noise, forward, update): the three phases of a step as callables, for timing.  ``fuse``: packed and pooled
    outputs between the layers (:func:`nesgpu_amd.modules.binary.fuse_packed_outputs`; same results)."""
    from .modules import binary
    layers, cin = [], in_channels
    for oc in (64, "M", 256, "M"):
        if oc == "M":
            layers.append(binary.BinarizedMaxPool2d())
        else:
            layers.append(binary.BinarizedConv2d(cin, oc, D, 3, batch_norm=True, padding=1, device=device))
            cin = oc
    layers += [torch.nn.Flatten(), binary.BinarizedLinear(cin * 64, classes, D, batch_norm=True, device=device)]
    net = torch.nn.Sequential(*layers)
    if fuse:
        binary.fuse_packed_outputs(net)
    g = _gen(seed)
    with torch.no_grad():
        for p in net.parameters():
            p.copy_(torch.randn(p.shape, generator=g).to(torch.float16).to(p.device))
    mods = [m for m in net.modules() if isinstance(m, binary.Binarized)]
    for i, m in enumerate(mods):
        m.set_seed(seed + 1 + i)
        m.perturbed_flag = True
    img = torch.randint(0, 256, (D, 32, 32, in_channels // 8), generator=g, dtype=torch.uint8).to(device)
    bits = binary.ExtractBits(torch.uint8)(img)                                       # [D,32,32,in_channels] bool
    fitness = torch.randn(D, generator=g).to(device)

    def set_noise():
        for m in mods:
            m.set_noise()

    def forward():
        with torch.no_grad():
            return net(bits)

    def update():
        for m in mods:
            m.update(fitness)

    set_noise()
    forward.model, forward.input = net, bits          # for callers that capture the forward (binary.capture)
    update.fitness = fitness
    return set_noise, forward, update


def linear_layer_config1(D=1024, device="cuda", seed=0):
    """Config 1 as a layer: BinarizedLinear(256, 256) without threshold, weights = sign XOR Bernoulli(0.01) flips,
    one packed input row per member; returns (layer wrapped in a PerturbedModel, packed input)."""
    from .modules import binary
    from .modules.base import PerturbedModel
    lin = binary.BinarizedLinear(256, 256, D, threshold=False, device=device, flip_probability=0.01)
    g = _gen(seed)
    with torch.no_grad():
        lin.weight.copy_((torch.randint(0, 2, lin.weight.shape, generator=g) * 2 - 1).to(torch.float16))
    x = ops.pack(_bits(g, (D, 256)).to(device), torch.int64)
    pm = PerturbedModel(torch.nn.Sequential(lin), D)
    pm.set_seed(seed + 1)
    pm.set_noise()
    return pm, x


BUILDERS = {1: linear_flip_materialised, 2: linear_flip_fused, 3: conv_int32, 4: conv_sign_pool, 5: cifar_net}


def wide_linear_law_step(D=4096, in_features=8192, out_features=1024, spread=0.1, sparse="auto", walk="auto", seed=0,
                         device="cuda"):
    """One NES step of configuration 5's 8192 -> 1024 layer under the reference's OWN law (per-weight probabilities
    sigmoid(5 w / mean|w|), modules/binary.py:59-60) through ``BinarizedLinear``: latent weights +-(1 + spread *
    N(0,1)), i.e. flip probabilities of 0.7 % and up with a tail that grows with ``spread``.  ``sparse`` / ``walk``:
    the layer's ``sparse`` argument and ``sparse_walk`` attribute.  Returns (layer, set_noise, forward, update)."""
    from .modules import binary
    g = _gen(seed)
    lin = binary.BinarizedLinear(in_features, out_features, D, threshold=True, pack_output=True, sparse=sparse,
                                 device=device)
    lin.sparse_walk = walk
    shape = (out_features, in_features)
    sign = torch.randint(0, 2, shape, generator=g) * 2 - 1
    with torch.no_grad():
        lin.weight.copy_((sign * (1.0 + spread * torch.randn(shape, generator=g))).to(torch.float16).to(device))
    lin.set_seed(seed + 1)
    lin.perturbed_flag = True
    x = torch.randint(-2 ** 62, 2 ** 62, (D, (in_features + 63) // 64), generator=g, dtype=torch.int64).to(device)
    fitness = torch.randn(D, generator=g).to(device)

    def forward():
        with torch.no_grad():
            return lin(x)

    lin.set_noise()
    return lin, lin.set_noise, forward, lambda: lin.update(fitness)

