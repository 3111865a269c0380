"""Binarized perturbed layers with the API of the reference's ``modules/binary.py``:
``BinarizedLinear`` (:80-109), ``BinarizedConv2d`` (:112-166), ``BinarizedMaxPool2d`` (:168-182),
``AsType`` (:11-18), ``ExtractBits`` (:20-29), on top of ``Binarized`` (:32-77).

Constructor signatures, attribute names, tensor layouts and the arithmetic of ``forward`` follow the
reference; the ops come from :mod:`nesgpu_amd.extensions.booleanOperations` (gfx950 kernels).  Known
defects of the reference snapshot are not reproduced: construction order (``Perturbed.__init__`` reading
``self.bias`` too early, modules/base.py:54,107) and ``threshold`` landing in the ``antithetic`` slot
(modules/binary.py:36 vs modules/base.py:47).

Additions, all opt-in: ``set_noise(words=...)`` samples from caller-supplied uint32 words (bit-exact
parity mode), ``set_noise(bias_generator=...)`` draws the bias noise from a given torch.Generator instead of the
global one, and ``BinarizedConv2d(pack_output=True[, pool_output=True])`` returns the thresholded map
already packed along channels (and 2x2 OR-pooled) from one fused kernel instead of a bool map;
``fuse_packed_outputs(model)`` switches those on wherever a reference-style ``nn.Sequential`` allows it.
``flip_probability=p`` (any layer) replaces the law sigmoid(5 w / mean|w|) by "sign of the latent weight, flipped with
probability p" (base XOR Bernoulli(p) flip mask).  ``set_noise`` draws with 16 bits per weight bit where the rows are
whole words (``half_draws``, a class attribute; same law, exact, see ``booleanOperations.sample_bits_philox``).  ``BinarizedLinear(sparse=...)`` keeps ``weight_noise`` as the
shared base plus per-member flip lists (:class:`booleanOperations.FlipRows`) instead of materialised weights: the ops
the layer calls (``bmm``, ``bmv_act_pack``, ``weighted_sum``) take either form and give the same results.
"""
import torch
from torch import nn
from torch.nn.parameter import Parameter

from ..extensions import booleanOperations
from .base import Perturbed, PerturbedModel  # noqa: F401


class AsType(nn.Module):
    """modules/binary.py:11-18."""

    def __init__(self, dtype):
        super().__init__()
        self.dtype = dtype

    def forward(self, x):
        return x.type(self.dtype)


class ExtractBits(nn.Module):
    """Expands every integer into its bits, LSB first, along the last axis (modules/binary.py:20-29).

    As in the reference, a bit counts as set when ``(value & mask) > 0``; for a SIGNED dtype the top mask is the
    (negative) sign bit, so that position is always False there (for torch.uint8, what image bytes come as, all eight
    bits are extracted).  ``sign_bit=True`` (not in the reference) extracts the sign bit of signed types as well."""

    def __init__(self, dtype, sign_bit=False):
        nn.Module.__init__(self)
        self.dtype = dtype
        self.bitlength = torch.iinfo(dtype).bits
        self.sign_bit = sign_bit
        # 1 << i; the top bit of a signed type is the sign bit, built by shifting rather than 2 ** i
        self.mask = torch.ones(self.bitlength, dtype=dtype) << torch.arange(self.bitlength, dtype=dtype)

    def forward(self, input):
        mask = self.mask.to(input.device)
        hit = input.unsqueeze(-1) & mask
        return ((hit != 0) if self.sign_bit else (hit > 0)).view(*input.shape[:-1], -1)


class Binarized(Perturbed, nn.Module):
    """Common part of the binary layers (modules/binary.py:32-77).

    ``weight`` is a latent fp16 matrix [rows, in_degree]; a member's binary weights are drawn per bit with
    probability sigmoid(5 * w / (mean|w| + 1e-5)) (modules/binary.py:59-62) and stored packed as
    ``weight_noise`` [directions, rows, ceil(in_degree/bits)]."""

    def __init__(self, in_degree, out_degree, directions, threshold=False, dtype=torch.int64, device="cuda",
                 flip_probability=None):
        nn.Module.__init__(self)
        Perturbed.__init__(self, directions)
        self.in_degree = in_degree
        self.out_degree = out_degree
        self.dtype = dtype
        self.threshold = threshold
        self.device = device
        self.directions = directions
        self.bias = None
        if flip_probability is not None and not 0.0 <= flip_probability <= 1.0:
            raise ValueError("flip_probability must lie in [0, 1]")
        self.flip_probability = flip_probability      # not in the reference: weights = sign(w) XOR Bernoulli(p)
        self.sparse = False                           # BinarizedLinear only: flip lists instead of weights
        self._cache = {}

    def reset_parameters(self):
        with torch.no_grad():
            self.weight.fill_(0)
            if self.threshold:
                self.bias.fill_(0)

    def probabilities(self):
        """fp16 [rows, in_degree] per-bit probabilities of a 1 (modules/binary.py:59-60): the tensor expression
        ``sigmoid((w / (w.abs().mean() + 1e-5) * 5).float()).half()`` with its roundings, in two small kernels (the mean of
        |w| is the exact one rounded once to fp16, where torch's adds in fp32 in its own order).  With
        ``flip_probability`` p: 1 - p where the latent weight is >= 0, p elsewhere."""
        with torch.no_grad():
            if self.flip_probability is not None:
                p = torch.tensor(self.flip_probability, dtype=torch.float32, device=self.weight.device)
                return torch.where(self.weight >= 0, 1.0 - p, p).half()
            if self.weight.is_cuda:
                return booleanOperations.probabilities_from_weights(self.weight)
            norm_weight = self.weight / (self.weight.abs().mean() + 1e-5) * 5
            return torch.sigmoid(norm_weight.float()).half()

    def _cached(self, key, tensor, make):
        """``make()`` once per version of ``tensor`` (a parameter): what depends only on the latent values."""
        tag = (tensor._version, tensor.data_ptr())
        hit = self._cache.get(key)
        if hit is None or hit[0] != tag:
            with torch.no_grad():
                hit = self._cache[key] = (tag, make())
        return hit[1]

    def sign_base(self):
        """Packed sign bits of the latent weights, [rows, ceil(in_degree/bits)] (bit = w >= 0)."""
        return self._cached("base", self.weight, lambda: booleanOperations.pack(self.weight.detach() >= 0, self.dtype))

    conv_taps = None     # conv layers: kx*ky, and the sampler also writes weight_noise_reshaped

    def set_noise(self, noise_scale=None, words=None, bias_generator=None):
        """modules/binary.py:54-64.  ``words`` (uint32 [directions, rows, in_degree]) replaces the
        generator: bit = words < floor(P * 2**32).  The bias noise comes from torch's global generator of the
        weight's device, as in the reference (:63-64): every call draws fresh values and no two layers share them;
        ``bias_generator`` (a torch.Generator on that device, not in the reference) makes it reproducible."""
        if self.seed is None:
            self.set_seed()
        if noise_scale is not None:
            self.set_noise_scale(noise_scale)
        sampled = None
        if words is not None:
            sampled = booleanOperations.sample_bits_from_words(
                booleanOperations.thresholds_from_p(self.probabilities()), words, self.dtype, conv_taps=self.conv_taps)
        elif self.conv_taps is None and self._sparse_now():
            sampled = self._sample_sparse()
        elif self.flip_probability is not None:
            T = min(int(self.flip_probability * 4294967296.0), 0xFFFFFFFF)
            words = booleanOperations.ceil_div(self.weight.size(1), torch.iinfo(self.dtype).bits)
            # short rows and few flips (a conv layer's filters): only the gaps between flips are drawn.  Measured on
            # 3x3 filters of 64 channels, population 4096: 2.3x the per-bit sampler's speed at p = 0.01, level with it
            # near p = 0.07; rows of a few bits gain nothing
            skip = (self.flip_probability <= 0.05 and self.weight.size(1) >= 32
                    and words <= booleanOperations.SKIP_DENSE_MAX_WORDS)
            if skip:
                sampled = booleanOperations.sample_bits_skip(T, self.directions, self.dtype, self.seed,
                                                             base=self.sign_base(), shape=tuple(self.weight.shape),
                                                             conv_taps=self.conv_taps)
            else:
                sampled = booleanOperations.sample_bits_philox(T, self.directions, self.dtype, self.seed,
                                                               base=self.sign_base(), shape=tuple(self.weight.shape),
                                                               conv_taps=self.conv_taps, half_draws=self._half_draws())
        elif self.weight.is_cuda:
            # sample_bits(P, directions, dtype, seed) of modules/binary.py:62 with the thresholds taken straight from
            # the latent weights
            sampled = booleanOperations.sample_bits_philox(booleanOperations.thresholds_from_weights(self.weight),
                                                           self.directions, self.dtype, self.seed,
                                                           conv_taps=self.conv_taps, half_draws=self._half_draws())
        else:
            sampled = booleanOperations.sample_bits(self.probabilities(), self.directions, self.dtype, self.seed,
                                                    conv_taps=self.conv_taps)
        if self.conv_taps is None:
            self.weight_noise = sampled
        else:
            # one kernel wrote both layouts: rows (what update sums over) and [D, kx*ky*Cw, out] (what conv multiplies)
            self.weight_noise, self.weight_noise_reshaped = sampled
        # (torch.rand(...) - .5) * 6 of the reference, the arithmetic in one kernel with the same roundings
        self.bias_noise = booleanOperations.bias_noise_scale_(
            torch.rand(size=(self.directions, self.out_degree), dtype=torch.float16, device=self.weight.device,
                       generator=bias_generator))

    def _sparse_now(self):
        return False

    # Generator draws of 16 bits per weight bit (two per generated word, ties decided exactly by a second stream)
    # wherever the rows are whole words: the generator's instructions bound set_noise.  False: one 32-bit draw per bit.
    half_draws = True

    def _half_draws(self):
        return self.half_draws and booleanOperations.half_draws_apply(self.weight.size(1), self.dtype)

    def int_thresholds(self, offset, floor=False):
        """int32 [directions, out] thresholds ``(bias + bias_noise) -> int + offset`` of the integer compare
        2*popc > threshold (modules/binary.py:157), made once per (bias, bias_noise) pair instead of on every
        forward."""
        noise = self.bias_noise
        tag = (self.bias._version, self.bias.data_ptr(), noise._version, offset, floor)
        hit = self._cache.get("thresh")
        if hit is None or hit[0] != tag or hit[2] is not noise:
            with torch.no_grad():
                t = self.bias + noise
                t = torch.floor(t.to(torch.float32)).to(torch.int32) if floor else t.type(torch.int32)
                hit = self._cache["thresh"] = (tag, t + offset, noise)   # holds the noise: its identity stays its own
        return hit[1]

    def free_memory(self):
        Perturbed.free_memory(self)
        self._cache = {}

    def update(self, weights, l1=0, l2=1e-3, exact=False):
        """modules/binary.py:67-77.  The sum over the population adds the members in blocks (``weighted_sum`` with
        ``fast=True``: fp32 roundings placed differently, far inside the reference's tolerance for the op,
        booloptests.py:284-285); ``exact=True`` adds them one by one in member order like the reference's kernel.
        The tensor expressions around it are one kernel each with the same roundings (``center_fitness``,
        ``grad_regularize_``, ``bias_grad`` of booleanOperations; the fitness mean is the exact one rounded once and
        the bias gradient is added in a fixed order, where torch's reductions have orders of their own)."""
        with torch.no_grad():
            weights = booleanOperations.center_fitness(weights)
            grad = booleanOperations.weighted_sum(self.weight_noise, weights, self.in_degree, fast=not exact)
            if l1 or l2:
                booleanOperations.grad_regularize_(grad, self.weight.detach(), l1, l2)
            self.weight.grad = grad
            if self.threshold:
                self.bias.grad = booleanOperations.bias_grad(weights, self.bias_noise)


class BinarizedLinear(Binarized):
    """modules/binary.py:80-109.  Input [directions, in_features] bool or [directions, Kw] packed: one input
    row per member (a batched matrix-VECTOR product, modules/binary.py:97)."""

    def __init__(self, in_features, out_features, directions, threshold=True, batch_norm=False, dtype=torch.int64,
                 device="cuda", pack_output=False, flip_probability=None, sparse="auto"):
        Binarized.__init__(self, in_features, out_features, directions, threshold, dtype, device, flip_probability)
        self.in_features = in_features
        self.out_features = out_features
        # True / False / "auto": base + flip lists when the layer is wide and its flip probabilities are small
        # (64-bit words, at least 2048 inputs, at most 65536 outputs)
        if sparse not in (True, False, "auto"):
            raise ValueError("sparse must be True, False or 'auto'")
        self.sparse = sparse
        # per-element laws in the sparse form: "thin" (one walk at the largest probability), "layered" (class by class)
        # or "auto" (whichever takes fewer steps)
        self.sparse_walk = "auto"
        # sparse="auto": how many versions of the weights a clearly dense law (mean flip probability of 0.06 or more)
        # stands before it is looked at again; 1: every version
        self.sparse_recheck = 8
        if pack_output and not threshold:
            raise NotImplementedError("packed output needs threshold=True")
        self.pack_output = pack_output    # not in the reference: return the thresholded row packed, from one kernel
        self.weight = Parameter(torch.zeros(out_features, in_features, dtype=torch.float16, device=device))
        if threshold:
            self.bias = Parameter(torch.zeros(out_features, dtype=torch.float16, device=device))
        self.batch_norm = batch_norm
        self.reset_parameters()

    # ---- sparse form: shared base + per-member flip lists ------------------------------------------------------------
    def _sparse_possible(self):
        return (self.dtype == torch.int64 and self.weight.is_cuda and self.in_features <= 511 * 64
                and self.out_features <= 65536)

    def _sparse_plan(self):
        """What the sparse sampler needs of the latent weights, made once per version of them: with
        ``flip_probability`` the packed sign bits; else the per-element law (base bits, flip probabilities, the skip
        sampler's table) and, read back once, its mean / largest / largest row-mean flip probability, from which the
        decision (``sparse="auto"``) and the lists' capacity follow."""
        def make():
            if self.flip_probability is not None:
                p = min(self.flip_probability, 1.0 - self.flip_probability)
                return dict(law=None, mean=p, peak=p, row=p)
            law = booleanOperations.flip_law_from_weights(self.weight)
            mean, row, peak = law.stats()                                           # the one read-back
            return dict(law=law, mean=mean, peak=peak, row=row)
        return self._cached("sparse_plan", self.weight, make)

    def _sparse_now(self):
        if self.sparse is False or not self._sparse_possible():
            if self.sparse is True:
                raise NotImplementedError("the sparse form needs 64-bit words on a GPU, at most 32704 inputs and 65536 "
                                          "outputs")
            return False
        if self.sparse is True:
            return True
        if self.in_features < 2048:
            return False
        if self.flip_probability is None:
            # a law that was far from sparse is not looked at again for the next sparse_recheck - 1 versions of the
            # weights (looking costs a few kernels and a read-back per version; staying dense a few steps too long
            # costs nothing but time)
            tag = (self.weight._version, self.weight.data_ptr())
            wait = self._cache.get("dense_for")
            if wait is not None and wait[0] != tag and wait[1] > 1:
                self._cache["dense_for"] = (tag, wait[1] - 1)
                return False
            if wait is not None and wait[0] == tag:
                return False
        plan = self._sparse_plan()
        # a row's lists cost a few steps per flip where the dense sampler draws every bit: worth it below about one
        # flip in twenty-five bits, whatever the largest probability (a law with a long tail is walked class by class)
        sparse = plan["mean"] <= 0.04
        self._cache.pop("dense_for", None)
        if not sparse and plan["mean"] >= 0.06 and self.sparse_recheck > 1 and self.flip_probability is None:
            self._cache["dense_for"] = ((self.weight._version, self.weight.data_ptr()), self.sparse_recheck)
        return sparse

    def _sample_sparse(self):
        plan = self._sparse_plan()
        cap = booleanOperations.flip_capacity(self.in_features, plan["row"])
        if plan["law"] is None:
            p = self.flip_probability
            base = self.sign_base() if p <= 0.5 else self._cached(
                "antibase", self.weight, lambda: booleanOperations.pack(self.weight.detach() < 0, self.dtype))
            T = min(int(min(p, 1.0 - p) * 4294967296.0), 0xFFFFFFFF)
            return booleanOperations.flip_rows_skip(base, self.in_features, self.directions, T, self.seed, cap=cap)
        if self._sparse_walk_now() == "layered":
            return booleanOperations.flip_rows_layered(plan["law"], self.directions, self.seed, cap)
        return booleanOperations.flip_rows_thin(plan["law"], self.directions, self.seed, cap)

    def _sparse_walk_now(self):
        """Which walk draws the lists of a per-element law: ``sparse_walk``, or for "auto" the one with fewer steps
        per row: thinning walks at the layer's largest probability; the class-by-class walk takes about three steps
        for two flips (every class accepts at least every second candidate) and a few per class."""
        if self.sparse_walk != "auto":
            return self.sparse_walk
        plan = self._sparse_plan()
        C = self.in_features
        return "layered" if C * plan["peak"] > 1.5 * C * plan["mean"] + 12 else "thin"

    def forward(self, input):
        if not self.perturbed_flag:
            raise NotImplementedError                     # modules/binary.py:108-109: no inference path
        packed_input = booleanOperations.pack(input, self.dtype) if input.dtype == torch.bool else input
        Z = self.directions
        dense = not isinstance(self.weight_noise, booleanOperations.FlipRows)
        if dense and self.threshold and self.batch_norm and self.in_features <= 65504 and (
                self.in_features <= 2048 or self.pack_output or Z * self.in_features <= 2 ** 24):
            # modules/binary.py:97-102 in one call: the weights are streamed once, the population mean of every output
            # comes from exact integer sums the way torch's fp16 mean forms it (the fp32 sum times the fp32 quotient of
            # the element counts), and the compare is exact.  Rows of more than 2048 bits: the reference's expression
            # rounds the activations to fp16 (for the mean and for the compare), and so does the call.  Its bits are
            # those of the tensor expression below as long as torch's fp32 sum over the population is exact (integers
            # up to 2**24); beyond that torch's sum depends on its summation order, the call's is the exact one rounded
            # once, and only short rows and packed outputs (which have no tensor expression) take it.
            return booleanOperations.bmv_bn_act(self.weight_noise, packed_input.view(Z, -1), self.bias.detach(),
                                                self.bias_noise, self.in_features, pack=self.pack_output,
                                                round_fp16=self.in_features > 2048)
        if self.pack_output and not self.batch_norm:
            # activation > t  <=>  2*popc - K > floor(t)  <=>  2*popc > floor(t) + K  (activation is an integer)
            thresh = self.int_thresholds(self.in_features, floor=True)
            return booleanOperations.bmv_act_pack(self.weight_noise, packed_input.view(self.directions, -1), thresh)
        if dense:
            activation = booleanOperations.bmv_pm1(self.weight_noise, packed_input.view(self.directions, -1),
                                                   self.in_features)                       # :97 in one kernel
        else:
            popc = booleanOperations.bmm(self.weight_noise, packed_input.view(self.directions, -1, 1))
            activation = 2 * popc.squeeze(dim=2) - self.in_features
        if self.threshold:
            thresh = (self.bias + self.bias_noise)
            if self.batch_norm:
                thresh = thresh + activation.type(torch.float16).mean(dim=0, keepdim=True)
            bits = activation > thresh
            return booleanOperations.pack(bits, self.dtype) if self.pack_output else bits
        return activation


class BinarizedConv2d(Binarized):
    """modules/binary.py:112-166.  Input [directions, H, W, C] bool (channels last) or
    [directions, H, W, Cw] packed; ``weight`` is [out*kx*ky, in]."""

    def __init__(self, in_channels, out_channels, directions, kernel_size, stride=1, padding=0, dilation=1, groups=1,
                 threshold=True, batch_norm=True, padding_mode='zeros', dtype=torch.int64, device="cuda",
                 pack_output=False, pool_output=False, flip_probability=None):
        Binarized.__init__(self, in_channels, out_channels, directions, threshold, dtype, device, flip_probability)
        if dilation != 1 or groups != 1 or padding_mode != "zeros":
            raise NotImplementedError
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.stride = stride
        self.padding = padding
        self.kernel_size = (kernel_size, kernel_size) if isinstance(kernel_size, int) else kernel_size
        self.conv_taps = self.kernel_size[0] * self.kernel_size[1]
        self.weight = Parameter(torch.zeros(out_channels * self.kernel_size[0] * self.kernel_size[1], in_channels,
                                            dtype=torch.float16, device=device))
        if threshold:
            self.bias = Parameter(torch.zeros(out_channels, dtype=torch.float16, device=device))
        self.batch_norm = batch_norm
        self.pack_output = pack_output
        self.pool_output = pool_output
        if (pack_output or pool_output) and not threshold:
            raise NotImplementedError("packed output needs threshold=True")
        self.weight_noise_reshaped = None
        self.weight_noise_tap = None
        self.reset_parameters()

    def reset_parameters(self):
        Binarized.reset_parameters(self)

    def set_noise(self, noise_scale=None, words=None, bias_generator=None):
        """modules/binary.py:134-137: [D, out*kx*ky, Cw] -> [D, kx*ky*Cw, out], out contiguous."""
        Binarized.set_noise(self, noise_scale, words, bias_generator)     # fills weight_noise_reshaped as well
        # narrow inputs (one word per pixel, at most half of it used): several taps share a word
        self.weight_noise_tap = None
        if booleanOperations.tap_packing_applies(self.in_channels, self.weight_noise.size(2), self.dtype):
            self.weight_noise_tap = booleanOperations.tap_pack_filter(
                self.weight_noise_reshaped, self.kernel_size[0] * self.kernel_size[1], self.in_channels)

    def forward(self, input):
        if not self.perturbed_flag:
            raise NotImplementedError
        if input.dtype == torch.bool:
            packed_input = booleanOperations.pack(input.reshape(-1, self.in_channels), self.dtype).view(
                *input.shape[:3], -1)
        else:
            packed_input = input
        offset = self.in_channels * self.kernel_size[0] * self.kernel_size[1]
        geom = (*self.kernel_size, self.padding, self.padding, self.stride, self.stride)
        filt, tapkw = self.weight_noise_reshaped, {}
        if getattr(self, "weight_noise_tap", None) is not None:
            filt, tapkw = self.weight_noise_tap, dict(in_bits=self.in_channels, filter_tap_packed=True)
        if self.threshold:
            if self.batch_norm and offset > 2048:
                # activations beyond fp16's exact integers: keep the reference's composition, roundings included
                activation = 2 * booleanOperations.conv(packed_input, filt, *geom, **tapkw) - offset
                thresh = self.bias + self.bias_noise + activation.type(torch.float16).mean(dim=[1, 2])
                return activation > thresh.unsqueeze(1).unsqueeze(1)
            if self.batch_norm:
                # modules/binary.py:147-155 without the int32 maps: the per-member mean over h,w needs only the sum of
                # the popcounts (exact integers), mean = fp16(float(sum of activations) / (h*w)); activations are
                # integers that fp16 holds exactly, so activation > thresh  <=>  2*popc > floor(thresh) + offset.
                thresh = booleanOperations.conv_bn_thresholds_from_input(
                    packed_input, filt, self.bias.detach(), self.bias_noise, *geom, channels=self.in_channels, **tapkw)
            else:
                thresh = self.int_thresholds(offset)
            if self.pack_output or self.pool_output:
                return booleanOperations.conv_act_pack(packed_input, filt, thresh, *geom, pool=self.pool_output,
                                                       **tapkw)
            return booleanOperations.conv_act(packed_input, filt, thresh, *geom, **tapkw)
        return 2 * booleanOperations.conv(packed_input, filt, *geom, **tapkw) - offset

    def free_memory(self):
        Binarized.free_memory(self)
        self.weight_noise_reshaped = None
        self.weight_noise_tap = None


class BinarizedMaxPool2d(nn.Module):
    """modules/binary.py:168-182."""

    def __init__(self, kernel_size=(2, 2), padding=(0, 0), stride=(2, 2), dtype=torch.int64):
        nn.Module.__init__(self)
        self.kernel_size = kernel_size
        self.padding = padding
        self.stride = stride
        self.dtype = dtype

    def forward(self, input):
        if input.dtype == torch.bool:
            packed_input = booleanOperations.pack(input.reshape(-1, input.size(3)), self.dtype).view(
                *input.shape[:3], -1)
        else:
            packed_input = input
        return booleanOperations.max_pool2d(packed_input, *self.kernel_size, *self.padding, *self.stride)


def fuse_packed_outputs(model, max_fan_in=2048):
    """Switches the fused outputs on in a reference-style stack of layers (not in the reference; results unchanged).

    Walks every ``nn.Sequential`` inside ``model``: a thresholding ``BinarizedConv2d`` followed by a 2x2 / stride 2 /
    no-padding ``BinarizedMaxPool2d`` gets ``pool_output=True`` and the pool becomes ``nn.Identity``; a thresholding
    conv or linear layer whose output goes (through ``nn.Flatten`` at most) into another binary layer, which accepts
    packed words, gets ``pack_output=True``.  A conv in front of ``nn.Flatten`` is only switched when its channel
    count fills whole words, so that the flattened packed words are the flattened bits, and layers with more than
    ``max_fan_in`` = 2048 inputs per output are left alone (their activations are beyond fp16's exact integers, where
    the reference's fp16 comparison and the fused integer comparison can differ: without batch norm they differ only
    for thresholds ``bias + bias_noise`` beyond +-2048, since rounding an activation to fp16 never moves it across a
    smaller threshold; ``max_fan_in=None`` fuses such layers too, for models whose biases stay below that).
    Returns the number of layers changed."""
    changed = 0
    for seq in [m for m in model.modules() if isinstance(m, nn.Sequential)]:
        layers = list(seq)
        for i, layer in enumerate(layers):
            if not isinstance(layer, (BinarizedConv2d, BinarizedLinear)) or not layer.threshold:
                continue
            # the fused kernels compare integers; the reference compares in fp16, which is the same thing as long as
            # the activations are integers that fp16 holds exactly
            if isinstance(layer, BinarizedConv2d):
                fan_in = layer.in_channels * layer.kernel_size[0] * layer.kernel_size[1]
            else:
                fan_in = layer.in_features
            if max_fan_in is not None and fan_in > max_fan_in:
                continue
            if fan_in > 2048 and layer.batch_norm:
                continue
            j = i + 1
            if isinstance(layer, BinarizedConv2d) and j < len(layers) and isinstance(layers[j], BinarizedMaxPool2d):
                pool = layers[j]
                if (tuple(pool.kernel_size), tuple(pool.padding), tuple(pool.stride)) == ((2, 2), (0, 0), (2, 2)) \
                        and pool.dtype == layer.dtype and not layer.pool_output:
                    layer.pool_output = True
                    seq[j] = nn.Identity()
                    layers[j] = seq[j]
                    changed += 1
                continue                      # a pool's output is packed either way
            if getattr(layer, "pool_output", False):
                continue                      # already packed (and pooled)
            through_flatten = False
            while j < len(layers) and isinstance(layers[j], (nn.Flatten, nn.Identity)):
                through_flatten = through_flatten or isinstance(layers[j], nn.Flatten)
                j += 1
            if j >= len(layers) or not isinstance(layers[j], (BinarizedConv2d, BinarizedLinear, BinarizedMaxPool2d)):
                continue
            if layers[j].dtype != layer.dtype or layer.pack_output:
                continue
            bits = torch.iinfo(layer.dtype).bits
            if isinstance(layer, BinarizedConv2d) and through_flatten and layer.out_channels % bits:
                continue
            if isinstance(layer, BinarizedLinear) and isinstance(layers[j], (BinarizedConv2d, BinarizedMaxPool2d)):
                continue                      # a linear layer's row is not an image
            layer.pack_output = True
            changed += 1
    return changed


def _noise_state(layer):
    """The tensors a layer's forward reads besides its input and its parameters, in a fixed order:
    [(name, tensor), ...].  A flip-list layer contributes its lists, their info words and the shared base."""
    out = []
    wn = layer.weight_noise
    if isinstance(wn, booleanOperations.FlipRows):
        out += [("entries", wn.entries), ("info", wn.info), ("overflow", wn.overflow), ("base", wn.base),
                ("base_codes", wn.base_expanded.codes)]
    elif wn is not None:
        out.append(("weight_noise", wn))
    for name in ("weight_noise_reshaped", "weight_noise_tap", "bias_noise"):
        t = getattr(layer, name, None)
        if t is not None:
            out.append((name, t))
    hit = layer._cache.get("thresh")
    if hit is not None:
        out.append(("thresh", hit[1]))
    return out


class CapturedForward:
    """A population forward recorded once as a HIP graph and replayed (not in the reference): a step of a small
    network is a handful of kernels of a few microseconds each, which eager launches from Python cannot keep fed.

    ``capture(model, example_input)`` runs the forward of ``model`` (an ``nn.Module`` of binary layers or a
    :class:`PerturbedModel`; ``set_noise`` must have been called) under graph capture.  The graph reads the layers'
    noise tensors at the addresses they had then, so new noise has to arrive there: :meth:`set_noise` draws it with
    the layers' own ``set_noise`` and copies it into those tensors (and makes them the layers' noise again), and
    brings the integer thresholds that depend on ``bias`` up to date.  Shapes must not change between draws (a
    flip-list layer keeps its capacity as long as its latent weights give the same one; otherwise capture again).
    ``forward(input)`` copies ``input`` into the graph's input tensor, replays, and returns the graph's output tensor
    (overwritten by the next replay).  ``batches=K``: ``example_input`` is [K, ...], K input batches evaluated on the same
    noise (a fitness evaluation over several minibatches per draw); the graph holds the K forwards and ``forward``
    returns the list of their K outputs from ONE replay, which matters for small networks: launching a graph from
    Python costs about 15 us whatever it holds."""

    def __init__(self, model, example_input, warmup=2, batches=None):
        self.model = model if isinstance(model, PerturbedModel) else PerturbedModel(model, None)
        self.layers = [m for m in self.model.perturbed_layers if isinstance(m, Binarized)]
        self.input = example_input.clone()
        self.batches = batches
        self._updates = {}
        run = self._forward_all
        with torch.no_grad():
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(max(1, warmup)):          # also fills the layers' threshold caches
                    run()
            torch.cuda.current_stream().wait_stream(side)
            self._static = [_noise_state(m) for m in self.layers]
            self._thresh_args = [m._cache["thresh"][0][3:5] if "thresh" in m._cache else None for m in self.layers]
            self._objects = [(m.weight_noise, getattr(m, "weight_noise_reshaped", None),
                              getattr(m, "weight_noise_tap", None), m.bias_noise) for m in self.layers]
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                self.output = run()

    def _forward_all(self):
        if self.batches is None:
            return self.model.forward(self.input)
        return [self.model.forward(self.input[b]) for b in range(self.batches)]

    def forward(self, input=None):
        if input is not None:
            self.input.copy_(input)
        self.graph.replay()
        return self.output

    __call__ = forward

    def set_noise(self, *args, **kwargs):
        """``set_noise`` of every layer, with the new noise copied to where the graph reads it."""
        with torch.no_grad():
            for m, static, targs, objs in zip(self.layers, self._static, self._thresh_args, self._objects):
                m._cache.pop("thresh", None)
                m.set_noise(*args, **kwargs)
                if targs is not None:
                    m.int_thresholds(*targs)
                fresh = _noise_state(m)
                if [(n, tuple(t.shape), t.dtype) for n, t in fresh] != [(n, tuple(t.shape), t.dtype) for n, t in static]:
                    raise RuntimeError("the layer's noise changed shape since the capture; capture again")
                for (_, dst), (_, src) in zip(static, fresh):
                    if dst.data_ptr() != src.data_ptr():
                        dst.copy_(src)
                # the graph's tensors are the layer's noise again (eager calls and update() see what the graph sees)
                m.weight_noise, reshaped, tap, m.bias_noise = objs
                if reshaped is not None:
                    m.weight_noise_reshaped = reshaped
                if tap is not None:
                    m.weight_noise_tap = tap
                if targs is not None:
                    thr = dict(static)["thresh"]
                    tag = (m.bias._version, m.bias.data_ptr(), m.bias_noise._version) + tuple(targs)
                    m._cache["thresh"] = (tag, thr, m.bias_noise)


    def update(self, weights, l1=0, l2=1e-3, exact=False):
        """``update`` of every layer (modules/binary.py:67-77) as one graph replay: recorded on the first call for a
        given (l1, l2, exact) and shape of ``weights``, replayed afterwards with ``weights`` copied into the graph's
        tensor.  The layers' ``.grad`` tensors are the graph's: the next replay overwrites them.  The graph reads the
        noise where this object's :meth:`set_noise` puts it."""
        key = (l1, l2, exact, weights.dtype, tuple(weights.shape))
        rec = self._updates.get(key)
        with torch.no_grad():
            if rec is None:
                static = weights.clone()
                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):
                    for m in self.layers:
                        m.update(static, l1, l2, exact)
                torch.cuda.current_stream().wait_stream(side)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    for m in self.layers:
                        m.update(static, l1, l2, exact)
                grads = [(m.weight.grad, m.bias.grad if m.threshold else None) for m in self.layers]
                rec = self._updates[key] = (graph, static, grads)
            graph, static, grads = rec
            static.copy_(weights)
            graph.replay()
            for m, (gw, gb) in zip(self.layers, grads):
                m.weight.grad = gw
                if gb is not None:
                    m.bias.grad = gb


def capture(model, example_input, warmup=2, batches=None):
    """See :class:`CapturedForward`."""
    return CapturedForward(model, example_input, warmup, batches)
