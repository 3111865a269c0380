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

    def __init__(self, in_degree, out_degree, directions, threshold=False, dtype=torch.int64, device="cuda"):
        nn.Module.__init__(self)
        Perturbed.__init__(self, directions)
        self.in_degree = in_degree
        self.out_degree = out_degree
        self.dtype = dtype
        self.threshold = threshold
        self.device = device
        self.directions = directions
        self.bias = None

    def reset_parameters(self):
        with torch.no_grad():
            self.weight.fill_(0)
            if self.threshold:
                self.bias.fill_(0)

    def probabilities(self):
        """fp16 [rows, in_degree] per-bit probabilities of a 1 (modules/binary.py:59-60)."""
        with torch.no_grad():
            norm_weight = self.weight / (self.weight.abs().mean() + 1e-5) * 5
            return torch.sigmoid(norm_weight.float()).half()

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
        P = self.probabilities()
        if words is None:
            sampled = booleanOperations.sample_bits(P, self.directions, self.dtype, self.seed, conv_taps=self.conv_taps)
        else:
            sampled = booleanOperations.sample_bits_from_words(
                booleanOperations.thresholds_from_p(P), words, self.dtype, conv_taps=self.conv_taps)
        if self.conv_taps is None:
            self.weight_noise = sampled
        else:
            # one kernel wrote both layouts: rows (what update sums over) and [D, kx*ky*Cw, out] (what conv multiplies)
            self.weight_noise, self.weight_noise_reshaped = sampled
        self.bias_noise = (torch.rand(size=(self.directions, self.out_degree), dtype=torch.float16,
                                      device=self.weight.device, generator=bias_generator) - .5) * 6

    def update(self, weights, l1=0, l2=1e-3):
        """modules/binary.py:67-77."""
        weights = weights.type(torch.float16)
        weights = (weights - weights.mean())
        self.weight.grad = booleanOperations.weighted_sum(self.weight_noise, weights.contiguous(), self.in_degree)
        if l1:
            self.weight.grad += l1 * torch.sign(self.weight)
        if l2:
            self.weight.grad += l2 * self.weight
        if self.threshold:
            self.bias.grad = weights @ self.bias_noise


class BinarizedLinear(Binarized):
    """modules/binary.py:80-109.  Input [directions, in_features] bool or [directions, Kw] packed: one input
    row per member (a batched matrix-VECTOR product, modules/binary.py:97)."""

    def __init__(self, in_features, out_features, directions, threshold=True, batch_norm=False, dtype=torch.int64,
                 device="cuda", pack_output=False):
        Binarized.__init__(self, in_features, out_features, directions, threshold, dtype, device)
        self.in_features = in_features
        self.out_features = out_features
        if pack_output and not threshold:
            raise NotImplementedError("packed output needs threshold=True")
        self.pack_output = pack_output    # not in the reference: return the thresholded row packed, from one kernel
        self.weight = Parameter(torch.zeros(out_features, in_features, dtype=torch.float16, device=device))
        if threshold:
            self.bias = Parameter(torch.zeros(out_features, dtype=torch.float16, device=device))
        self.batch_norm = batch_norm
        self.reset_parameters()

    def forward(self, input):
        if not self.perturbed_flag:
            raise NotImplementedError                     # modules/binary.py:108-109: no inference path
        packed_input = booleanOperations.pack(input, self.dtype) if input.dtype == torch.bool else input
        if self.threshold and self.batch_norm and (self.in_features <= 2048 or self.pack_output):
            # modules/binary.py:97-102 in one call: the weights are streamed once, the population mean of every output
            # comes from exact integer sums, mean = fp16(float(sum of activations) / directions), and the compare is
            # exact (activations up to 2048 are exact in fp16, which is what the reference compares in)
            return booleanOperations.bmv_bn_act(self.weight_noise, packed_input.view(self.directions, -1),
                                                self.bias.detach(), self.bias_noise, self.in_features,
                                                pack=self.pack_output)
        Z = self.directions
        if (self.threshold and self.batch_norm and self.in_features <= 65504 and Z & (Z - 1) == 0
                and Z * self.in_features <= 2 ** 24):
            # Longer rows: the reference's expression rounds the activations to fp16 (for the mean and for the
            # compare).  The same call does that too, and gives the very bits of the tensor expression below as long
            # as torch's fp32 sum over the population is exact (integers below 2**24) and its multiplication by
            # 1 / directions is a division (a power of two).
            return booleanOperations.bmv_bn_act(self.weight_noise, packed_input.view(Z, -1), self.bias.detach(),
                                                self.bias_noise, self.in_features, round_fp16=True)
        if self.pack_output:
            # activation > t  <=>  2*popc - K > floor(t)  <=>  2*popc > floor(t) + K  (activation is an integer)
            thresh = torch.floor((self.bias + self.bias_noise).to(torch.float32)).to(torch.int32) + self.in_features
            return booleanOperations.bmv_act_pack(self.weight_noise, packed_input.view(self.directions, -1), thresh)
        popc = booleanOperations.bmm(self.weight_noise, packed_input.view(self.directions, -1, 1))
        activation = 2 * popc.squeeze(dim=2) - self.in_features
        if self.threshold:
            thresh = (self.bias + self.bias_noise)
            if self.batch_norm:
                thresh = thresh + activation.type(torch.float16).mean(dim=0, keepdim=True)
            return activation > thresh
        return activation


class BinarizedConv2d(Binarized):
    """modules/binary.py:112-166.  Input [directions, H, W, C] bool (channels last) or
    [directions, H, W, Cw] packed; ``weight`` is [out*kx*ky, in]."""

    def __init__(self, in_channels, out_channels, directions, kernel_size, stride=1, padding=0, dilation=1, groups=1,
                 threshold=True, batch_norm=True, padding_mode='zeros', dtype=torch.int64, device="cuda",
                 pack_output=False, pool_output=False):
        Binarized.__init__(self, in_channels, out_channels, directions, threshold, dtype, device)
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
                thresh = (self.bias + self.bias_noise).type(torch.int32) + offset
            if self.pack_output or self.pool_output:
                return booleanOperations.conv_act_pack(packed_input, filt, thresh, *geom, pool=self.pool_output,
                                                       **tapkw)
            return booleanOperations.conv_act(packed_input, filt, thresh, *geom, **tapkw)
        return 2 * booleanOperations.conv(packed_input, filt, *geom, **tapkw) - offset

    def free_memory(self):
        Perturbed.free_memory(self)
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


def fuse_packed_outputs(model):
    """Switches the fused outputs on in a reference-style stack of layers (not in the reference; results unchanged).

    Walks every ``nn.Sequential`` inside ``model``: a thresholding ``BinarizedConv2d`` followed by a 2x2 / stride 2 /
    no-padding ``BinarizedMaxPool2d`` gets ``pool_output=True`` and the pool becomes ``nn.Identity``; a thresholding
    conv or linear layer whose output goes (through ``nn.Flatten`` at most) into another binary layer, which accepts
    packed words, gets ``pack_output=True``.  A conv in front of ``nn.Flatten`` is only switched when its channel
    count fills whole words, so that the flattened packed words are the flattened bits, and layers with more than
    2048 inputs per output are left alone (their activations are beyond fp16's exact integers, where the reference's
    fp16 comparison and the fused integer comparison can differ).  Returns the number of layers changed."""
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
            if fan_in > 2048:
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
