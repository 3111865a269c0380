"""The C-ABI shared library without a GPU: it loads, exports every symbol include/nesbin.h declares, and
rejects bad arguments with a status code before launching anything.  No compute calls here."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "nesbin.h")


@pytest.fixture(scope="module")
def lib():
    from nesgpu_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        import __graft_entry__ as g
        g.build()
    return _lib.load()


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nb_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_what_the_binding_lists():
    from nesgpu_amd import _lib
    assert declared_symbols() == sorted(_lib.exported_symbols())


def test_every_declared_symbol_is_exported(lib):
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_version_and_error_string(lib):
    assert lib.nb_version() >= 100
    assert isinstance(lib.nb_last_error_string(), bytes)


def test_bad_arguments_are_rejected_without_a_launch(lib):
    from nesgpu_amd import _lib
    one = ctypes.c_void_p(8)          # a non-NULL, 8-byte aligned dummy; never dereferenced on these paths
    odd = ctypes.c_void_p(12)
    # negative shape
    assert lib.nb_pack_i64(one, one, -1, 3, None) == 2
    assert b"negative" in lib.nb_last_error_string()
    # NULL pointer with a non-empty shape
    assert lib.nb_bmm_i64(None, one, one, 1, 1, 1, 1, None) == 1
    assert lib.nb_bmm_i64(one, None, one, 1, 1, 1, 2, None) == 1
    # misaligned words
    assert lib.nb_bmm_i64(one, odd, one, 1, 1, 1, 2, None) == 3
    # conv window larger than the padded input
    assert lib.nb_conv_i64(one, one, one, 1, 2, 2, 1, 1, 5, 5, 0, 0, 1, 1, 0, None) == 2
    # tap packing needs one word per pixel and at most half a word of channels
    assert lib.nb_conv_i64(one, one, one, 1, 8, 8, 2, 4, 3, 3, 1, 1, 1, 1, 16, None) == 2
    assert lib.nb_conv_i64(one, one, one, 1, 8, 8, 1, 4, 3, 3, 1, 1, 1, 1, 40, None) == 2
    assert lib.nb_tap_pack_filter_i64(one, one, 1, 9, 4, 0, None) == 2
    # zero stride
    assert lib.nb_max_pool2d_i64(one, one, 1, 4, 4, 1, 2, 2, 0, 0, 0, 2, None) == 2
    # weighted_sum: more output bits than a row's words hold
    assert lib.nb_weighted_sum_i64(one, one, one, 4, 2, 1, 65, None) == 2
    assert b"zbits" in lib.nb_last_error_string()
    assert lib.nb_weighted_sum_i32(one, one, one, 4, 2, 2, 65, None) == 2
    assert lib.nb_weighted_sum_fast_i64(one, one, one, 4, 2, 1, 65, None) == 2
    assert lib.nb_weighted_sum_fast_i32(one, one, one, -1, 2, 2, 64, None) == 2
    # the skip sampler as packed words: no output, rows of more than 8 words
    assert lib.nb_sample_conv_skip_i64(None, None, one, one, 1, 0, 0, 2, 4, 9, 64, None) == 2
    assert lib.nb_sample_skip_i64(one, one, one, 1, 0, 0, 2, 4, 576, None) == 4
    assert lib.nb_sample_skip_i32(one, one, one, 1, 0, 0, 2, 4, 288, None) == 4
    # the update helpers: negative lengths, a misaligned fp32 pointer
    assert lib.nb_center_fitness_f16(one, one, -1, None) == 2
    assert lib.nb_center_fitness_f32(one, ctypes.c_void_p(10), 4, None) == 3
    assert lib.nb_grad_regularize(one, one, 0.1, 0.1, -1, None) == 2
    assert lib.nb_bias_grad(one, one, one, -1, 4, None) == 2
    assert lib.nb_bias_noise_scale(one, -1, None) == 2
    # the linear layer's activation: more input bits than the rows hold
    assert lib.nb_bmv_pm1_i64(one, one, one, 1, 1, 1, 65, None) == 2
    assert lib.nb_bmv_pm1_i32(one, one, one, 1, 1, 2, 65, None) == 2
    # 16-bit draws: rows that are not whole words, a stream offset that is not a multiple of 8
    assert lib.nb_sample_philox16_i64(one, None, None, 5, 1, 0, 0, 2, 3, 70, None) == 4
    assert lib.nb_sample_philox16_i32(one, None, None, 5, 1, 0, 4, 2, 3, 64, None) == 4
    assert lib.nb_sample_conv_philox16_i64(None, one, None, None, 5, 1, 0, 0, 2, 3, 9, 64, None) == 1
    # conv batch-norm thresholds: a pixel count below one, a misaligned fp16 pointer
    assert lib.nb_conv_bn_thresholds(one, one, one, one, 2, 3, 144, 0, None) == 2
    assert lib.nb_conv_bn_thresholds(one, one, ctypes.c_void_p(9), one, 2, 3, 144, 64, None) == 3
    assert lib.nb_conv_bn_thresholds(None, None, None, None, 0, 3, 144, 64, None) == 0
    # the same thresholds from the layer's input: a window larger than the padded image (no output pixel), a missing
    # bias, a misaligned noise pointer, an empty population
    args = (1, 2, 2, 1, 4, 5, 5, 0, 0, 1, 1, 0, 100, None)
    assert lib.nb_conv_bn_thresholds_from_input_i64(one, one, one, one, one, *args) == 2
    args = (1, 8, 8, 1, 4, 3, 3, 1, 1, 1, 1, 0, 576, None)
    assert lib.nb_conv_bn_thresholds_from_input_i64(one, one, one, None, one, *args) == 1
    assert lib.nb_conv_bn_thresholds_from_input_i32(one, one, one, one, ctypes.c_void_p(9), *args) == 3
    assert lib.nb_conv_bn_thresholds_from_input_i64(None, None, None, None, None, 0, 8, 8, 1, 4, 3, 3, 1, 1, 1, 1, 0, 576,
                                                    None) == 0
    # sampler thresholds: a NULL probability array, an odd fp16 address, an empty array
    assert lib.nb_thresholds_from_p(one, None, 4, None) == 1
    assert lib.nb_thresholds_from_p(one, ctypes.c_void_p(9), 4, None) == 3
    assert lib.nb_thresholds_from_p(None, None, 0, None) == 0
    # flip lists: the overflow count has to go somewhere, entries are read 16 bytes at a time, R <= 65536, a
    # capacity of at most 8191 pieces per row; the skip sampler needs its table
    big = ctypes.c_void_p(256)
    assert lib.nb_flip_fill_i64(big, one, None, one, one, 2, 64, 1, 4, None) == 1
    assert lib.nb_flip_fill_i64(one, one, one, one, one, 2, 64, 1, 4, None) == 3
    assert lib.nb_flip_fill_i64(big, one, one, one, one, 2, 65537, 1, 4, None) == 2
    assert lib.nb_bmv_flip_i64(one, one, big, one, one, 2, 64, 1, 8192, None) == 2
    assert lib.nb_flip_skip_i64(big, one, one, one, None, 1, 0, 0, 2, 64, 64, 4, None) == 1
    assert lib.nb_flip_skip_thin_i64(big, one, one, ctypes.c_void_p(9), one, 1, 0, 0, 2, 64, 64, 4, None) == 3
    assert lib.nb_flip_weighted_sum_i64(one, big, one, one, ctypes.c_void_p(9), 2, 64, 64, 4, None) == 3
    assert lib.nb_flip_skip_layered_i64(big, one, one, one, None, one, 1, 0, 0, 2, 64, 64, 4, None) == 1     # cls missing
    assert lib.nb_flip_skip_layered_i64(big, one, one, ctypes.c_void_p(6), one, one, 1, 0, 0, 2, 64, 64, 4, None) == 3
    assert lib.nb_flip_skip_layered_i64(big, one, one, one, one, one, 1, 0, 0, 2, 64, 512 * 64, 4, None) == 2  # row too long
    assert lib.nb_flip_law_layers(one, None, one, 4, 64, None) == 1
    assert lib.nb_flip_law_layers(one, one, one, 4, 512 * 64, None) == 2
    assert lib.nb_flip_law_layers(None, None, None, 0, 64, None) == 0
    assert lib.nb_flip_layer_tables(None, None) == 1
    assert lib.nb_flip_law_stats(one, one, one, None, 4, 64, None) == 1
    assert lib.nb_flip_law_stats(one, one, one, one, 0, 64, None) == 2
    assert lib.nb_flip_layer_table_words() == 16 * 4100
    assert lib.nb_flip_law_from_weights(one, one, None, one, 4, 64, one, None) == 1
    assert lib.nb_thresholds_from_weights(one, one, 4, ctypes.c_void_p(4), None) == 3
    assert lib.nb_skip_table_words() == 4100 and lib.nb_law_workspace_bytes() == 2048
    # empty problems succeed without touching the pointers
    assert lib.nb_pack_i64(None, None, 0, 64, None) == 0
    assert lib.nb_bmm_i32(None, None, None, 0, 5, 5, 5, None) == 0
    assert lib.nb_conv_i64(None, None, None, 0, 8, 8, 1, 4, 3, 3, 1, 1, 1, 1, 0, None) == 0
    assert lib.nb_sample_from_words_i64(None, None, None, 0, None, 0, 3, 64, None) == 0
    with pytest.raises(RuntimeError, match="negative"):
        _lib.call("nb_unpack_i32", one, one, -2, 1, None)


def test_python_ops_refuse_cpu_tensors():
    import torch
    from nesgpu_amd.extensions import booleanOperations as ops
    x = torch.zeros(4, 64, dtype=torch.bool)
    with pytest.raises(RuntimeError, match="CUDA"):
        ops.pack(x, torch.int64)
    with pytest.raises(AssertionError):
        ops.pack(torch.zeros(4, dtype=torch.bool), torch.int64)          # rank check first, as the reference
    with pytest.raises(TypeError):
        ops._suffix(torch.int8)
    a = torch.zeros(2, 3, 4, dtype=torch.int64)
    with pytest.raises(AssertionError):
        ops.bmm(a, torch.zeros(2, 5, 1, dtype=torch.int64))             # contraction mismatch
    assert ops.next_pow2_clip(9, 512) == 16 and ops.next_pow2_clip(300, 512) == 512 and ops.ceil_div(7, 2) == 4


def test_layer_construction_and_lifecycle_on_cpu():
    import torch
    from nesgpu_amd.modules import binary
    lin = binary.BinarizedLinear(100, 10, 8, device="cpu")
    conv = binary.BinarizedConv2d(16, 32, 8, 3, padding=1, device="cpu")
    pool = binary.BinarizedMaxPool2d()
    assert lin.weight.shape == (10, 100) and lin.weight.dtype == torch.float16 and lin.bias.shape == (10,)
    assert conv.weight.shape == (32 * 9, 16) and conv.kernel_size == (3, 3)
    assert pool.kernel_size == (2, 2) and pool.stride == (2, 2)
    model = torch.nn.Sequential(conv, pool, torch.nn.Flatten(), lin)
    pm = binary.PerturbedModel(model, 8)
    assert pm.perturbed_layers == [conv, lin]
    pm.set_seed(5)
    assert conv.seed == 5 and lin.seed == 5
    pm.free_memory()
    assert lin.weight_noise is None and conv.weight_noise_reshaped is None
    with pytest.raises(NotImplementedError):
        lin(torch.zeros(8, 100, dtype=torch.bool))                        # not in perturbed mode
    with pytest.raises(NotImplementedError):
        binary.BinarizedConv2d(3, 3, 2, 3, dilation=2, device="cpu")
    eb = binary.ExtractBits(torch.int64)
    v = torch.tensor([[5, -1]], dtype=torch.int64)
    bits = eb(v)
    assert bits.shape == (1, 128) and bits[0, :3].tolist() == [True, False, True]
    # (value & mask) > 0 as in the reference (modules/binary.py:29): the sign bit of a signed type never counts
    assert bits[0, 64:127].all() and not bits[0, 127]
    assert binary.ExtractBits(torch.int64, sign_bit=True)(v)[0, 64:].all()
    u8 = binary.ExtractBits(torch.uint8)(torch.tensor([[0x81, 0xFF]], dtype=torch.uint8))
    assert u8.shape == (1, 16) and u8[0].tolist() == [True] + [False] * 6 + [True] + [True] * 8
