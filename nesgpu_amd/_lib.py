"""ctypes binding of libnesbin.so (the C ABI declared in include/nesbin.h).

The library is loaded lazily on first use and there is no fallback: if it has not been built
(`python -c "import __graft_entry__ as g; g.build()"` or `make -C nesgpu_amd/csrc`) every op
raises ``RuntimeError``.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnesbin.so")
_lib = None

NB_OK = 0
NB_ERR_HIP_BASE = 1000

_I64, _I32, _U32, _U64, _PTR = ctypes.c_int64, ctypes.c_int, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_void_p
_GEOM = [_I32] * 6

# name -> argument types (without the `_i64`/`_i32` suffix expansion); every entry returns int
_SUFFIXED = {
    "nb_pack": [_PTR, _PTR, _I64, _I64, _PTR],
    "nb_unpack": [_PTR, _PTR, _I64, _I64, _PTR],
    "nb_int8pack": [_PTR, _PTR, _I64, _I64, _PTR],
    "nb_bmm": [_PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _PTR],
    "nb_bmv_pm1": [_PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _PTR],
    "nb_bmm_act": [_PTR, _PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _PTR],
    "nb_bmv_act_pack": [_PTR, _PTR, _PTR, _PTR, _I64, _I64, _I64, _PTR],
    "nb_im2col": [_PTR, _PTR, _I64, _I64, _I64, _I64] + _GEOM + [_PTR],
    "nb_conv": [_PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _I64] + _GEOM + [_I32, _PTR],
    "nb_conv_popc_sums": [_PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _I64] + _GEOM + [_I32, _PTR],
    "nb_conv_bn_thresholds_from_input": [_PTR, _PTR, _PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _I64] + _GEOM
                                        + [_I32, _I64, _PTR],
    "nb_conv_act": [_PTR, _PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _I64] + _GEOM + [_I32, _PTR],
    "nb_conv_act_pack": [_PTR, _PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _I64] + _GEOM + [_I32, _I32, _PTR],
    "nb_tap_pack_filter": [_PTR, _PTR, _I64, _I64, _I64, _I32, _PTR],
    "nb_max_pool2d": [_PTR, _PTR, _I64, _I64, _I64, _I64] + _GEOM + [_PTR],
    "nb_sample_from_words": [_PTR, _PTR, _PTR, _U32, _PTR, _I64, _I64, _I64, _PTR],
    "nb_sample_philox": [_PTR, _PTR, _PTR, _U32, _U64, _U64, _U64, _I64, _I64, _I64, _PTR],
    "nb_sample_philox16": [_PTR, _PTR, _PTR, _U32, _U64, _U64, _U64, _I64, _I64, _I64, _PTR],
    "nb_sample_conv_philox16": [_PTR, _PTR, _PTR, _PTR, _U32, _U64, _U64, _U64, _I64, _I64, _I64, _I64, _PTR],
    "nb_sample_conv_from_words": [_PTR, _PTR, _PTR, _PTR, _U32, _PTR, _I64, _I64, _I64, _I64, _PTR],
    "nb_sample_conv_philox": [_PTR, _PTR, _PTR, _PTR, _U32, _U64, _U64, _U64, _I64, _I64, _I64, _I64, _PTR],
    "nb_seeded_bmv_from_words": [_PTR, _PTR, _PTR, _U32, _PTR, _PTR, _I64, _I64, _I64, _PTR],
    "nb_seeded_bmv_philox": [_PTR, _PTR, _PTR, _U32, _PTR, _U64, _U64, _U64, _I64, _I64, _I64, _PTR],
    "nb_seeded_bmv_philox16": [_PTR, _PTR, _PTR, _U32, _PTR, _U64, _U64, _U64, _I64, _I64, _I64, _PTR],
    "nb_sample_skip": [_PTR, _PTR, _PTR, _U64, _U64, _U64, _I64, _I64, _I64, _PTR],
    "nb_sample_conv_skip": [_PTR, _PTR, _PTR, _PTR, _U64, _U64, _U64, _I64, _I64, _I64, _I64, _PTR],
    "nb_weighted_sum": [_PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _PTR],
    "nb_weighted_sum_fast": [_PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _PTR],
    "nb_bmv_bn_act": [_PTR, _PTR, _PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _I32, _PTR, _I64, _PTR],
}
_PLAIN = {
    "nb_philox_words": [_PTR, _U64, _U64, _U64, _I64, _PTR],
    "nb_thresholds_from_p": [_PTR, _PTR, _I64, _PTR],
    "nb_conv_engine": [_I32],
    "nb_conv_last_engine": [],
    "nb_flip_count_i64": [_PTR, _PTR, _PTR, _I64, _I64, _I64, _PTR],
    "nb_flip_fill_i64": [_PTR, _PTR, _PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _PTR],
    "nb_flip_to_dense_i64": [_PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _PTR],
    "nb_skip_table": [_PTR, _PTR, _PTR],
    "nb_flip_skip_i64": [_PTR, _PTR, _PTR, _PTR, _PTR, _U64, _U64, _U64, _I64, _I64, _I64, _I64, _PTR],
    "nb_flip_skip_thin_i64": [_PTR, _PTR, _PTR, _PTR, _PTR, _U64, _U64, _U64, _I64, _I64, _I64, _I64, _PTR],
    "nb_flip_law_stats": [_PTR, _PTR, _PTR, _PTR, _I64, _I64, _PTR],
    "nb_flip_layer_tables": [_PTR, _PTR],
    "nb_flip_law_layers": [_PTR, _PTR, _PTR, _I64, _I64, _PTR],
    "nb_flip_skip_layered_i64": [_PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _U64, _U64, _U64, _I64, _I64, _I64, _I64, _PTR],
    "nb_thresholds_from_weights": [_PTR, _PTR, _I64, _PTR, _PTR],
    "nb_probabilities_from_weights": [_PTR, _PTR, _I64, _PTR, _PTR],
    "nb_flip_law_from_weights": [_PTR, _PTR, _PTR, _PTR, _I64, _I64, _PTR, _PTR],
    "nb_expand_fp4_i64": [_PTR, _PTR, _I64, _I64, _I64, _I64, _PTR],
    "nb_bmm_nt_fp4": [_PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _I64, _I64, _PTR],
    "nb_bmv_flip_i64": [_PTR, _PTR, _PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _PTR],
    "nb_bmv_flip_act_pack_i64": [_PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _PTR],
    "nb_flip_weighted_sum_i64": [_PTR, _PTR, _PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _PTR],
    "nb_bmv_bn_act_static_i64": [_PTR, _PTR, _PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _I32, _PTR],
    "nb_conv_bn_thresholds": [_PTR, _PTR, _PTR, _PTR, _I64, _I64, _I64, _I64, _PTR],
    "nb_center_fitness_f16": [_PTR, _PTR, _I64, _PTR],
    "nb_center_fitness_f32": [_PTR, _PTR, _I64, _PTR],
    "nb_grad_regularize": [_PTR, _PTR, ctypes.c_float, ctypes.c_float, _I64, _PTR],
    "nb_bias_grad": [_PTR, _PTR, _PTR, _I64, _I64, _PTR],
    "nb_bias_noise_scale": [_PTR, _I64, _PTR],
}
# entry points that return a size (int64) instead of a status
_SIZES = {
    "nb_bmv_bn_workspace_bytes": [_I64, _I64],
    "nb_bmv_bn_static_bytes": [],
    "nb_skip_table_words": [],
    "nb_flip_layer_table_words": [],
    "nb_law_workspace_bytes": [],
}


def exported_symbols():
    """Every symbol include/nesbin.h declares."""
    names = ["nb_version", "nb_last_error_string"] + list(_PLAIN) + list(_SIZES)
    for base in _SUFFIXED:
        names += [base + "_i64", base + "_i32"]
    return names


def load():
    global _lib
    if _lib is not None:
        return _lib
    path = os.environ.get("NESBIN_LIB", LIB_PATH)
    if not os.path.exists(path):
        raise RuntimeError(
            "libnesbin.so is not built (looked at %s); run `make -C nesgpu_amd/csrc` or "
            "`python -c 'import __graft_entry__ as g; g.build()'`. There is no CPU fallback." % path)
    lib = ctypes.CDLL(path)
    lib.nb_version.restype = ctypes.c_int
    lib.nb_version.argtypes = []
    lib.nb_last_error_string.restype = ctypes.c_char_p
    lib.nb_last_error_string.argtypes = []
    for base, args in _SUFFIXED.items():
        for suf in ("_i64", "_i32"):
            fn = getattr(lib, base + suf)
            fn.restype = ctypes.c_int
            fn.argtypes = args
    for name, args in _PLAIN.items():
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int
        fn.argtypes = args
    for name, args in _SIZES.items():
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int64
        fn.argtypes = args
    _lib = lib
    return lib


_fns = {}


def call(name, *args):
    """Call an entry point and turn a non-zero status into RuntimeError."""
    fn = _fns.get(name)
    if fn is None:
        fn = _fns[name] = getattr(load(), name)
    rc = fn(*args)
    if rc != NB_OK:
        msg = load().nb_last_error_string().decode("utf-8", "replace")
        raise RuntimeError("%s failed with status %d: %s" % (name, rc, msg))
