"""Helpers shared by CPU and GPU tests to read the committed fixtures in tests/golden/."""
import json
import os

import numpy as np

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load_ops():
    return np.load(os.path.join(GOLDEN_DIR, "ops_small.npz"), allow_pickle=False)


def load_philox():
    with open(os.path.join(GOLDEN_DIR, "philox_rocrand.json")) as f:
        return json.load(f)


TAGS = {"i64": np.int64, "i32": np.int32}
BMM_CASES = ["a", "b", "c"]
CONV_CASES = ["k3p1s1", "k1p0s1", "k7p2s3", "k3p2s2", "k3p0s1"]
POOL_CASES = ["s2", "odd", "pad", "k3"]
SMP_CASES = ["w64", "rag", "big"]
PACK_WIDTHS = [1, 3, 63, 64, 65, 200]


def torch_mean_fp16(sums, out_elems, in_elems):
    """What torch's fp16 ``mean`` gives on the GPU for exact integer sums up to 2**24 in magnitude: the fp32 sum times
    the fp32 quotient float32(out_elems) / float32(in_elems) of the result's and the input's element counts, the exact
    product rounded ONCE, to fp16 (no intermediate rounding to fp32; a double holds the product of two floats exactly,
    and numpy rounds a double to fp16 directly)."""
    factor = np.float32(out_elems) / np.float32(in_elems)
    return (np.asarray(sums).astype(np.float32).astype(np.float64) * np.float64(factor)).astype(np.float16)
