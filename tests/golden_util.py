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
