"""Writes tests/golden/ops_small.npz: seeded inputs and expected outputs for every op on the
path, computed ONLY with the unpacked numpy / torch-CPU formulation in oracle/unpacked.py
(numpy.packbits, +-1 integer matmul, grouped torch.conv2d with pad value -1, F.max_pool2d:
the ground-truth forms of booloptests.py:94-163).  The reference holds no vectors of its own
for this path, and none of its code is imported or run here.

Both the C oracle (CPU tests) and the HIP kernels (GPU tests) are compared with this file.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import unpacked as U  # noqa: E402


def main():
    g = np.random.default_rng(20240)
    out = {}
    for tag, dtype in (("i64", np.int64), ("i32", np.int32)):
        # pack: ragged widths around the word size
        for C in (1, 3, 63, 64, 65, 200):
            bits = g.integers(0, 2, size=(7, C)).astype(bool)
            out[f"pack_{tag}_C{C}_in"] = bits
            out[f"pack_{tag}_C{C}_out"] = U.pack_bits(bits, dtype)
        # bmm / bmm_act: M, N, K not multiples of any tile; N = 1 (linear form) included
        for name, (Z, M, K, N) in {"a": (3, 37, 150, 5), "b": (4, 19, 256, 1), "c": (2, 70, 64, 67)}.items():
            a = g.integers(0, 2, size=(Z, M, K)).astype(bool)
            b = g.integers(0, 2, size=(Z, K, N)).astype(bool)
            A = U.pack_bits(a.reshape(Z * M, K), dtype).reshape(Z, M, -1)
            B = np.ascontiguousarray(
                U.pack_bits(b.transpose(0, 2, 1).reshape(Z * N, K), dtype).reshape(Z, N, -1).transpose(0, 2, 1))
            popc = U.popc_bmm_bits(a, b)
            thr = (g.integers(0, K, size=(Z, N)) + K // 2).astype(np.int32)
            out[f"bmm_{tag}_{name}_A"] = A
            out[f"bmm_{tag}_{name}_B"] = B
            out[f"bmm_{tag}_{name}_C"] = popc
            out[f"bmm_{tag}_{name}_thr"] = thr
            out[f"bmm_{tag}_{name}_act"] = 2 * popc > thr[:, None, :]
        # conv / conv_act / im2col: a slice of the reference sweep plus odd channel counts
        for name, (D, S, C, O, fs, pad, st) in {
            "k3p1s1": (3, 10, 16, 5, 3, 1, 1), "k1p0s1": (2, 10, 1, 64, 1, 0, 1), "k7p2s3": (2, 10, 3, 4, 7, 2, 3),
            "k3p2s2": (2, 9, 70, 6, 3, 2, 2), "k3p0s1": (2, 8, 64, 64, 3, 0, 1),
        }.items():
            xb = g.integers(0, 2, size=(D, S, S, C)).astype(bool)
            fb = g.integers(0, 2, size=(D, O, fs, fs, C)).astype(bool)
            xp = U.pack_bits(xb.reshape(-1, C), dtype).reshape(D, S, S, -1)
            fp = U.pack_bits(fb.reshape(-1, C), dtype).reshape(D, O, fs, fs, -1)
            fr = np.ascontiguousarray(fp.transpose(0, 2, 3, 4, 1).reshape(D, -1, O))
            popc = U.conv_popc_torch(xb, fb, pad, st)
            K = fs * fs * C
            thr = (g.integers(0, K, size=(D, O)) - K // 2 + K).astype(np.int32)
            cols = U.im2col_bits(xb, fs, fs, pad, pad, st, st)
            colsp = U.pack_bits(cols.reshape(-1, C), dtype).reshape(D, cols.shape[1], -1)
            out[f"conv_{tag}_{name}_x"] = xp
            out[f"conv_{tag}_{name}_f"] = fr
            out[f"conv_{tag}_{name}_popc"] = popc
            out[f"conv_{tag}_{name}_thr"] = thr
            out[f"conv_{tag}_{name}_act"] = 2 * popc > thr[:, None, None, :]
            out[f"conv_{tag}_{name}_cols"] = colsp
            out[f"conv_{tag}_{name}_geom"] = np.array([fs, fs, pad, pad, st, st], dtype=np.int32)
        # max pool: the reference's 2x2/s2 case via F.max_pool2d, padded cases via the OR window
        for name, (B, S, C, geom) in {
            "s2": (3, 10, 16, (2, 2, 0, 0, 2, 2)), "odd": (2, 7, 100, (2, 2, 0, 0, 2, 2)),
            "pad": (2, 8, 5, (2, 2, 1, 1, 2, 2)), "k3": (2, 9, 64, (3, 3, 1, 0, 2, 1)),
        }.items():
            xb = g.integers(0, 2, size=(B, S, S, C)).astype(bool)
            xp = U.pack_bits(xb.reshape(-1, C), dtype).reshape(B, S, S, -1)
            if name in ("s2", "odd"):
                pooled = U.max_pool_bits_torch(xb)
            else:
                pooled = U.or_pool2x2_bits(xb, *geom)
            out[f"pool_{tag}_{name}_x"] = xp
            out[f"pool_{tag}_{name}_geom"] = np.array(geom, dtype=np.int32)
            out[f"pool_{tag}_{name}_out"] = U.pack_bits(pooled.reshape(-1, C), dtype).reshape(*pooled.shape[:3], -1)
        # threshold sampling from supplied words, flip form and fused matrix-vector product
        for name, (n, R, C) in {"w64": (3, 4, 64), "rag": (4, 5, 100), "big": (2, 3, 512)}.items():
            words = g.integers(0, 2 ** 32, size=(n, R, C), dtype=np.uint64).astype(np.uint32)
            thr = g.integers(0, 2 ** 32, size=(R, C), dtype=np.uint64).astype(np.uint32)
            T = 214748364
            baseb = g.integers(0, 2, size=(R, C)).astype(bool)
            xb = g.integers(0, 2, size=(n, C)).astype(bool)
            smp = (words < thr[None])
            flp = (words < T) ^ baseb[None]
            out[f"smp_{tag}_{name}_words"] = words
            out[f"smp_{tag}_{name}_thr"] = thr
            out[f"smp_{tag}_{name}_base"] = U.pack_bits(baseb, dtype)
            out[f"smp_{tag}_{name}_x"] = U.pack_bits(xb, dtype)
            out[f"smp_{tag}_{name}_sample"] = U.pack_bits(smp.reshape(n * R, C), dtype).reshape(n, R, -1)
            out[f"smp_{tag}_{name}_flip"] = U.pack_bits(flp.reshape(n * R, C), dtype).reshape(n, R, -1)
            out[f"smp_{tag}_{name}_bmv_sample"] = (smp != xb[:, None, :]).sum(2).astype(np.int32)
            out[f"smp_{tag}_{name}_bmv_flip"] = (flp != xb[:, None, :]).sum(2).astype(np.int32)
    np.savez_compressed(os.path.join(HERE, "ops_small.npz"), **out)
    print(len(out), "arrays")


if __name__ == "__main__":
    main()
