"""Writes tests/golden/philox_rocrand.json: Philox4x32-10 words produced by rocRAND's own
host-callable engine (/opt/rocm/include/rocrand/rocrand_philox4x32_10.h, a system header, not
part of the reference) for a few (seed, subsequence, offset) triples.  The fixture pins the
generator-mode word stream independently of this repository's implementations.

Run from the repository root:  python tests/golden/make_philox_golden.py
"""
import json
import os
import subprocess
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))

CASES = [  # (seed, subsequence, offset, count)
    (0, 0, 0, 16),
    (0x123456789ABCDEF, 5, 0, 16),
    (42, 0xFFFFFFFF, 4 * 0xFFFFFFFF, 12),          # counter word 0 about to wrap into word 1
    (0xDEADBEEFCAFEF00D, 0x100000003, 6, 13),      # unaligned offset, subsequence above 32 bits
    (7, 1, 1023, 9),
]

SRC = r"""
#include <hip/hip_runtime.h>
#include <rocrand/rocrand_philox4x32_10.h>
#include <cstdio>
#include <cstdlib>
int main(int argc, char** argv) {
    unsigned long long seed = strtoull(argv[1], 0, 0), sub = strtoull(argv[2], 0, 0), off = strtoull(argv[3], 0, 0);
    int n = atoi(argv[4]);
    rocrand_state_philox4x32_10 st;
    rocrand_init(seed, sub, off, &st);
    for (int i = 0; i < n; i++) printf("%u\n", rocrand(&st));
    return 0;
}
"""


def main():
    out = []
    with tempfile.TemporaryDirectory() as td:
        src = os.path.join(td, "g.cpp")
        exe = os.path.join(td, "g")
        with open(src, "w") as f:
            f.write(SRC)
        subprocess.check_call(["hipcc", "-O1", src, "-o", exe])
        for seed, sub, off, n in CASES:
            txt = subprocess.check_output([exe, str(seed), str(sub), str(off), str(n)], text=True)
            out.append({"seed": seed, "subsequence": sub, "offset": off,
                        "words": [int(t) for t in txt.split()]})
    # Random123 known-answer vectors for philox4x32-10 (kat_vectors of the Random123
    # distribution, D. E. Shaw Research): (counter[4], key[2]) -> out[4].
    kat = [
        {"ctr": [0, 0, 0, 0], "key": [0, 0],
         "out": [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]},
        {"ctr": [0xFFFFFFFF] * 4, "key": [0xFFFFFFFF] * 2,
         "out": [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]},
        {"ctr": [0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], "key": [0xA4093822, 0x299F31D0],
         "out": [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]},
    ]
    with open(os.path.join(HERE, "philox_rocrand.json"), "w") as f:
        json.dump({"rocrand": out, "random123_kat": kat}, f, indent=1)


if __name__ == "__main__":
    main()
