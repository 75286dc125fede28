"""Writes tests/golden/philox_vectors.json: outputs of torch's own host-callable
Philox engine (at::Philox4_32, ATen/core/PhiloxRNGEngine.h, a header of the
installed torch, not of the reference) for a list of (seed, subsequence,
offset-in-blocks) triples, next to the outputs of this library's
csrc/philox.h::dropout_draw for the matching (seed, offset = 4*blocks, group).
The two columns are asserted equal here; the fixture then pins the numpy
restatement in oracle/oslo_oracle.py without a compiler.

    python tests/golden/make_philox_vectors.py
"""

import json
import os
import subprocess
import tempfile

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))

CASES = [
    (0, 0, 0), (1234, 0, 0), (1234, 1, 0), (1234, 0, 1), (1234, 7, 3),
    (0xDEADBEEFCAFEF00D, 0x1_0000_0005, 0x2_0000_0001),
    (67280421310721, 123456789, 987654321),
    (2**64 - 1, 2**64 - 1, 2**62 - 1),
]

SRC = r"""
#include <ATen/core/PhiloxRNGEngine.h>
#include <cstdio>
#include <cstdlib>
#include "philox.h"
int main(int argc, char** argv) {
  for (int i = 1; i + 2 < argc; i += 3) {
    unsigned long long seed = strtoull(argv[i], 0, 10), sub = strtoull(argv[i+1], 0, 10),
                       blk = strtoull(argv[i+2], 0, 10);
    at::Philox4_32 e(seed, sub, blk);
    unsigned a[4]; for (int j = 0; j < 4; ++j) a[j] = e();
    oslo::Philox4 d = oslo::dropout_draw(seed, blk * 4ull, sub);
    printf("%u %u %u %u %u %u %u %u\n", a[0], a[1], a[2], a[3], d.w[0], d.w[1], d.w[2], d.w[3]);
  }
}
"""


def main():
    inc = os.path.join(os.path.dirname(torch.__file__), "include")
    with tempfile.TemporaryDirectory() as tmp:
        src = os.path.join(tmp, "v.cpp")
        exe = os.path.join(tmp, "v")
        open(src, "w").write(SRC)
        subprocess.check_call(["g++", "-std=c++17", "-O1", f"-I{inc}",
                               f"-I{os.path.join(ROOT, 'oslo_amd', 'csrc')}", src, "-o", exe])
        args = [str(v) for case in CASES for v in case]
        out = subprocess.check_output([exe, *args], text=True)
    vectors = []
    for case, line in zip(CASES, out.strip().splitlines()):
        w = [int(t) for t in line.split()]
        assert w[:4] == w[4:], (case, w)  # at::Philox4_32 == csrc/philox.h on the host
        vectors.append({"seed": case[0], "group": case[1], "offset": case[2] * 4, "words": w[:4]})
    path = os.path.join(HERE, "philox_vectors.json")
    json.dump({"source": "at::Philox4_32 (torch %s), checked equal to csrc/philox.h" % torch.__version__,
               "vectors": vectors}, open(path, "w"), indent=1)
    print("wrote", path)


if __name__ == "__main__":
    main()
