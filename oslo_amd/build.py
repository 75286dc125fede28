"""Builds ``liboslo_amd.so`` (the C-ABI kernel library) in-tree with hipcc.

Takes the place of the reference's JIT builder
(oslo/fused_kernels_utils.py:53-216), which drives nvcc through
``torch.utils.cpp_extension.load`` at first use. Here the library is built
ahead of time for gfx950 only and loaded with ctypes; nothing is compiled when
a model runs.

    python -m oslo_amd.build

Environment variables make a second build for measurements without touching
the one in the tree: ``OSLO_AMD_LIB=/some/where/lib.so`` is where the library
is written (and where ``oslo_amd._lib`` then loads it from);
``OSLO_BWD_COMBINED_MAX_DIM=256`` compiles the attention backward with dK and
dV in one pass at head_dim 256 as well (it spills there; the default, 128, is
what measures fastest); ``OSLO_STORED_WAVES=4`` and ``OSLO_STORED_BUFFERS=5``
give the pass of that backward that reads the tile store blocks of 128 keys
instead of 256, and five tiles per tensor in LDS instead of three.
"""

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
_VARIANT = os.environ.get("OSLO_AMD_LIB")
LIB_PATH = _VARIANT or os.path.join(os.path.dirname(os.path.abspath(__file__)), "liboslo_amd.so")
OBJ_DIR = (_VARIANT + ".objs") if _VARIANT else os.path.join(CSRC, "build")

SOURCES = [
    "runtime.hip",
    "softmax_causal.hip",
    "softmax_masked.hip",
    "softmax_window.hip",
    "bias_gelu.hip",
    "bias_dropout_add.hip",
    "ngram_repeat_block.hip",
    "rotary.hip",
    "linear_rows.hip",
    "attention_decode.hip",
    "attention_prefill.hip",
    "attention_prefill_bwd.hip",
    "dataset_index.hip",
]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -ffp-contract=off: products and sums are rounded separately unless the source
# asks for an fma, so results do not depend on what the optimiser fuses.
# packed-fp32-ops is switched off: v_pk_*_f32 forms are not used on this part.
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++20",
    "-fPIC",
    "-ffp-contract=off",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


# The two prompt-attention sources name M0 as clobbered by their hand-written
# loads into LDS (they set it themselves inside the asm statement). M0 is a
# reserved register to the compiler, which says so once per instantiation of
# every such statement, thousands of lines per build; silenced for these two
# files only, so that -Wall stays readable for everything else.
EXTRA_FLAGS = {
    "attention_prefill.hip": ["-Wno-inline-asm"],
    "attention_prefill_bwd.hip": ["-Wno-inline-asm"],
}
if os.environ.get("OSLO_STORED_BUFFERS"):
    EXTRA_FLAGS["attention_prefill_bwd.hip"].append("-DOSLO_STORED_BUFFERS=" + str(int(os.environ["OSLO_STORED_BUFFERS"])))
if os.environ.get("OSLO_STORED_WAVES"):
    EXTRA_FLAGS["attention_prefill_bwd.hip"].append("-DOSLO_STORED_WAVES=" + str(int(os.environ["OSLO_STORED_WAVES"])))
if os.environ.get("OSLO_BWD_COMBINED_MAX_DIM"):
    EXTRA_FLAGS["attention_prefill_bwd.hip"].append(
        "-DOSLO_BWD_COMBINED_MAX_DIM=" + str(int(os.environ["OSLO_BWD_COMBINED_MAX_DIM"])))


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the target feature; drop that
    err = "\n".join(
        line for line in proc.stderr.splitlines()
        if "packed-fp32-ops" not in line and "is not a recognized feature" not in line
    )
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build_library(verbose=True):
    """Compiles every kernel source for gfx950 and links the shared library."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 1)) as pool:
        objs = list(pool.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build_library()
