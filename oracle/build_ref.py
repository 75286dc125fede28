"""Builds the one part of the reference that compiles from its own source file
with the tools in this image: the dataset index builders of
oslo/fused_kernels/bindings/pybind_datasets.cpp (plain C++ with pybind11; the
CUDA kernels need nvcc and are not buildable here). The source is compiled
where it lies; only the extension module lands in oracle/_ref/. Test
infrastructure: nothing under oslo_amd/ imports it.

    python oracle/build_ref.py [/root/reference]
"""

import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
OUT_DIR = os.path.join(HERE, "_ref")
MODULE = "oslo_datasets"


def output_path():
    return os.path.join(OUT_DIR, MODULE + sysconfig.get_config_var("EXT_SUFFIX"))


def build_reference(reference_root="/root/reference"):
    """Returns the path of the built module, or None when the reference's
    sources are not there (the GPU box: the prebuilt file is used)."""
    src_dir = os.path.join(reference_root, "oslo", "fused_kernels")
    src = os.path.join(src_dir, "bindings", "pybind_datasets.cpp")
    if not os.path.exists(src):
        return None
    import torch
    from torch.utils import cpp_extension

    os.makedirs(OUT_DIR, exist_ok=True)
    out = output_path()
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-w",
           f"-DTORCH_EXTENSION_NAME={MODULE}", "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    for inc in cpp_extension.include_paths() + [sysconfig.get_paths()["include"],
                                                os.path.join(src_dir, "includes")]:
        cmd += ["-I", inc]
    cmd += [src, "-o", out, f"-L{torch_lib}", f"-Wl,-rpath,{torch_lib}",
            "-ltorch_python", "-ltorch", "-ltorch_cpu", "-lc10"]
    subprocess.run(cmd, check=True)
    return out


if __name__ == "__main__":
    path = build_reference(*sys.argv[1:2])
    print("built " + path if path else "reference sources not found; nothing built")
