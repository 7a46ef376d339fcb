"""Builds oracle/_ref/: the reference's own host wave buffer, compiled from where it lies.

TEST INFRASTRUCTURE ONLY.  Of the reference's native sources for this path only
library/retroinfer/retroinfer_kernels/src/wave_buffer_cpu.cpp (with thread_pool.hpp) is plain C++
against the torch and pybind11 headers; the other two need nvcc and a CUTLASS checkout and are not
buildable here.  The file is compiled with g++ directly (not through the reference's setup.py) into a
Python extension module that tests/test_wavebuf_ref.py loads to check the block cache restatement
(oracle/wavebuf.py) and the library's host manager against the real thing.  Nothing is copied: the
source stays under the reference tree, only the built module lands in oracle/_ref/ (git-ignored).

Usage: python oracle/build_ref.py [reference root, default /root/reference]
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
OUT_DIR = os.path.join(HERE, "_ref")
MODULE = "WaveBufferRef"
SRC = "library/retroinfer/retroinfer_kernels/src/wave_buffer_cpu.cpp"


def module_path():
    return os.path.join(OUT_DIR, MODULE + sysconfig.get_config_var("EXT_SUFFIX"))


def build(ref_root="/root/reference", verbose=True):
    """Returns the path of the built module, or None when the reference tree is absent."""
    src = os.path.join(ref_root, SRC)
    if not os.path.isfile(src):
        return None
    import torch
    from torch.utils import cpp_extension
    os.makedirs(OUT_DIR, exist_ok=True)
    inc = [p for p in cpp_extension.include_paths() if os.path.isdir(p)] + [sysconfig.get_paths()["include"]]
    lib_dir = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-fopenmp", "-w",
           f"-DTORCH_EXTENSION_NAME={MODULE}", "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    cmd += [f"-I{p}" for p in inc]
    cmd += [src, "-o", module_path(), f"-L{lib_dir}", "-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_python",
            f"-Wl,-rpath,{lib_dir}"]
    if verbose:
        print("[oracle/_ref]", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return module_path()


if __name__ == "__main__":
    p = build(*sys.argv[1:2])
    print(p if p else "reference tree not found: nothing built")
