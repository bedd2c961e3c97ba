"""Compiles the reference's own host codec / packer (tmq/tmq_native.cpp with rangecoder.h and
bitstream.h) from the sources where they lie in the reference tree into oracle/_ref/ -- a
checker for the tests. The built library is kept out of version control; it travels to a GPU machine
with the rest of the tree like the library's own binaries, where only the tests may load it (they run
from the committed fixtures when it is absent). One g++ command on the reference's own
file; the reference's build system is not run. The CUDA file needs nvcc and is not buildable
in this image.

    python3 oracle/build_ref.py /root/reference
"""
import os
import subprocess
import sys
import sysconfig


def main(ref):
    src = os.path.join(ref, "tmq", "tmq_native.cpp")
    if not os.path.exists(src):
        print("reference source not found:", src)
        return 0
    import torch
    from torch.utils import cpp_extension as ce
    here = os.path.dirname(os.path.abspath(__file__))
    out_dir = os.path.join(here, "_ref")
    os.makedirs(out_dir, exist_ok=True)
    out = os.path.join(out_dir, "tmq_native.so")
    lib_dir = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-shared", "-fPIC", "-std=c++17", "-w", "-DTORCH_EXTENSION_NAME=tmq_native",
           "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    for inc in ce.include_paths() + [sysconfig.get_paths()["include"]]:
        cmd += ["-isystem", inc]
    cmd += [src, "-o", out, f"-L{lib_dir}", "-lc10", "-ltorch", "-ltorch_cpu", "-ltorch_python",
            f"-Wl,-rpath,{lib_dir}"]
    print("+", " ".join(cmd), flush=True)
    return subprocess.call(cmd)


if __name__ == "__main__":
    sys.exit(main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference"))
