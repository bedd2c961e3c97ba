"""Builds tmq_amd/tmq_hip_ext.so: the PyTorch extension (torch_ext.cpp) that exposes the reference's
binding names over libtmq_hip.so. One g++ command; libtmq_hip.so must have been built first
(`make -C tmq_amd/csrc`).

    python3 tmq_amd/csrc/build_ext.py
"""
import os
import subprocess
import sys
import sysconfig


def main():
    import torch
    from torch.utils import cpp_extension as ce
    here = os.path.dirname(os.path.abspath(__file__))
    pkg = os.path.dirname(here)
    root = os.path.dirname(pkg)
    out = os.path.join(pkg, "tmq_hip_ext.so")
    lib_dir = os.path.join(os.path.dirname(torch.__file__), "lib")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["g++", "-O2", "-shared", "-fPIC", "-std=c++17", "-w", "-DTORCH_EXTENSION_NAME=tmq_hip_ext",
           "-DTORCH_API_INCLUDE_EXTENSION_H", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    for inc in ce.include_paths() + [sysconfig.get_paths()["include"], os.path.join(rocm, "include")]:
        cmd += ["-isystem", inc]
    cmd += ["-I", os.path.join(root, "include"), os.path.join(here, "torch_ext.cpp"), "-o", out,
            f"-L{pkg}", "-ltmq_hip", f"-L{lib_dir}", "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_hip",
            "-ltorch_python", f"-L{os.path.join(rocm, 'lib')}", "-lamdhip64",
            "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{lib_dir}", f"-Wl,-rpath,{os.path.join(rocm, 'lib')}"]
    print("+", " ".join(cmd), flush=True)
    return subprocess.call(cmd)


if __name__ == "__main__":
    sys.exit(main())
