"""Builds flute_extended/_C_native (csrc/torch_binding.cpp) against this interpreter's torch.

Host C++ only (no device code, no hipify): g++ with torch's headers, linked to
libflute_hip.so next to it, libc10_hip for the current-stream query and torch_python for
the tensor casters.  The result lands in ../flute_extended/ so that it ships with the tree.
usage: python build_torch_binding.py
"""
import os
import subprocess
import sys
import sysconfig


def build() -> str:
    import torch
    from torch.utils import cpp_extension as ce

    here = os.path.dirname(os.path.abspath(__file__))
    pkg = os.path.dirname(here)
    root = os.path.dirname(pkg)
    out = os.path.join(pkg, "flute_extended", "_C_native" + sysconfig.get_config_var("EXT_SUFFIX"))
    rocm = ce.ROCM_HOME or "/opt/rocm"
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_C_native",
           "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    for name in ("COMPILER_TYPE", "STDLIB", "BUILD_ABI"):
        val = getattr(torch._C, f"_PYBIND11_{name}", None)
        if val is not None:
            cmd.append(f'-DPYBIND11_{name}="{val}"')
    for inc in ce.include_paths() + [sysconfig.get_paths()["include"], os.path.join(rocm, "include"),
                                     os.path.join(root, "include")]:
        cmd += ["-isystem" if "torch" in inc or "rocm" in inc else "-I", inc]
    cmd += [os.path.join(here, "torch_binding.cpp"), "-o", out,
            "-L" + torch_lib, "-L" + os.path.join(pkg, "lib"),
            "-lflute_hip", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch", "-ltorch_python",
            "-Wl,-rpath,$ORIGIN/../lib", "-Wl,-rpath," + torch_lib]
    subprocess.run(cmd, check=True)
    return out


if __name__ == "__main__":
    print(build())
