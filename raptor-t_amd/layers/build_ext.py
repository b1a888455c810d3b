"""Builds the pybind module `raptor_t` (the layer functors in this directory) in-tree:
`raptor-t_amd/lib/raptor_t*.so`, linked against libraptor_t_hip.so and libtorch.
Plain C++ (no device code): the GPU work is behind the C ABI.

    python raptor-t_amd/layers/build_ext.py [--force]
"""
import os
import subprocess
import sys
import sysconfig

import torch
from torch.utils import cpp_extension as ce

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(os.path.dirname(HERE), "lib")
SRCS = ["tensor_set.cpp", "semaphore.cpp", "metadata.cpp", "kernels.cpp", "multi_headed_attention.cpp",
        "bert_attention.cpp", "bert_intermediate.cpp", "bert_output.cpp", "pybind.cpp"]


def main():
    force = "--force" in sys.argv
    os.makedirs(LIB, exist_ok=True)
    obj_dir = os.path.join(os.path.dirname(HERE), "build", "layers")
    os.makedirs(obj_dir, exist_ok=True)
    target = os.path.join(LIB, "raptor_t" + sysconfig.get_config_var("EXT_SUFFIX"))
    inc = ce.include_paths() + [sysconfig.get_paths()["include"], "/opt/rocm/include"]
    flags = ["-O2", "-std=c++17", "-fPIC", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
             "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
             "-DTORCH_EXTENSION_NAME=raptor_t", "-DTORCH_API_INCLUDE_EXTENSION_H", "-Wno-deprecated-declarations"]
    flags += ["-I" + p for p in inc]
    deps = [os.path.join(HERE, f) for f in os.listdir(HERE) if f.endswith(".h")]
    deps.append(os.path.join(os.path.dirname(os.path.dirname(HERE)), "include", "raptor_t_hip.h"))
    newest_dep = max(os.path.getmtime(d) for d in deps)
    procs, objs = [], []
    for src in SRCS:
        obj = os.path.join(obj_dir, src.replace(".cpp", ".o"))
        objs.append(obj)
        s = os.path.join(HERE, src)
        if force or not os.path.exists(obj) or os.path.getmtime(obj) < max(os.path.getmtime(s), newest_dep):
            procs.append((src, subprocess.Popen(["g++"] + flags + ["-c", s, "-o", obj])))
    for src, p in procs:
        if p.wait() != 0:
            raise SystemExit("compiling %s failed" % src)
    tlib = ce.library_paths()[0]
    cmd = ["g++", "-shared", "-o", target] + objs + [
        "-L" + LIB, "-lraptor_t_hip", "-L" + tlib, "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip",
        "-ltorch_python", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + tlib]
    subprocess.check_call(cmd)
    print("built", target)


if __name__ == "__main__":
    main()
