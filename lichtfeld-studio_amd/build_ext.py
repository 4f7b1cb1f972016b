"""Build gsx_torch_ext.so: the C++ host layer (csrc/host/gsplat_ops.cpp: the at::Tensor functions of gsplat/Ops.h;
csrc/host/fastgs_api.cpp: fast_gs::rasterization::forward_wrapper / backward_wrapper; both over the C ABI) plus its pybind11 module, in-tree, linked against libgsx.so (rpath $ORIGIN) and LibTorch.

    python build_ext.py

Host code only: g++ compiles it; the kernels live in libgsx.so (build.py).
"""
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
HOST = os.path.join(HERE, "csrc", "host")
OBJ = os.path.join(HERE, "build")
OUT = os.path.join(HERE, "gsx_torch_ext.so")
CXX = os.environ.get("CXX", "g++")


def _flags():
    import pybind11
    import torch
    from torch.utils import cpp_extension as ce
    inc = [*ce.include_paths("cuda"), pybind11.get_include(), sysconfig.get_paths()["include"],
           os.path.join(ROOT, "include")]
    cflags = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-Wno-deprecated-declarations", "-Wno-attributes",
              "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=gsx_torch_ext",
              f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
              *[f"-I{p}" for p in inc]]
    libdirs = [p for p in ce.library_paths("cuda") if os.path.isdir(p)]
    ldflags = ["-shared", *[f"-L{p}" for p in libdirs], f"-L{HERE}", "-lgsx", "-lc10", "-lc10_hip", "-ltorch_cpu",
               "-ltorch_hip", "-ltorch", "-ltorch_python", "-lamdhip64",
               "-Wl,-rpath,$ORIGIN", *[f"-Wl,-rpath,{p}" for p in libdirs]]
    return cflags, ldflags


def _compile(args):
    src, cflags = args
    obj = os.path.join(OBJ, os.path.basename(src) + ".o")
    cmd = [CXX, *cflags, "-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"{' '.join(cmd)}\n{r.stderr}")
    if r.stderr.strip():
        print(r.stderr, file=sys.stderr)
    return obj


def build():
    if not os.path.exists(os.path.join(HERE, "libgsx.so")):
        raise RuntimeError("libgsx.so is missing: run build.py first")
    os.makedirs(OBJ, exist_ok=True)
    cflags, ldflags = _flags()
    srcs = [os.path.join(HOST, "gsplat_ops.cpp"), os.path.join(HOST, "fastgs_api.cpp"), os.path.join(HOST, "ops_path.cpp"),
            os.path.join(HOST, "train_step.cpp"),
            os.path.join(HOST, "bindings.cpp")]
    with ThreadPoolExecutor(max_workers=5) as ex:
        objs = list(ex.map(_compile, [(s, cflags) for s in srcs]))
    subprocess.run([CXX, *objs, *ldflags, "-o", OUT], check=True)
    return OUT


if __name__ == "__main__":
    print(build())
