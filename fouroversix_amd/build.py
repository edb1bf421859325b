"""Build the gfx950 shared library (``libfouroversix_hip.so``) with hipcc, and the PyTorch
binding on top of its C ABI (``_C.so``: host C++ only, compiled with g++).

    python fouroversix_amd/build.py [--force]

(run as a script: importing the package needs the libraries this builds)

hipcc cross-compiles for gfx950 without a GPU.  The flags matter for bit-exactness:
no fp contraction (fused multiply-adds only where the source spells them), correctly
rounded fp32 division, fp32 denormals kept, and no packed-fp32 instructions.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB_PATH = os.path.join(HERE, "libfouroversix_hip.so")
OBJ_DIR = os.path.join(CSRC, "build")

SOURCES = ["fos_common.hip", "fos_quantize.hip", "fos_quantize_fast.hip", "fos_quantize_tiles.hip", "fos_gemm.hip", "fos_dequantize.hip", "fos_transform.hip", "fos_mxfp4.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-fno-gpu-flush-denormals-to-zero",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    f"-I{INCLUDE}",
    f"-I{CSRC}",
]


def _deps(src: str) -> list[str]:
    return [src] + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")] + [
        os.path.join(INCLUDE, f) for f in os.listdir(INCLUDE)
    ]


def _compile(name: str, force: bool) -> str:
    src = os.path.join(CSRC, name)
    obj = os.path.join(OBJ_DIR, name.replace(".hip", ".o"))
    if not force and os.path.exists(obj) and all(os.path.getmtime(obj) >= os.path.getmtime(d) for d in _deps(src)):
        return obj
    cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "packed-fp32-ops"
    err = "\n".join(line for line in res.stderr.splitlines() if noise not in line)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {name}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


BINDING_SRC = os.path.join(CSRC, "torch_ops.cpp")
BINDING_PATH = os.path.join(HERE, "_C.so")
BINDING_OBJ = os.path.join(OBJ_DIR, "torch_ops.o")


def _compile_binding(force: bool) -> str:
    """torch_ops.cpp -> object file (host code only: the operators call the C ABI)."""
    deps = [BINDING_SRC] + [os.path.join(INCLUDE, f) for f in os.listdir(INCLUDE)]
    if not force and os.path.exists(BINDING_OBJ) and all(os.path.getmtime(BINDING_OBJ) >= os.path.getmtime(d) for d in deps):
        return BINDING_OBJ
    import sysconfig

    import torch
    from torch.utils import cpp_extension

    cmd = [
        os.environ.get("CXX", "g++"), "-std=c++17", "-O2", "-fPIC", "-c", BINDING_SRC, "-o", BINDING_OBJ,
        "-DTORCH_EXTENSION_NAME=_C", "-DTORCH_API_INCLUDE_EXTENSION_H", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
        f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
        *[f"-I{p}" for p in cpp_extension.include_paths()], f"-I{sysconfig.get_paths()['include']}",
        "-I/opt/rocm/include", f"-I{INCLUDE}", "-Wno-deprecated-declarations",
    ]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"compiling torch_ops.cpp failed:\n{res.stderr[-4000:]}")
    return BINDING_OBJ


def _link_binding(obj: str, force: bool) -> str:
    if not force and os.path.exists(BINDING_PATH) and os.path.getmtime(BINDING_PATH) >= max(os.path.getmtime(obj), os.path.getmtime(LIB_PATH)):
        return BINDING_PATH
    from torch.utils import cpp_extension

    torch_lib = cpp_extension.library_paths()[0]
    cmd = [
        os.environ.get("CXX", "g++"), "-shared", "-fPIC", "-o", BINDING_PATH, obj,
        f"-L{HERE}", "-l:libfouroversix_hip.so", f"-L{torch_lib}", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip",
        "-ltorch_python", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}",
    ]
    subprocess.run(cmd, check=True)
    return BINDING_PATH


def build(force: bool = False) -> str:
    """Compile every HIP source and link the shared library, then the PyTorch binding; returns the
    library's path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES) + 1)) as pool:
        binding = pool.submit(_compile_binding, force)
        objs = list(pool.map(lambda n: _compile(n, force), SOURCES))
        binding_obj = binding.result()
    if force or not os.path.exists(LIB_PATH) or any(os.path.getmtime(o) > os.path.getmtime(LIB_PATH) for o in objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
        subprocess.run(cmd, check=True)
    _link_binding(binding_obj, force)
    return LIB_PATH


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
