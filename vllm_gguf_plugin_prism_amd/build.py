"""Build libgguf_hip.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

``python -m vllm_gguf_plugin_prism_amd.build`` compiles every ``csrc/*.hip`` and
links them into ``vllm_gguf_plugin_prism_amd/libgguf_hip.so``.  hipcc cross-compiles,
so no GPU is needed.  The grid-code header is regenerated from ``tables/`` first.
"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB = PKG / "libgguf_hip.so"
PROBES_SRC = CSRC / "probes" / "probes.hip"      # measurement probes for bench.py, a library of their own
PROBES_LIB = PKG / "libgguf_probes.so"
TORCH_BINDING_SRC = CSRC / "torch_binding" / "gguf_torch_ops.cpp"   # torch.ops._C_gguf.* compiled (host code)
TORCH_BINDING_LIB = PKG / "_C_gguf_native.so"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 VALU forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _compile(src: Path, obj: Path) -> None:
    cmd = [HIPCC, *FLAGS, "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if "is not a recognized feature" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{err}")


def build_torch_binding() -> Path:
    """The compiled torch operator library over the C ABI (csrc/torch_binding): host code only, built with the C++
    compiler against the headers of the torch that is installed, linked against libgguf_hip.so beside it."""
    import torch
    from torch.utils import cpp_extension

    cxx = os.environ.get("CXX", "g++")
    tmp = TORCH_BINDING_LIB.with_suffix(".so.tmp")
    torch_lib = Path(torch.__file__).resolve().parent / "lib"
    cmd = [cxx, "-std=c++17", "-O2", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           *[f"-I{d}" for d in cpp_extension.include_paths()], "-I/opt/rocm/include", f"-I{PKG.parent / 'include'}",
           str(TORCH_BINDING_SRC), "-o", str(tmp), f"-L{torch_lib}", "-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_hip", "-lc10_hip",
           f"-L{PKG}", "-lgguf_hip", "-Wl,-rpath,$ORIGIN"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("the torch binding failed to build:\n" + res.stderr)
    os.replace(tmp, TORCH_BINDING_LIB)
    return TORCH_BINDING_LIB


def build(verbose: bool = True) -> Path:
    from .tables import grids

    header = CSRC / "grid_codes.h"
    text = grids.emit_c_header()
    if not header.exists() or header.read_text() != text:
        header.write_text(text)
    objdir = PKG / "build"
    objdir.mkdir(exist_ok=True)
    srcs = sorted(CSRC.glob("*.hip"))
    objs = [objdir / (s.stem + ".o") for s in srcs]
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        list(pool.map(_compile, srcs, objs))
    tmp = LIB.with_suffix(".so.tmp")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stderr)
    os.replace(tmp, LIB)
    probes_obj = objdir / "probes.o"
    _compile(PROBES_SRC, probes_obj)
    tmp = PROBES_LIB.with_suffix(".so.tmp")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", str(probes_obj), "-o", str(tmp)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link of the probe library failed:\n" + res.stderr)
    os.replace(tmp, PROBES_LIB)
    build_torch_binding()
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources", file=sys.stderr)
    return LIB


if __name__ == "__main__":
    build()
