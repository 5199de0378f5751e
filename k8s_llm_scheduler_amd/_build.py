"""Build the native extension ``k8s_llm_scheduler_amd/ops/_C*.so`` for gfx950.

Plain ``hipcc`` invocations (no hipify, no torch.utils.cpp_extension JIT cache): every ``.hip``
kernel file is compiled with ``--offload-arch=gfx950``, the runtime ``.cpp`` files and the
pybind11 bindings are host code, and only ``torch_stream.cpp`` sees PyTorch headers (to pick up
the current PyTorch HIP stream).  Objects are cached under ``build/`` and rebuilt when a source
or any header is newer.  Cross-compiles without a GPU.

    python -m k8s_llm_scheduler_amd._build [-j N] [--force] [-v] [--checked]

``--lean`` builds ``ops/_C_lean*.so`` (``-DK8S_LEAN``, objects under ``build/native_lean``): the runtime, the sampler and
the kernels of the fp32-stream model designs only -- what a fresh checkout compiles before it replays a trace of such a
model; it is loaded when the full module is absent, and every matrix product then runs on the any-shape GEMM.

``--checked`` builds the bounds-checked variant ``ops/_C_checked*.so`` (``-DK8S_CHECKED``, objects under
``build/native_checked``; loaded instead of ``_C`` when ``K8S_CHECKED=1``): kernels range-check every index they
derive from data and record violations for the host (csrc/kernels/common.h).
"""

from __future__ import annotations

import argparse
import concurrent.futures as cf
import os
import subprocess
import sys
import sysconfig
from pathlib import Path
from typing import List

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
BUILD = PKG.parent / "build" / "native"
ARCH = os.environ.get("K8S_HIP_ARCH", "gfx950")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# Kernels added since the packed-fp32 rule are built without the packed fp32 instructions (v_pk_add/mul/fma_f32), which
# -O3 otherwise forms from ordinary float code.  The older kernel files keep the flags they were validated with: with
# the option on every file, the two-rank fused GEMV all-reduce check of tests/test_multigpu.py reported a wrong sum.
NO_PACKED_FP32 = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
NO_PACKED_FP32_FILES = {"stream32.hip", "mixers.hip", "moe.hip", "window_attn.hip", "gated_scan.hip", "delta_scan.hip"}
# the lean module: kernels of the fp32-stream designs, the sampler, the small shared kernels; the block allocator
LEAN_KERNELS = NO_PACKED_FP32_FILES | {"sampler.hip", "misc.hip", "norm.hip"}
LEAN_RUNTIME = {"block_allocator.cpp"}


def ext_path(checked: bool = False, lean: bool = False) -> Path:
    name = "_C_lean" if lean else "_C_checked" if checked else "_C"
    return PKG / "ops" / (name + sysconfig.get_config_var("EXT_SUFFIX"))


def _torch_dirs():
    import torch

    root = Path(torch.__file__).resolve().parent
    return root / "include", root / "lib", bool(torch._C._GLIBCXX_USE_CXX11_ABI)


def _headers() -> List[Path]:
    return list(CSRC.rglob("*.h"))


def _stale(obj: Path, src: Path, headers: List[Path]) -> bool:
    if not obj.exists():
        return True
    t = obj.stat().st_mtime
    return src.stat().st_mtime > t or any(h.stat().st_mtime > t for h in headers)


def _run(cmd: List[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"command failed ({r.returncode}): {' '.join(cmd)}\n{r.stdout}\n{r.stderr}")


def build(jobs: int = 0, force: bool = False, verbose: bool = False, checked: bool = False, lean: bool = False) -> Path:
    import pybind11

    if checked and lean:
        raise ValueError("the lean module has no checked variant")
    tinc, tlib, cxx11 = _torch_dirs()
    bdir = BUILD.parent / "native_lean" if lean else BUILD.parent / "native_checked" if checked else BUILD
    bdir.mkdir(parents=True, exist_ok=True)
    headers = _headers()
    common = ["-O3", "-fPIC", "-std=c++17", f"-I{CSRC}", f"-D_GLIBCXX_USE_CXX11_ABI={int(cxx11)}"]
    if checked:
        common += ["-DK8S_CHECKED", "-DK8S_MODULE_NAME=_C_checked"]
    if lean:
        common += ["-DK8S_LEAN", "-DK8S_MODULE_NAME=_C_lean"]
    py_inc = sysconfig.get_paths()["include"]
    units = []
    for src in sorted((CSRC / "kernels").glob("*.hip")):
        if lean and src.name not in LEAN_KERNELS:
            continue
        units.append((src, ["-x", "hip", f"--offload-arch={ARCH}", "-munsafe-fp-atomics",
                            *(NO_PACKED_FP32 if src.name in NO_PACKED_FP32_FILES else [])]))
    for src in sorted((CSRC / "runtime").glob("*.cpp")):
        if lean and src.name not in LEAN_RUNTIME:
            continue
        units.append((src, []))
    units.append((CSRC / "bindings.cpp", [f"-I{pybind11.get_include()}", f"-I{py_inc}", "-fvisibility=hidden"]))
    units.append((CSRC / "torch_stream.cpp", [f"-I{tinc}", f"-I{tinc / 'torch/csrc/api/include'}",
                                               "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-w"]))
    objs = []
    todo = []
    for src, flags in units:
        obj = bdir / (src.relative_to(CSRC).as_posix().replace("/", "__") + ".o")
        objs.append(obj)
        if force or _stale(obj, src, headers):
            todo.append([HIPCC, *common, *flags, "-c", str(src), "-o", str(obj)])
    n = jobs or min(8, os.cpu_count() or 4)
    with cf.ThreadPoolExecutor(max_workers=n) as ex:
        for f in [ex.submit(_run, c, verbose) for c in todo]:
            f.result()
    out = ext_path(checked, lean)
    if todo or force or not out.exists() or any(o.stat().st_mtime > out.stat().st_mtime for o in objs):
        tmp = out.with_suffix(".tmp.so")
        _run([HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", str(tmp), *map(str, objs),
              f"-L{tlib}", "-lc10_hip", "-lc10", *([] if lean else ["-lrccl"]), f"-Wl,-rpath,{tlib}",
              "-Wl,--no-as-needed"], verbose)
        os.replace(tmp, out)
    return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("-j", "--jobs", type=int, default=0)
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-v", "--verbose", action="store_true")
    ap.add_argument("--checked", action="store_true", help="bounds-checked kernels: ops/_C_checked*.so")
    ap.add_argument("--lean", action="store_true", help="runtime + fp32-stream model kernels only: ops/_C_lean*.so")
    a = ap.parse_args(argv)
    p = build(a.jobs, a.force, a.verbose, a.checked, a.lean)
    print(p)
    return 0


if __name__ == "__main__":
    sys.exit(main())
