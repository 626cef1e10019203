"""Build libdiffulex_amd.so (the C-ABI library with the gfx950 kernels) and _torch_ops.so (the
PyTorch operator library that binds it) in-tree.

    python -m diffulex_amd.build

compiles every kernel source under ``csrc/`` with hipcc for gfx950 and links them into
``diffulex_amd/libdiffulex_amd.so``, then compiles ``csrc/torch_ext.cpp`` (host code) against
PyTorch's headers into ``diffulex_amd/_torch_ops.so``, which finds the kernel library next to
itself.  hipcc cross-compiles, so no GPU is needed.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libdiffulex_amd.so"
OPS_PATH = PKG_DIR / "_torch_ops.so"
STEP_BENCH_PATH = PKG_DIR / "build" / "step_bench"
ARCH = "gfx950"

# packed-fp32 instructions are kept out of the generated code on purpose
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-Wno-inline-asm",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
SOURCES = ["capi.cpp", "kv_cache.hip", "metadata.hip", "paged_attn.hip", "rotary.hip"]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the gfx950 kernels cannot be built")
    return exe


def _compile(src: Path, obj: Path) -> None:
    cmd = [_hipcc(), *HIP_FLAGS, *os.environ.get("DFX_EXTRA_FLAGS", "").split(), "-x", "hip", "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the packed-fp32 feature name; that warning is expected
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def _generator():
    import importlib.util
    spec = importlib.util.spec_from_file_location("gen_pipe_step", CSRC / "gen_pipe_step.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _generate() -> None:
    """Run the source generators under csrc/ (the hand-scheduled tile step of the streaming kernel)."""
    _generator().main()


def build_step_bench(verbose: bool = True) -> Path:
    """The microbenchmark of the generated tile step (csrc/step_bench.hip): an executable, with the
    timing variants of the blocks it compares the step with generated into build/."""
    obj_dir = PKG_DIR / "build"
    obj_dir.mkdir(exist_ok=True)
    gen = _generator()
    for only in ("mfma", "valu", "lds"):
        gen.main(out=str(obj_dir / f"step_only_{only}.h"), only=only, namespace=f"dfx_only_{only}")
    cmd = [_hipcc(), *[f for f in HIP_FLAGS if f != "-fPIC"], f"-I{CSRC}", "-x", "hip", str(CSRC / "step_bench.hip"), "-o", str(STEP_BENCH_PATH)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for step_bench.hip:\n{res.stderr[-4000:]}")
    if verbose:
        print(f"built {STEP_BENCH_PATH} ({STEP_BENCH_PATH.stat().st_size} bytes)")
    return STEP_BENCH_PATH


def build(verbose: bool = True) -> Path:
    _generate()
    obj_dir = PKG_DIR / "build"
    obj_dir.mkdir(exist_ok=True)
    objs = [obj_dir / (Path(s).stem + ".o") for s in SOURCES]
    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as pool:
        list(pool.map(lambda so: _compile(CSRC / so[0], so[1]), zip(SOURCES, objs)))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} ({LIB_PATH.stat().st_size} bytes)")
    build_torch_ops(verbose)
    build_step_bench(verbose)
    return LIB_PATH


def build_torch_ops(verbose: bool = True) -> Path:
    """The TORCH_LIBRARY module: host C++ only, linked against PyTorch and libdiffulex_amd.so."""
    import torch
    from torch.utils import cpp_extension
    torch_lib = Path(torch.__file__).resolve().parent / "lib"
    tmp = OPS_PATH.with_suffix(".so.tmp")
    cmd = [_hipcc(), "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           *[f"-I{p}" for p in cpp_extension.include_paths("cuda")], str(CSRC / "torch_ext.cpp"), "-o", str(tmp),
           f"-L{torch_lib}", "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip",
           f"-L{PKG_DIR}", f"-l:{LIB_PATH.name}", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for torch_ext.cpp:\n{res.stderr[-4000:]}")
    os.replace(tmp, OPS_PATH)
    if verbose:
        print(f"built {OPS_PATH} ({OPS_PATH.stat().st_size} bytes)")
    return OPS_PATH


if __name__ == "__main__":
    build()
