"""Loads (building on first use) the host-side hook library for csrc helper code."""
import ctypes as C
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "host", "host_hooks.cpp")
LIB = os.path.join(HERE, "host", "libdfx_hosthooks.so")


def build():
    subprocess.run(["hipcc", "-x", "hip", "--cuda-host-only", "-O2", "-std=c++17", "-shared", "-fPIC", SRC, "-o", LIB],
                   check=True, capture_output=True)


def load():
    deps = [SRC, os.path.join(HERE, "..", "diffulex_amd", "csrc", "partition.h"),
            os.path.join(HERE, "..", "diffulex_amd", "csrc", "fp8_e4m3.h")]
    if not os.path.exists(LIB) or any(os.path.getmtime(d) > os.path.getmtime(LIB) for d in deps):
        build()
    lib = C.CDLL(LIB)
    vp, i32, i64 = C.c_void_p, C.c_int, C.c_int64
    lib.hook_quantise_e4m3.argtypes = [vp, C.c_float, vp, i64]
    lib.hook_e4m3_to_f32.argtypes = [vp, vp, i64]
    lib.hook_bf16_round.argtypes = [vp, vp, i64]
    lib.hook_effective_workgroups.restype = i32
    lib.hook_effective_workgroups.argtypes = [i64, i64, i32, i32]
    lib.hook_walk_segments.restype = i64
    lib.hook_walk_segments.argtypes = [vp, vp, vp, i32, i32, i32, i32, i32, vp, i64]
    lib.hook_walk_segments_masked.restype = i64
    lib.hook_walk_segments_masked.argtypes = [vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, vp, i64]
    lib.hook_enumerate_units.restype = i32
    lib.hook_enumerate_units.argtypes = [i32, i32, i32, i32, i32, i32, i32, vp, i32]
    lib.hook_combine_slots.restype = i32
    lib.hook_combine_slots.argtypes = [vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, i32, vp, i32]
    lib.hook_sweep_head.restype = i32
    lib.hook_sweep_head.argtypes = [vp, i32, i32, i32, vp]
    lib.hook_owners_with_bounds.restype = None
    lib.hook_owners_with_bounds.argtypes = [vp, i32, i32, i64, i64, vp, vp]
    return lib
