"""What the compiler made of the streaming kernels' tile loops (CPU test: hipcc cross-compiles).

The asynchronous tile loads are waited for by hand (exact ``s_waitcnt vmcnt(n)``), which only
works while the compiler has no reason to wait inside the loop itself: a load of its own that is
pending on some path into the loop, or a register spilled to scratch, makes it drain the load
queue in every iteration.  Such regressions cost 10-30 % and change no result, so they are
checked on the generated code: per tile loop the expected matrix instructions, no scratch access, and no
``vmcnt`` wait beyond the hand-placed ones.
"""
import collections
import re
import shutil
import subprocess
from pathlib import Path

import pytest

from diffulex_amd import build as dbuild

ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def isa(tmp_path_factory):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(hipcc).exists():
        pytest.skip("hipcc not available")
    out = tmp_path_factory.mktemp("isa") / "paged_attn.s"
    cmd = [hipcc, *dbuild.HIP_FLAGS, "-I", str(ROOT / "include"), "-S", "--cuda-device-only", "-x", "hip",
           str(ROOT / "diffulex_amd" / "csrc" / "paged_attn.hip"), "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True)
    return out.read_text()


def _tile_loop(isa_text, mangled_prefix):
    """Instructions of the innermost loop that contains every matrix instruction of the kernel and its
    tile loads (a jump from a peeled iteration into the middle of the loop looks like a smaller one)."""
    m = re.search(r"^(%s\w*):" % re.escape(mangled_prefix), isa_text, re.M)
    assert m, mangled_prefix
    body = [l.strip() for l in isa_text[m.start():isa_text.index("s_endpgm", m.start())].split("\n")]
    mfma = [i for i, l in enumerate(body) if l.startswith("v_mfma")]
    labels = {mm.group(1): i for i, l in enumerate(body) for mm in [re.match(r"^(\.LBB\d+_\d+):", l)] if mm}
    best = None
    for i, l in enumerate(body):
        mm = re.search(r"s_c?branch\S*\s+(\.LBB\d+_\d+)", l)
        if mm and mm.group(1) in labels:
            t = labels[mm.group(1)]
            if t < mfma[0] and i > mfma[-1] and (best is None or i - t < best[1] - best[0]) and \
                    any(x.startswith("global_load_lds") for x in body[t:i]):
                best = (t, i)
    assert best, "no loop around the matrix instructions"
    return [l for l in body[best[0]:best[1] + 1] if l and not l.startswith((";", "."))]


# kernel, hand-placed vmcnt waits in its loop (three alternatives of wait_younger; the FP8 kernel
# also waits inside the branch that copies fresh bf16 rows, once per load round of a wave)
KERNELS = [
    ("_ZN3dfx24paged_attn_stream_kernelILi128ELi1ELi8ELb0ELb0E", 3),
    ("_ZN3dfx24paged_attn_stream_kernelILi128ELi1ELi4ELb1ELb0E", 3),
    ("_ZN3dfx24paged_attn_stream_kernelILi128ELi1ELi4ELb0ELb0E", 3),
    ("_ZN3dfx24paged_attn_stream_kernelILi64ELi1ELi8ELb0ELb0E", 3),
    ("_ZN3dfx24paged_attn_stream_kernelILi64ELi1ELi4ELb1ELb0E", 3),
    ("_ZN3dfx24paged_attn_stream_kernelILi128ELi1ELi8ELb0ELb1E", 3),   # the distinct cache layout
    ("_ZN3dfx28paged_attn_stream_fp8_kernelILi128ELi1ELi8E", 3 + 2),
    ("_ZN3dfx28paged_attn_stream_fp8_kernelILi128ELi1ELi4E", 3 + 3),
]


@pytest.mark.parametrize("kernel,max_waits", KERNELS)
def test_tile_loop_has_no_spills_and_no_compiler_waits(isa, kernel, max_waits):
    loop = _tile_loop(isa, kernel)
    ops = collections.Counter(l.split()[0] for l in loop)
    assert ops["v_mfma_f32_32x32x16_bf16"] == (32 if "ILi128E" in kernel else 16)   # head_dim / 4 per 64-token tile
    assert not [l for l in loop if l.startswith("scratch_")], "a register of the tile loop lives in scratch"
    waits = [l for l in loop if l.startswith("s_waitcnt") and "vmcnt" in l]
    assert len(waits) <= max_waits, waits
    # nothing may wait for memory between the barrier and the end of the step in the bf16 kernels
    if "fp8" not in kernel:
        after_barrier = loop[max(i for i, l in enumerate(loop) if l.startswith("s_barrier")):]
        assert not [l for l in after_barrier if "vmcnt" in l]
    assert ops["global_load_lds_dwordx4"] in (2, 4, 8)   # a wave's share of the 64 * head_dim * elt * 2 bytes of a tile


PIPE_KERNELS = ["_ZN3dfx22paged_attn_pipe_kernelILi8ELb0ELb0ELi128E", "_ZN3dfx22paged_attn_pipe_kernelILi8ELb1ELb0ELi128E",
                "_ZN3dfx22paged_attn_pipe_kernelILi8ELb0ELb1ELi128E",   # the distinct cache layout
                "_ZN3dfx22paged_attn_pipe_kernelILi8ELb0ELb0ELi64E",    # head_dim 64
                "_ZN3dfx26paged_attn_pipe_fp8_kernelILi8E"]


@pytest.mark.parametrize("kernel", PIPE_KERNELS)
def test_pipelined_kernel_leaves_the_generated_blocks_registers_alone(isa, kernel):
    """The generated blocks of csrc/attn_pipe_gen.h keep their state in v32..v127 / a32..a127 across
    compiler-generated code, which is only sound while the compiler allocates nothing there
    (amdgpu_num_vgpr(32) on the kernel).  Checked on the generated code: outside the assembly
    blocks no register above v31 / a31 is named, and the tile loop has no scratch access."""
    m = re.search(r"^(%s\w*):" % re.escape(kernel), isa, re.M)
    assert m, kernel
    body = isa[m.start():isa.index("s_endpgm", m.start())].split("\n")
    in_asm, top_v, top_a, blocks = False, 0, 0, 0
    for line in body:
        t = line.strip()
        if t.startswith(";;#ASMSTART"):
            in_asm, blocks = True, blocks + 1
            continue
        if t.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if in_asm or not t or t.startswith((";", ".")):
            continue
        for mm in re.finditer(r"\b([va])(\d+)\b", t):
            if mm.group(1) == "v":
                top_v = max(top_v, int(mm.group(2)))
            else:
                top_a = max(top_a, int(mm.group(2)))
        for mm in re.finditer(r"\b([va])\[(\d+):(\d+)\]", t):
            if mm.group(1) == "v":
                top_v = max(top_v, int(mm.group(3)))
            else:
                top_a = max(top_a, int(mm.group(3)))
    assert blocks > 20
    assert top_v <= 31 and top_a <= 31, (top_v, top_a)
    # the kernel's register count covers the blocks' registers
    i = isa.index(".amdhsa_kernel " + m.group(1))
    assert int(re.search(r"\.amdhsa_next_free_vgpr (\d+)", isa[i:i + 3000]).group(1)) == 256
    assert int(re.search(r"\.amdhsa_accum_offset (\d+)", isa[i:i + 3000]).group(1)) == 128
    loop = _tile_loop(isa, kernel)
    ops = collections.Counter(l.split()[0] for l in loop)
    # first tile of a run 16, two steps 32 each, two steps 32 + 16 each, two plain steps 32 each (head_dim 64: half)
    assert ops["v_mfma_f32_32x32x16_bf16"] == (88 if "ELi64E" in kernel else 176)
    # (the FP8 kernel carries more per-item state in scalar registers, some of which the compiler parks in
    # scratch until the item's rows are written: behind the steps, where no tile load is waited for by count)
    mfma = [i for i, l in enumerate(loop) if l.startswith("v_mfma")]
    steps = loop[mfma[0]:mfma[-1] + 1] if "fp8" in kernel else loop
    assert not [l for l in steps if l.startswith("scratch_")], "a register of the tile loop lives in scratch"
    # and the compiler waits for no load of its own between the steps' matrix instructions, except in the
    # FP8 kernel's copies of fresh rows (hand-placed, one per matrix and copy of the general step)
    in_asm, waits = False, 0
    m = re.search(r"^(%s\w*):" % re.escape(kernel), isa, re.M)
    body = [l.strip() for l in isa[m.start():isa.index("s_endpgm", m.start())].split("\n")]
    mf = [i for i, l in enumerate(body) if l.startswith("v_mfma")]
    for l in body[mf[0]:mf[-1] + 1]:
        if l.startswith(";;#ASMSTART"):
            in_asm = True
        elif l.startswith(";;#ASMEND"):
            in_asm = False
        elif not in_asm and l.startswith("s_waitcnt") and "vmcnt" in l:
            waits += 1
    assert waits <= (6 if "fp8" in kernel else 0), waits


def test_timing_variants_of_the_step_hold_one_class_of_instructions(tmp_path):
    """csrc/step_bench.hip compares the step with variants of its blocks that hold the matrix instructions, the
    softmax arithmetic or the operand reads alone (gen_pipe_step.main(only=...)): each in a namespace of its
    own, and generating them leaves the library's header as it is."""
    gen = dbuild._generator()
    lib_header = (ROOT / "diffulex_amd" / "csrc" / "attn_pipe_gen.h").read_text()
    counts = {}
    for only in (None, "mfma", "valu", "lds"):
        out = tmp_path / f"{only}.h"
        gen.main(out=str(out), only=only, namespace="dfx" if only is None else f"dfx_only_{only}")
        text = out.read_text()
        step = text[text.index("void pipe_step_ab_x("):text.index("void pipe_step_ba_x(")]
        counts[only] = (step.count("v_mfma_f32"), step.count("v_exp_f32"), step.count("ds_read_"))
        assert (f"namespace dfx_only_{only} {{" in text) == (only is not None)
    assert gen.main(out=str(tmp_path / "again.h")) and (tmp_path / "again.h").read_text() == lib_header == (tmp_path / "None.h").read_text()
    mfma, exp2, reads = counts[None]
    assert (mfma, exp2) == (32, 32) and reads == 16 + 32
    assert counts["mfma"] == (mfma, 0, 0) and counts["valu"] == (0, exp2, 0) and counts["lds"] == (0, 0, reads)
