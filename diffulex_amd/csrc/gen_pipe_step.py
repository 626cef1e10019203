#!/usr/bin/env python3
"""Generates attn_pipe_gen.h: the software-pipelined tile step of the streaming paged-attention
kernel as hand-scheduled gfx950 assembly on registers the compiler never touches.

    python diffulex_amd/csrc/gen_pipe_step.py        (diffulex_amd/build.py runs it before compiling)

Why.  The matrix unit and the vector ALU of a SIMD only work at the same time if one wave's
instruction stream alternates between them: a 32x32x16 matrix instruction occupies its pipeline
for 8 passes, in whose shadow the wave can issue four or five independent vector instructions.
One step therefore computes S^T = K Q^T of the NEXT tile and O^T += V^T P^T of the CURRENT tile,
with the softmax of the current tile (exp2, row sum, bf16 rounding) and the row maximum of the
next one cut into pieces between the matrix instructions.  Both waves of a SIMD reach the start of
a phase together (behind the step's barrier), where the matrix unit would idle until the first
operands have come from LDS: phase X does a dozen of its vector instructions there, and the first
operands of phase Y are requested from the tail of phase X.  Left to the compiler, loop-carried
matrix state around inline assembly is copied between registers (or spilled) at control-flow
merges.  The kernel that uses these blocks is therefore compiled with amdgpu_num_vgpr(32): the
compiler allocates v0..v31 and a0..a31 only, and the matrix state lives in the registers above,
which appear in no operand list -- only in the clobber list of pipe_reserve(), so that the
kernel's register count covers them.

Register map (head_dim 128; one 32-row query block per wave; 128 + 128 registers per lane):
    a[32:95]   O^T accumulators, 32-row d block db in a[32 + 16 db : 47 + 16 db]
    a[96:127]  Q operand, contraction slab s in a[96 + 4 s : 99 + 4 s]
    v[48:79]   score set A: tokens 0..31 in v[48:63], tokens 32..63 in v[64:79]
    v[80:111]  score set B
    v[112:127] operand ring: four 4-register buffers (K operands in phase X, V^T in phase Y)
    v[32:42]   temporaries: exp2 pair, K operand address, 8 V^T operand addresses
    v[43:44]   the lane's byte offsets inside a band of cached rows (tile loads, pipe_issue_band)
    v[45:47]   cache of one-byte codes: the lane's LDS addresses for pipe_widen;
               two-byte elements: v[45:46] the lane's byte offsets inside a band of fresh rows (pipe_issue_band_fresh)
    v[0:31], a[0:31]  the compiler's
The two score sets swap roles every step (steps AB and BA), so nothing is ever moved.  P (the
bf16 pairs, the B operand of the second product) overwrites the current score set as it is
consumed: pair j of the 16 (token block j / 8) goes to register j of the set, whose score
(element j of token block 0) an earlier or the same pair has read by then.

Hazards handled here by construction (the compiler does not see inside the blocks):
  * vector-ALU result -> matrix instruction operand: 2 wait states (an s_nop 1 is emitted when the
    producer is closer than that);
  * transcendental result -> any reader: at least one instruction in between;
  * matrix result -> vector-ALU reader: the readers (row maximum of the next tile) come at least
    four matrix instructions later, or behind 18 wait states; every block that reads the O^T
    accumulators with the vector ALU starts with those wait states;
  * LDS operands: exact s_waitcnt lgkmcnt(n) on the in-order LDS return queue; a block starts
    with lgkmcnt(0) so that only its own reads are in the queue.
"""
from __future__ import annotations

import os

HERE = os.path.dirname(os.path.abspath(__file__))

HD = 128
ROWB = HD * 2
NSLAB = HD // 16            # 8
NDB = HD // 32              # 4


def set_head_dim(hd):
    """The blocks generated from here on are for this head_dim (128, or 64: half the contraction slabs of S^T, half
    the d blocks of O^T -- a[32:63] -- and of the Q operand -- a[96:111]; a tile row is 128 bytes, a K or V tile 8 KiB)."""
    global HD, ROWB, NSLAB, NDB, MAT_BYTES
    HD, ROWB, NSLAB, NDB = hd, hd * 2, hd // 16, hd // 32
    MAT_BYTES = 64 * ROWB


COMPILER_REGS = 32          # v0..v31 and a0..a31 are the compiler's (amdgpu_num_vgpr(32))
O_BASE, Q_BASE = 32, 96
TMP, NTMP = 32, 11
SA, SB, RING = 48, 80, 112
T_EXP = [TMP + 0, TMP + 1]  # exp2 arguments / results of the pair in flight
T_ADDR = TMP + 2            # K operand address of the slab being read (phase X); scratch elsewhere
T_VADDR = TMP + 3           # 8 V^T operand addresses (phase Y)
LOAD_OFF = 43               # two registers: byte offsets of the lane's chunk in its two rows of a band of cached rows
WIDEN_ADDR = 45             # three registers: LDS addresses for pipe_widen (cache of one-byte codes)
FRESH_OFF = 45              # two registers: LOAD_OFF for a band of fresh rows (two-byte cache elements: no pipe_widen there)
MAT_BYTES = 64 * ROWB       # K tile; the V tile of a ring stage follows it
# Tile layout the blocks being generated read: 'u' (cache in the unified layout: both tiles row-major, 16-byte chunks
# swizzled by the row) or 'd' (distinct layout: K tile chunk-major [HD / 8][64 tokens][16 bytes], V tile d-major
# [HD][64 tokens] with chunks swizzled by (d / 2) % 8; the key rows feed S^T with quads 1 and 2 of every 16 swapped, so
# that a lane's 8 scores of a 16-token slab are 8 consecutive tokens, as a chunk of a V^T row holds them).
LAYOUT = "u"
CHUNK_COL_BYTES = 64 * 16
NEG_INF = "0xff800000"
FRONT_X = 12                # vector instructions of phase X ahead of its first matrix instruction
MFMA_TO_VALU = ["s_nop 15", "s_nop 1"]  # 18 wait states: the longest the ISA asks for
# Timing variants for step_bench.hip (never for the library): the step blocks with only one class of their
# instructions -- "mfma", "valu" (the softmax arithmetic) or "lds" (the operand reads).  Their results are meaningless.
ONLY = None
NAMESPACE = "dfx"
SOFTMAX_OPS = ("v_fma_f32", "v_exp_f32", "v_add_f32", "v_cvt_pk_bf16_f32", "v_max3_f32", "v_max_f32")


def vr(base, n=1):
    return f"v{base}" if n == 1 else f"v[{base}:{base + n - 1}]"


def ar(base, n=1):
    return f"a{base}" if n == 1 else f"a[{base}:{base + n - 1}]"


NBUF = 4                    # operand ring buffers (4 registers each): operands are read NBUF - 1 matrix instructions ahead


def ring(n, cnt=4, sub=0):
    """Registers sub .. sub + cnt - 1 of operand ring buffer n % NBUF."""
    return vr(RING + 4 * (n % NBUF) + sub, cnt)


def swizzle(row):
    if HD == 64:  # (TileLayout<64>::swizzle: 128-byte rows, odd rows already sit 64 banks further)
        return (((row >> 1) & 1) << 2) | ((row >> 2) & 3)
    return ((row & 3) << 2) | ((row >> 2) & 3)


def join(ins):
    return "\\n\\t".join(ins)


class Block:
    """Instruction list with LDS queue tracking and the vector-ALU -> matrix operand hazard."""

    def __init__(self):
        self.ins = []
        self.lds_queue = []         # tags of outstanding LDS reads, oldest first
        self.recent_valu_defs = []  # register sets written by the last two instructions

    def _push(self, text, defs=()):
        self.ins.append(text)
        self.recent_valu_defs = (self.recent_valu_defs + [set(defs)])[-2:]

    def valu(self, text, defs):
        if ONLY in ("mfma", "lds") and text.split()[0] in SOFTMAX_OPS:
            return
        self._push(text, defs)

    def other(self, text):
        self._push(text)

    def lds_read(self, text, tag):
        if ONLY in ("mfma", "valu"):
            return
        self._push(text)
        self.lds_queue.append(tag)

    def wait_lds(self, tag):
        """Wait until the read `tag` has returned (reads return in order)."""
        if tag not in self.lds_queue:
            return
        younger = len(self.lds_queue) - 1 - self.lds_queue.index(tag)
        self._push(f"s_waitcnt lgkmcnt({younger})")
        self.lds_queue = self.lds_queue[len(self.lds_queue) - younger:]

    def mfma(self, dst, a, b, c, reads):
        """reads: registers (numbers) of vector operands a/b/c written by the vector ALU."""
        if ONLY in ("valu", "lds"):
            return
        if any(set(reads) & d for d in self.recent_valu_defs):
            self._push("s_nop 1")
        self._push(f"v_mfma_f32_32x32x16_bf16 {dst}, {a}, {b}, {c}")

    def text(self):
        return join(self.ins)


def pair_instrs(cur, pr):
    """The 7 vector instructions of element pair pr (0..15) of score set `cur`: two exp2 arguments,
    two exp2, two row-sum additions, one bf16 pair.  Operands: %[c] scale (SGPR), %[nm] minus the
    running maximum, %[l] the row sum."""
    tb, i = pr >> 3, pr & 7
    s0, s1 = cur + 16 * tb + 2 * i, cur + 16 * tb + 2 * i + 1
    t0, t1 = T_EXP
    p = cur + pr
    return [
        (f"v_fma_f32 {vr(t0)}, {vr(s0)}, %[c], %[nm]", {t0}),
        (f"v_fma_f32 {vr(t1)}, {vr(s1)}, %[c], %[nm]", {t1}),
        (f"v_exp_f32 {vr(t0)}, {vr(t0)}", {t0}),
        (f"v_exp_f32 {vr(t1)}, {vr(t1)}", {t1}),
        (f"v_add_f32 %[l], %[l], {vr(t0)}", set()),
        (f"v_add_f32 %[l], %[l], {vr(t1)}", set()),
        (f"v_cvt_pk_bf16_f32 {vr(p)}, {vr(t0)}, {vr(t1)}", {p}),
    ]


def vaddr_instrs():
    """V^T operand addresses vx[z] = %[v0] ^ const_z."""
    out = []
    if LAYOUT == "d":  # one per 16-token slab z = 2 tb + sl: chunk 2 z + half; the d block is an immediate offset
        for z in range(4):
            out.append((f"v_mov_b32 {vr(T_VADDR)}, %[v0]", {T_VADDR}) if z == 0 else
                       (f"v_xor_b32 {vr(T_VADDR + z)}, {z * 32:#x}, %[v0]", {T_VADDR + z}))
        return out
    for z in range(2 * NDB):
        const = (((z >> 1) * 4) ^ swizzle((z & 1) * 8)) * 16
        if z == 0:
            out.append((f"v_mov_b32 {vr(T_VADDR)}, %[v0]", {T_VADDR}))
        else:
            out.append((f"v_xor_b32 {vr(T_VADDR + z)}, {const:#x}, %[v0]", {T_VADDR + z}))
    return out


def max_instrs(nxt):
    """Maximum of the lane's 32 scores of set `nxt` into %[mx] (one lane: half a query row)."""
    out = [(f"v_max3_f32 %[mx], {vr(nxt)}, {vr(nxt + 1)}, {vr(nxt + 2)}", set())]
    regs = list(range(nxt + 3, nxt + 32))
    while regs:
        if len(regs) >= 2:
            out.append((f"v_max3_f32 %[mx], %[mx], {vr(regs[0])}, {vr(regs[1])}", set()))
            regs = regs[2:]
        else:
            out.append((f"v_max_f32 %[mx], %[mx], {vr(regs[0])}", set()))
            regs = regs[1:]
    return out


def emit_valu(b, stream, n):
    for _ in range(n):
        if stream:
            text, defs = stream.pop(0)
            b.valu(text, defs)


def phase_x(b, nxt, stream, quotas, front=0, tail_read=None):
    """S^T of the next tile into set `nxt`: 16 matrix instructions (slab-major, token block minor),
    K operands read three ahead through the ring, `front` vector instructions between the first
    reads and the first matrix instruction (work for the time the reads take), `quotas[i]` behind the
    i-th.  tail_read(j): issues operand read j (0..2) of the phase that follows, in the places of the
    K reads the last three matrix instructions no longer need (the ring buffer each goes to was last
    read by the matrix instruction issued just before, as with the K reads).
    (LDS instructions take their address when they issue, in program order: the address register
    may be rewritten for the next slab right behind the read.)"""
    n = 2 * NSLAB

    def read(i):
        slab, tb = i >> 1, i & 1
        if LAYOUT == "d":  # chunk column 2 slab + half, tokens 32 tb ..: every offset an immediate
            b.lds_read(f"ds_read_b128 {ring(i)}, %[k0] offset:{slab * 2 * CHUNK_COL_BYTES + tb * 32 * 16}", ("k", i))
            return
        if tb == 0 and slab > 0:
            b.valu(f"v_xor_b32 {vr(T_ADDR)}, {slab * 32:#x}, %[k0]", {T_ADDR})
        addr = "%[k0]" if slab == 0 else vr(T_ADDR)
        b.lds_read(f"ds_read_b128 {ring(i)}, {addr} offset:{tb * 32 * ROWB}", ("k", i))

    A = NBUF - 1
    for i in range(A):
        read(i)
    emit_valu(b, stream, front)
    for i in range(n):
        if i + A < n:
            read(i + A)
        elif tail_read is not None:
            tail_read(i + A - n)
        b.wait_lds(("k", i))
        slab, tb = i >> 1, i & 1
        dst = vr(nxt + 16 * tb, 16)
        b.mfma(dst, ring(i), ar(Q_BASE + 4 * slab, 4), "0" if slab == 0 else dst, reads=())
        emit_valu(b, stream, quotas[i])


def y_operand_read(b, j):
    """Read of the V^T operand of matrix instruction j of phase Y into ring buffer j % 4."""
    tb, sl, db = j // (2 * NDB), (j // NDB) & 1, j % NDB
    if LAYOUT == "d":  # row 32 db + lane % 32 of V^T, the 8 tokens of the lane's half of the slab: one read
        b.lds_read(f"ds_read_b128 {ring(j)}, {vr(T_VADDR + 2 * tb + sl)} offset:{db * 32 * 128}", ("v", j, 1))
        return
    for ii in range(2):
        off = (tb * 32 + sl * 16 + ii * 8) * ROWB
        b.lds_read(f"ds_read_b64_tr_b16 {ring(j, 2, 2 * ii)}, {vr(T_VADDR + 2 * db + ii)} offset:{off}",
                   ("v", j, ii))


def phase_y(b, cur, stream, quotas, hoisted=False):
    """O^T += V^T P^T of the current tile: 16 matrix instructions ordered (token block, 16-token
    slab, d block), V^T operands (two transposing 8-byte reads each) three instructions ahead; the
    first three reads are in flight already if `hoisted` (phase X has issued them: b.lds_queue)."""
    n = 4 * NDB
    A = NBUF - 1
    if not hoisted:
        for j in range(A):
            y_operand_read(b, j)
    for j in range(n):
        if j + A < n:
            y_operand_read(b, j + A)
        b.wait_lds(("v", j, 1))
        tb, sl, db = j // (2 * NDB), (j // NDB) & 1, j % NDB
        acc = ar(O_BASE + 16 * db, 16)
        p = cur + 8 * tb + 4 * sl
        b.mfma(acc, ring(j), vr(p, 4), acc, reads=range(p, p + 4))
        emit_valu(b, stream, quotas[j])


def spread(total, slots):
    """`total` instructions over `slots` matrix instructions, as evenly as integers allow."""
    return [((i + 1) * total) // slots - (i * total) // slots for i in range(slots)]


def step_blocks(cur, nxt, has_next):
    """The two halves of a step.  X: S^T of the next tile with pairs 0..8 of the current set and the
    V^T addresses in its shadow (no next tile: the vector instructions alone).  Y: O^T += V^T P^T with
    pairs 9..13 behind its first 8 matrix instructions (pairs 8..11 feed the 9th, pairs 12..15 the
    13th), pairs 14, 15 and the row maximum of the next set behind the rest.  The halves are separate
    blocks so that a wave can issue its tile loads between them."""
    pairs = [pair_instrs(cur, pr) for pr in range(16)]
    flat = lambda ps: [ins for p in ps for ins in p]
    sx = vaddr_instrs() + flat(pairs[:9])  # (the addresses first: the tail of phase X reads with them)
    y1 = flat(pairs[9:14])
    y2a = flat(pairs[14:16])
    bx = Block()
    bx.other("s_waitcnt lgkmcnt(0)")
    by = Block()
    half, quarter = 2 * NDB, NDB  # of the 4 * NDB matrix instructions of phase Y (head_dim 128: 8 and 4)
    if has_next:
        # The matrix unit would idle while a phase's first operands travel from LDS (both waves of a SIMD reach
        # that point together, behind the step's barrier).  Phase X therefore does FRONT_X of its vector
        # instructions there, and phase Y's first three operands are requested from the tail of phase X.
        phase_x(bx, nxt, sx, spread(len(sx) - FRONT_X, 2 * NSLAB), FRONT_X, lambda j: y_operand_read(bx, j))
        # (phase Y starts with those reads in the queue and no wait of its own: whatever the compiler puts between
        # the two blocks is younger than they are, and the queue returns in order)
        by.lds_queue, bx.lds_queue = bx.lds_queue, []
        y2 = y2a + max_instrs(nxt)
        qa = spread(len(y2a) + 4, quarter)
        sy = y1 + y2
        quotas = spread(len(y1), half) + qa + spread(len(y2) - sum(qa), quarter)
    else:
        emit_valu(bx, sx, len(sx))
        by.other("s_waitcnt lgkmcnt(0)")
        sy = y1 + y2a
        quotas = spread(len(y1), half) + spread(len(y2a), quarter) + [0] * quarter
    # every pair is complete before the matrix instruction that reads it: instruction j (token block tb, slab sl)
    # reads pairs 8 tb + 4 sl .. + 3; pairs 0..8 are done in phase X, pair p > 8 with instruction 7 (p - 8) of phase Y
    for j in range(4 * NDB):
        last_pair = 8 * (j // (2 * NDB)) + 4 * ((j // NDB) & 1) + 3
        assert sum(quotas[:j]) >= 7 * max(0, last_pair - 8), (HD, j)
    phase_y(by, cur, sy, quotas, hoisted=has_next)
    assert not sx and not sy and not bx.lds_queue and not by.lds_queue
    return bx.text(), by.text()


def first_scores_block(nxt):
    """S^T of a run's first tile into set `nxt` and its lane maximum, with nothing to overlap."""
    b = Block()
    b.other("s_waitcnt lgkmcnt(0)")
    phase_x(b, nxt, [], [0] * (2 * NSLAB))
    for t in MFMA_TO_VALU:
        b.other(t)
    for text, defs in max_instrs(nxt):
        b.valu(text, defs)
    return b.text()


def mask_block(s, hole_rows):
    """Masks score set `s`: element (tb, e) of the lane is token tb * 32 + (e / 4) * 8 + e % 4 of the
    tile (plus 4 for the upper half of the wave, which %[thr] accounts for) and is set to -inf if
    that token number is >= %[thr] or if bit (token / hole_rows) of %[holes] is set; then the lane
    maximum of the masked set into %[mx].  The set's matrix results are ready (caller)."""
    t, ninf = T_ADDR, T_EXP[0]
    ins = [f"v_mov_b32 {vr(ninf)}, {NEG_INF}"]  # (a literal and vcc in one instruction exceed the constant bus)
    for g in range(8):  # groups of 4 elements = 8 tokens
        tb, q = g >> 2, g & 3
        bit = (g * 8) // hole_rows
        ins += [f"s_bitcmp1_b32 %[holes], {bit}", "s_cselect_b64 vcc, -1, 0",
                f"v_cndmask_b32 {vr(t)}, %[thr], -1, vcc"]
        for j in range(4):
            reg = s + 16 * tb + 4 * q + j
            # token of the element (the wave's upper half sits 4 higher, 8 with the swapped quads: in %[thr])
            token = g * 8 + j if LAYOUT == "u" else tb * 32 + (q >> 1) * 16 + (q & 1) * 4 + j
            ins += [f"v_cmp_lt_i32 vcc, {token}, {vr(t)}",
                    f"v_cndmask_b32 {vr(reg)}, {vr(ninf)}, {vr(reg)}, vcc"]
    ins += [text for text, _ in max_instrs(s)]
    return join(ins)


def rotate_pairs(ins, x1, x2, cos, sin, y1, y2, t):
    """Rotates the two bf16 pairs in registers x1 (elements e, e + 1 of the lower half of a head row) and
    x2 (the same elements of the upper half) by the angles whose cosines / sines are in registers cos,
    cos + 1 / sin, sin + 1: y1 = x1 * cos - x2 * sin, y2 = x2 * cos + x1 * sin, every product and the sum
    rounded on their own (the reference evaluates them as separate fp32 tensor operations:
    diffulex/layer/rotary_embedding.py:13-16), then rounded to nearest even to bf16.  t: 8 scratch registers."""
    a_lo, a_hi, b_lo, b_hi, p, q, r, u = range(t, t + 8)
    ins += [f"v_lshlrev_b32 {vr(a_lo)}, 16, {vr(x1)}", f"v_and_b32 {vr(a_hi)}, 0xffff0000, {vr(x1)}",
            f"v_lshlrev_b32 {vr(b_lo)}, 16, {vr(x2)}", f"v_and_b32 {vr(b_hi)}, 0xffff0000, {vr(x2)}"]
    for a, b, c, sn, o1, o2 in ((a_lo, b_lo, cos, sin, p, q), (a_hi, b_hi, cos + 1, sin + 1, r, u)):
        ins += [f"v_mul_f32 {vr(o1)}, {vr(a)}, {vr(c)}", f"v_mul_f32 {vr(o2)}, {vr(b)}, {vr(sn)}",
                f"v_sub_f32 {vr(o1)}, {vr(o1)}, {vr(o2)}",                    # y1 = x1 c - x2 s
                f"v_mul_f32 {vr(o2)}, {vr(b)}, {vr(c)}", f"v_mul_f32 {vr(a)}, {vr(a)}, {vr(sn)}",
                f"v_add_f32 {vr(o2)}, {vr(o2)}, {vr(a)}"]                      # y2 = x2 c + x1 s
    ins += [f"v_cvt_pk_bf16_f32 {vr(y1)}, {vr(p)}, {vr(r)}", f"v_cvt_pk_bf16_f32 {vr(y2)}, {vr(q)}, {vr(u)}"]


def rope_queries_fns():
    """Rotary embedding of the query rows in the Q operand registers, in two blocks: the request for the
    cosines / sines of the lane's elements (2 x 32 floats of its position's table row, into the score sets,
    which are free between two items), and the rotation once they and the query rows have landed.  The lane
    holds, of its row, elements 16 s + 8 h .. + 7 in slab s (h: the wave's half): slabs s and s + 4 are the
    two halves a rotation mixes."""
    loads = []
    for s in range(NSLAB // 2):
        for j in range(2):
            loads.append(f"global_load_dwordx4 {vr(SA + 8 * s + 4 * j, 4)}, %[t], off offset:{(16 * s + 4 * j) * 4}")
            loads.append(f"global_load_dwordx4 {vr(SB + 8 * s + 4 * j, 4)}, %[t], off offset:{(HD // 2 + 16 * s + 4 * j) * 4}")
    ins = ["s_waitcnt vmcnt(0)"]
    x1, x2, t = RING, RING + 1, TMP
    for s in range(NSLAB // 2):
        for j in range(4):
            lo, hi = Q_BASE + 4 * s + j, Q_BASE + 4 * (s + NSLAB // 2) + j
            ins += [f"v_accvgpr_read_b32 {vr(x1)}, {ar(lo)}", f"v_accvgpr_read_b32 {vr(x2)}, {ar(hi)}"]
            rotate_pairs(ins, x1, x2, SA + 8 * s + 2 * j, SB + 8 * s + 2 * j, RING + 2, RING + 3, t)
            ins += [f"v_accvgpr_write_b32 {ar(lo)}, {vr(RING + 2)}", f"v_accvgpr_write_b32 {ar(hi)}, {vr(RING + 3)}"]
    ins.append("s_nop 1")  # (a matrix instruction may read the operand next)
    return (asm_fn("pipe_issue_rope_angles", "const void* table_row", join(loads), ins=['[t] "v"(table_row)'], clobbers=["memory"],
                   comment="Requests the cosines and sines of the lane's query elements: `table_row` is the lane's position's row of\n"
                           "the angle table plus 8 h floats.  They go to the score sets, which are free between two items.") +
            asm_fn("pipe_rope_queries", "", join(ins), clobbers=["memory"],
                   comment="Rotates the query row in the Q operand registers by the angles pipe_issue_rope_angles() has requested:\n"
                           "the arithmetic of dfx_rope_kv_store, bit for bit.  Waits for every load of the wave in flight (the\n"
                           "angles, the query rows); the operand ring is free (between two items)."))


def rope_row_fn(with_v=False):
    """Rotary embedding of one pair of 16-byte chunks (c, c + 8) of a fresh K head row, in the blocks' registers:
    the kernel's per-item rotation of the fresh K rows (the compiler's 32 registers would not hold it).  with_v:
    the same chunks of the V row travel with them, from v_chunk to v_dst (their cache slot, two-byte elements),
    through registers of score set B: one trip to memory instead of two."""
    ins = [f"global_load_dwordx4 {vr(SA, 4)}, %[k], off", f"global_load_dwordx4 {vr(SA + 4, 4)}, %[k], off offset:{HD}",
           f"global_load_dwordx4 {vr(SA + 8, 4)}, %[t], off", f"global_load_dwordx4 {vr(SA + 12, 4)}, %[t], off offset:16",
           f"global_load_dwordx4 {vr(SA + 16, 4)}, %[t], off offset:{HD * 2}",
           f"global_load_dwordx4 {vr(SA + 20, 4)}, %[t], off offset:{HD * 2 + 16}"]
    if with_v:
        ins += [f"global_load_dwordx4 {vr(SB, 4)}, %[v], off", f"global_load_dwordx4 {vr(SB + 4, 4)}, %[v], off offset:{HD}"]
    ins.append("s_waitcnt vmcnt(0)")
    if with_v:
        ins += [f"global_store_dwordx4 %[vd], {vr(SB, 4)}, off", f"global_store_dwordx4 %[vd], {vr(SB + 4, 4)}, off offset:{HD}"]
    for j in range(4):
        rotate_pairs(ins, SA + j, SA + 4 + j, SA + 8 + 2 * j, SA + 16 + 2 * j, SA + 24 + j, SA + 28 + j, TMP)
    ins += [f"v_mov_b32 %{j}, {vr(SA + 24 + j)}" for j in range(8)]
    outs = [f'"=v"(lo[{j}])' for j in range(4)] + [f'"=v"(hi[{j}])' for j in range(4)]
    name = "pipe_rope_row_with_v" if with_v else "pipe_rope_row"
    args = ", const void* v_chunk, void* v_dst" if with_v else ""
    extra_ins = ', [v] "v"(v_chunk), [vd] "v"(v_dst)' if with_v else ""
    extra_doc = ("\n// The same chunks of the V row go from v_chunk to v_dst (16 bytes each, HD bytes apart on both sides) in the same\n"
                 "// trip to memory, through score set B." if with_v else "")
    return f'''// Rotates chunks c and c + 8 (16 bytes each, HD bytes apart) of the head row at `k_chunk` by the angles of
// the table row at `table_chunk` (the position's row plus 8 c floats): the arithmetic of dfx_rope_kv_store, bit
// for bit.  Uses score set A; waits for every load of the wave in flight.{extra_doc}
DFX_D void {name}(const void* k_chunk, const void* table_chunk{args}, uint32_t (&lo)[4], uint32_t (&hi)[4]) {{
    asm volatile("{join(ins)}"
                 : {", ".join(outs)}
                 : [k] "v"(k_chunk), [t] "v"(table_chunk){extra_ins}
                 : "memory");
}}

'''


def asm_fn(name, args, body, outs=(), ins=(), clobbers=(), comment=None):
    head = "".join(f"// {line}\n" for line in (comment or "").split("\n") if line)
    ops = f"\n                 : {', '.join(outs)}\n                 : {', '.join(ins)}"
    clob = ", ".join(f'"{c}"' for c in clobbers)
    if clob:
        ops += f"\n                 : {clob}"
    return f'''{head}DFX_D void {name}({args}) {{
    asm volatile("{body}"{ops});
}}

'''


def step_fns(name, cur, nxt, has_next, comment=None):
    x, y = step_blocks(cur, nxt, has_next)
    fx = asm_fn(name + "_x", ("uint32_t k_next, " if has_next else "") + "float c, float neg_m, float& l_run", x,
                ['[l] "+v"(l_run)'], (['[k0] "v"(k_next)'] if has_next else []) + ['[c] "s"(c)', '[nm] "v"(neg_m)'],
                ["memory"], comment)
    # (phase X has written the V^T operand addresses from v_cur: it takes it as well)
    fx = fx.replace('[c] "s"(c)', '[v0] "v"(v_cur), [c] "s"(c)').replace("float c, float neg_m", "uint32_t v_cur, float c, float neg_m", 1)
    fy = asm_fn(name + "_y", "float c, float neg_m, float& l_run" + (", float& mx" if has_next else ""), y,
                ['[l] "+v"(l_run)'] + (['[mx] "=&v"(mx)'] if has_next else []), ['[c] "s"(c)', '[nm] "v"(neg_m)'], ["memory"])
    return fx + fy


def head_dim_64_family():
    """The blocks whose code depends on head_dim, once more for head_dim 64 (pipe64_*): same register map with
    half the O^T accumulators (a[32:63]) and half the Q operand (a[96:111]); a wave fetches its 8 rows of a tile with
    one load per matrix.  Masks, the accessors of the accumulators and of a requested piece are shared."""
    global LAYOUT
    LAYOUT = "u"
    set_head_dim(64)
    pre, what = "pipe64_", "  head_dim 64."
    parts = []
    parts.append(asm_fn(pre + "zero_outputs", "", join(f"v_accvgpr_write_b32 {ar(O_BASE + i)}, 0" for i in range(16 * NDB)),
                        comment="O^T = 0." + what))
    resc = list(MFMA_TO_VALU)
    for g in range(0, 16 * NDB, 4):
        resc += [f"v_accvgpr_read_b32 {vr(TMP + i - g)}, {ar(O_BASE + i)}" for i in range(g, g + 4)]
        resc += [f"v_mul_f32 {vr(TMP + i - g)}, {vr(TMP + i - g)}, %[alpha]" for i in range(g, g + 4)]
        resc += [f"v_accvgpr_write_b32 {ar(O_BASE + i)}, {vr(TMP + i - g)}" for i in range(g, g + 4)]
    parts.append(asm_fn(pre + "rescale_outputs", "float alpha", join(resc), ins=['[alpha] "v"(alpha)'],
                        comment="O^T *= alpha, behind the wait states for the matrix results." + what))
    ql = [f"global_load_dwordx4 {ar(Q_BASE + 4 * s, 4)}, %[p], off offset:{s * 32}" for s in range(NSLAB)]
    parts.append(asm_fn(pre + "issue_queries", "const void* row", join(ql), ins=['[p] "v"(row)'], clobbers=["memory"],
                        comment="Q operand: requests the lane's half (slab s at byte 32 s) of the 128-byte query row at `row`." + what))
    parts.append(asm_fn(pre + "set_load_offsets", "uint32_t o0", f"v_mov_b32 {vr(LOAD_OFF)}, %0", ins=['"v"(o0)'],
                        comment="Once per kernel: the lane's byte offset (row * row stride + swizzled chunk * 16) for the one\n"
                                "wave-wide load that fetches its wave's 8 rows (128 bytes each) of a tile of cached rows." + what))
    issue = [f"s_add_u32 m0, %[d], 0", f"global_load_lds_dwordx4 {vr(LOAD_OFF)}, %[kb] nt",
             f"s_add_u32 m0, %[d], {MAT_BYTES}", f"global_load_lds_dwordx4 {vr(LOAD_OFF)}, %[vb] nt"]
    parts.append(asm_fn(pre + "issue_band", "const void* k_rows, const void* v_rows, uint32_t lds_dst", join(issue),
                        ins=['[kb] "s"(k_rows)', '[vb] "s"(v_rows)', '[d] "s"(lds_dst)'], clobbers=["memory", "m0", "scc"],
                        comment="The wave's two direct-to-LDS loads of a tile whose 8 rows of the wave are all cached rows." + what))
    req = [f"global_load_dwordx4 {vr(SA + 4 * c, 4)}, %[p{c // 4}], off offset:{(c % 4) * 1024} sc1" for c in range(2 * NDB + 1)]
    parts.append(asm_fn(pre + "request_partial", "const void* p0, const void* p1", join(req),
                        ins=['[p0] "v"(p0)', '[p1] "v"(p1)'], clobbers=["memory"],
                        comment="pipe_request_partial() for a block of four chunks and the statistics (p1: 4 KiB behind p0)." + what))
    parts.append(asm_fn(pre + "first_scores", "uint32_t k_next, float& mx", first_scores_block(SA),
                        ['[mx] "=&v"(mx)'], ['[k0] "v"(k_next)'], ["memory"],
                        "S^T of a run's first tile into score set A, and the lane's maximum." + what))
    parts.append(step_fns(pre + "step_ab", SA, SB, True, "One step, in two halves (_x then _y), as pipe_step_ab." + what))
    parts.append(step_fns(pre + "step_ba", SB, SA, True))
    parts.append(step_fns(pre + "last_a", SA, SB, False, "Last step of a run: no next tile." + what))
    parts.append(step_fns(pre + "last_b", SB, SA, False))
    set_head_dim(128)
    return "".join(parts)


def generate():
    reserved = [f"v{i}" for i in range(COMPILER_REGS, 128)] + [f"a{i}" for i in range(COMPILER_REGS, 128)]
    parts = ['''// GENERATED by gen_pipe_step.py -- do not edit.  The generator's header describes the register
// map, the schedule and the hazards the blocks take care of themselves.
//
// These blocks keep their state (score sets, O^T accumulators, Q operand) in v32..v127 and
// a32..a127 without naming those registers in any operand list.  They may only be used in a kernel
// compiled with __attribute__((amdgpu_num_vgpr(32))), whose compiler-allocated registers end at
// v31 / a31, and which calls pipe_reserve() once.
#pragma once

#include "dfx_common.h"

namespace ''' + NAMESPACE + ''' {
''' + ("" if NAMESPACE == "dfx" else "using namespace ::dfx;\n") + '''
''']
    parts.append(asm_fn("pipe_reserve", "", "", clobbers=reserved,
                        comment="Makes the kernel's register count cover the registers of the blocks below (no instruction)."))
    parts.append(asm_fn("pipe_zero_outputs", "", join(f"v_accvgpr_write_b32 {ar(O_BASE + i)}, 0" for i in range(16 * NDB)),
                        comment="O^T = 0."))
    # rescale: four at a time so that each read has three instructions behind it before its use
    resc = list(MFMA_TO_VALU)
    for g in range(0, 16 * NDB, 4):
        resc += [f"v_accvgpr_read_b32 {vr(TMP + i - g)}, {ar(O_BASE + i)}" for i in range(g, g + 4)]
        resc += [f"v_mul_f32 {vr(TMP + i - g)}, {vr(TMP + i - g)}, %[alpha]" for i in range(g, g + 4)]
        resc += [f"v_accvgpr_write_b32 {ar(O_BASE + i)}, {vr(TMP + i - g)}" for i in range(g, g + 4)]
    parts.append(asm_fn("pipe_rescale_outputs", "float alpha", join(resc), ins=['[alpha] "v"(alpha)'],
                        comment="O^T *= alpha (per lane: one query row per lane column), behind the wait states for the matrix results."))
    # queries: 8 x 16-byte loads of the lane's row half straight into the Q operand registers
    ql = [f"global_load_dwordx4 {ar(Q_BASE + 4 * s, 4)}, %[p], off offset:{s * 32}" for s in range(NSLAB)]
    parts.append(asm_fn("pipe_issue_queries", "const void* row", join(ql), ins=['[p] "v"(row)'], clobbers=["memory"],
                        comment="Q operand: requests the lane's half (64 bytes of every 128: slab s at byte 32 s) of the query row at\n"
                                "`row` (lanes without a row of their own pass any readable row: their columns of S^T and O^T are\n"
                                "never stored).  The caller waits for the loads (vmcnt) before the next matrix instruction, and\n"
                                "no matrix instruction that reads the previous Q operand may still be in flight."))
    parts.append(asm_fn("pipe_set_load_offsets", "uint32_t o0, uint32_t o1",
                        join(f"v_mov_b32 {vr(LOAD_OFF + j)}, %{j}" for j in range(2)), ins=['"v"(o0)', '"v"(o1)'],
                        comment="Once per kernel: the lane's byte offsets (row * row stride + swizzled chunk * 16) for the two\n"
                                "wave-wide loads that fetch its wave's 8 rows of a tile of cached rows."))
    issue = []
    for j in range(2):
        issue += [f"s_add_u32 m0, %[d], {j * 1024}", f"global_load_lds_dwordx4 {vr(LOAD_OFF + j)}, %[kb] nt",
                  f"s_add_u32 m0, %[d], {MAT_BYTES + j * 1024}", f"global_load_lds_dwordx4 {vr(LOAD_OFF + j)}, %[vb] nt"]
    parts.append(asm_fn("pipe_issue_band", "const void* k_rows, const void* v_rows, uint32_t lds_dst", join(issue),
                        ins=['[kb] "s"(k_rows)', '[vb] "s"(v_rows)', '[d] "s"(lds_dst)'], clobbers=["memory", "m0", "scc"],
                        comment="The wave's four direct-to-LDS loads of a tile whose 8 rows of the wave are all cached rows (K rows at\n"
                                "k_rows, V rows at v_rows, both wave-uniform; lds_dst: the wave's place in the K tile of the ring stage):\n"
                                "no vector instruction, the offsets are those of pipe_set_load_offsets."))
    parts.append(asm_fn("pipe_set_fresh_offsets", "uint32_t o0, uint32_t o1",
                        join(f"v_mov_b32 {vr(FRESH_OFF + j)}, %{j}" for j in range(2)), ins=['"v"(o0)', '"v"(o1)'],
                        comment="Once per kernel (two-byte cache elements): the same offsets for the K rows of a band of fresh rows,\n"
                                "which lie a token of k_new apart."))
    issue_fresh = []
    for j in range(2):  # K rows with the offsets of pipe_set_fresh_offsets, V rows with those of pipe_set_load_offsets
        issue_fresh += [f"s_add_u32 m0, %[d], {j * 1024}", f"global_load_lds_dwordx4 {vr(FRESH_OFF + j)}, %[kb] nt",
                        f"s_add_u32 m0, %[d], {MAT_BYTES + j * 1024}", f"global_load_lds_dwordx4 {vr(LOAD_OFF + j)}, %[vb] nt"]
    parts.append(asm_fn("pipe_issue_band_fresh", "const void* k_rows, const void* v_rows, uint32_t lds_dst",
                        join(issue_fresh),
                        ins=['[kb] "s"(k_rows)', '[vb] "s"(v_rows)', '[d] "s"(lds_dst)'], clobbers=["memory", "m0", "scc"],
                        comment="pipe_issue_band() for a full band of fresh rows in a launch without a cache: the K rows lie a token of\n"
                                "k_new apart (pipe_set_fresh_offsets), the V rows a token of v_new (pipe_set_load_offsets, free there)."))
    issue8 = [f"s_add_u32 m0, %[d], 0", f"global_load_lds_dwordx4 {vr(LOAD_OFF)}, %[kb] nt",
              f"s_add_u32 m0, %[d], {MAT_BYTES // 2}", f"global_load_lds_dwordx4 {vr(LOAD_OFF)}, %[vb] nt"]
    parts.append(asm_fn("pipe_issue_band_fp8", "const void* k_rows, const void* v_rows, uint32_t lds_dst", join(issue8),
                        ins=['[kb] "s"(k_rows)', '[vb] "s"(v_rows)', '[d] "s"(lds_dst)'], clobbers=["memory", "m0", "scc"],
                        comment="The same for a cache of one-byte codes: a wave's 8 rows of a tile are one load each for K and V (the\n"
                                "first offset of pipe_set_load_offsets), and the V codes of a stage follow its K codes."))
    parts.append(asm_fn("pipe_set_widen_addresses", "uint32_t raw, uint32_t lo, uint32_t hi",
                        join(f"v_mov_b32 {vr(WIDEN_ADDR + j)}, %{j}" for j in range(3)), ins=['"v"(raw)', '"v"(lo)', '"v"(hi)'],
                        comment="Once per kernel (cache of one-byte codes): LDS addresses of the 16 codes the lane widens in stage 0 of the\n"
                                "ring (K; V follows at pipe_widen's offsets) and of the two 16-byte chunks they become in widened tile 0."))
    w = Block()
    ta, tb2 = TMP, TMP + 1
    w.valu(f"v_add_u32 {vr(ta)}, %[rk], {vr(WIDEN_ADDR)}", {ta})
    w.valu(f"v_add_u32 {vr(tb2)}, %[rv], {vr(WIDEN_ADDR)}", {tb2})
    w.other(f"ds_read_b128 {vr(RING, 4)}, {vr(ta)}")
    w.other(f"ds_read_b128 {vr(RING + 4, 4)}, {vr(tb2)}")
    for j, (sel, which) in enumerate((("wk", 1), ("wk", 2), ("wv", 1), ("wv", 2))):
        w.valu(f"v_add_u32 {vr(TMP + 2 + j)}, %[{sel}], {vr(WIDEN_ADDR + which)}", {TMP + 2 + j})
    def widen(src, dst):  # 4 registers of codes -> 8 registers of bf16 pairs; dst may end on src's last registers
        for q in range(4):
            w.valu(f"v_cvt_scalef32_pk_bf16_fp8 {vr(dst + 2 * q)}, {vr(src + q)}, 1.0", {dst + 2 * q})
            w.valu(f"v_cvt_scalef32_pk_bf16_fp8 {vr(dst + 2 * q + 1)}, {vr(src + q)}, 1.0 op_sel:[1,0,0]", {dst + 2 * q + 1})
    w.other("s_waitcnt lgkmcnt(1)")
    widen(RING, RING + 8)
    w.other(f"ds_write_b128 {vr(TMP + 2)}, {vr(RING + 8, 4)}")
    w.other(f"ds_write_b128 {vr(TMP + 3)}, {vr(RING + 12, 4)}")
    w.other("s_waitcnt lgkmcnt(2)")
    widen(RING + 4, RING)   # (register RING + 4 + q is read by the instructions that write RING + 2q, 2q + 1 <= RING + 4 + q: in order)
    w.other(f"ds_write_b128 {vr(TMP + 4)}, {vr(RING, 4)}")
    w.other(f"ds_write_b128 {vr(TMP + 5)}, {vr(RING + 4, 4)}")
    parts.append(asm_fn("pipe_widen", "uint32_t raw_k, uint32_t raw_v, uint32_t wide_k, uint32_t wide_v", w.text(),
                        ins=['[rk] "s"(raw_k)', '[rv] "s"(raw_v)', '[wk] "s"(wide_k)', '[wv] "s"(wide_v)'], clobbers=["memory"],
                        comment="Widens the lane's 16 K codes at raw_k and 16 V codes at raw_v (byte offsets from the address given for\n"
                                "stage 0) into the widened tiles at wide_k and wide_v (byte offsets from widened tile 0): both reads first,\n"
                                "one instruction per pair of codes (exact), in the operand ring's registers, which are free between the\n"
                                "blocks of two steps.  The writes are waited for by whatever waits for LDS next (lgkmcnt)."))
    # a stored piece of a cut item (a block of 8 chunks and the statistics, 1 KiB apart, 16 bytes per lane) into
    # score set A and the first registers of set B, all nine loads in flight at once
    req = []
    for c in range(9):
        req.append(f"global_load_dwordx4 {vr(SA + 4 * c, 4)}, %[p{c // 3}], off offset:{(c % 3) * 1024} sc1")
    parts.append(asm_fn("pipe_request_partial", "const void* p0, const void* p1, const void* p2", join(req),
                        ins=['[p0] "v"(p0)', '[p1] "v"(p1)', '[p2] "v"(p2)'], clobbers=["memory"],
                        comment="Requests the lane's nine 16-byte pieces of a stored block (p0: the lane's address in the block's first\n"
                                "chunk; p1, p2: 3 and 6 KiB further) with device scope into the score sets, which are free between two\n"
                                "runs.  The caller waits for the loads (vmcnt) before pipe_partial_chunk()."))
    for c in range(9):
        outs = [f'"=v"(x[{e}])' for e in range(4)]
        body = join(f"v_mov_b32 %{e}, {vr(SA + 4 * c + e)}" for e in range(4))
        parts.append(f'''DFX_D u32x4 pipe_partial_chunk_{c}() {{
    uint32_t x[4];
    asm volatile("{body}"
                 : {", ".join(outs)});
    return u32x4{{x[0], x[1], x[2], x[3]}};
}}

''')
    parts.append('''// Piece c (0..7: chunks, 8: the statistics; a compile-time constant after unrolling) of what
// pipe_request_partial() has loaded.
DFX_D u32x4 pipe_partial_chunk(int c) {
    switch (c) {
''' + "".join(f"        case {c}: return pipe_partial_chunk_{c}();\n" for c in range(8)) + '''        default: return pipe_partial_chunk_8();
    }
}

''')
    parts.append(rope_queries_fns())
    parts.append(rope_row_fn())
    parts.append(rope_row_fn(with_v=True))
    for d in range(NDB):
        outs = [f'"=v"(x[{e}])' for e in range(16)]
        body = join(f"v_accvgpr_read_b32 %{e}, {ar(O_BASE + 16 * d + e)}" for e in range(16))
        parts.append(f'''DFX_D f32x16 pipe_get_output_{d}() {{
    float x[16];
    asm volatile("{body}"
                 : {", ".join(outs)});
    f32x16 v;
#pragma unroll
    for (int e = 0; e < 16; ++e) v[e] = x[e];
    return v;
}}

''')
        ins = [f'"v"(v[{e}])' for e in range(16)]
        body = join(f"v_accvgpr_write_b32 {ar(O_BASE + 16 * d + e)}, %{e}" for e in range(16))
        parts.append(f'''DFX_D void pipe_set_output_{d}(const f32x16& v) {{
    asm volatile("{body}"
                 :
                 : {", ".join(ins)});
}}

''')
    parts.append('''// d block db of the O^T accumulators (db a compile-time constant after unrolling).  The caller
// has waited for the matrix results (pipe_outputs_ready()).
DFX_D f32x16 pipe_get_output(int db) {
    switch (db) {
        case 0: return pipe_get_output_0();
        case 1: return pipe_get_output_1();
        case 2: return pipe_get_output_2();
        default: return pipe_get_output_3();
    }
}
DFX_D void pipe_set_output(int db, const f32x16& v) {
    switch (db) {
        case 0: pipe_set_output_0(v); break;
        case 1: pipe_set_output_1(v); break;
        case 2: pipe_set_output_2(v); break;
        default: pipe_set_output_3(v); break;
    }
}

DFX_D void pipe_outputs_ready() { asm volatile("s_nop 15\\n\\ts_nop 1" ::: "memory"); }

''')
    for nm, s in (("a", SA), ("b", SB)):
        hide = [f"v_mov_b32 {vr(s)}, {NEG_INF}"] + [f"v_mov_b32 {vr(s + j)}, {vr(s)}" for j in range(1, 32)] + [f"v_mov_b32 %[mx], {vr(s)}"]
        parts.append(asm_fn(f"pipe_hide_{nm}", "float& mx", join(hide), ['[mx] "=&v"(mx)'], [], [],
                            f"Score set {nm.upper()} of a tile the wave's rows see nothing of: every score and the lane's maximum -inf (what the\n"
                            "mask blocks make of such a tile; any tile layout and head_dim).  The set's matrix results are ready."))
    global LAYOUT
    for LAYOUT, pre, what in (("u", "pipe_", ""), ("d", "pipe_d_", "  Tiles of a cache in the distinct layout.")):
        parts.append(asm_fn(pre + "first_scores", "uint32_t k_next, float& mx", first_scores_block(SA),
                            ['[mx] "=&v"(mx)'], ['[k0] "v"(k_next)'], ["memory"],
                            "S^T of a run's first tile (LDS address k_next: tile + the lane's K operand offset) into score\nset A, and the lane's maximum." + what))
        for hole_rows in (8, 16):
            for nm, s in (("a", SA), ("b", SB)):
                parts.append(asm_fn(f"{pre}mask_{nm}_{hole_rows}", "int thr, uint32_t holes, float& mx", mask_block(s, hole_rows),
                                    ['[mx] "=&v"(mx)'], ['[thr] "v"(thr)', '[holes] "s"(holes)'], ["vcc", "scc"],
                                    f"Mask of score set {nm.upper()} (tokens >= thr of the tile, and the {hole_rows}-token bands whose bit in `holes` is set,\n"
                                    "become -inf) and the lane's maximum of the masked set." + what))
        parts.append(step_fns(pre + "step_ab", SA, SB, True,
                              "One step, in two halves (_x then _y): softmax and O^T += V^T P^T of the current score set (A; v_cur:\n"
                              "LDS address of the V tile + the lane's V^T operand offset), S^T of the next tile into the other set\n"
                              "and its lane maximum." + what))
        parts.append(step_fns(pre + "step_ba", SB, SA, True))
        parts.append(step_fns(pre + "last_a", SA, SB, False, "Last step of a run: no next tile." + what))
        parts.append(step_fns(pre + "last_b", SB, SA, False))
    LAYOUT = "u"
    parts.append(asm_fn("pipe_d_set_load_offsets", "uint32_t k, uint32_t v0, uint32_t v1",
                        join(f"v_mov_b32 {vr(LOAD_OFF + j)}, %{j}" for j in range(3)), ins=['"v"(k)', '"v"(v0)', '"v"(v1)'],
                        comment="Once per kernel (distinct layout): the lane's byte offsets for the wave's loads of a full tile of cached\n"
                                "rows: inside a chunk column of K (its token), and inside the (page, head) of V for the two rows of V^T it\n"
                                "fetches a chunk of (row * row stride + the chunk its place in the row holds)."))
    issue_d = [f"s_add_u32 m0, %[d], 0", f"global_load_lds_dwordx4 {vr(LOAD_OFF)}, %[k0] nt",
               f"s_add_u32 m0, %[d], 1024", f"global_load_lds_dwordx4 {vr(LOAD_OFF)}, %[k1] nt",
               f"s_add_u32 m0, %[d], {MAT_BYTES}", f"global_load_lds_dwordx4 {vr(LOAD_OFF + 1)}, %[vb] nt",
               f"s_add_u32 m0, %[d], {MAT_BYTES + 1024}", f"global_load_lds_dwordx4 {vr(LOAD_OFF + 2)}, %[vb] nt"]
    parts.append(asm_fn("pipe_d_issue_band", "const void* k_col0, const void* k_col1, const void* v_rows, uint32_t lds_dst", join(issue_d),
                        ins=['[k0] "s"(k_col0)', '[k1] "s"(k_col1)', '[vb] "s"(v_rows)', '[d] "s"(lds_dst)'], clobbers=["memory", "m0", "scc"],
                        comment="The wave's four direct-to-LDS loads of a full tile of cached rows in the distinct layout: its two chunk\n"
                                "columns of K (64 tokens of each at k_col0 / k_col1) and its 16 rows of V^T (v_rows: the tile's first token\n"
                                "in row 0 of the (page, head)); lds_dst: the wave's place in the K tile of the ring stage."))
    parts.append(head_dim_64_family())
    parts.append(f"}}  // namespace {NAMESPACE}\n")
    return "".join(parts)


def main(out=None, only=None, namespace="dfx"):
    """Writes the blocks to `out` (default: attn_pipe_gen.h beside this file, what the library is built from).
    only / namespace: a timing variant for step_bench.hip in a namespace of its own."""
    global ONLY, NAMESPACE
    out = out or os.path.join(HERE, "attn_pipe_gen.h")
    ONLY, NAMESPACE = only, namespace
    try:
        text = generate()
    finally:
        ONLY, NAMESPACE = None, "dfx"
    if not os.path.exists(out) or open(out).read() != text:
        with open(out, "w") as f:
            f.write(text)
    return out


if __name__ == "__main__":
    print(main())
