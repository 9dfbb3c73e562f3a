#!/usr/bin/env python3
"""Writes ``scan_asm.inc``: the instruction-level K step of the large-tile routing scan (``score_scan4_kernel``).

The scan's 256 x 256 tile is computed by four wavefronts, one per SIMD, 128 x 128 each: sixteen 32 x 32
accumulators in the 256 accumulation registers a0-a255, operand fragments double-buffered in v128-v191.  One K step
(64 elements of K: 64 MFMAs per wavefront) is one asm statement whose issue order is fixed here:

* sub-step s (16 MFMAs on fragment slot s & 1) carries the eight LDS reads of sub-step s + 1 behind its first eight
  MFMAs, one read per MFMA;
* the eight 1 KB blocks of the K_r tile two steps ahead are requested during sub-step 0 and those of the query tile
  two steps ahead during sub-step 3, one ``buffer_load_dwordx4 ... lds`` behind every second MFMA (the compute unit's
  address unit takes about that long per load of four wavefronts), M0 set one instruction earlier;
* the step's only wait for memory (everything but the eight newest loads) and the workgroup barrier sit at the start
  of sub-step 3, the barrier behind that sub-step's first MFMA so that the matrix pipe runs while the wavefronts meet;
  behind the barrier the stages this step has finished with are refilled and the first fragments of the next step
  are read.

LDS: two stages of the query tile at 0 / 0x8000, three of the K_r tile at 0x10000 / 0x18000 / 0x20000, rows of 128
bytes whose 16-byte units are XOR-swizzled by (row >> 1) & 7.

Registers the statements own (the kernel's compiler-allocated code stays below v128 and uses no accumulation
registers): v128-v159 / v160-v191 fragment slots (A0-A3, B0-B3), v192-v199 LDS addresses of the step, v200-v207
per-lane LDS offsets of sub-steps 0-3 (A, then B), v208-v215 global offsets of the wavefront's eight 1 KB blocks,
v216-v223 tile pool and prefetch values (see the kernel), v224-v239 the maxima of the sixteen accumulator blocks of
the tile just finished (block (i, j) in v224 + 4 i + j; in the folding form the maxima over the four row blocks, column
block j in v224 + j), v240-v247 scratch of the reduction and the fold, v248-v252 per-lane constants of the fold,
s76-s95 scratch.

The reduction of a finished tile (per lane the maximum of each block's sixteen values: sixteen reads of accumulation
registers and eight three-way maxima per block) rides in the first sub-step of the next tile's first K step, block
(i, j) in front of the MFMA that overwrites it: with one wavefront per SIMD the matrix pipe runs under it.  When the
wavefront's four row blocks belong to one query whose rows all count and the tile lies inside the bank, the fold of the
column maxima over the chunks of a document (half-wave swap, order-preserving key, segmented max-scan over the 64
lanes by row moves, one atomic per document run) follows in the same statement, dealt out behind the MFMAs of
sub-steps 1 and 2; its atomics are issued behind the step's wait so that the wait does not count them.

Run ``python gen_scan_asm.py`` after changing the schedule; the generated file is committed.
"""
import os
import sys

F = [128, 160]
VT = 192
VADDR_A, VADDR_B = 200, 204
VOFF = 208
VMAX = 224
VRED = 240           # 8 scratch registers; the fold's temporaries: pair p in v(240 + 4 p) .. v(243 + 4 p)
V_LOWMASK, V_DISTBASE, V_L32P1, V_IS31, V_L15 = 248, 249, 250, 251, 252
VDOC = 220           # documents of the wavefront's columns: pair p in v(220 + p)
S_HALF = "s[86:87]"  # lanes 32 - 63
S_M0, S_AN, S_BN, S_BLD = "s92", "s93", "s94", "s95"
B0, BEND = 0x10000, 0x28000

# MFMA order inside a sub-step and the order in which the next sub-step's fragments are read (what is needed first)
ORDER = [(0, 0), (0, 1), (1, 0), (1, 1), (0, 2), (0, 3), (1, 2), (1, 3),
         (2, 0), (2, 1), (2, 2), (2, 3), (3, 0), (3, 1), (3, 2), (3, 3)]
READS = [("a", 0), ("b", 0), ("b", 1), ("a", 1), ("b", 2), ("b", 3), ("a", 2), ("a", 3)]


def acc(i, j):
    b = (i * 4 + j) * 16
    return f"a[{b}:{b + 15}]"


def fa(slot, i):
    b = F[slot] + i * 4
    return f"v[{b}:{b + 3}]"


def fb(slot, j):
    b = F[slot] + 16 + j * 4
    return f"v[{b}:{b + 3}]"


def reduce_block(i, j, joined=False):
    """Per-lane maximum of accumulator block (i, j) into v(VMAX + 4 i + j); joined: into v(VMAX + j), over the row
    blocks i as well.  Two halves of eight values, each a tree of depth three (a wavefront that is alone on its SIMD
    waits out every dependent instruction)."""
    b = (i * 4 + j) * 16
    m = f"v{VMAX + j}" if joined else f"v{VMAX + i * 4 + j}"
    r = [f"v{VRED + x}" for x in range(8)]
    out = []
    for h in range(2):
        out += [f"v_accvgpr_read_b32 {r[x]}, a{b + 8 * h + x}" for x in range(8)]
        out.append(f"v_max3_f32 {r[0]}, {r[0]}, {r[1]}, {r[2]}")
        out.append(f"v_max3_f32 {r[3]}, {r[3]}, {r[4]}, {r[5]}")
        out.append(f"v_max3_f32 {r[0]}, {r[0]}, {r[3]}, {r[6]}")
        if h == 0 and not (joined and i > 0):
            out.append(f"v_max_f32 {m}, {r[0]}, {r[7]}")
        else:
            out.append(f"v_max3_f32 {m}, {m}, {r[0]}, {r[7]}")
    return out


def fold_pair(p):
    """Document fold of column blocks 2p / 2p + 1 (maxima over the rows in v(VMAX + 2p), v(VMAX + 2p + 1), documents of
    the 64 columns in v(VDOC + p)): returns (instructions, the masked atomic).  [okey]: the query's row of keys."""
    R, H, doc = f"v{VMAX + 2 * p}", f"v{VMAX + 2 * p + 1}", f"v{VDOC + p}"
    t0, t1, t2, t3 = (f"v{VRED + 4 * p + x}" for x in range(4))
    sc = f"s[{80 + 2 * p}:{81 + 2 * p}]"        # a condition
    shl, shh = f"s{76 + 2 * p}", f"s{77 + 2 * p}"   # run heads, one bit per lane
    sx = "s[88:89]"                             # exec saved around the atomic
    o = []
    o.append(f"v_permlane32_swap_b32 {R}, {H}")            # lower 32 lanes: block 2p, upper 32: block 2p + 1
    o.append(f"v_max_f32 {R}, {R}, {H}")
    o.append(f"v_ashrrev_i32 {t0}, 31, {R}")               # order-preserving key of the float
    o.append(f"v_or_b32 {t0}, 0x80000000, {t0}")
    o.append(f"v_xor_b32 {R}, {R}, {t0}")
    o.append(f"v_mov_b32 {t1}, {doc}")                     # the document of the lane below (lane 0: its own)
    o.append(f"v_mov_b32_dpp {t1}, {doc} wave_shr:1 row_mask:0xf bank_mask:0xf")
    o.append(f"v_cmp_ne_u32_e64 s[{shl[1:]}:{shh[1:]}], {t1}, {doc}")
    o.append(f"s_or_b32 {shl}, {shl}, 1")                  # lanes 0 and 32 open a run
    o.append(f"s_or_b32 {shh}, {shh}, 1")
    o.append(f"v_mov_b32 {t1}, {shl}")
    o.append(f"v_mov_b32 {t2}, {shh}")
    o.append(f"v_cndmask_b32_e64 {t1}, {t1}, {t2}, {S_HALF}")      # the heads of the lane's half
    o.append(f"v_and_b32 {t2}, v{V_LOWMASK}, {t1}")        # heads at or below the lane (never empty)
    o.append(f"v_ffbh_u32 {t2}, {t2}")
    o.append(f"v_add_u32 {t2}, {t2}, v{V_DISTBASE}")       # distance from the run's first lane: l32 - 31 + leading zeros
    o.append(f"v_lshrrev_b32 {t3}, v{V_L32P1}, {t1}")
    o.append(f"v_and_b32 {t3}, 1, {t3}")
    o.append(f"v_or_b32 {t3}, {t3}, v{V_IS31}")            # non-zero: last lane of its run
    for k in (1, 2, 4, 8):                                 # segmented max-scan inside the rows of 16 lanes
        o.append(f"v_max_u32_dpp {t0}, {R}, {R} row_shr:{k} row_mask:0xf bank_mask:0xf bound_ctrl:0")
        o.append(f"v_cmp_le_u32_e64 {sc}, {k}, {t2}")
        o.append(f"v_cndmask_b32_e64 {R}, {R}, {t0}, {sc}")
    o.append(f"v_mov_b32 {t0}, 0")                         # lane 15 of the lower row joins the runs that cross into the upper
    o.append(f"v_mov_b32_dpp {t0}, {R} row_bcast:15 row_mask:0xa bank_mask:0xf")
    o.append(f"v_max_u32 {t0}, {t0}, {R}")
    o.append(f"v_cmp_gt_u32_e64 {sc}, {t2}, v{V_L15}")
    o.append(f"v_cndmask_b32_e64 {R}, {R}, {t0}, {sc}")
    o.append(f"v_lshlrev_b32 {t0}, 2, {doc}")
    o.append(f"v_cmp_ne_u32_e64 {sc}, 0, {t3}")
    atomic = [f"s_and_saveexec_b64 {sx}, {sc}", f"global_atomic_umax {t0}, {R}, %[okey]", f"s_mov_b64 exec, {sx}"]
    return o, atomic


def interleave(a, b):
    out = []
    for x, y in zip(a, b):
        out += [x, y]
    return out + a[len(b):] + b[len(a):]


def written_vgprs(line):
    """Vector registers an instruction writes (first operand of v_* / ds_read*; v_permlane32_swap writes both)."""
    import re
    op, _, rest = line.partition(" ")
    if not (op.startswith("v_") or op.startswith("ds_read")) or op.startswith("v_mfma") or op.startswith("v_cmp"):
        return set()
    ops = [x.strip() for x in rest.split(",")]
    targets = ops[:2] if op.startswith("v_permlane") else ops[:1]
    regs = set()
    for t in targets:
        m = re.match(r"v\[(\d+):(\d+)\]", t)
        if m:
            regs |= set(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            m = re.match(r"v(\d+)$", t)
            if m:
                regs.add(int(m.group(1)))
    return regs


def fix_lane_move_hazards(lines):
    """A DPP operand or a half-wave swap reads its registers two wait states after a VALU write at the earliest."""
    import re
    out = []
    for line in lines:
        op = line.split(" ")[0]
        if op.endswith("_dpp") or op.startswith("v_permlane"):
            reads = {int(x) for x in re.findall(r"\bv(\d+)\b", line)}
            dist = 0
            need = 0
            for prev in reversed(out):
                if dist >= 2:
                    break
                if written_vgprs(prev) & reads:
                    need = 2 - dist
                    break
                dist += int(prev.split(" ")[1]) + 1 if prev.startswith("s_nop") else 1
            if need:
                out.append(f"s_nop {need - 1}")
        out.append(line)
    return out


def kstep(fresh, reduce=None):
    """One K step.  Operands: [sa] / [sb] LDS stage of the step's query / K_r tile (advanced to the next step's),
    [ra] / [rb] resources the loads of this step read, [k] their byte offset inside a row, [woff] wave * 8 KB.
    fresh: a tile's first step (the first sub-step multiplies into zero); reduce: it also reduces the accumulators the
    previous tile left, "blocks" to one maximum per block, "fold" on to the key plane ([okey]: the query's keys)."""
    out = []
    e = out.append
    fillers, atomics = [], []
    if reduce == "fold":
        (a0, at0), (a1, at1) = fold_pair(0), fold_pair(1)
        fillers = interleave(a0, a1)
        atomics = at0 + at1
    per_slot = -(-len(fillers) // 32)
    # The step's scalar and address arithmetic stands behind its first MFMAs, not in front of them (a wavefront that
    # is alone on its SIMD pays for every instruction the matrix pipe does not run under): `early` is what the first
    # LDS read and the first tile load need, `later` the rest, three instructions per MFMA.
    early = [f"s_mov_b32 {S_M0}, m0",
             f"v_add_u32 v{VT}, %[sa], v{VADDR_A + 1}", f"v_add_u32 v{VT + 1}, %[sb], v{VADDR_B + 1}",
             f"s_sub_u32 {S_BLD}, %[sb], 0x8000", f"s_cmp_lt_u32 {S_BLD}, {B0:#x}",
             f"s_cselect_b32 {S_BLD}, {BEND - 0x8000:#x}, {S_BLD}", f"s_add_u32 {S_BLD}, {S_BLD}, %[woff]"]
    later = [f"s_add_u32 {S_BN}, %[sb], 0x8000", f"s_cmp_eq_u32 {S_BN}, {BEND:#x}", f"s_cselect_b32 {S_BN}, {B0:#x}, {S_BN}",
             f"s_xor_b32 {S_AN}, %[sa], 0x8000", f"v_add_u32 v{VT + 2}, %[sa], v{VADDR_A + 2}", f"v_add_u32 v{VT + 3}, %[sb], v{VADDR_B + 2}",
             f"v_add_u32 v{VT + 4}, %[sa], v{VADDR_A + 3}", f"v_add_u32 v{VT + 5}, %[sb], v{VADDR_B + 3}", f"v_add_u32 v{VT + 6}, {S_AN}, v{VADDR_A}",
             f"v_add_u32 v{VT + 7}, {S_BN}, v{VADDR_B}"]
    if reduce == "fold":
        later += ["s_mov_b32 s86, 0", "s_mov_b32 s87, -1"]
    for sub in range(4):
        slot, nslot = sub & 1, (sub & 1) ^ 1
        va, vb = (VT + 2 * sub, VT + 2 * sub + 1) if sub < 3 else (VT + 6, VT + 7)
        e("s_waitcnt vmcnt(8) lgkmcnt(0)" if sub == 3 else "s_waitcnt lgkmcnt(0)")
        nload = 0
        for n, (i, j) in enumerate(ORDER):
            do_load = sub in (0, 3) and n % 2 == 1
            if do_load:
                if nload > 0:
                    e("s_add_u32 m0, m0, 0x400")
                elif sub == 0:
                    e(f"s_mov_b32 m0, {S_BLD}")
                else:
                    e("s_add_u32 m0, %[sa], %[woff]")
            c = "0" if (fresh and sub == 0) else acc(i, j)
            if reduce and sub == 0:
                out.extend(reduce_block(i, j, joined=reduce == "fold"))
            e(f"v_mfma_f32_32x32x16_bf16 {acc(i, j)}, {fa(slot, i)}, {fb(slot, j)}, {c}")
            if sub == 3 and n == 0:
                e("s_barrier")
            if sub == 0 and n == 0:
                out.extend(early)
            if sub == 0 and n >= 1:
                for _ in range(3):
                    if later:
                        e(later.pop(0))
            if sub in (1, 2):
                for _ in range(per_slot):
                    if fillers:
                        e(fillers.pop(0))
            if sub == 3 and n in (10, 12) and atomics:
                for _ in range(3):
                    e(atomics.pop(0))
            rd = n if sub < 3 else n - 1
            if 0 <= rd < 8:
                kind, idx = READS[rd]
                if kind == "a":
                    e(f"ds_read_b128 {fa(nslot, idx)}, v{va} offset:{idx * 4096}")
                else:
                    e(f"ds_read_b128 {fb(nslot, idx)}, v{vb} offset:{idx * 4096}")
            if do_load:
                if sub == 0:
                    e(f"buffer_load_dwordx4 v{VOFF + nload}, %[rb], %[k] offen nt lds")
                else:
                    e(f"buffer_load_dwordx4 v{VOFF + nload}, %[ra], %[k] offen lds")
                nload += 1
    e(f"s_mov_b32 %[sa], {S_AN}")
    e(f"s_mov_b32 %[sb], {S_BN}")
    e(f"s_mov_b32 m0, {S_M0}")
    assert not fillers and not atomics and not later
    return fix_lane_move_hazards(out)


def define(name, lines):
    body = " \\\n".join(f'  "{l}\\n\\t"' for l in lines)
    return f"#define {name} \\\n{body}\n"


def main():
    parts = ["// Generated by gen_scan_asm.py (the schedule and the register map are described there).  Do not edit.\n"]
    parts.append(define("MSA_SCAN4_KSTEP", kstep(False)))
    parts.append(define("MSA_SCAN4_KSTEP_FRESH", kstep(True)))
    parts.append(define("MSA_SCAN4_KSTEP_FRESH_REDUCE", kstep(True, "blocks")))
    parts.append(define("MSA_SCAN4_KSTEP_FRESH_FOLD", kstep(True, "fold")))
    # the reduction by itself, behind a workgroup's last tile (an MFMA's result may be read 18 wait states after its
    # issue at the earliest)
    parts.append(define("MSA_SCAN4_REDUCE", ["s_nop 15", "s_nop 7"] + [l for (i, j) in ORDER for l in reduce_block(i, j)]))
    parts.append(define("MSA_SCAN4_MAX_READ", [f"v_mov_b32 %{x}, v{VMAX + x}" for x in range(16)]))
    # fragments of sub-step 0 out of the stages [sa] / [sb] into slot 0 (in front of the first step)
    lines = [f"v_add_u32 v{VT + 6}, %[sa], v{VADDR_A}", f"v_add_u32 v{VT + 7}, %[sb], v{VADDR_B}"]
    for kind, idx in READS:
        lines.append(f"ds_read_b128 {fa(0, idx) if kind == 'a' else fb(0, idx)}, v{VT + 6 if kind == 'a' else VT + 7} offset:{idx * 4096}")
    parts.append(define("MSA_SCAN4_FRAGS0", lines))
    # the wavefront's eight blocks of one operand tile into the LDS stage at [dst] (+ wave * 8 KB already added)
    for name, nt in (("MSA_SCAN4_LOAD8", ""), ("MSA_SCAN4_LOAD8_NT", " nt")):
        lines = [f"s_mov_b32 {S_M0}, m0", "s_mov_b32 m0, %[dst]", "s_nop 4"]
        for i in range(8):
            lines.append(f"buffer_load_dwordx4 v{VOFF + i}, %[r], %[k] offen{nt} lds")
            if i < 7:
                lines += ["s_add_u32 m0, m0, 0x400", "s_nop 0"]
        lines.append(f"s_mov_b32 m0, {S_M0}")
        parts.append(define(name, lines))
    parts.append(define("MSA_SCAN4_SET_ADDR", [f"v_mov_b32 v{VADDR_A + s}, %{s}" for s in range(8)]))
    parts.append(define("MSA_SCAN4_SET_VOFF", [f"v_mov_b32 v{VOFF + s}, %{s}" for s in range(8)]))
    # the fold's per-lane constants from l32 = lane & 31 (operand 0)
    parts.append(define("MSA_SCAN4_SET_FOLD", [
        f"v_lshlrev_b32 v{V_LOWMASK}, %0, 2", f"v_add_u32 v{V_LOWMASK}, -1, v{V_LOWMASK}",      # (2 << l32) - 1
        f"v_add_u32 v{V_DISTBASE}, -31, %0", f"v_add_u32 v{V_L32P1}, 1, %0",
        f"v_cmp_eq_u32 vcc, 31, %0", f"v_cndmask_b32 v{V_IS31}, 0, 1, vcc", f"v_and_b32 v{V_L15}, 15, %0"]))
    regs = [f"v{r}" for r in range(128, 256)] + [f"a{r}" for r in range(256)] + [f"s{r}" for r in range(76, 96)] + ["vcc", "scc", "memory"]
    parts.append("#define MSA_SCAN4_CLOBBERS " + ", ".join(f'"{x}"' for x in regs) + "\n")
    text = "\n".join(parts)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "scan_asm.inc")
    if len(sys.argv) > 1 and sys.argv[1] == "--check":
        return 0 if open(path).read() == text else 1
    open(path, "w").write(text)
    return 0


if __name__ == "__main__":
    sys.exit(main())
