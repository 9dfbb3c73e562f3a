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
v216-v223 tile pool and prefetch values (see the kernel), s90-s95 scratch.

Run ``python gen_scan_asm.py`` after changing the schedule; the generated file is committed.
"""
import os
import sys

F = [128, 160]
VT = 192
VADDR_A, VADDR_B = 200, 204
VOFF = 208
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


def kstep(fresh):
    """One K step.  Operands: [sa] / [sb] LDS stage of the step's query / K_r tile (advanced to the next step's),
    [ra] / [rb] resources the loads of this step read, [k] their byte offset inside a row, [woff] wave * 8 KB."""
    out = []
    e = out.append
    e(f"s_mov_b32 {S_M0}, m0")
    e(f"s_add_u32 {S_BN}, %[sb], 0x8000")
    e(f"s_cmp_eq_u32 {S_BN}, {BEND:#x}")
    e(f"s_cselect_b32 {S_BN}, {B0:#x}, {S_BN}")
    e(f"s_sub_u32 {S_BLD}, %[sb], 0x8000")
    e(f"s_cmp_lt_u32 {S_BLD}, {B0:#x}")
    e(f"s_cselect_b32 {S_BLD}, {BEND - 0x8000:#x}, {S_BLD}")
    e(f"s_xor_b32 {S_AN}, %[sa], 0x8000")
    for s in (1, 2, 3):
        e(f"v_add_u32 v{VT + 2 * (s - 1)}, %[sa], v{VADDR_A + s}")
        e(f"v_add_u32 v{VT + 2 * (s - 1) + 1}, %[sb], v{VADDR_B + s}")
    e(f"v_add_u32 v{VT + 6}, {S_AN}, v{VADDR_A}")
    e(f"v_add_u32 v{VT + 7}, {S_BN}, v{VADDR_B}")
    e(f"s_add_u32 {S_BLD}, {S_BLD}, %[woff]")
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
            e(f"v_mfma_f32_32x32x16_bf16 {acc(i, j)}, {fa(slot, i)}, {fb(slot, j)}, {c}")
            if sub == 3 and n == 0:
                e("s_barrier")
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
    return out


def define(name, lines):
    body = " \\\n".join(f'  "{l}\\n\\t"' for l in lines)
    return f"#define {name} \\\n{body}\n"


def main():
    parts = ["// Generated by gen_scan_asm.py (the schedule and the register map are described there).  Do not edit.\n"]
    parts.append(define("MSA_SCAN4_KSTEP", kstep(False)))
    parts.append(define("MSA_SCAN4_KSTEP_FRESH", kstep(True)))
    # the eight accumulator blocks' registers, 16 floats each
    for n in range(16):
        parts.append(define(f"MSA_SCAN4_ACC_READ_{n}", [f"v_accvgpr_read_b32 %{x}, a{n * 16 + x}" for x in range(16)]))
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
    regs = [f"v{r}" for r in range(128, 256)] + [f"a{r}" for r in range(256)] + ["s90", "s91", "s92", "s93", "s94", "s95", "scc", "memory"]
    parts.append("#define MSA_SCAN4_CLOBBERS " + ", ".join(f'"{x}"' for x in regs) + "\n")
    text = "\n".join(parts)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "scan_asm.inc")
    if len(sys.argv) > 1 and sys.argv[1] == "--check":
        return 0 if open(path).read() == text else 1
    open(path, "w").write(text)
    return 0


if __name__ == "__main__":
    sys.exit(main())
