#!/usr/bin/env python3
"""Writes ``flash_asm.inc``: the instruction-level tile step of the wide flash-attention kernel (``flash_wide_kernel``).

One wavefront per SIMD owns 64 (token, head) columns in two blocks of 32 (cb = 0, 1).  Per tile of 64 keys it computes
S^T[64 keys x 64 cols] = K . Q^T (32 MFMAs, every K fragment from LDS feeding both column blocks) and
O^T[128 dims x 64 cols] += V^T . P^T (32 MFMAs, every V^T fragment likewise), half the LDS operand reads per MFMA of the
32-column kernel, and all of the softmax's VALU work is dealt out behind those MFMAs in a fixed order.

Step t (tile index i = (t - first) % 6 selects the statement: LDS slots and score buffers are immediates):
  half A   MFMAs: O += V(t-1)^T . P(t-1)^T.   VALU: (mask,) column maxima of S(t), the growth test of the running
           reference maximum, the first exponentials of tile t.  Before the 29th MFMA the step's one wait
           (everything but the eight newest tile loads, all LDS reads) and behind it the workgroup barrier.
  half B   MFMAs: S(t+1) = K(t+1) . Q^T.   VALU: the other exponentials of tile t.  The wavefront's share of the
           tile loads K(t+3), V(t+2) (one ``buffer_load_dwordx4 ... lds`` behind every fourth MFMA).
Between the halves the kernel rescales O when a reference maximum grew (FLASHW_RESCALE, rare).

Scores and probabilities share registers: S(t) lives in one of two 64-register buffers (X = v128-v191 for even i,
Y = v192-v255 for odd i; block (cb, rb) at + 32 cb + 16 rb, element e of a block = key 32 rb + 8 (e >> 2) + 4 half +
(e & 3)); the exponentials of element pair k of a block are packed to bf16 into the block's register k (k < 4) or
8 + k - 4 (k >= 4), i.e. in place behind the elements already consumed, which leaves the B operands of the second
product (keys 16 jj .. + 16 of a column block: four consecutive registers) where the next step's half A reads them.

Registers the statements own (compiler-allocated code stays below v56 and uses no accumulation registers):
  v56-v63   LDS address of the lane's K fragment of contraction step ks (slot 0, key rows 0-31)
  v64-v67   LDS address of the lane's V^T fragment of dim block d (V ring base included, slot 0, keys 0-15)
  v68-v71 / v72-v75   global offsets of the wavefront's four 1 KB blocks of a K / V tile
  v76, v77  running reference maximum m of the lane's column (log2 units), per column block
  v78-v81   row sums (two partial sums per column block: v78 + 2 cb, v79 + 2 cb)
  v82, v83  alpha = 2^(m_old - m_new) of the step, per column block (1 when nothing grew)
  v84, v85  masked steps: column limit minus the tile's first key minus 4 half, per column block (the limits
            minus 4 half wait in a192, a193)
  v86-v95   temporaries
  v96-v127  free
  a0-a127   O^T: block (cb, d) at 64 cb + 16 d;   a128-a191   Q^T fragments: (cb, ks) at 128 + 32 cb + 4 ks
  a196-a211 K fragment ring (4 x 4), a212-a227 V^T fragment ring (4 x 4): fragments are read from LDS a pair ahead
            (the next pair is requested, then one wait covers the pair about to be multiplied), straight into
            accumulation registers: returns into the vector registers compete with the VALU instructions of a
            wavefront that is alone on its SIMD (a half step measured 13 % shorter this way)
  s84-s95   scratch
LDS: K ring at 0 / 0x4000 / 0x8000, V ring at 0xC000 / 0x10000 / 0x14000 (96 KB); behind them 16 KB per wavefront
for the query rows of its next block (two column blocks of 32 rows x 256 bytes).

Hazards kept by construction: a VALU read of an MFMA result stands at least 24 wait states behind the MFMA; a
half-wave swap reads its operands two wait states after their VALU write; one instruction between a write of M0
and the load that uses it.
"""
import os
import re
import sys

V_FIRST = 56        # the statements own v56 - v255
V_KAT, V_VAT, V_KOFF, V_VOFF = 56, 64, 68, 72
V_M, V_L, V_ALPHA, V_REL = 76, 78, 82, 84
V_T = 86            # 10 temporaries
A_KF, A_VA = 196, 212    # fragment rings, in accumulation registers
RING = 4            # fragments per ring
BUF = [128, 192]
KSLOT, VSLOT = 0x4000, 0x4000
VBASE = 0xC000
S_M0 = "s92"
GROW = "0x40c00000"     # 6.0: the reference maximum moves only when a column's maximum grew by more than 2^6
NINF = "0xff800000"


def o_acc(cb, d):
    b = 64 * cb + 16 * d
    return f"a[{b}:{b + 15}]"


def q_frag(cb, ks):
    b = 128 + 32 * cb + 4 * ks
    return f"a[{b}:{b + 3}]"


def s_blk(buf, cb, rb):
    b = BUF[buf] + 32 * cb + 16 * rb
    return f"v[{b}:{b + 15}]"


def p_frag(buf, cb, jj):
    b = BUF[buf] + 32 * cb + 16 * (jj >> 1) + 8 * (jj & 1)
    return f"v[{b}:{b + 3}]"


def kf(f):
    b = A_KF + 4 * (f % RING)
    return f"a[{b}:{b + 3}]"


def va(f):
    b = A_VA + 4 * (f % RING)
    return f"a[{b}:{b + 3}]"


def k_read(f, slot):
    ks, rb = f >> 1, f & 1
    return [f"ds_read_b128 {kf(f)}, v{V_KAT + ks} offset:{slot * KSLOT + rb * 8192}"]


def v_read(f, slot):
    jj, d = f >> 2, f & 3
    b = A_VA + 4 * (f % RING)
    off = slot * VSLOT + jj * 4096
    return [f"ds_read_b64_tr_b16 a[{b}:{b + 1}], v{V_VAT + d} offset:{off}",
            f"ds_read_b64_tr_b16 a[{b + 2}:{b + 3}], v{V_VAT + d} offset:{off + 2048}"]


# ------------------------------------------------------------------------------------------------- VALU streams
def interleave(*streams):
    out = []
    n = max(len(s) for s in streams)
    for i in range(n):
        for s in streams:
            if i < len(s):
                out.append(s[i])
    return out


def mask_ops(buf):
    """Scores of keys at or past the column's limit become -inf."""
    ninf = f"v{V_T + 9}"
    out = [f"v_mov_b32 {ninf}, {NINF}"]
    for cb in range(2):                 # a192 + cb: the column's limit minus 4 half; [t64]: the tile's first key
        out.append(f"v_accvgpr_read_b32 v{V_REL + cb}, a{192 + cb}")
    for cb in range(2):
        out.append(f"v_subrev_u32 v{V_REL + cb}, %[t64], v{V_REL + cb}")
    for rb in range(2):
        for e in range(16):
            o = 32 * rb + 8 * (e >> 2) + (e & 3)
            for cb in range(2):
                r = BUF[buf] + 32 * cb + 16 * rb + e
                out.append(f"v_cmp_lt_i32 vcc, {o}, v{V_REL + cb}")
                out.append(f"v_cndmask_b32 v{r}, {ninf}, v{r}, vcc")
    return out


def max_ops(buf, cb):
    """Maximum of the lane's 32 scores of column block cb into v(V_T + cb) (two chains of three-way maxima)."""
    e = [BUF[buf] + 32 * cb + x for x in range(32)]
    r0, r1 = f"v{V_T + 2 + 2 * cb}", f"v{V_T + 3 + 2 * cb}"
    out = [f"v_max3_f32 {r0}, v{e[0]}, v{e[1]}, v{e[2]}", f"v_max3_f32 {r1}, v{e[3]}, v{e[4]}, v{e[5]}"]
    x = 6
    which = 0
    while x < 32:
        r = r0 if which == 0 else r1
        out.append(f"v_max3_f32 {r}, {r}, v{e[x]}, v{e[x + 1]}")
        x += 2
        which ^= 1
    out.append(f"v_max_f32 v{V_T + cb}, {r0}, {r1}")
    return out


def growth_ops(cb):
    """m and alpha of column block cb from the tile's maximum in v(V_T + cb); sets %[flag] when m moved.  Returns
    (straight-line part, the conditional part as one unit that must not be split)."""
    t0, t1 = f"v{V_T + 6 + 2 * cb}", f"v{V_T + 7 + 2 * cb}"
    m, al = f"v{V_M + cb}", f"v{V_ALPHA + cb}"
    la, lb = f"v{V_L + 2 * cb}", f"v{V_L + 2 * cb + 1}"
    cond = f"s[{84 + 2 * cb}:{85 + 2 * cb}]"
    lab = f"Lflashw_%=_{cb}"
    head = [f"v_mul_f32 {t0}, %[c], v{V_T + cb}",
            f"v_max_f32 {t0}, {t0}, {m}",
            f"v_mov_b32 {t1}, {t0}",
            f"v_mov_b32 {al}, 1.0",
            f"v_add_f32 v{V_T + cb}, {GROW}, {m}",
            f"v_permlane32_swap_b32 {t0}, {t1}",
            f"v_max_f32 {t0}, {t0}, {t1}",                      # the column's maximum, in both halves
            f"v_cmp_gt_f32_e64 {cond}, {t0}, v{V_T + cb}"]
    unit = [f"s_cmp_lg_u64 {cond}, 0",
            f"s_cbranch_scc0 {lab}",
            f"v_sub_f32 {al}, {m}, {t0}",
            f"v_exp_f32 {al}, {al}",
            f"v_mov_b32 {m}, {t0}",
            "s_mov_b32 %[flag], 1",
            f"v_mul_f32 {la}, {la}, {al}",
            f"v_mul_f32 {lb}, {lb}, {al}",
            f"{lab}:"]
    return head, unit


def exp_stages(buf, rb, k, tbase):
    """Exponentials of element pair k of blocks (0, rb) and (1, rb), packed in place, and their row sums, as three
    stages of independent instructions (a stage depends on the one before it)."""
    st = [[], [], []]
    for cb in range(2):
        b = BUF[buf] + 32 * cb + 16 * rb
        e0, e1 = b + 2 * k, b + 2 * k + 1
        dst = b + k if k < 4 else b + 8 + (k - 4)
        t0, t1 = f"v{tbase + 2 * cb}", f"v{tbase + 2 * cb + 1}"
        m = f"v{V_M + cb}"
        st[0] += [f"v_fma_f32 {t0}, v{e0}, %[c], -{m}", f"v_fma_f32 {t1}, v{e1}, %[c], -{m}"]
        st[1] += [f"v_exp_f32 {t0}, {t0}", f"v_exp_f32 {t1}, {t1}"]
        # (row sums by fp32 additions: one v_dot2c_f32_bf16 per pair on the packed values measured 3.7 % slower)
        st[2] += [f"v_cvt_pk_bf16_f32 v{dst}, {t0}, {t1}", f"v_add_f32 v{V_L + 2 * cb}, v{V_L + 2 * cb}, {t0}",
                  f"v_add_f32 v{V_L + 2 * cb + 1}, v{V_L + 2 * cb + 1}, {t1}"]
    return st


def exp_stream(buf, first, count):
    """Groups first .. first + count - 1 of a tile (a group: one element pair of both column blocks) as one
    instruction stream, software-pipelined so that no instruction stands right behind the one it depends on:
    ... fma(n + 1), exp(n + 1), pack(n) and sums(n) ...  Two sets of temporaries alternate."""
    groups = []
    for n in range(first, first + count):
        rb, k = n >> 3, n & 7
        groups.append(exp_stages(buf, rb, k, V_T + 4 * (n % 2) + 2))
    out = []
    for n in range(len(groups) + 1):
        if n < len(groups):
            out += groups[n][0] + groups[n][1]
        if 0 <= n - 1 < len(groups):
            out += groups[n - 1][2]
    return out


N_GROUPS_A = 5        # exponential groups dealt out in half A (of 16); the others ride in half B


# ------------------------------------------------------------------------------------------------- hazards
def written_vgprs(line):
    op, _, rest = line.partition(" ")
    if not op.startswith("v_") or op.startswith("v_mfma") or op.startswith("v_cmp"):
        return set()
    ops = [x.strip() for x in rest.split(",")]
    targets = ops[:2] if op.startswith("v_permlane") else ops[:1]
    regs = set()
    for t in targets:
        m = re.match(r"v(\d+)$", t)
        if m:
            regs.add(int(m.group(1)))
    return regs


def fix_swap_hazards(lines):
    """A half-wave swap reads its registers two wait states after a VALU write at the earliest."""
    out = []
    for line in lines:
        if line.startswith("v_permlane"):
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


class Lds:
    """Counts LDS reads in program order so that a wait can name how many newer ones may stay in flight."""

    def __init__(self):
        self.issued = 0
        self.done_at = {}
        self.waited = 0         # reads up to this count are known to have returned

    def issue(self, key, lines, out):
        out.extend(lines)
        self.issued += len(lines)
        self.done_at[key] = self.issued

    def seed(self, key, n):
        self.issued += n
        self.done_at[key] = self.issued

    def wait(self, key, out):
        if self.done_at[key] <= self.waited:
            return
        newer = self.issued - self.done_at[key]
        out.append(f"s_waitcnt lgkmcnt({min(newer, 15)})")
        self.waited = self.done_at[key]

    def all_done(self):
        self.waited = self.issued


def spread(fillers, slots):
    """Deals the filler instructions out over `slots` places as evenly as possible; an item that is a list stays in
    one place (a branch and its target)."""
    units = [x if isinstance(x, list) else [x] for x in fillers]
    total = sum(len(u) for u in units)
    per = [[] for _ in range(slots)]
    idx = 0
    count = 0
    for u in units:
        per[idx] += u
        count += len(u)
        while idx < slots - 1 and count >= (idx + 1) * total / slots:
            idx += 1
    return per


def flat(fillers):
    return [l for x in fillers for l in (x if isinstance(x, list) else [x])]


# ------------------------------------------------------------------------------------------------- the halves
def half_a(i, has_pv=True, masked=False, valu=True, sync=True):
    """Half A of step i (see the module text).  Operands: [c] scale * log2(e), [flag] out: a reference maximum moved."""
    buf, pbuf = i & 1, (i & 1) ^ 1
    vslot = (i + 2) % 3                 # V(t - 1)
    kslot_next = (i + 1) % 3            # K(t + 1), read by half B
    out = []
    fillers = []
    if valu:
        if masked:
            fillers += mask_ops(buf)
        fillers += interleave(max_ops(buf, 0), max_ops(buf, 1))
        (h0, u0), (h1, u1) = growth_ops(0), growth_ops(1)
        fillers += interleave(h0, h1)
        fillers += [u0, u1]
        fillers += exp_stream(buf, 0, N_GROUPS_A)
        out.append("s_mov_b32 %[flag], 0")
    tail_sync = ["s_barrier"] + k_read(0, kslot_next) + k_read(1, kslot_next) if sync else []
    if not has_pv:
        out += ["s_nop 15", "s_nop 7"] + flat(fillers)
        if sync:
            out += ["s_waitcnt vmcnt(8) lgkmcnt(0)"] + tail_sync
        return fix_swap_hazards(out)
    lds = Lds()
    lds.seed(0, 2)
    lds.seed(1, 2)
    per = spread(fillers, 30) if fillers else [[] for _ in range(30)]
    for n in range(32):
        f, cb = n >> 1, n & 1
        jj, d = f >> 2, f & 3
        if n % 4 == 0:                  # a pair of fragments: request the next pair, wait for this one
            for x in (f + 2, f + 3):
                if x < 16:
                    lds.issue(x, v_read(x, vslot), out)
            if n == 28 and sync:
                out.append("s_waitcnt vmcnt(8) lgkmcnt(0)")
                lds.all_done()
            else:
                lds.wait(f + 1, out)
        out.append(f"v_mfma_f32_32x32x16_bf16 {o_acc(cb, d)}, {va(f)}, {p_frag(pbuf, cb, jj)}, {o_acc(cb, d)}")
        if n == 28 and sync:
            out += tail_sync
        if n >= 2:
            out += per[n - 2]
    return fix_swap_hazards(out)


def half_b(i, has_qk=True, valu=True, loads=True, prefetch_own=False, prefetch_next=True):
    """Half B of step i.  Operands: [c]; [rk] / [rv] resources of the tiles K(t + 3) / V(t + 2); [ldsw] LDS address of
    the wavefront's first 1 KB block of ring slot 0."""
    buf, sbuf = i & 1, (i & 1) ^ 1
    kslot = (i + 1) % 3                 # K(t + 1)
    kload, vload = i % 3, (i + 2) % 3   # slots of K(t + 3), V(t + 2)
    vslot_next = i % 3                  # V(t), read by the next step's half A
    out = []
    fillers = []
    if valu:
        fillers += exp_stream(buf, N_GROUPS_A, 16 - N_GROUPS_A)
    tail = v_read(0, vslot_next) + v_read(1, vslot_next) if prefetch_next else []
    if not has_qk:
        return fix_swap_hazards(out + flat(fillers) + tail)
    lds = Lds()
    if prefetch_own:
        lds.issue(0, k_read(0, kslot), out)
        lds.issue(1, k_read(1, kslot), out)
    else:
        lds.seed(0, 1)
        lds.seed(1, 1)
    if loads:
        out.append(f"s_mov_b32 {S_M0}, m0")
    per = spread(fillers, 32) if fillers else [[] for _ in range(32)]
    load_at = {3 + 4 * j: ("k", j) for j in range(4)}
    load_at.update({19 + 4 * j: ("v", j) for j in range(4)})
    for n in range(32):
        ks, rb, cb = n >> 2, (n >> 1) & 1, n & 1
        f = n >> 1
        if n % 4 == 0:
            for x in (f + 2, f + 3):
                if x < 16:
                    lds.issue(x, k_read(x, kslot), out)
            lds.wait(f + 1, out)
        if loads and n in load_at:
            kind, j = load_at[n]
            base = kload * KSLOT if kind == "k" else VBASE + vload * VSLOT
            out.append(f"s_add_u32 m0, %[ldsw], {base + 0x400 * j:#x}")
        c = "0" if ks == 0 else s_blk(sbuf, cb, rb)
        out.append(f"v_mfma_f32_32x32x16_bf16 {s_blk(sbuf, cb, rb)}, {kf(f)}, {q_frag(cb, ks)}, {c}")
        out += per[n]
        if loads and n in load_at:
            kind, j = load_at[n]
            if kind == "k":
                out.append(f"buffer_load_dwordx4 v{V_KOFF + j}, %[rk], 0 offen lds")
            else:
                out.append(f"buffer_load_dwordx4 v{V_VOFF + j}, %[rv], 0 offen lds")
    out += tail
    if loads:
        out.append(f"s_mov_b32 m0, {S_M0}")
    return fix_swap_hazards(out)


def rescale():
    """O *= alpha per column block (behind half A, when its flag says a reference maximum moved)."""
    out = ["s_nop 15", "s_nop 7"]
    for cb in range(2):
        for base in range(0, 64, 8):
            regs = [64 * cb + base + x for x in range(8)]
            out += [f"v_accvgpr_read_b32 v{V_T + 2 + x}, a{r}" for x, r in enumerate(regs)]
            out += [f"v_mul_f32 v{V_T + 2 + x}, v{V_T + 2 + x}, v{V_ALPHA + cb}" for x in range(8)]
            out += [f"v_accvgpr_write_b32 a{r}, v{V_T + 2 + x}" for x, r in enumerate(regs)]
    return out


def define(name, lines):
    body = " \\\n".join(f'  "{l}\\n\\t"' for l in lines)
    return f"#define {name} \\\n{body}\n"


def main():
    parts = ["// Generated by gen_flash_asm.py (the schedule and the register map are described there).  Do not edit.\n"]
    for i in range(6):
        parts.append(define(f"FLASHW_A{i}", half_a(i)))
        parts.append(define(f"FLASHW_A{i}_M", half_a(i, masked=True)))
        parts.append(define(f"FLASHW_B{i}", half_b(i)))
        parts.append(define(f"FLASHW_B{i}_LAST", half_b(i, has_qk=False)))
        parts.append(define(f"FLASHW_PV{i}", half_a(i, valu=False, sync=False)))
    parts.append(define("FLASHW_A_FIRST", half_a(0, has_pv=False)))
    parts.append(define("FLASHW_A_FIRST_M", half_a(0, has_pv=False, masked=True)))
    parts.append(define("FLASHW_QK_FIRST", half_b(5, valu=False, loads=False, prefetch_own=True, prefetch_next=False)))
    parts.append(define("FLASHW_RESCALE", rescale()))
    # the wavefront's four 1 KB blocks of one K / V tile into the LDS ring at [dst] (wave offset already added)
    for name, voff in (("FLASHW_LOAD4_K", V_KOFF), ("FLASHW_LOAD4_V", V_VOFF)):
        lines = [f"s_mov_b32 {S_M0}, m0", "s_mov_b32 m0, %[dst]", "s_nop 4"]
        for j in range(4):
            lines.append(f"buffer_load_dwordx4 v{voff + j}, %[r], 0 offen lds")
            if j < 3:
                lines += ["s_add_u32 m0, m0, 0x400", "s_nop 0"]
        lines.append(f"s_mov_b32 m0, {S_M0}")
        parts.append(define(name, lines))
    parts.append(define("FLASHW_SET_KAT", [f"v_mov_b32 v{V_KAT + s}, %{s}" for s in range(8)]))
    parts.append(define("FLASHW_SET_VAT", [f"v_mov_b32 v{V_VAT + s}, %{s}" for s in range(4)]))
    parts.append(define("FLASHW_SET_KOFF", [f"v_mov_b32 v{V_KOFF + s}, %{s}" for s in range(4)]))
    parts.append(define("FLASHW_SET_VOFF", [f"v_mov_b32 v{V_VOFF + s}, %{s}" for s in range(4)]))
    parts.append(define("FLASHW_SET_LIMIT", ["v_accvgpr_write_b32 a192, %0", "v_accvgpr_write_b32 a193, %1"]))
    # m = a large negative finite number (a column that never sees a key keeps it and its sums stay zero), sums zero
    init = [f"v_mov_b32 v{V_M + cb}, 0xf149f2ca" for cb in range(2)] + [f"v_mov_b32 v{V_L + x}, 0" for x in range(4)]
    init += [f"v_accvgpr_write_b32 a{r}, 0" for r in range(128)]
    parts.append(define("FLASHW_INIT", init))
    for cb in range(2):
        for d in range(4):
            b = 64 * cb + 16 * d
            parts.append(define(f"FLASHW_GET_O{cb}_{d}", [f"v_accvgpr_read_b32 %{x}, a{b + x}" for x in range(16)]))
    # four 1 KB blocks of the wavefront's query rows into its private LDS region ([dst], then + 1 KB each): a block
    # is four rows of 256 bytes, lane l fetching the piece that belongs at position l % 16 of row l / 16
    lines = [f"s_mov_b32 {S_M0}, m0", "s_mov_b32 m0, %[dst]", "s_nop 4"]
    for j in range(4):
        lines.append(f"buffer_load_dwordx4 %[o{j}], %[r], 0 offen lds")
        if j < 3:
            lines += ["s_add_u32 m0, m0, 0x400", "s_nop 0"]
    lines.append(f"s_mov_b32 m0, {S_M0}")
    parts.append(define("FLASHW_LOADQ4", lines))
    # Q^T operand fragments out of that region ([qoff]: its LDS address; rows swizzled like a K tile's, so the K
    # fragment addresses serve) into the accumulation registers they stay in
    lines = [f"v_add_u32 v{V_T + ks}, %[qoff], v{V_KAT + ks}" for ks in range(8)]
    for cb in range(2):
        for ks in range(8):
            b = 128 + 32 * cb + 4 * ks
            lines.append(f"ds_read_b128 a[{b}:{b + 3}], v{V_T + ks} offset:{8192 * cb}")
    lines.append("s_waitcnt lgkmcnt(0)")
    parts.append(define("FLASHW_Q_FROM_LDS", lines))
    parts.append(define("FLASHW_DRAIN", ["s_nop 15", "s_nop 7"]))
    parts.append(define("FLASHW_GET_ML", [f"v_mov_b32 %0, v{V_M}", f"v_mov_b32 %1, v{V_M + 1}",
                                          f"v_add_f32 %2, v{V_L}, v{V_L + 1}", f"v_add_f32 %3, v{V_L + 2}, v{V_L + 3}"]))
    regs = [f"v{r}" for r in range(V_FIRST, 256)] + [f"a{r}" for r in range(256)] + [f"s{r}" for r in range(84, 96)] + ["vcc", "scc", "memory"]
    parts.append("#define FLASHW_CLOBBERS " + ", ".join(f'"{x}"' for x in regs) + "\n")
    text = "\n".join(parts)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "flash_asm.inc")
    if len(sys.argv) > 1 and sys.argv[1] == "--check":
        return 0 if os.path.exists(path) and open(path).read() == text else 1
    open(path, "w").write(text)
    return 0


if __name__ == "__main__":
    sys.exit(main())
