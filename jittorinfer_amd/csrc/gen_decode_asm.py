#!/usr/bin/env python3
"""Generates mla_decode_asm.inc: the hand-scheduled gfx950 instruction stream of the pipelined MLA decode kernel
(one inline-asm block inside mla_decode_kernel.hip).  Usage: python gen_decode_asm.py > mla_decode_asm.inc

Why a generator: the kernel keeps Q (144 VGPRs) and the O accumulator (256 AGPRs) resident, which leaves ~110
registers for everything else; the instruction order (MFMA issue slots filled with LDS reads and softmax VALU work)
and the register map are fixed here instead of being left to a compiler that spills under that pressure.

Work of one wave (32 attention rows, all 512 output columns), per 32-token tile `it`:
    phase A   S_next = K[it+1] . Q^T      36 MFMA, interleaved with  softmax(S_cur) -> P (hi, lo)   (VALU)
                                          and the address arithmetic + issue of the LDS-DMA loads of tile it+2
    phase B   O^T += V[it]^T . P^T        32 V^T fragments (ds_read_b64_tr_b16 x2 each), 64 MFMA (hi and lo halves of P)
    end       s_waitcnt vmcnt(0); s_barrier   (tile it+2 has landed for every wave)
Register roles of S_cur/S_next swap every tile, so the loop body is emitted twice.
"""
import sys

DEBUG = "--debug" in sys.argv
NO_LOOP_DMA = "--no-loop-dma" in sys.argv   # timing experiments only (wrong results)
NO_PV = "--no-pv" in sys.argv
NO_QK = "--no-qk" in sys.argv
NO_SM = "--no-softmax" in sys.argv
DMA_PLACE = "pv" if "--dma-pv" in sys.argv else "bulk" if "--dma-bulk" in sys.argv else "a"
NO_STORE = "--no-store" in sys.argv
NO_QLOAD = "--no-qload" in sys.argv
F16 = "--f16" in sys.argv  # f16 KV: f16 MFMA, single P (no lo half)
MF = "v_mfma_f32_32x32x16_f16" if F16 else "v_mfma_f32_32x32x16_bf16"
CVT = "v_cvt_pk_f16_f32" if F16 else "v_cvt_pk_bf16_f32"
SPLIT = not F16

PITCH = 1168
TILE_BYTES = 32 * PITCH
NBUF = 4
HOFF = NBUF * TILE_BYTES       # hand-off area written by the C++ prologue: 32 bytes per thread
DMA_PER_TILE = 10              # LDS-DMA instructions each wave issues per tile
CPR = 73                       # 16-byte chunks per padded row
WAVE_CHUNKS = 8 * CPR          # 584: each wave moves rows 8w..8w+7 of a tile
TAU = 8.0

# ---- VGPR map
Q0 = 0
SA, SB = 144, 160
PHI, PLO = 176, 184
KF = 192   # 4 fragments x 4
VF = 208   # 4 fragments x 4
T = list(range(224, 232))
OPTR, MLPTR = 232, 234
KADDR_LANE, VADDR_LANE, MRUN, LRUN, NEGM = 236, 237, 238, 239, 240
DROW, DCOL, VOFF, PAGES = 241, 242, 243, 244
LANE, KADDR, VADDR, TMAX = 245, 246, 247, 248
X0, X1, X2 = 249, 250, 251
N_VGPR = 252
DBG, TIDR = 230, 248   # debug builds only: T[6:7] holds the debug pointer until the main loop; TMAX's register keeps tid
# ---- SGPR map (all inside the clobbered range s40..s79)
KV, BT, KVB, KVE, CL2, NPP, NB1, FLG = 40, 42, 44, 45, 46, 47, 48, 49
NT, IT, OFF0, OFF1, OFF2, WAVE, TB, TMP, NVM1 = 50, 51, 52, 53, 54, 55, 56, 58, 59
EXS, S0, S1, S2, S3, DMAB, NVAL, THR, PG0, RSC, SPITCH, SCLS, OFF3, VMW, OSTR, QP = 60, 62, 63, 64, 65, 66, 67, 68, 69, 70, 72, 73, 74, 75, 76, 78

out = []
uid = [0]


def e(s):
    out.append(s)


def label(prefix):
    uid[0] += 1
    return "L%s_%d_%%=" % (prefix, uid[0])


def v(i, n=1):
    return "v%d" % i if n == 1 else "v[%d:%d]" % (i, i + n - 1)


def a(i, n=1):
    return "a%d" % i if n == 1 else "a[%d:%d]" % (i, i + n - 1)


def s(i, n=1):
    return "s%d" % i if n == 1 else "s[%d:%d]" % (i, i + n - 1)


class Lds:
    """Tracks outstanding LDS reads so that each use waits for exactly the reads that precede it."""

    def __init__(self):
        self.pending = []

    def read(self, line, tag):
        e(line)
        self.pending.append(tag)

    def need(self, tag):
        if tag in self.pending:
            after = len(self.pending) - 1 - self.pending.index(tag)
            e("s_waitcnt lgkmcnt(%d)" % after)
            self.pending = self.pending[len(self.pending) - after:]

    def drain(self):
        if self.pending:
            e("s_waitcnt lgkmcnt(0)")
            self.pending = []


lds = Lds()


def interleave(mfma_slots, valu, per_slot):
    """mfma_slots: list of callables emitting one MFMA slot (its LDS prefetch + the MFMA); valu: list of lines."""
    vi = 0
    n = len(mfma_slots)
    for i, slot in enumerate(mfma_slots):
        slot()
        remaining_slots = n - i
        take = max(per_slot, -(-(len(valu) - vi) // remaining_slots)) if vi < len(valu) else 0
        for _ in range(take):
            if vi < len(valu):
                e(valu[vi])
                vi += 1
    while vi < len(valu):
        e(valu[vi])
        vi += 1


# ---------------------------------------------------------------------------------------------------------------
def dma_tile_lines(tile_sreg, off_sreg):
    """Instruction list (to be interleaved) that issues the LDS-DMA loads of tile index s[tile_sreg] into the buffer
    at LDS offset s[off_sreg].  Scalar part first (tile base address), then 10 slots."""
    L = []
    # t0 = kv_begin + 32*tile ; nvalid-1 = min(32, kv_end - t0) - 1
    L.append("s_lshl_b32 %s, %s, 5" % (s(S0), s(tile_sreg)))
    L.append("s_add_u32 %s, %s, %s" % (s(S0), s(S0), s(KVB)))                      # S0 = t0
    L.append("s_sub_u32 %s, %s, %s" % (s(S1), s(KVE), s(S0)))
    L.append("s_min_u32 %s, %s, 32" % (s(S1), s(S1)))
    L.append("s_sub_u32 %s, %s, 1" % (s(NVM1), s(S1)))
    # page lookup (branch-free: the list below gets interleaved with MFMA slots, so no label may sit inside it)
    L.append("s_lshr_b32 %s, %s, 7" % (s(S1), s(S0)))                             # logical page
    L.append("s_sub_u32 %s, %s, %s" % (s(S1), s(S1), s(PG0)))                     # index into the preloaded lanes
    L.append("v_readlane_b32 %s, %s, %s" % (s(S2), v(PAGES), s(S1)))
    L.append("s_lshl_b32 %s, %s, 7" % (s(S2), s(S2)))
    L.append("s_and_b32 %s, %s, 127" % (s(S3), s(S0)))
    L.append("s_add_u32 %s, %s, %s" % (s(S2), s(S2), s(S3)))                      # pool row when paged
    L.append("s_cmp_eq_u64 %s, 0" % s(BT, 2))
    L.append("s_cselect_b32 %s, %s, %s" % (s(S0), s(S0), s(S2)))                  # no table: the logical row itself
    # tile base = kv + row * nb1   (64-bit)
    L.append("s_mul_hi_u32 %s, %s, %s" % (s(S1), s(S0), s(NB1)))
    L.append("s_mul_i32 %s, %s, %s" % (s(S0), s(S0), s(NB1)))
    L.append("s_add_u32 %s, %s, %s" % (s(TB), s(KV), s(S0)))
    L.append("s_addc_u32 %s, %s, %s" % (s(TB + 1), s(KV + 1), s(S1)))
    # LDS destination of this wave's first slot
    L.append("s_mul_i32 %s, %s, %d" % (s(DMAB), s(WAVE), WAVE_CHUNKS * 16))
    L.append("s_add_u32 %s, %s, %s" % (s(DMAB), s(DMAB), s(off_sreg)))
    # per-lane chunk walk: local chunk cl = 64*j + lane -> (row_l, col); row = 8*wave + row_l
    L.append("v_mov_b32 %s, %s" % (v(DCOL), v(LANE)))
    L.append("s_lshl_b32 %s, %s, 3" % (s(S2), s(WAVE)))
    L.append("v_mov_b32 %s, %s" % (v(DROW), s(S2)))
    for j in range(10):
        L.append("v_min_u32 %s, %s, %s" % (v(X0), s(NVM1), v(DROW)))
        L.append("v_min_u32 %s, 71, %s" % (v(X1), v(DCOL)))
        L.append("v_lshlrev_b32 %s, 4, %s" % (v(X1), v(X1)))
        L.append("v_mad_u32_u24 %s, %s, %s, %s" % (v(VOFF), v(X0), s(NB1), v(X1)))
        if j == 9:
            # 8 chunks left per wave: lanes 0..7 only.  One atomic group: nothing may be scheduled inside the exec window.
            L.append("\\n\\t".join(["s_add_u32 m0, %s, %d" % (s(DMAB), j * 1024),
                                    "s_mov_b64 %s, exec" % s(EXS, 2),
                                    "s_mov_b64 exec, 0xff",
                                    "global_load_lds_dwordx4 %s, %s" % (v(VOFF), s(TB, 2)),
                                    "s_mov_b64 exec, %s" % s(EXS, 2)]))
        else:
            L.append("\\n\\t".join(["s_add_u32 m0, %s, %d" % (s(DMAB), j * 1024),
                                    "s_nop 0",
                                    "global_load_lds_dwordx4 %s, %s" % (v(VOFF), s(TB, 2))]))
            # advance 64 chunks: col += 64; if (col >= 73) { col -= 73; row += 1 }
            L.append("v_add_u32 %s, 64, %s" % (v(DCOL), v(DCOL)))
            L.append("v_cmp_le_u32 vcc, %d, %s" % (CPR, v(DCOL)))
            L.append("v_subrev_u32 %s, %d, %s" % (v(X2), CPR, v(DCOL)))
            L.append("v_add_u32 %s, 1, %s" % (v(X0), v(DROW)))
            L.append("s_nop 0")
            L.append("v_cndmask_b32 %s, %s, %s, vcc" % (v(DCOL), v(DCOL), v(X2)))
            L.append("v_cndmask_b32 %s, %s, %s, vcc" % (v(DROW), v(DROW), v(X0)))
    return L


def qk_slots(sreg, kaddr):
    """36 MFMA slots of S = K.Q^T into v[sreg:sreg+15]; K fragments come through a ring of 4."""
    if NO_QK:
        return [(lambda: None) for _ in range(36)]
    slots = []
    depth = 3

    def mk(ks):
        def slot():
            # keep `depth` reads in flight
            if ks == 0:
                for p in range(depth):
                    lds.read("ds_read_b128 %s, %s offset:%d" % (v(KF + 4 * (p % 4), 4), v(kaddr), p * 32), ("k", p))
            if ks + depth < 36:
                p = ks + depth
                lds.read("ds_read_b128 %s, %s offset:%d" % (v(KF + 4 * (p % 4), 4), v(kaddr), p * 32), ("k", p))
            lds.need(("k", ks))
            c = "0" if ks == 0 else v(sreg, 16)
            e("%s %s, %s, %s, %s" % (MF, v(sreg, 16), v(KF + 4 * (ks % 4), 4), v(Q0 + 4 * ks, 4), c))
        return slot
    for ks in range(36):
        slots.append(mk(ks))
    return slots


def softmax_part1(sreg):
    """tile max -> TMAX (log2 units), uniform test whether any row's max moved by more than TAU."""
    if NO_SM:
        return ["s_mov_b64 %s, 0" % s(RSC, 2)]
    L = []
    m = [T[0], T[1], T[2], T[3], T[4]]
    L.append("v_max3_f32 %s, %s, %s, %s" % (v(m[0]), v(sreg + 0), v(sreg + 1), v(sreg + 2)))
    L.append("v_max3_f32 %s, %s, %s, %s" % (v(m[1]), v(sreg + 3), v(sreg + 4), v(sreg + 5)))
    L.append("v_max3_f32 %s, %s, %s, %s" % (v(m[2]), v(sreg + 6), v(sreg + 7), v(sreg + 8)))
    L.append("v_max3_f32 %s, %s, %s, %s" % (v(m[3]), v(sreg + 9), v(sreg + 10), v(sreg + 11)))
    L.append("v_max3_f32 %s, %s, %s, %s" % (v(m[4]), v(sreg + 12), v(sreg + 13), v(sreg + 14)))
    L.append("v_max3_f32 %s, %s, %s, %s" % (v(m[0]), v(m[0]), v(m[1]), v(sreg + 15)))
    L.append("v_max3_f32 %s, %s, %s, %s" % (v(m[0]), v(m[0]), v(m[2]), v(m[3])))
    L.append("v_max_f32 %s, %s, %s" % (v(m[0]), v(m[0]), v(m[4])))
    L.append("v_mov_b32 %s, %s" % (v(m[1]), v(m[0])))
    L.append("s_nop 1")
    L.append("v_permlane32_swap_b32 %s, %s" % (v(m[0]), v(m[1])))
    L.append("s_nop 1")
    L.append("v_max_f32 %s, %s, %s" % (v(TMAX), v(m[0]), v(m[1])))
    L.append("v_mul_f32 %s, %s, %s" % (v(TMAX), s(CL2), v(TMAX)))          # log2 units (c_log2 > 0)
    L.append("v_add_f32 %s, %s, %s" % (v(m[2]), s(THR), v(MRUN)))           # m_run + TAU  (-inf stays -inf)
    L.append("v_cmp_gt_f32 %s, %s, %s" % (s(RSC, 2), v(TMAX), v(m[2])))
    return L


def rescale_block(ret_label):
    """Rare path: m_new = max(m_run, tmax); alpha = 2^(m_run - m_new) (0 when m_run = -inf); acc *= alpha; l *= alpha."""
    e("v_max_f32 %s, %s, %s" % (v(T[0]), v(MRUN), v(TMAX)))                 # m_new
    e("v_sub_f32 %s, %s, %s" % (v(T[1]), v(MRUN), v(T[0])))                 # m_run - m_new (NaN when both -inf)
    e("v_exp_f32 %s, %s" % (v(T[1]), v(T[1])))
    e("v_mov_b32 %s, 0xff800000" % v(T[2]))
    e("v_cmp_eq_f32 vcc, %s, %s" % (v(MRUN), v(T[2])))
    e("s_nop 1")
    e("v_cndmask_b32 %s, %s, 0, vcc" % (v(T[1]), v(T[1])))                  # alpha
    e("v_mov_b32 %s, %s" % (v(MRUN), v(T[0])))
    e("v_mul_f32 %s, %s, %s" % (v(LRUN), v(LRUN), v(T[1])))
    e("s_nop 7")
    e("s_nop 7")
    e("s_nop 3")                                                            # last MFMA writes to acc are long done
    for i in range(0, 256, 4):
        for j in range(4):
            e("v_accvgpr_read_b32 %s, %s" % (v(T[3 + j]), a(i + j)))
        for j in range(4):
            e("v_mul_f32 %s, %s, %s" % (v(T[3 + j]), v(T[3 + j]), v(T[1])))
        for j in range(4):
            e("v_accvgpr_write_b32 %s, %s" % (a(i + j), v(T[3 + j])))
    e("s_nop 7")
    e("s_nop 7")
    e("s_branch %s" % ret_label)


def softmax_part2(sreg):
    if NO_SM:
        return []
    L = []
    # p = 2^(s*c - m)
    for k in range(16):
        L.append("v_fma_f32 %s, %s, %s, %s" % (v(sreg + k), v(sreg + k), s(CL2), v(NEGM)))
    for k in range(16):
        L.append("v_exp_f32 %s, %s" % (v(sreg + k), v(sreg + k)))
    # running sum (this lane's 16 tokens)
    L.append("v_add_f32 %s, %s, %s" % (v(T[0]), v(sreg + 0), v(sreg + 1)))
    L.append("v_add_f32 %s, %s, %s" % (v(T[1]), v(sreg + 2), v(sreg + 3)))
    for k in range(4, 16, 2):
        L.append("v_add_f32 %s, %s, %s" % (v(T[0]), v(T[0]), v(sreg + k)))
        L.append("v_add_f32 %s, %s, %s" % (v(T[1]), v(T[1]), v(sreg + k + 1)))
    L.append("v_add_f32 %s, %s, %s" % (v(T[0]), v(T[0]), v(T[1])))
    L.append("v_add_f32 %s, %s, %s" % (v(LRUN), v(LRUN), v(T[0])))
    # P^T operands: k-step kk uses elements 8kk .. 8kk+7
    for j in range(8):
        L.append("%s %s, %s, %s" % (CVT, v(PHI + j), v(sreg + 2 * j), v(sreg + 2 * j + 1)))
    if SPLIT:
        for j in range(8):
            t0, t1 = T[2 + (j % 3) * 2], T[3 + (j % 3) * 2]
            L.append("v_lshlrev_b32 %s, 16, %s" % (v(t0), v(PHI + j)))
            L.append("v_and_b32 %s, 0xffff0000, %s" % (v(t1), v(PHI + j)))
            L.append("v_sub_f32 %s, %s, %s" % (v(t0), v(sreg + 2 * j), v(t0)))
            L.append("v_sub_f32 %s, %s, %s" % (v(t1), v(sreg + 2 * j + 1), v(t1)))
            L.append("%s %s, %s, %s" % (CVT, v(PLO + j), v(t0), v(t1)))
    return L


def mask_tail(sreg):
    """Last tile only: tokens >= n_valid get score -inf.  element k is token 8*(k/4) + 4g + k%4."""
    lab = label("full")
    e("s_cmp_ge_u32 %s, 32" % s(NVAL))
    e("s_cbranch_scc1 %s" % lab)
    e("v_mov_b32 %s, 0xff800000" % v(T[0]))
    e("v_lshrrev_b32 %s, 5, %s" % (v(T[2]), v(LANE)))
    e("v_lshlrev_b32 %s, 2, %s" % (v(T[2]), v(T[2])))                       # 4g
    for k in range(16):
        e("v_add_u32 %s, %d, %s" % (v(T[1]), 8 * (k // 4) + (k % 4), v(T[2])))
        e("v_cmp_gt_u32 vcc, %s, %s" % (s(NVAL), v(T[1])))                  # valid if n_valid > token
        e("s_nop 1")
        e("v_cndmask_b32 %s, %s, %s, vcc" % (v(sreg + k), v(T[0]), v(sreg + k)))
    e("%s:" % lab)


def pv_phase(vaddr, extra=None):
    """O^T += V^T.P^T: 16 d-blocks x 2 k-steps; fragment ring of 4; d-blocks in pairs so dependent MFMAs alternate.
    `extra`: instruction lines spread evenly between the MFMA pairs (whole-slot groups only)."""
    frags = [(kk, db) for kk in range(2) for db in range(16)]
    extra = list(extra or [])
    per_pair = -(-len(extra) // 16)

    def rd(idx):
        kk, db = frags[idx]
        r = VF + 4 * (idx % 4)
        base = 16 * kk * PITCH + db * 64
        lds.read("ds_read_b64_tr_b16 %s, %s offset:%d" % (v(r, 2), v(vaddr), base), ("v", idx, 0))
        lds.read("ds_read_b64_tr_b16 %s, %s offset:%d" % (v(r + 2, 2), v(vaddr), base + 8 * PITCH), ("v", idx, 1))
    depth = 3
    for p in range(depth):
        rd(p)
    for pair in range(16):
        i0, i1 = 2 * pair, 2 * pair + 1
        # issue order: hi(i0), hi(i1), lo(i0), lo(i1) with prefetches in between
        kk0, db0 = frags[i0]
        kk1, db1 = frags[i1]
        if i0 + depth < 32:
            rd(i0 + depth)
        lds.need(("v", i0, 1))
        e("%s %s, %s, %s, %s" % (MF, a(16 * db0, 16), v(VF + 4 * (i0 % 4), 4), v(PHI + 4 * kk0, 4), a(16 * db0, 16)))
        lds.need(("v", i1, 1))
        e("%s %s, %s, %s, %s" % (MF, a(16 * db1, 16), v(VF + 4 * (i1 % 4), 4), v(PHI + 4 * kk1, 4), a(16 * db1, 16)))
        if SPLIT:
            e("%s %s, %s, %s, %s" % (MF, a(16 * db0, 16), v(VF + 4 * (i0 % 4), 4), v(PLO + 4 * kk0, 4), a(16 * db0, 16)))
            if i1 + depth < 32:
                rd(i1 + depth)
            e("%s %s, %s, %s, %s" % (MF, a(16 * db1, 16), v(VF + 4 * (i1 % 4), 4), v(PLO + 4 * kk1, 4), a(16 * db1, 16)))
        else:
            if i1 + depth < 32:
                rd(i1 + depth)
        for _ in range(per_pair):
            if extra:
                e(extra.pop(0))
    for ln in extra:
        e(ln)


def half_iteration(s_cur, s_next, tag):
    """Tile IT: QK of tile IT+1 into s_next interleaved with softmax of s_cur; then PV of tile IT."""
    e("; ---- half %s" % tag)
    # n_valid of tile IT
    e("s_lshl_b32 %s, %s, 5" % (s(S0), s(IT)))
    e("s_add_u32 %s, %s, %s" % (s(S0), s(S0), s(KVB)))
    e("s_sub_u32 %s, %s, %s" % (s(NVAL), s(KVE), s(S0)))
    e("s_min_u32 %s, %s, 32" % (s(NVAL), s(NVAL)))
    mask_tail(s_cur)
    # addresses for this half
    e("v_add_u32 %s, %s, %s" % (v(KADDR), s(OFF1), v(KADDR_LANE)))
    e("v_add_u32 %s, %s, %s" % (v(VADDR), s(OFF0), v(VADDR_LANE)))
    slots = qk_slots(s_next, KADDR)
    # DMA of tile IT+3 (skipped when it does not exist)
    e("s_add_u32 %s, %s, 3" % (s(TMP), s(IT)))
    e("s_mov_b32 %s, 0" % s(VMW))
    lab_nodma, lab_after = label("nodma"), label("afterdma")
    e("s_cmp_ge_u32 %s, %s" % (s(TMP), s(NT)))
    e("s_cbranch_scc1 %s" % lab_nodma)
    if NO_LOOP_DMA:
        e("s_branch %s" % lab_nodma)
    e("s_mov_b32 %s, 1" % s(VMW))
    dma = dma_tile_lines(TMP, OFF3)
    if DMA_PLACE != "a":
        if DMA_PLACE == "bulk":
            for ln in dma:
                e(ln)
        e("s_branch %s" % lab_nodma)   # the compute part is the DMA-free code below
        dma = []
    # part 1 of the softmax + DMA issue share the first MFMA slots
    p1 = softmax_part1(s_cur)
    n1 = 8
    interleave(slots[:n1], p1 + dma[:46], 8)  # 22 set-up lines + two whole DMA slots (vcc must not live across the cut)
    rest_dma = dma[46:]
    lab_resc, lab_back = label("resc"), label("back")
    e("s_cmp_lg_u64 %s, 0" % s(RSC, 2))
    e("s_cbranch_scc1 %s" % lab_resc)
    e("%s:" % lab_back)
    # -m (0 when still -inf)
    pre = ["v_mov_b32 %s, 0xff800000" % v(T[0]),
           "v_cmp_eq_f32 vcc, %s, %s" % (v(MRUN), v(T[0])),
           "v_sub_f32 %s, 0, %s" % (v(NEGM), v(MRUN)),
           "s_nop 0",
           "v_cndmask_b32 %s, %s, 0, vcc" % (v(NEGM), v(NEGM))]
    p2 = softmax_part2(s_cur)
    interleave(slots[n1:], pre + rest_dma + p2, 6)
    e("s_branch %s" % lab_after)
    # ---- same thing without the DMA (last two tiles)
    e("%s:" % lab_nodma)
    saved = list(lds.pending)
    lds.pending = []
    slots2 = qk_slots(s_next, KADDR)
    p1b = softmax_part1(s_cur)
    interleave(slots2[:n1], p1b, 4)
    lab_resc2, lab_back2 = label("resc"), label("back")
    e("s_cmp_lg_u64 %s, 0" % s(RSC, 2))
    e("s_cbranch_scc1 %s" % lab_resc2)
    e("%s:" % lab_back2)
    interleave(slots2[n1:], list(pre) + softmax_part2(s_cur), 4)
    e("%s:" % lab_after)
    assert not lds.pending and not saved
    # ---- PV of tile IT
    if not NO_PV:
        if DMA_PLACE == "pv":
            # DMA of tile IT+3 issued from inside the PV phase (VALU is otherwise idle there)
            lab_pvnodma, lab_pvdone = label("pvnodma"), label("pvdone")
            e("s_cmp_eq_u32 %s, 0" % s(VMW))
            e("s_cbranch_scc1 %s" % lab_pvnodma)
            pv_phase(VADDR, dma_tile_lines(TMP, OFF3))
            lds.drain()
            e("s_branch %s" % lab_pvdone)
            e("%s:" % lab_pvnodma)
            pv_phase(VADDR)
            lds.drain()
            e("%s:" % lab_pvdone)
        else:
            pv_phase(VADDR)
    lds.drain()
    # ---- end of tile: the DMA of tile IT+2 has landed (the one of tile IT+3, issued in this iteration, may still be
    # in flight: loads complete in order, so vmcnt(DMA_PER_TILE) is enough); everyone is done with tile IT
    lab_w0, lab_wd = label("w0"), label("wd")
    e("s_cmp_eq_u32 %s, 0" % s(VMW))
    e("s_cbranch_scc1 %s" % lab_w0)
    e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
    e("s_branch %s" % lab_wd)
    e("%s:" % lab_w0)
    e("s_waitcnt vmcnt(0)")
    e("%s:" % lab_wd)
    e("s_barrier")
    e("s_mov_b32 %s, %s" % (s(TMP), s(OFF0)))
    e("s_mov_b32 %s, %s" % (s(OFF0), s(OFF1)))
    e("s_mov_b32 %s, %s" % (s(OFF1), s(OFF2)))
    e("s_mov_b32 %s, %s" % (s(OFF2), s(OFF3)))
    e("s_mov_b32 %s, %s" % (s(OFF3), s(TMP)))
    e("s_add_u32 %s, %s, 1" % (s(IT), s(IT)))
    return (lab_resc, lab_back), (lab_resc2, lab_back2)


def main():
    # ------------------------------------------------------------------ entry: inputs -> fixed registers
    e("s_mov_b64 %s, %%[kv]" % s(KV, 2))
    e("s_mov_b64 %s, %%[bt]" % s(BT, 2))
    e("s_mov_b32 %s, %%[kvb]" % s(KVB))
    e("s_mov_b32 %s, %%[kve]" % s(KVE))
    e("s_mov_b32 %s, %%[cl2]" % s(CL2))
    e("s_mov_b32 %s, %%[npp]" % s(NPP))
    e("s_mov_b32 %s, %%[nb1]" % s(NB1))
    e("s_mov_b32 %s, %%[flg]" % s(FLG))
    e("s_mov_b32 %s, %%[ntl]" % s(NT))
    e("s_mov_b32 %s, %%[ostr]" % s(OSTR))
    e("s_mov_b64 %s, %%[qp]" % s(QP, 2))
    e("v_mov_b32 %s, %%[tid]" % v(X0))
    if DEBUG:
        e("v_mov_b32 %s, %s" % (v(TIDR), v(X0)))
    e("s_mov_b32 %s, 0x%08x" % (s(THR), 0x41000000))  # TAU = 8.0f
    e("v_and_b32 %s, 63, %s" % (v(LANE), v(X0)))
    e("v_lshrrev_b32 %s, 6, %s" % (v(X1), v(X0)))
    e("s_nop 0")
    e("v_readfirstlane_b32 %s, %s" % (s(WAVE), v(X1)))
    # hand-off record of this thread
    e("v_lshlrev_b32 %s, 5, %s" % (v(X0), v(X0)))
    e("v_add_u32 %s, %d, %s" % (v(X0), HOFF, v(X0)))
    e("ds_read_b128 %s, %s" % (v(T[0], 4), v(X0)))
    e("ds_read_b128 %s, %s offset:16" % (v(T[4], 4), v(X0)))
    e("s_waitcnt lgkmcnt(0)")
    e("v_mov_b32 %s, %s" % (v(OPTR), v(T[2])))
    e("v_mov_b32 %s, %s" % (v(OPTR + 1), v(T[3])))
    e("v_mov_b32 %s, %s" % (v(MLPTR), v(T[4])))
    e("v_mov_b32 %s, %s" % (v(MLPTR + 1), v(T[5])))
    # lane geometry
    e("v_and_b32 %s, 31, %s" % (v(X0), v(LANE)))                       # rl
    e("v_lshrrev_b32 %s, 5, %s" % (v(X1), v(LANE)))                    # g
    e("v_lshlrev_b32 %s, 2, %s" % (v(DROW), v(X1)))                    # 4g (DROW is free here)
    e("v_lshlrev_b32 %s, 4, %s" % (v(X2), v(X1)))                      # 16g
    e("s_mov_b32 %s, %d" % (s(SPITCH), PITCH))
    e("v_mad_u32_u24 %s, %s, %s, %s" % (v(KADDR_LANE), v(X0), s(SPITCH), v(X2)))
    e("v_bfe_u32 %s, %s, 2, 2" % (v(X0), v(LANE)))                     # (lane & 15) >> 2
    e("v_add_u32 %s, %s, %s" % (v(X0), v(DROW), v(X0)))                # 4g + ...
    e("v_bfe_u32 %s, %s, 4, 1" % (v(X1), v(LANE)))                     # (lane >> 4) & 1
    e("v_lshlrev_b32 %s, 5, %s" % (v(X1), v(X1)))                      # *16 elements *2 bytes
    e("v_and_b32 %s, 3, %s" % (v(X2), v(LANE)))
    e("v_lshlrev_b32 %s, 3, %s" % (v(X2), v(X2)))                      # *4 elements *2 bytes
    e("v_add_u32 %s, %s, %s" % (v(X1), v(X1), v(X2)))
    e("v_mad_u32_u24 %s, %s, %s, %s" % (v(VADDR_LANE), v(X0), s(SPITCH), v(X1)))
    # ------------------------------------------------------------------ page ids of this split -> one lane each
    lab_nobt = label("nobt")
    e("s_lshr_b32 %s, %s, 7" % (s(PG0), s(KVB)))
    e("v_mov_b32 %s, 0" % v(PAGES))
    e("s_cmp_eq_u64 %s, 0" % s(BT, 2))
    e("s_cbranch_scc1 %s" % lab_nobt)
    e("s_add_u32 %s, %s, 127" % (s(S0), s(KVE)))
    e("s_lshr_b32 %s, %s, 7" % (s(S0), s(S0)))
    e("s_sub_u32 %s, %s, %s" % (s(S0), s(S0), s(PG0)))                   # pages in this split (<= 64)
    e("v_cmp_gt_u32 vcc, %s, %s" % (s(S0), v(LANE)))
    e("s_mov_b64 %s, exec" % s(EXS, 2))
    e("s_nop 1")
    e("s_and_b64 exec, exec, vcc")
    e("v_add_u32 %s, %s, %s" % (v(X0), s(PG0), v(LANE)))
    e("v_lshlrev_b32 %s, 2, %s" % (v(X0), v(X0)))
    e("global_load_dword %s, %s, %s" % (v(PAGES), v(X0), s(BT, 2)))
    e("s_waitcnt vmcnt(0)")
    e("s_mov_b64 exec, %s" % s(EXS, 2))
    e("v_max_i32 %s, 0, %s" % (v(PAGES), v(PAGES)))
    e("v_min_i32 %s, %s, %s" % (v(PAGES), s(NPP), v(PAGES)))
    e("%s:" % lab_nobt)
    # ------------------------------------------------------------------ state
    e("v_mov_b32 %s, 0xff800000" % v(MRUN))
    e("v_mov_b32 %s, 0" % v(LRUN))
    e("s_mov_b32 %s, 0" % s(OFF0))
    e("s_mov_b32 %s, %d" % (s(OFF1), TILE_BYTES))
    e("s_mov_b32 %s, %d" % (s(OFF2), 2 * TILE_BYTES))
    e("s_mov_b32 %s, %d" % (s(OFF3), 3 * TILE_BYTES))
    e("s_mov_b32 %s, 0" % s(IT))
    for i in range(256):
        e("v_accvgpr_write_b32 %s, 0" % a(i))
    # ------------------------------------------------------------------ prologue: tiles 0, 1, 2, S of tile 0
    e("s_mov_b32 %s, 0" % s(TMP))
    for ln in dma_tile_lines(TMP, OFF0):
        e(ln)
    lab_one = label("one")
    lab_three, lab_pw = label("three"), label("pw")
    e("s_cmp_lt_u32 %s, 2" % s(NT))
    e("s_cbranch_scc1 %s" % lab_one)
    e("s_mov_b32 %s, 1" % s(TMP))
    for ln in dma_tile_lines(TMP, OFF1):
        e(ln)
    e("s_cmp_lt_u32 %s, 3" % s(NT))
    e("s_cbranch_scc1 %s" % lab_one)
    e("s_mov_b32 %s, 2" % s(TMP))
    for ln in dma_tile_lines(TMP, OFF2):
        e(ln)
    e("%s:" % lab_one)
    # ------------------------------------------------------------------ Q operands: 36 coalesced 16-byte loads per lane from
    # the packed image, issued behind the tile DMAs (one memory latency for everything)
    e("v_lshlrev_b32 %s, 4, %s" % (v(X0), v(LANE)))
    e("s_mul_i32 %s, %s, %d" % (s(S0), s(WAVE), 36 * 1024))
    e("s_add_u32 %s, %s, %s" % (s(QP), s(QP), s(S0)))
    e("s_addc_u32 %s, %s, 0" % (s(QP + 1), s(QP + 1)))
    for ks in range(36):
        if ks and ks % 4 == 0:
            e("s_add_u32 %s, %s, 4096" % (s(QP), s(QP)))
            e("s_addc_u32 %s, %s, 0" % (s(QP + 1), s(QP + 1)))
        e("global_load_dwordx4 %s, %s, %s offset:%d" % (v(Q0 + 4 * ks, 4), v(X0), s(QP, 2), (ks % 4) * 1024))
    e("s_waitcnt vmcnt(0)")
    e("s_barrier")
    if DEBUG:
        # FLG bit 1: dump LDS tile 0 (2336 chunks) to the debug pointer and stop
        lab = label("nodump1")
        e("s_bitcmp1_b32 %s, 1" % s(FLG))
        e("s_cbranch_scc0 %s" % lab)
        for k in range(10):
            lab2 = label("skipchunk")
            e("v_add_u32 %s, %d, %s" % (v(X1), 256 * k, v(TIDR)))
            e("v_cmp_gt_u32 vcc, %d, %s" % (32 * CPR, v(X1)))
            e("s_mov_b64 %s, exec" % s(EXS, 2))
            e("s_nop 1")
            e("s_and_b64 exec, exec, vcc")
            e("v_lshlrev_b32 %s, 4, %s" % (v(X1), v(X1)))
            e("v_add_u32 %s, %s, %s" % (v(X2), s(OFF0), v(X1)))
            e("ds_read_b128 %s, %s" % (v(SA, 4), v(X2)))
            e("v_add_co_u32 %s, vcc, %s, %s" % (v(SB), v(DBG), v(X1)))
            e("s_nop 1")
            e("v_addc_co_u32 %s, vcc, 0, %s, vcc" % (v(SB + 1), v(DBG + 1)))
            e("s_waitcnt lgkmcnt(0)")
            e("global_store_dwordx4 %s, %s, off" % (v(SB, 2), v(SA, 4)))
            e("s_mov_b64 exec, %s" % s(EXS, 2))
        e("s_waitcnt vmcnt(0)")
        e("s_endpgm")
        e("%s:" % lab)
    e("v_add_u32 %s, %s, %s" % (v(KADDR), s(OFF0), v(KADDR_LANE)))
    for slot in qk_slots(SA, KADDR):
        slot()
    if DEBUG:
        lab = label("nodump2")
        e("s_bitcmp1_b32 %s, 2" % s(FLG))
        e("s_cbranch_scc0 %s" % lab)
        e("s_nop 7")
        e("s_nop 7")
        e("s_nop 7")
        e("v_lshlrev_b32 %s, 6, %s" % (v(X1), v(TIDR)))
        e("v_add_co_u32 %s, vcc, %s, %s" % (v(DBG), v(DBG), v(X1)))
        e("s_nop 1")
        e("v_addc_co_u32 %s, vcc, 0, %s, vcc" % (v(DBG + 1), v(DBG + 1)))
        for k in range(4):
            e("global_store_dwordx4 %s, %s, off offset:%d" % (v(DBG, 2), v(SA + 4 * k, 4), 16 * k))
        e("s_waitcnt vmcnt(0)")
        e("s_endpgm")
        e("%s:" % lab)
    # ------------------------------------------------------------------ main loop (two halves: S roles swap)
    lab_loop, lab_end = label("loop"), label("end")
    e("%s:" % lab_loop)
    r1 = half_iteration(SA, SB, "A")
    e("s_cmp_ge_u32 %s, %s" % (s(IT), s(NT)))
    e("s_cbranch_scc1 %s" % lab_end)
    r2 = half_iteration(SB, SA, "B")
    e("s_cmp_lt_u32 %s, %s" % (s(IT), s(NT)))
    e("s_cbranch_scc1 %s" % lab_loop)
    e("s_branch %s" % lab_end)
    # out-of-line rescale blocks
    for pairs in (r1, r2):
        for resc, back in pairs:
            e("%s:" % resc)
            rescale_block(back)
    e("%s:" % lab_end)
    # ------------------------------------------------------------------ epilogue
    e("s_nop 7")
    e("s_nop 7")
    e("s_nop 7")
    # l_tot = l(lane) + l(lane ^ 32)
    e("v_mov_b32 %s, %s" % (v(T[0]), v(LRUN)))
    e("v_mov_b32 %s, %s" % (v(T[1]), v(LRUN)))
    e("s_nop 1")
    e("v_permlane32_swap_b32 %s, %s" % (v(T[0]), v(T[1])))
    e("s_nop 1")
    e("v_add_f32 %s, %s, %s" % (v(LRUN), v(T[0]), v(T[1])))
    # scale: 1/l when this launch writes the final output, 1 otherwise
    lab_part = label("part")
    e("v_rcp_f32 %s, %s" % (v(T[2]), v(LRUN)))
    # one Newton step: r = r * (2 - l*r)   (keeps the quotient within 1 ulp; l = 0 still gives inf/NaN)
    e("s_nop 0")
    e("v_fma_f32 %s, -%s, %s, 2.0" % (v(T[3]), v(LRUN), v(T[2])))
    e("v_mul_f32 %s, %s, %s" % (v(T[3]), v(T[2]), v(T[3])))
    e("s_mov_b32 %s, 0x1f8" % s(SCLS))
    e("v_cmp_class_f32 vcc, %s, %s" % (v(T[3]), s(SCLS)))   # finite?  (normal/denormal/zero, either sign)
    e("s_nop 1")
    e("v_cndmask_b32 %s, %s, %s, vcc" % (v(T[2]), v(T[2]), v(T[3])))
    e("%s:" % lab_part)
    # rows past n_rows store nothing
    e("v_cmp_ne_u64 vcc, 0, %s" % v(OPTR, 2))
    e("s_mov_b64 %s, exec" % s(EXS, 2))
    e("s_nop 1")
    e("s_and_b64 exec, exec, vcc")
    # O^T block i, element 4j+c is column 32 i + 8 j + 4 g + c.
    # Final output (FLG bit 0): row-major rows of dst; the out pointer already includes the 4*g float offset.
    # Split-K partial: layout [column/4][row][4 floats] so that the 32 lanes of a half-wave write 512 contiguous bytes;
    # the out pointer already includes (g*n_rows + row)*16 bytes and every (i, j) step advances it by 2*n_rows*16 bytes.
    lab_pstore, lab_sdone = label("pstore"), label("sdone")
    if NO_STORE:
        e("s_branch %s" % lab_sdone)
    e("s_bitcmp1_b32 %s, 0" % s(FLG))
    e("s_cbranch_scc0 %s" % lab_pstore)
    for i in range(16):
        for j in range(4):
            r = T[4] if (i * 4 + j) % 2 == 0 else SA  # alternate two 4-register staging groups
            for c in range(4):
                e("v_accvgpr_read_b32 %s, %s" % (v(r + c), a(16 * i + 4 * j + c)))
            for c in range(4):
                e("v_mul_f32 %s, %s, %s" % (v(r + c), v(r + c), v(T[2])))
            e("global_store_dwordx4 %s, %s, off offset:%d" % (v(OPTR, 2), v(r, 4), (32 * i + 8 * j) * 4))
    e("s_branch %s" % lab_sdone)
    e("%s:" % lab_pstore)
    # partial: O / l of this split as f16, layout [column/4][row][4 halves]; T[2] holds 1/l here as well
    for i in range(16):
        for j in range(4):
            r = T[4] if (i * 4 + j) % 2 == 0 else SA
            for c in range(4):
                e("v_accvgpr_read_b32 %s, %s" % (v(r + c), a(16 * i + 4 * j + c)))
            for c in range(4):
                e("v_mul_f32 %s, %s, %s" % (v(r + c), v(r + c), v(T[2])))
            e("v_cvt_pk_f16_f32 %s, %s, %s" % (v(r), v(r), v(r + 1)))
            e("v_cvt_pk_f16_f32 %s, %s, %s" % (v(r + 1), v(r + 2), v(r + 3)))
            e("s_nop 0")
            e("global_store_dwordx2 %s, %s, off" % (v(OPTR, 2), v(r, 2)))
            e("v_add_co_u32 %s, vcc, %s, %s" % (v(OPTR), s(OSTR), v(OPTR)))
            e("s_nop 1")
            e("v_addc_co_u32 %s, vcc, 0, %s, vcc" % (v(OPTR + 1), v(OPTR + 1)))
    e("%s:" % lab_sdone)
    # (m, l) of this split, written by the g == 0 lane of each row when a pointer was handed over
    e("v_cmp_ne_u64 vcc, 0, %s" % v(MLPTR, 2))
    e("s_nop 1")
    e("s_and_b64 exec, exec, vcc")
    e("v_mov_b32 %s, %s" % (v(T[0]), v(MRUN)))
    e("v_mov_b32 %s, %s" % (v(T[1]), v(LRUN)))
    e("s_nop 0")
    e("global_store_dwordx2 %s, %s, off" % (v(MLPTR, 2), v(T[0], 2)))
    e("s_mov_b64 exec, %s" % s(EXS, 2))
    e("s_waitcnt vmcnt(0)")

    print("// generated by gen_decode_asm.py%s -- do not edit" % (" --f16" if F16 else ""))
    for ln in out:
        print('"%s\\n\\t"' % ln)


main()
