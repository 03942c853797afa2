#!/usr/bin/env python3
"""Generates mla_decode_asm*.inc: the hand-scheduled gfx950 instruction streams of the pipelined MLA decode kernel
(one inline-asm block each inside mla_decode_kernel.hip).  Usage: python gen_decode_asm.py [--f16 | --q8 | --cvt] [--mask [--bias]]
> mla_decode_asm[_f16|_q8|_cvt][_mask|_bias].inc

Why a generator: the kernel keeps Q (144 VGPRs) and the O accumulator (256 AGPRs) resident, which leaves ~110
registers for everything else; the instruction order (MFMA issue slots filled with LDS reads and softmax VALU work)
and the register map are fixed here instead of being left to a compiler that spills under that pressure.

Work of one wave (32 attention rows, all 512 output columns), per 32-token tile `it`:
    part 1   36 MFMA of S = K[it+1].Q^T alternating with the first 36 MFMA of O^T += V[it]^T.P[it]^T (independent
             accumulators), with the address arithmetic + issue of the LDS-DMA loads of tile it+3 in their shadow
    part 2   the remaining P.V MFMAs of tile it with softmax(S[it+1]) -> P[it+1] (in place) in their shadow
    end      deferred accumulator rescale (rare), s_waitcnt vmcnt; s_barrier   (tile it+2 has landed for every wave)
The two 16-register score/P groups swap roles every tile, so the loop body is emitted twice.
"""
import sys

CLKP = "--clk-parts" in sys.argv    # with --clk: accumulate the cycles of part 1 / part 2 of the iterations instead of the waits
CLK = "--clk" in sys.argv or CLKP           # timing experiments only: s_memtime stamps, written to the hand-off area at the end
MASK = "--mask" in sys.argv  # additive f16 mask rows (one per query token), added to the scaled scores
Q8 = "--q8" in sys.argv    # Q8_0 KV: raw tiles staged in LDS, dequantized to an f16 tile one tile ahead, then the f16 path
CVTB = "--cvt" in sys.argv  # bf16 KV converted in place to f16 inside LDS one tile ahead (exact between 2^-14 and 65504, saturating
                            # beyond), then the f16 path: 68 MFMAs per tile instead of the 100 the hi + lo halves of a bf16 P need
F16 = "--f16" in sys.argv or Q8 or CVTB  # f16 KV: f16 MFMA, single P (no lo half)
MF = "v_mfma_f32_32x32x16_f16" if F16 else "v_mfma_f32_32x32x16_bf16"
CVT = "v_cvt_pk_f16_f32" if F16 else "v_cvt_pk_bf16_f32"
SPLIT = not F16
BIAS = "--bias" in sys.argv  # mask builds of the f16 kinds: ALiBi slope per head on the mask values, tanh soft cap on the logits (see bias_block)
assert (MASK and not SPLIT and not CLK) or not BIAS

PITCH = 1168
TILE_BYTES = 32 * PITCH
NBUF = 3 if Q8 else 4          # 16-bit tiles resident in LDS
Q8_ROW = 612                   # 18 blocks of (f16 d, 32 x int8)
RAW_TILE = 32 * Q8_ROW         # 19584 = 1224 x 16 bytes; Q8_0 builds keep two raw tiles behind the 16-bit tiles
RAW0 = NBUF * TILE_BYTES
RAW1 = RAW0 + RAW_TILE
HOFF = RAW1 + RAW_TILE if Q8 else NBUF * TILE_BYTES   # hand-off area written by the C++ prologue: 32 bytes per thread
DMA_PER_TILE = 5 if Q8 else 10 # LDS-DMA instructions each wave issues per tile
# Tile copies of the unmasked 16-bit programs carry the non-temporal hint: a decode step reads every key once, and cells streamed
# through the L2s without it push out what is read again (the operand image, the partials).  Not the masked programs (prompt chunks
# re-read their cells from one row block to the next) and not the Q8_0 programs (their kernel measured 3 % slower with it).
NT_HINT = "" if MASK or Q8 else " nt"
# The f16 partial rows and the (m, l) pairs go to another kernel, on other XCDs: stored at device scope they are written through as
# they are produced instead of at the kernel's end (see gen_decode_cs_asm.py)
PARTIAL_SCOPE = " sc1"
Q8_WAVE_CHUNKS = 306           # a wave copies 306 of the 1224 16-byte chunks of a raw tile
CPR = 73                       # 16-byte chunks per padded row
WAVE_CHUNKS = 8 * CPR          # 584: each wave moves rows 8w..8w+7 of a tile
TAU = 8.0
P1_PV = 24 if SPLIT else 12   # P.V MFMAs issued among the 36 QK^T MFMAs; the rest cover the softmax
P1_LEAD = 3                   # P.V MFMAs at the head of an iteration (they cover the first K fragment reads)

# ---- VGPR map
Q0 = 0
SA, SB = 144, 160   # two 16-register groups: scores of one tile, converted in place to its P^T operands
KF, KRING = 176, (3 if Q8 else 4) if MASK else 5   # K fragment ring (x 4 registers); what a masked build takes from it goes to the mask values
ALPHA = 196
RELOAD_PTRS = Q8 and MASK           # the output pointers are read again from the hand-off record in the epilogue: their registers carry MOFF
MOFF = 232 if RELOAD_PTRS else 197  # mask builds: byte offset of this lane's first mask element inside a tile's 64 mask bytes
# V^T fragment ring (x 4 registers); 220..223 go to the mask values / the dequantizer / the converter.  v252..v255 are never used: the clobber list of the asm block ends at v251, and the compiler
# keeps what lives across the block there (among it the lanes it spills scalar registers to).
VF, VRING = 200, 5 if MASK or Q8 else 6
assert 30 % VRING == 0   # the hand-over between tiles relies on the last two fragments of a tile sitting in ring slots 0 and 1
MKR = [192, 193, 194, 195] + ([188, 189, 190, 191] if Q8 else [220, 221, 222, 223])   # mask builds: the 16 f16 mask values of this lane's 16 tokens of a tile
T = list(range(224, 232))
OPTR, MLPTR = 232, 234
KADDR_LANE, VADDR_LANE, MRUN, LRUN, NEGM = 236, 237, 238, 239, 240
DROW, DCOL, VOFF, PAGES = 241, 242, 243, 244
LANE, KADDR, VADDR, TMAX = 245, 246, 247, 248
X0, X1, X2 = 249, 250, 251
SLOPE = 252         # bias builds: ALiBi slope of this lane's row (one register more than the other builds own)
N_VGPR = 253 if BIAS else 252
# ---- SGPR map (all inside the clobbered range s40..s79)
KV, BT, KVB, KVE, CL2, NPP, NB1, FLG = 40, 42, 44, 45, 46, 47, 48, 49
NT, IT, OFF0, OFF1, OFF2, WAVE, TB, TMP, NVM1 = 50, 51, 52, 53, 54, 55, 56, 58, 59
RAWC, RAWN, SH, SHM2, PSEL = 74, 77, 78, 79, 72   # Q8_0 builds: raw buffer to dequantize / to load into (OFF3's and a free register), byte shifts and the
                                                  # v_perm selector of the dequantizer (QP's and SPITCH's registers once the prologue is done with them)
RAWB, DSTB, DZ = 197, 198, 199                    # Q8_0 builds: per-lane raw window / f16 destination offsets, all-ones where this lane's row is valid
SCL, L2E, MSK = (82, 73, 80) if Q8 else (77, 73, 78)   # mask builds: scale, log2(e) (the register of SCLS until the epilogue), mask base (QP's registers once Q is loaded;
                                                        # Q8_0 builds keep the dequantizer's scalars there and take s80..s83)
ONES = 83   # f16 builds: packed (1.0, 1.0)
K1, K2 = CL2, NPP   # bias builds: 2 log2(e) scale / softcap (the input that carries c_log2 elsewhere) and -2 softcap, 0 = no soft cap
                    # (NPP's register once the page ids are clamped; until then it waits in the upper half of RSC)
EXS, S0, S1, S2, S3, DMAB, NVAL, THR, PG0, RSC, SPITCH, SCLS, OFF3, VMW, OSTR, QP = 60, 62, 63, 64, 65, 66, 67, 68, 69, 70, 72, 73, 74, 75, 76, 78

out = []
uid = [0]


def e(s):
    out.append(s)


def label(prefix):
    uid[0] += 1
    return "L%s_%d_%%=" % (prefix, uid[0])


def v(i, n=1):
    assert 0 <= i and i + n - 1 < N_VGPR, (i, n)   # v252..v255 belong to the compiler
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
            after = min(len(self.pending) - 1 - self.pending.index(tag), 15)   # the counter field has 4 bits
            e("s_waitcnt lgkmcnt(%d)" % after)
            self.pending = self.pending[len(self.pending) - after:] if after else []

    def drain(self):
        if self.pending:
            e("s_waitcnt lgkmcnt(0)")
            self.pending = []


lds = Lds()


def stamp(k):
    """--clk builds: shader-clock time stamp k into s[80+2k:81+2k]."""
    if CLK:
        e("s_memtime %s" % s(100 if k == 6 else 80 + 2 * k, 2))
        e("s_waitcnt lgkmcnt(0)")


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
                emit_item(valu[vi])
                vi += 1
    while vi < len(valu):
        emit_item(valu[vi])
        vi += 1


def emit_item(x):
    """A shadow item is a line or a callable that emits lines (LDS accesses go through the tracker)."""
    if x is None:
        return
    if callable(x):
        x()
    else:
        e(x)


# ---------------------------------------------------------------------------------------------------------------
PGZ = 75   # prologue only (VMW's register): id of the split's first page, handed over as a scalar


def tile_base_lines(tile_sreg, first_page_scalar=False):
    """Scalar lines: s[TB:TB+1] = address of the first row of tile s[tile_sreg]; s[NVM1] = its valid rows - 1.
    first_page_scalar: a tile inside the split's first page takes the page id from s[PGZ] instead of the lane of PAGES
    (the prologue's tiles, issued while the vector load of the page ids may still be in flight)."""
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
    if first_page_scalar:
        L.append("s_cmp_eq_u32 %s, 0" % s(S1))
        L.append("s_cselect_b32 %s, %s, %s" % (s(S2), s(PGZ), s(S2)))
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
    return L


DQ_LOFF = 227   # lane * 16 for the flat raw-tile copy; as DQ_OUT + 3 the last register the dequantizer overwrites afterwards


def q8_dma_lines(tile_sreg, raw_sreg, first_page_scalar=False):
    """Q8_0 builds: the 19584 bytes of tile s[tile_sreg] (32 packed rows, contiguous in the pool) -> the raw buffer at
    LDS offset s[raw_sreg], as a flat copy: 306 chunks per wave, 4 full LDS-DMA instructions and one of 50 lanes."""
    L = tile_base_lines(tile_sreg, first_page_scalar)
    L.append("s_mul_i32 %s, %s, %d" % (s(DMAB), s(WAVE), Q8_WAVE_CHUNKS * 16))
    L.append("s_add_u32 %s, %s, %s" % (s(TB), s(TB), s(DMAB)))
    L.append("s_addc_u32 %s, %s, 0" % (s(TB + 1), s(TB + 1)))
    L.append("s_add_u32 %s, %s, %s" % (s(DMAB), s(DMAB), s(raw_sreg)))
    L.append("v_lshlrev_b32 %s, 4, %s" % (v(DQ_LOFF), v(LANE)))
    # no instruction offset on an LDS-DMA load: it would move the LDS address as well; the scalar base steps instead
    for j in range(4):
        L.append("\\n\\t".join(["s_add_u32 m0, %s, %d" % (s(DMAB), j * 1024),
                                "s_nop 0",
                                "global_load_lds_dwordx4 %s, %s" % (v(DQ_LOFF), s(TB, 2)),
                                "s_add_u32 %s, %s, 1024" % (s(TB), s(TB)),
                                "s_addc_u32 %s, %s, 0" % (s(TB + 1), s(TB + 1))]))
    L.append("\\n\\t".join(["s_add_u32 m0, %s, %d" % (s(DMAB), 4 * 1024),
                            "s_mov_b64 %s, exec" % s(EXS, 2),
                            "s_mov_b32 exec_lo, -1",
                            "s_mov_b32 exec_hi, 0x3ffff",                      # lanes 0..49
                            "global_load_lds_dwordx4 %s, %s" % (v(DQ_LOFF), s(TB, 2)),
                            "s_mov_b64 exec, %s" % s(EXS, 2)]))
    return L


DQ_OUT = 224                                  # T[0:3]: the 8 f16 values of a unit
DQ_W = [(228, 229, 241), (230, 231, 251), (222, 223, 250)]   # three 12-byte raw windows: the reads of the next two units are in flight during a unit's arithmetic
DQ_D = [249, 221]                             # the block scales of the two units in flight
RAWA, DSTA, RAWD = 242, 243, 220


def q8_dequant_items(raw_sreg, dst_sreg, tile_plus):
    """Q8_0 builds: raw tile at LDS offset s[raw_sreg] -> f16 tile at s[dst_sreg] (padded row layout).  A unit is
    8 values (one 16-byte destination chunk); a wave does 576 units in 9 steps: waves 0/1 the even blocks of rows
    0-15/16-31, waves 2/3 the odd blocks, lane = (row, quarter of the block).  The int8 values of an even block start
    2 bytes past a 4-byte boundary, those of an odd block on one: a unit reads the 12-byte window from that boundary and
    the same code shifts by s[SH] = 2 or 0 bytes; the block's f16 scale is read on its own (2-byte aligned).
    value = f16(q) * d in packed f16: one rounding of an exact product, the same number as f16(q * f32(d)).
    Rows past the end of the sequence become zeros (their bytes are not KV data).  tile_plus: the tile is IT + tile_plus."""
    I = []
    # valid rows of that tile: clamp(kv_end - kv_begin - 32*(IT + tile_plus), 0, 32), times the row pitch of the f16 tile
    I.append("s_add_u32 %s, %s, %d" % (s(S0), s(IT), tile_plus))
    I.append("s_lshl_b32 %s, %s, 5" % (s(S0), s(S0)))
    I.append("s_add_u32 %s, %s, %s" % (s(S0), s(S0), s(KVB)))
    I.append("s_sub_i32 %s, %s, %s" % (s(S0), s(KVE), s(S0)))
    I.append("s_max_i32 %s, %s, 0" % (s(S0), s(S0)))
    I.append("s_min_i32 %s, %s, 32" % (s(S0), s(S0)))
    I.append("s_mul_i32 %s, %s, %d" % (s(S0), s(S0), PITCH))
    I.append("v_cmp_gt_u32 vcc, %s, %s" % (s(S0), v(DSTB)))                      # row * PITCH + (< PITCH) < n_valid * PITCH
    I.append("v_add_u32 %s, %s, %s" % (v(RAWA), s(raw_sreg), v(RAWB)))
    I.append("v_add_u32 %s, %s, %s" % (v(DSTA), s(dst_sreg), v(DSTB)))
    I.append("v_cndmask_b32_e64 %s, 0, -1, vcc" % v(DZ))
    # the scale of (row, block 2u + parity) sits 8q (+ 2 for odd blocks) bytes before the window
    I.append("v_and_b32 %s, 3, %s" % (v(RAWD), v(LANE)))
    I.append("v_lshlrev_b32 %s, 3, %s" % (v(RAWD), v(RAWD)))
    I.append("v_add_u32 %s, %s, %s" % (v(RAWD), s(SHM2), v(RAWD)))
    I.append("v_sub_u32 %s, %s, %s" % (v(RAWD), v(RAWA), v(RAWD)))

    def reads_w(u):
        w = DQ_W[u % 3]
        def f0():
            lds.read("ds_read2_b32 %s, %s offset0:%d offset1:%d" % (v(w[0], 2), v(RAWA), 17 * u, 17 * u + 1), ("r", u, 0))
        def f1():
            lds.read("ds_read_b32 %s, %s offset:%d" % (v(w[2]), v(RAWA), 68 * u + 8), ("r", u, 1))
        return [f0, f1]

    def reads_d(u):
        def f2():
            lds.read("ds_read_u16 %s, %s offset:%d" % (v(DQ_D[u & 1]), v(RAWD), 68 * u), ("r", u, 2))
        return [f2]

    I += reads_w(0) + reads_d(0) + reads_w(1)
    for u in range(9):
        w, d = DQ_W[u % 3], DQ_D[u & 1]
        if u + 1 < 9:
            I += reads_d(u + 1)
        if u + 2 < 9:
            I += reads_w(u + 2)
        def first(u=u, w=w):
            lds.need(("r", u, 2))
            lds.need(("r", u, 1))
            e("v_alignbyte_b32 %s, %s, %s, %s" % (v(w[0]), v(w[1]), v(w[0]), s(SH)))      # values 0..3
        I.append(first)
        I.append("v_alignbyte_b32 %s, %s, %s, %s" % (v(w[1]), v(w[2]), v(w[1]), s(SH)))   # values 4..7
        I.append("v_perm_b32 %s, %s, %s, %s" % (v(d), v(d), v(d), s(PSEL)))              # d in both halves
        I.append("v_and_b32 %s, %s, %s" % (v(d), v(d), v(DZ)))
        for h in range(2):
            for j in range(4):
                el = 2 * j + h
                I.append("v_cvt_f16_i16_sdwa %s, sext(%s) dst_sel:WORD_%d dst_unused:%s src0_sel:BYTE_%d" % (
                    v(DQ_OUT + j), v(w[el // 4]), h, "UNUSED_PAD" if h == 0 else "UNUSED_PRESERVE", el % 4))
        for j in range(4):
            I.append("v_pk_mul_f16 %s, %s, %s" % (v(DQ_OUT + j), v(DQ_OUT + j), v(d)))
        def wr(u=u):
            lds.read("ds_write_b128 %s, %s offset:%d" % (v(DSTA), v(DQ_OUT, 4), 128 * u), ("w", u))
        I.append(wr)
    return I


# --cvt builds: this lane's byte offset inside a tile (v198 is free in every build without a dequantizer), and for the address and
# two temporaries the registers of NEGM, ALPHA and TMAX: those live from the softmax to the end of an iteration, the converter
# runs in part 1 and in the prologue
CVL, CADDR, CT0, CT1 = 198, 240, 196, 248


def cvt_items(off_sreg):
    """--cvt builds: the bf16 tile at LDS offset s[off_sreg] -> f16, in place.  A wave converts the eight rows it loaded
    itself (so only its own loads have to be back, no barrier): lane = (row, 16-byte column chunk mod 8), nine units of
    16 bytes 128 bytes apart.  Per 32-bit word: both halves widened to f32, v_cvt_pkrtz_f16_f32 (exact inside the f16
    range; round-toward-zero makes larger magnitudes 65504 instead of infinity).  The data registers are T[0:7], free
    in the part of the iteration that carries these items."""
    I = ["v_add_u32 %s, %s, %s" % (v(CADDR), s(off_sreg), v(CVL))]
    D = [T[0], T[4]]

    def rd(u):
        return lambda: lds.read("ds_read_b128 %s, %s offset:%d" % (v(D[u & 1], 4), v(CADDR), 128 * u), ("r", u))

    I.append(rd(0))
    for u in range(9):
        d = D[u & 1]
        if u + 1 < 9:
            I.append(rd(u + 1))
        def first(u=u, d=d):
            lds.need(("r", u))
            e("v_lshlrev_b32 %s, 16, %s" % (v(CT0), v(d)))
        I.append(first)
        for j in range(4):
            if j:
                I.append("v_lshlrev_b32 %s, 16, %s" % (v(CT0), v(d + j)))
            I.append("v_and_b32 %s, 0xffff0000, %s" % (v(CT1), v(d + j)))
            I.append("v_cvt_pkrtz_f16_f32 %s, %s, %s" % (v(d + j), v(CT0), v(CT1)))
        I.append("s_nop 0")
        I.append(lambda u=u, d=d: lds.read("ds_write_b128 %s, %s offset:%d" % (v(CADDR), v(d, 4), 128 * u), ("w", u)))
    return I


PT = [241, 242, 243, 249, 250]   # 16-bit tiles: per-lane byte offsets of the 10 LDS-DMA slots, two 16-bit values per register
DT = [251, 199]                  # address temporaries of the slots


def dma_table_lines():
    """Once per kernel: where the 16 bytes that lane l of LDS-DMA slot j copies sit inside a tile.  The LDS side of a slot
    is 64 consecutive 16-byte chunks of the padded tile (73 chunks per row, the 73rd is padding); the global side is
    row * nb1 + min(column chunk, 71) * 16 -- at most 31 * 1152 + 1136, so two offsets share a register.  The walk
    over (row, column chunk) is done here and never again: per tile a slot costs two VALU instructions."""
    L = []
    row, col, x0, x1, x2 = T[0], T[1], T[2], T[3], T[4]
    L.append("v_mov_b32 %s, %s" % (v(col), v(LANE)))
    L.append("s_lshl_b32 %s, %s, 3" % (s(S2), s(WAVE)))
    L.append("v_mov_b32 %s, %s" % (v(row), s(S2)))                     # a wave copies rows 8w .. 8w+7
    for j in range(10):
        L.append("v_min_u32 %s, 71, %s" % (v(x1), v(col)))
        L.append("v_lshlrev_b32 %s, 4, %s" % (v(x1), v(x1)))
        L.append("v_mad_u32_u24 %s, %s, %s, %s" % (v(x0), v(row), s(NB1), v(x1)))
        if j % 2 == 0:
            L.append("v_mov_b32 %s, %s" % (v(PT[j // 2]), v(x0)))
        else:
            L.append("v_lshl_or_b32 %s, %s, 16, %s" % (v(PT[j // 2]), v(x0), v(PT[j // 2])))
        if j < 9:
            # advance 64 chunks: col += 64; if (col >= 73) { col -= 73; row += 1 }
            L.append("v_add_u32 %s, 64, %s" % (v(col), v(col)))
            L.append("v_cmp_le_u32 vcc, %d, %s" % (CPR, v(col)))
            L.append("v_subrev_u32 %s, %d, %s" % (v(x2), CPR, v(col)))
            L.append("v_add_u32 %s, 1, %s" % (v(x0), v(row)))
            L.append("s_nop 0")
            L.append("v_cndmask_b32 %s, %s, %s, vcc" % (v(col), v(col), v(x2)))
            L.append("v_cndmask_b32 %s, %s, %s, vcc" % (v(row), v(row), v(x0)))
    return L


def dma_tile_lines(tile_sreg, off_sreg, first_page_scalar=False):
    """Instruction list (to be interleaved) that issues the LDS-DMA loads of tile index s[tile_sreg] into the buffer
    at LDS offset s[off_sreg].  Scalar part first (tile base address), then 10 slots whose per-lane offsets come from
    the table of dma_table_lines.  Rows past the end of the sequence are replaced by the last 16 bytes of the last valid
    row (any finite data will do: their probabilities are exactly 0): one v_min against that offset."""
    L = tile_base_lines(tile_sreg, first_page_scalar)
    L.append("s_mul_i32 %s, %s, %s" % (s(S3), s(NVM1), s(NB1)))
    L.append("s_add_u32 %s, %s, %d" % (s(S3), s(S3), 71 * 16))
    # LDS destination of this wave's first slot
    L.append("s_mul_i32 %s, %s, %d" % (s(DMAB), s(WAVE), WAVE_CHUNKS * 16))
    L.append("s_add_u32 %s, %s, %s" % (s(DMAB), s(DMAB), s(off_sreg)))
    for j in range(10):
        t = DT[j & 1]
        if j % 2 == 0:
            L.append("v_and_b32 %s, 0xffff, %s" % (v(t), v(PT[j // 2])))
        else:
            L.append("v_lshrrev_b32 %s, 16, %s" % (v(t), v(PT[j // 2])))
        L.append("v_min_u32 %s, %s, %s" % (v(t), s(S3), v(t)))
        if j == 9:
            # 8 chunks left per wave: lanes 0..7 only.  One atomic group: nothing may be scheduled inside the exec window.
            L.append("\\n\\t".join(["s_add_u32 m0, %s, %d" % (s(DMAB), j * 1024),
                                    "s_mov_b64 %s, exec" % s(EXS, 2),
                                    "s_mov_b64 exec, 0xff",
                                    "global_load_lds_dwordx4 %s, %s%s" % (v(t), s(TB, 2), NT_HINT),
                                    "s_mov_b64 exec, %s" % s(EXS, 2)]))
        else:
            L.append("\\n\\t".join(["s_add_u32 m0, %s, %d" % (s(DMAB), j * 1024),
                                    "s_nop 0",
                                    "global_load_lds_dwordx4 %s, %s%s" % (v(t), s(TB, 2), NT_HINT)]))
    return L


def k_read(kaddr, p):
    lds.read("ds_read_b128 %s, %s offset:%d" % (v(KF + 4 * (p % KRING), 4), v(kaddr), p * 32), ("k", p))


def k_warm(kaddr):
    """First K fragments of a tile into the ring."""
    for p in range(KRING - 1):
        k_read(kaddr, p)


def qk_slots(sreg, kaddr):
    """36 MFMA slots of S = K.Q^T into v[sreg:sreg+15]; K fragments come through a ring (k_warm first)."""
    depth = KRING - 1

    def mk(ks):
        def slot():
            lds.need(("k", ks))
            c = "0" if ks == 0 else v(sreg, 16)
            e("%s %s, %s, %s, %s" % (MF, v(sreg, 16), v(KF + 4 * (ks % KRING), 4), v(Q0 + 4 * ks, 4), c))
            # the next fragment read goes right behind the MFMA, ahead of the VALU work of this slot: an LDS read that
            # follows VALU instructions in the shadow of an MFMA delays the next MFMA by 8 cycles more than one that leads them
            if ks + depth < 36:
                k_read(kaddr, ks + depth)
        return slot
    return [mk(ks) for ks in range(36)]


V_FRAGS = [(kk, db) for kk in range(2) for db in range(16)]


def v_read(vaddr, idx):
    kk, db = V_FRAGS[idx]
    r = VF + 4 * (idx % VRING)
    base = 16 * kk * PITCH + db * 64
    lds.read("ds_read_b64_tr_b16 %s, %s offset:%d" % (v(r, 2), v(vaddr), base), ("v", idx, 0))
    lds.read("ds_read_b64_tr_b16 %s, %s offset:%d" % (v(r + 2, 2), v(vaddr), base + 8 * PITCH), ("v", idx, 1))


def v_warm(vaddr):
    """First V^T fragments of a tile into the ring (issued at the end of the previous tile)."""
    for idx in range(VRING - 1):
        v_read(vaddr, idx)


def canon_tags():
    """LDS reads in flight at the top of every iteration, in issue order (see tile_handover)."""
    vt = lambda idx: [("v", idx, 0), ("v", idx, 1)]
    kt = [("k", p) for p in range(KRING - 1)]
    t = []
    for idx in range(2, VRING - 1):
        t += vt(idx)
    return t + kt + vt(0) + vt(1)


def tile_handover(kaddr_off, vaddr_off, last_slots, sync):
    """The hand-over from tile IT to tile IT+1, placed before the last two P.V MFMAs of tile IT so that it costs no
    MFMA time: first fragment reads of the next iteration (V^T of tile IT+1 from the buffer at s[vaddr_off], K of tile
    IT+2 from s[kaddr_off]) around the wait for the tile loads and the workgroup barrier (`sync` emits them).
    Ring slots 0 and 1 of the V^T ring are still needed by the last two MFMAs, so fragments 0 and 1 follow them."""
    lds.need(("v", 31, 1))          # every read of tile IT's buffer has returned: the buffer may be overwritten
    e("v_add_u32 %s, %s, %s" % (v(VADDR), s(vaddr_off), v(VADDR_LANE)))
    for idx in range(2, VRING - 1):
        v_read(VADDR, idx)
    if Q8 or CVTB:
        lds.need(("w", 8))              # this wave's share of the next f16 tile is written
    sync()
    e("v_add_u32 %s, %s, %s" % (v(KADDR), s(kaddr_off), v(KADDR_LANE)))
    k_warm(KADDR)
    for n in range(2):
        if n < len(last_slots):
            last_slots[n]()
        v_read(VADDR, n)
    assert lds.pending == canon_tags(), (lds.pending, canon_tags())


def pv_slots(vaddr, greg):
    """MFMA slots of O^T += V^T.P^T for the tile whose P^T operands sit in group `greg`
    (hi halves of k-step kk in greg+8kk .. +3, lo halves in greg+8kk+4 .. +7).  16 d-blocks x 2 k-steps, fragments
    through a ring (v_warm first), d-blocks in pairs so that MFMAs on the same accumulator are never adjacent."""
    depth = VRING - 1

    def mf(idx, lo, pre):
        kk, db = V_FRAGS[idx]
        def slot():
            lds.need(("v", idx, 1))
            e("%s %s, %s, %s, %s" % (MF, a(16 * db, 16), v(VF + 4 * (idx % VRING), 4), v(greg + 8 * kk + (4 if lo else 0), 4), a(16 * db, 16)))
            for p in pre:
                v_read(vaddr, p)
        return slot
    slots = []
    for pair in range(16):
        i0, i1 = 2 * pair, 2 * pair + 1
        n0 = [i0 + depth] if i0 + depth < 32 else []
        n1 = [i1 + depth] if i1 + depth < 32 else []
        slots.append(mf(i0, False, n0))
        if SPLIT:
            slots.append(mf(i1, False, []))
            slots.append(mf(i0, True, []))
            slots.append(mf(i1, True, n1))   # fragment i0's ring slot is only reused by reads issued after its last MFMA
        else:
            slots.append(mf(i1, False, n1))
    return slots


def mask_loads(tile_sreg):
    """Mask builds: the 64 mask bytes of tile s[tile_sreg] for this lane's query token -> MKR (four 8-byte loads)."""
    e("s_lshl_b32 %s, %s, 6" % (s(S0), s(tile_sreg)))
    e("s_add_u32 %s, %s, %s" % (s(S0), s(MSK), s(S0)))
    e("s_addc_u32 %s, %s, 0" % (s(S1), s(MSK + 1)))
    for j in range(4):
        e("global_load_dwordx2 %s, %s, %s offset:%d" % (v(MKR[2 * j], 2), v(MOFF), s(S0, 2), 16 * j))


def softmax_lines(sreg):
    """Softmax of the scores in group sreg, as one list of VALU lines (no branches):
    tile max -> lazy max update (new max only where it grew by more than TAU) -> ALPHA (rescale factor of O and l,
    1 where the max stayed) and RSC (non-zero when some lane changed its max; the accumulators are rescaled by the
    caller once the MFMAs of the current tile are done) -> p = 2^(s*c - m) -> l += sum p -> P^T operands in place:
    k-step kk: hi halves in sreg+8kk..+3, lo halves in sreg+8kk+4..+7."""
    L = []
    m = [T[0], T[1], T[2], T[3], T[4]]
    if MASK:
        # u = s * scale + mask (ggml-cpu.c:12048-12057 order), element k = token 8(k/4) + 4g + k%4
        for k in range(16):
            if BIAS:   # the logits were scaled (and capped) by bias_block(): u += slope * mask
                L.append("v_fma_mix_f32 %s, %s, %s, %s op_sel:[%d,0,0] op_sel_hi:[1,0,0]" % (v(sreg + k), v(MKR[2 * (k // 4) + (k % 4) // 2]), v(SLOPE), v(sreg + k), k % 2))
                continue
            t = T[5 + (k & 1)]
            L.append("v_cvt_f32_f16_sdwa %s, %s dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:WORD_%d" % (v(t), v(MKR[2 * (k // 4) + (k % 4) // 2]), k % 2))
            L.append("v_fma_f32 %s, %s, %s, %s" % (v(sreg + k), v(sreg + k), s(SCL), v(t)))
    CS = L2E if MASK else CL2           # factor from the values in sreg to log2 units
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
    L.append("v_mul_f32 %s, %s, %s" % (v(TMAX), s(CS), v(TMAX)))           # log2 units (the factor is > 0)
    L.append("v_add_f32 %s, %s, %s" % (v(m[2]), s(THR), v(MRUN)))           # m_run + TAU  (-inf stays -inf)
    L.append("v_sub_f32 %s, %s, %s" % (v(m[3]), v(MRUN), v(TMAX)))          # m_run - tmax
    L.append("v_exp_f32 %s, %s" % (v(m[3]), v(m[3])))                       # 2^(m_run - tmax); 0 when m_run = -inf
    L.append("v_cmp_gt_f32 vcc, %s, %s" % (v(TMAX), v(m[2])))               # this lane's max moves
    L.append("s_mov_b64 %s, vcc" % s(RSC, 2))
    L.append("s_nop 1")
    L.append("v_cndmask_b32 %s, 1.0, %s, vcc" % (v(ALPHA), v(m[3])))
    L.append("v_cndmask_b32 %s, %s, %s, vcc" % (v(MRUN), v(MRUN), v(TMAX)))
    L.append("v_mul_f32 %s, %s, %s" % (v(LRUN), v(LRUN), v(ALPHA)))
    # -m (0 when still -inf)
    L.append("v_mov_b32 %s, 0xff800000" % v(m[0]))
    L.append("v_cmp_eq_f32 vcc, %s, %s" % (v(MRUN), v(m[0])))
    L.append("v_sub_f32 %s, 0, %s" % (v(NEGM), v(MRUN)))
    L.append("s_nop 0")
    L.append("v_cndmask_b32 %s, %s, 0, vcc" % (v(NEGM), v(NEGM)))
    # p = 2^(s*c - m)
    for k in range(16):
        L.append("v_fma_f32 %s, %s, %s, %s" % (v(sreg + k), v(sreg + k), s(CS), v(NEGM)))
    for k in range(16):
        L.append("v_exp_f32 %s, %s" % (v(sreg + k), v(sreg + k)))
    # running sum (this lane's 16 tokens).  With a hi/lo pair the operands carry p to 2^-17 and the f32 values are summed;
    # a single f16 operand is p rounded to 11 bits, and there the sum is taken over the rounded values further down: the
    # output stays an exact weighted mean of V rows (with weights that moved by 2^-12), so a dominant key's V value is not
    # scaled by the rounding of its own weight.
    if SPLIT:
        L.append("v_add_f32 %s, %s, %s" % (v(T[0]), v(sreg + 0), v(sreg + 1)))
        L.append("v_add_f32 %s, %s, %s" % (v(T[1]), v(sreg + 2), v(sreg + 3)))
        for k in range(4, 16, 2):
            L.append("v_add_f32 %s, %s, %s" % (v(T[0]), v(T[0]), v(sreg + k)))
            L.append("v_add_f32 %s, %s, %s" % (v(T[1]), v(T[1]), v(sreg + k + 1)))
        L.append("v_add_f32 %s, %s, %s" % (v(T[0]), v(T[0]), v(T[1])))
        L.append("v_add_f32 %s, %s, %s" % (v(LRUN), v(LRUN), v(T[0])))
    # P^T operands in place.  k-step kk owns registers b = sreg+8kk .. +7, holding p of tokens
    # (8(2kk)+4g+0..3, 8(2kk+1)+4g+0..3); pairs (b0,b1) (b2,b3) (b4,b5) (b6,b7) become hi -> b0..b3, lo -> b4..b7.
    for kk in range(2):
        b = sreg + 8 * kk
        if not SPLIT:
            for j in range(4):
                L.append("%s %s, %s, %s" % (CVT, v(b + j), v(b + 2 * j), v(b + 2 * j + 1)))
            # l += the eight rounded values of this k-step: dot products with (1, 1), two chains
            for j in range(4):
                acc = T[j & 1]
                c = "0" if kk == 0 and j < 2 else v(acc)
                L.append("v_dot2_f32_f16 %s, %s, %s, %s" % (v(acc), v(b + j), s(ONES), c))
            if kk == 1:
                L.append("s_nop 2")   # a dot product's result may be read by another kind of VALU instruction three wait states later
                L.append("v_add_f32 %s, %s, %s" % (v(T[0]), v(T[0]), v(T[1])))
                L.append("v_add_f32 %s, %s, %s" % (v(LRUN), v(LRUN), v(T[0])))
            continue
        H, X, Y = T[0], T[1], T[2]
        Lo = [T[3], T[4], T[5], T[6]]
        for j in range(4):
            L.append("%s %s, %s, %s" % (CVT, v(H), v(b + 2 * j), v(b + 2 * j + 1)))
            L.append("v_lshlrev_b32 %s, 16, %s" % (v(X), v(H)))
            L.append("v_and_b32 %s, 0xffff0000, %s" % (v(Y), v(H)))
            L.append("v_sub_f32 %s, %s, %s" % (v(X), v(b + 2 * j), v(X)))
            L.append("v_sub_f32 %s, %s, %s" % (v(Y), v(b + 2 * j + 1), v(Y)))
            L.append("%s %s, %s, %s" % (CVT, v(Lo[j]), v(X), v(Y)))
            L.append("v_mov_b32 %s, %s" % (v(b + j), v(H)))       # b+j <= b+2j: already consumed
        for j in range(4):
            L.append("v_mov_b32 %s, %s" % (v(b + 4 + j), v(Lo[j])))
    return L


def rescale_block(ret_label):
    """Rare path, entered only when no MFMA is in flight on the accumulators: acc *= ALPHA (per lane = per row)."""
    e("s_nop 7")
    e("s_nop 7")
    e("s_nop 3")
    for i in range(0, 256, 4):
        for j in range(4):
            e("v_accvgpr_read_b32 %s, %s" % (v(T[3 + j]), a(i + j)))
        for j in range(4):
            e("v_mul_f32 %s, %s, %s" % (v(T[3 + j]), v(T[3 + j]), v(ALPHA)))
        for j in range(4):
            e("v_accvgpr_write_b32 %s, %s" % (a(i + j), v(T[3 + j])))
    e("s_nop 7")
    e("s_nop 7")
    e("s_branch %s" % ret_label)


def bias_block(sreg):
    """Bias builds (ggml-cpu.c:12041-12057: u = softcap * tanh(s * scale / softcap) + slope(head) * mask), once the scores of a tile are
    complete: s <- s * scale, or, with a soft cap, -2 softcap / (1 + 2^(s K1)) = softcap * tanh(s * scale / softcap) - softcap (a
    constant added to every logit of a row changes neither the probabilities nor the split-K merge).  The launcher hands scale /
    softcap, 2 log2(e) scale / softcap and -2 softcap where the plain builds find scale, scale log2(e) and nothing.  Ahead of
    mask_tail(): the cap is bounded, so a key past the end of the sequence that was already at -inf would come back with a finite
    logit."""
    lab_plain, lab_done = label("nocap"), label("capd")
    e("s_cmp_eq_u32 %s, 0" % s(K2))
    e("s_cbranch_scc1 %s" % lab_plain)
    for k in range(16):
        e("v_mul_f32 %s, %s, %s" % (v(sreg + k), s(K1), v(sreg + k)))
    for k in range(16):
        e("v_exp_f32 %s, %s" % (v(sreg + k), v(sreg + k)))
    for k in range(16):
        e("v_add_f32 %s, 1.0, %s" % (v(sreg + k), v(sreg + k)))
    for k in range(16):
        e("v_rcp_f32 %s, %s" % (v(sreg + k), v(sreg + k)))
    for k in range(16):
        e("v_mul_f32 %s, %s, %s" % (v(sreg + k), s(K2), v(sreg + k)))
    e("s_branch %s" % lab_done)
    e("%s:" % lab_plain)
    for k in range(16):
        e("v_mul_f32 %s, %s, %s" % (v(sreg + k), s(SCL), v(sreg + k)))
    e("%s:" % lab_done)


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


def iteration(g_cur, g_next, tag):
    """Tile IT (its P^T operands are in g_cur): the 64 (32) P.V MFMAs, the first 36 of them alternating with the 36
    MFMAs of S = K.Q^T of tile IT+1 (into g_next; independent accumulators, so the MFMA pipe never waits on a
    dependency), the rest carrying the softmax of tile IT+1 in their shadow.  The LDS-DMA loads of tile IT+3 are
    issued from the first part.  Returns the (label, return label) pairs of the out-of-line rescale blocks."""
    e("; ---- iteration %s" % tag)
    resc = []
    if CLKP:
        e("s_memtime s[94:95]")
    # n_valid of tile IT+1
    e("s_add_u32 %s, %s, 1" % (s(S0), s(IT)))
    e("s_lshl_b32 %s, %s, 5" % (s(S0), s(S0)))
    e("s_add_u32 %s, %s, %s" % (s(S0), s(S0), s(KVB)))
    e("s_sub_u32 %s, %s, %s" % (s(NVAL), s(KVE), s(S0)))
    e("s_min_u32 %s, %s, 32" % (s(NVAL), s(NVAL)))
    e("s_mov_b32 %s, 0" % s(VMW))
    e("s_mov_b64 %s, 0" % s(RSC, 2))
    lab_last, lab_nodma, lab_p2, lab_end = label("last"), label("nodma"), label("p2"), label("iend")
    e("s_add_u32 %s, %s, 1" % (s(TMP), s(IT)))
    e("s_cmp_ge_u32 %s, %s" % (s(TMP), s(NT)))
    e("s_cbranch_scc1 %s" % lab_last)
    if MASK:
        mask_loads(TMP)              # mask of tile IT+1: behind the loads of tile IT+2, ahead of those of tile IT+3
    e("s_add_u32 %s, %s, 3" % (s(TMP), s(IT)))
    e("s_cmp_ge_u32 %s, %s" % (s(TMP), s(NT)))
    e("s_cbranch_scc1 %s" % lab_nodma)

    def part1(dma):
        lds.pending = canon_tags()
        qk = qk_slots(g_next, KADDR)
        pv = pv_slots(VADDR, g_cur)
        n1 = min(P1_PV, len(pv))
        lead = min(P1_LEAD, n1)
        merged = list(pv[:lead])
        for n in range(36):
            merged.append(qk[n])
            merged.extend(pv[lead + n * (n1 - lead) // 36:lead + (n + 1) * (n1 - lead) // 36])
        interleave(merged, dma, 2)
        return pv[n1:]

    # ---- part 1 with the DMA of tile IT+3
    e("s_mov_b32 %s, 1" % s(VMW))
    if Q8:
        q8_dma = q8_dma_lines(TMP, RAWN)
        rest_a = part1(q8_dma + q8_dequant_items(RAWC, OFF2, 2))
    elif CVTB:
        cv_dma = dma_tile_lines(TMP, OFF3)
        rest_a = part1(cv_dma + cvt_items(OFF2))
    else:
        rest_a = part1(dma_tile_lines(TMP, OFF3))
    state_a = list(lds.pending)
    e("s_branch %s" % lab_p2)
    # ---- part 1 without it (tiles IT+3.. do not exist)
    e("%s:" % lab_nodma)
    # (Q8_0: empty items in place of the loads, so that the dequantizer's LDS accesses fall into the same slots on both paths)
    rest_b = part1([None] * len(q8_dma) + q8_dequant_items(RAWC, OFF2, 2) if Q8 else [None] * len(cv_dma) + cvt_items(OFF2) if CVTB else [])
    assert lds.pending == state_a and len(rest_a) == len(rest_b), (lds.pending, state_a)
    # ---- part 2: remaining P.V MFMAs of tile IT, softmax of tile IT+1 in their shadow
    e("%s:" % lab_p2)
    if CLKP:
        e("s_memtime s[96:97]")
    head = rest_b[:2]
    for sl in head:
        sl()
    e("s_nop 7")                       # the last QK^T MFMA has written g_next
    if len(head) < 2:
        e("s_nop 7")
    if BIAS:
        bias_block(g_next)             # (ahead of mask_tail: the soft cap maps -inf to a finite value)
    mask_tail(g_next)
    if MASK:
        lab_m0, lab_md = label("m0"), label("md")
        e("s_cmp_eq_u32 %s, 0" % s(VMW))
        e("s_cbranch_scc1 %s" % lab_m0)
        e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
        e("s_branch %s" % lab_md)
        e("%s:" % lab_m0)
        e("s_waitcnt vmcnt(0)")
        e("%s:" % lab_md)
    body = rest_b[2:]
    tail = body[-2:] if len(body) >= 2 else []
    interleave(body[:len(body) - len(tail)], softmax_lines(g_next), 4)

    def sync():
        # the DMA of tile IT+2 has landed (the one of tile IT+3, issued in this iteration, may still be in flight:
        # loads complete in order, so vmcnt(DMA_PER_TILE) is enough); every wave is done with tile IT's buffer
        lab_w0, lab_wd = label("w0"), label("wd")
        if CLK and not CLKP:
            e("s_memtime s[94:95]")
            e("s_waitcnt lgkmcnt(0)")
        if Q8 or CVTB:
            e("s_waitcnt vmcnt(0)")     # the raw tile loaded during this iteration is dequantized / converted in the next one
        else:
            e("s_cmp_eq_u32 %s, 0" % s(VMW))
            e("s_cbranch_scc1 %s" % lab_w0)
            e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
            e("s_branch %s" % lab_wd)
            e("%s:" % lab_w0)
            e("s_waitcnt vmcnt(0)")
            e("%s:" % lab_wd)
        if CLK and not CLKP:
            e("s_memtime s[96:97]")
            e("s_waitcnt lgkmcnt(0)")
            e("s_sub_u32 s94, s96, s94")
            e("s_add_u32 s92, s92, s94")       # cycles spent waiting for the tile loads
        e("s_barrier")
        if CLK and not CLKP:
            e("s_memtime s[98:99]")
            e("s_waitcnt lgkmcnt(0)")
            e("s_sub_u32 s98, s98, s96")
            e("s_add_u32 s93, s93, s98")       # cycles spent in the barrier
    tile_handover(OFF2, OFF1, tail, sync)
    if CLKP:
        e("s_memtime s[98:99]")
        e("s_waitcnt lgkmcnt(0)")
        e("s_sub_u32 s98, s98, s96")
        e("s_sub_u32 s96, s96, s94")
        e("s_add_u32 s92, s92, s96")       # part 1
        e("s_add_u32 s93, s93, s98")       # part 2
    e("s_branch %s" % lab_end)
    # ---- last tile: P.V only
    e("%s:" % lab_last)
    lds.pending = canon_tags()
    for sl in pv_slots(VADDR, g_cur):
        sl()
    lds.drain()
    e("%s:" % lab_end)
    # ---- the accumulators take the new row maxima now that no MFMA of tile IT is left to issue
    lab_resc, lab_back = label("resc"), label("back")
    e("s_cmp_lg_u64 %s, 0" % s(RSC, 2))
    e("s_cbranch_scc1 %s" % lab_resc)
    e("%s:" % lab_back)
    resc.append((lab_resc, lab_back))
    e("s_mov_b32 %s, %s" % (s(TMP), s(OFF0)))
    e("s_mov_b32 %s, %s" % (s(OFF0), s(OFF1)))
    e("s_mov_b32 %s, %s" % (s(OFF1), s(OFF2)))
    if Q8:
        e("s_mov_b32 %s, %s" % (s(OFF2), s(TMP)))
        e("s_mov_b32 %s, %s" % (s(TMP), s(RAWC)))
        e("s_mov_b32 %s, %s" % (s(RAWC), s(RAWN)))
        e("s_mov_b32 %s, %s" % (s(RAWN), s(TMP)))
    else:
        e("s_mov_b32 %s, %s" % (s(OFF2), s(OFF3)))
        e("s_mov_b32 %s, %s" % (s(OFF3), s(TMP)))
    e("s_add_u32 %s, %s, 1" % (s(IT), s(IT)))
    return resc


LAB_EXIT = "Lexit_%="


def main():
    # ------------------------------------------------------------------ entry: inputs -> fixed registers
    stamp(0)
    if CLK:
        e("s_mov_b32 s92, 0")
        e("s_mov_b32 s93, 0")
    # Nothing of the compiled code ahead of the program may still be in flight: a scalar load whose value that code no longer needs
    # (hoisted above a branch, say) may have been given a register of this program's, and would land on top of what the program
    # has put there since -- the hardware keeps no order between a load's return and later writes to its destination.
    e("s_waitcnt vmcnt(0) lgkmcnt(0)")
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
    e("s_mov_b32 %s, %%[pg0]" % s(PGZ))
    e("s_mov_b64 %s, %%[qp]" % s(QP, 2))
    e("v_mov_b32 %s, %%[tid]" % v(X0))
    e("s_mov_b32 %s, 0x%08x" % (s(THR), 0x41000000))  # TAU = 8.0f
    if not SPLIT:
        e("s_mov_b32 %s, 0x3c003c00" % s(ONES))
    if MASK:
        e("s_mov_b32 %s, %%[scl]" % s(SCL))
        e("s_mov_b32 %s, 0x3fb8aa3b" % s(L2E))
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
    if not RELOAD_PTRS:
        e("v_mov_b32 %s, %s" % (v(OPTR), v(T[2])))
        e("v_mov_b32 %s, %s" % (v(OPTR + 1), v(T[3])))
        e("v_mov_b32 %s, %s" % (v(MLPTR), v(T[4])))
        e("v_mov_b32 %s, %s" % (v(MLPTR + 1), v(T[5])))
    if MASK:
        e("v_mov_b32 %s, %s" % (v(MOFF), v(T[0])))
    if BIAS:
        # the last 8 bytes of the record: the slope of this thread's row's head, and -2 softcap
        e("v_mov_b32 %s, %s" % (v(SLOPE), v(T[6])))
        e("v_readfirstlane_b32 %s, %s" % (s(RSC + 1), v(T[7])))
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
    # FLG bit 4: V is columns 64 .. 575 of the rows instead of 0 .. 511 (second pass of a 576-wide V)
    e("s_bitcmp1_b32 %s, 4" % s(FLG))
    e("s_cselect_b32 %s, 128, 0" % s(S0))
    e("v_add_u32 %s, %s, %s" % (v(VADDR_LANE), s(S0), v(VADDR_LANE)))
    if CVTB:
        # in-place conversion: lane = (row 8 wave + lane / 8, column chunk lane % 8 of every group of eight chunks)
        e("v_lshrrev_b32 %s, 3, %s" % (v(CVL), v(LANE)))
        e("s_lshl_b32 %s, %s, 3" % (s(S0), s(WAVE)))
        e("v_add_u32 %s, %s, %s" % (v(CVL), s(S0), v(CVL)))
        e("v_and_b32 %s, 7, %s" % (v(CT0), v(LANE)))
        e("v_lshlrev_b32 %s, 4, %s" % (v(CT0), v(CT0)))
        e("v_mad_u32_u24 %s, %s, %s, %s" % (v(CVL), v(CVL), s(SPITCH), v(CT0)))
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
    e("s_mov_b64 exec, %s" % s(EXS, 2))
    e("%s:" % lab_nobt)
    # ------------------------------------------------------------------ Q operands: 36 coalesced 16-byte loads per lane from
    # the packed image, in flight together with the page ids
    nq = 36
    e("v_lshlrev_b32 %s, 4, %s" % (v(X0), v(LANE)))
    e("s_mul_i32 %s, %s, %d" % (s(S0), s(WAVE), 36 * 1024))
    e("s_add_u32 %s, %s, %s" % (s(QP), s(QP), s(S0)))
    e("s_addc_u32 %s, %s, 0" % (s(QP + 1), s(QP + 1)))
    # a wave without a valid row (FLG bit 5) never uses Q: it skips the loads (its part of the image is not written either)
    lab_noq = label("noq")
    if nq and not Q8:
        e("s_bitcmp1_b32 %s, 5" % s(FLG))
        e("s_cbranch_scc1 %s" % lab_noq)
    for ks in range(nq):
        if ks and ks % 4 == 0:
            e("s_add_u32 %s, %s, 4096" % (s(QP), s(QP)))
            e("s_addc_u32 %s, %s, 0" % (s(QP + 1), s(QP + 1)))
        e("global_load_dwordx4 %s, %s, %s offset:%d" % (v(Q0 + 4 * ks, 4), v(X0), s(QP, 2), (ks % 4) * 1024))
    e("%s:" % lab_noq)
    n_early = nq
    if MASK:
        # mask rows start at key kv_begin of this split; QP's registers are free now
        e("s_mov_b64 %s, %%[msk]" % s(MSK, 2))
        e("s_lshl_b32 %s, %s, 1" % (s(S0), s(KVB)))
        e("s_add_u32 %s, %s, %s" % (s(MSK), s(MSK), s(S0)))
        e("s_addc_u32 %s, %s, 0" % (s(MSK + 1), s(MSK + 1)))
        e("s_mov_b32 %s, 0" % s(TMP))
        mask_loads(TMP)
        n_early += 4
    # ------------------------------------------------------------------ state
    e("v_mov_b32 %s, 0xff800000" % v(MRUN))
    e("v_mov_b32 %s, 0" % v(LRUN))
    e("s_mov_b32 %s, 0" % s(OFF0))
    e("s_mov_b32 %s, %d" % (s(OFF1), TILE_BYTES))
    e("s_mov_b32 %s, %d" % (s(OFF2), 2 * TILE_BYTES))
    e("s_mov_b32 %s, %d" % (s(OFF3), 3 * TILE_BYTES))
    e("s_mov_b32 %s, 0" % s(IT))
    if not Q8:
        for ln in dma_table_lines():
            e(ln)
    # The first tiles can be requested before the page ids are there when the split starts on a page boundary (always,
    # except for masked key ranges): they lie in the first page, whose id came as a scalar.  Otherwise wait for the ids
    # (loads return in order: only the Q and mask loads may still be in flight).
    lab_al = label("aligned")
    e("s_and_b32 %s, %s, 127" % (s(S0), s(KVB)))
    e("s_cmp_eq_u32 %s, 0" % s(S0))
    e("s_cbranch_scc1 %s" % lab_al)
    if nq and not Q8:
        lab_wq, lab_wqd = label("wq"), label("wqd")
        e("s_bitcmp1_b32 %s, 5" % s(FLG))
        e("s_cbranch_scc0 %s" % lab_wq)
        e("s_waitcnt vmcnt(%d)" % (n_early - nq))     # no Q loads behind the page ids
        e("s_branch %s" % lab_wqd)
        e("%s:" % lab_wq)
        e("s_waitcnt vmcnt(%d)" % n_early)
        e("%s:" % lab_wqd)
    else:
        e("s_waitcnt vmcnt(%d)" % n_early)
    e("v_max_i32 %s, 0, %s" % (v(PAGES), v(PAGES)))
    e("v_min_i32 %s, %s, %s" % (v(PAGES), s(NPP), v(PAGES)))
    e("%s:" % lab_al)

    def acc_init():
        for i in range(256):
            e("v_accvgpr_write_b32 %s, 0" % a(i))

    def page_clamp():
        # (again for the path that already waited: harmless) page ids outside the pool can only come from table entries
        # that are never used; clamped so that no address leaves the pool
        e("v_max_i32 %s, 0, %s" % (v(PAGES), v(PAGES)))
        e("v_min_i32 %s, %s, %s" % (v(PAGES), s(NPP), v(PAGES)))
        if BIAS:
            e("s_mov_b32 %s, %s" % (s(K2), s(RSC + 1)))
    stamp(6)
    if Q8:
        # ------------------------------------------------------------------ Q8_0: per-lane offsets of the dequantizer
        e("v_lshrrev_b32 %s, 2, %s" % (v(X0), v(LANE)))
        e("s_and_b32 %s, %s, 1" % (s(S0), s(WAVE)))
        e("s_lshl_b32 %s, %s, 4" % (s(S0), s(S0)))
        e("v_add_u32 %s, %s, %s" % (v(X0), s(S0), v(X0)))                  # row = 16*(wave&1) + lane/4
        e("v_and_b32 %s, 3, %s" % (v(X1), v(LANE)))                        # quarter of the block
        e("s_lshr_b32 %s, %s, 1" % (s(S1), s(WAVE)))                       # 0: even blocks, 1: odd blocks
        e("v_lshlrev_b32 %s, 3, %s" % (v(X2), v(X1)))
        e("s_mov_b32 %s, %d" % (s(S2), Q8_ROW))
        e("v_mad_u32_u24 %s, %s, %s, %s" % (v(RAWB), v(X0), s(S2), v(X2)))  # row*612 + 8q: window of (even block 0, quarter q)
        e("s_mul_i32 %s, %s, 36" % (s(S2), s(S1)))
        e("v_add_u32 %s, %s, %s" % (v(RAWB), s(S2), v(RAWB)))              # odd blocks: + 34 + 2: their values are 4-byte aligned
        e("v_lshlrev_b32 %s, 4, %s" % (v(X2), v(X1)))
        e("v_mad_u32_u24 %s, %s, %s, %s" % (v(DSTB), v(X0), s(SPITCH), v(X2)))
        e("s_lshl_b32 %s, %s, 6" % (s(S2), s(S1)))
        e("v_add_u32 %s, %s, %s" % (v(DSTB), s(S2), v(DSTB)))              # odd blocks: + 32 columns
        e("s_lshl_b32 %s, %s, 1" % (s(SHM2), s(S1)))                       # 0 / 2
        e("s_sub_u32 %s, 2, %s" % (s(SH), s(SHM2)))                        # 2 / 0
        e("s_mov_b32 %s, 0x01000100" % s(PSEL))
        e("s_mov_b32 %s, %d" % (s(RAWC), RAW0))
        e("s_mov_b32 %s, %d" % (s(RAWN), RAW1))
        # ------------------------------------------------------------------ raw tiles 0 and 1 -> LDS, tile 0 -> f16
        lab_w0, lab_wd = label("pw0"), label("pwd")
        e("s_mov_b32 %s, 0" % s(TMP))
        for ln in q8_dma_lines(TMP, RAWC, True):
            e(ln)
        acc_init()
        e("s_cmp_lt_u32 %s, 2" % s(NT))
        e("s_cbranch_scc1 %s" % lab_w0)
        e("s_mov_b32 %s, 1" % s(TMP))
        for ln in q8_dma_lines(TMP, RAWN, True):
            e(ln)
        e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
        e("s_branch %s" % lab_wd)
        e("%s:" % lab_w0)
        e("s_waitcnt vmcnt(0)")
        e("%s:" % lab_wd)
        page_clamp()
        e("s_barrier")
        for it_ in q8_dequant_items(RAWC, OFF0, 0):
            emit_item(it_)
        lds.need(("w", 8))
        e("s_waitcnt vmcnt(0)")
        e("s_barrier")                      # f16 tile 0 complete, raw tile 1 landed, raw buffer 0 free
        lab_n2 = label("pn2")
        e("s_cmp_lt_u32 %s, 3" % s(NT))
        e("s_cbranch_scc1 %s" % lab_n2)
        e("s_mov_b32 %s, 2" % s(TMP))
        for ln in q8_dma_lines(TMP, RAWC, True):
            e(ln)
        e("%s:" % lab_n2)
        for it_ in q8_dequant_items(RAWN, OFF1, 1):
            emit_item(it_)
        # ---------------------------------------------------------------- waves without a valid row (FLG bit 5): they keep their share
        # of the loads and of the dequantisation and meet the others at every barrier, and issue no MFMA, no fragment read
        # and no softmax
        lab_busy, lab_iloop, lab_inodma, lab_iend = (label(x) for x in ("busy", "iloop", "inodma", "iend"))
        busy_pending = list(lds.pending)
        e("s_bitcmp1_b32 %s, 5" % s(FLG))
        e("s_cbranch_scc0 %s" % lab_busy)
        lds.drain()                                     # this wave's share of f16 tile 1 is written
        e("s_waitcnt vmcnt(0)")                         # raw tile 2 has landed
        e("s_barrier")
        e("%s:" % lab_iloop)
        e("s_add_u32 %s, %s, 1" % (s(TMP), s(IT)))
        e("s_cmp_ge_u32 %s, %s" % (s(TMP), s(NT)))
        e("s_cbranch_scc1 %s" % lab_iend)               # the last tile has no successor to prepare
        e("s_add_u32 %s, %s, 3" % (s(TMP), s(IT)))
        e("s_cmp_ge_u32 %s, %s" % (s(TMP), s(NT)))
        e("s_cbranch_scc1 %s" % lab_inodma)
        for ln in q8_dma_lines(TMP, RAWN):
            e(ln)
        e("%s:" % lab_inodma)
        for it_ in q8_dequant_items(RAWC, OFF2, 2):
            emit_item(it_)
        lds.drain()
        e("s_waitcnt vmcnt(0)")
        e("s_barrier")
        e("s_mov_b32 %s, %s" % (s(TMP), s(OFF0)))
        e("s_mov_b32 %s, %s" % (s(OFF0), s(OFF1)))
        e("s_mov_b32 %s, %s" % (s(OFF1), s(OFF2)))
        e("s_mov_b32 %s, %s" % (s(OFF2), s(TMP)))
        e("s_mov_b32 %s, %s" % (s(TMP), s(RAWC)))
        e("s_mov_b32 %s, %s" % (s(RAWC), s(RAWN)))
        e("s_mov_b32 %s, %s" % (s(RAWN), s(TMP)))
        e("s_add_u32 %s, %s, 1" % (s(IT), s(IT)))
        e("s_branch %s" % lab_iloop)
        e("%s:" % lab_iend)
        e("s_waitcnt vmcnt(0)")
        e("s_branch %s" % LAB_EXIT)
        e("%s:" % lab_busy)
        lds.pending = busy_pending
    else:
        # ------------------------------------------------------------------ tiles 0, 1, 2 -> LDS; go on as soon as Q and tile 0 are there
        lab_w0, lab_w1, lab_wd = label("pw0"), label("pw1"), label("pwd")
        e("s_mov_b32 %s, 0" % s(TMP))
        for ln in dma_tile_lines(TMP, OFF0, True):
            e(ln)
        acc_init()
        e("s_cmp_lt_u32 %s, 2" % s(NT))
        e("s_cbranch_scc1 %s" % lab_w0)
        e("s_mov_b32 %s, 1" % s(TMP))
        for ln in dma_tile_lines(TMP, OFF1, True):
            e(ln)
        e("s_cmp_lt_u32 %s, 3" % s(NT))
        e("s_cbranch_scc1 %s" % lab_w1)
        e("s_mov_b32 %s, 2" % s(TMP))
        for ln in dma_tile_lines(TMP, OFF2, True):
            e(ln)
        e("s_waitcnt vmcnt(%d)" % (2 * DMA_PER_TILE))
        e("s_branch %s" % lab_wd)
        e("%s:" % lab_w1)
        e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
        e("s_branch %s" % lab_wd)
        e("%s:" % lab_w0)
        e("s_waitcnt vmcnt(0)")
        e("%s:" % lab_wd)
        page_clamp()
        if CVTB:
            # this wave's rows of tile 0 -> f16; once every wave has done that, the same for tile 1 (its loads may still be in
            # flight with those of tile 2 behind them); tile 2 is converted by iteration 0
            for it_ in cvt_items(OFF0):
                emit_item(it_)
            lds.drain()
        e("s_barrier")
        if CVTB:
            lab_c1, lab_c1d = label("c1"), label("c1d")
            e("s_cmp_lt_u32 %s, 3" % s(NT))
            e("s_cbranch_scc1 %s" % lab_c1)
            e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
            e("s_branch %s" % lab_c1d)
            e("%s:" % lab_c1)
            e("s_waitcnt vmcnt(0)")
            e("%s:" % lab_c1d)
            for it_ in cvt_items(OFF1):
                emit_item(it_)
            # waves without a valid row: their share of the loads and of the conversion, every barrier, nothing else
            lab_busy, lab_iloop, lab_inodma, lab_iend = (label(x) for x in ("busy", "iloop", "inodma", "iend"))
            busy_pending = list(lds.pending)
            e("s_bitcmp1_b32 %s, 5" % s(FLG))
            e("s_cbranch_scc0 %s" % lab_busy)
            lds.drain()
            e("s_waitcnt vmcnt(0)")
            e("s_barrier")
            e("%s:" % lab_iloop)
            e("s_add_u32 %s, %s, 1" % (s(TMP), s(IT)))
            e("s_cmp_ge_u32 %s, %s" % (s(TMP), s(NT)))
            e("s_cbranch_scc1 %s" % lab_iend)
            e("s_add_u32 %s, %s, 3" % (s(TMP), s(IT)))
            e("s_cmp_ge_u32 %s, %s" % (s(TMP), s(NT)))
            e("s_cbranch_scc1 %s" % lab_inodma)
            for ln in dma_tile_lines(TMP, OFF3):
                e(ln)
            e("%s:" % lab_inodma)
            for it_ in cvt_items(OFF2):
                emit_item(it_)
            lds.drain()
            e("s_waitcnt vmcnt(0)")
            e("s_barrier")
            e("s_mov_b32 %s, %s" % (s(TMP), s(OFF0)))
            e("s_mov_b32 %s, %s" % (s(OFF0), s(OFF1)))
            e("s_mov_b32 %s, %s" % (s(OFF1), s(OFF2)))
            e("s_mov_b32 %s, %s" % (s(OFF2), s(OFF3)))
            e("s_mov_b32 %s, %s" % (s(OFF3), s(TMP)))
            e("s_add_u32 %s, %s, 1" % (s(IT), s(IT)))
            e("s_branch %s" % lab_iloop)
            e("%s:" % lab_iend)
            e("s_waitcnt vmcnt(0)")
            e("s_branch %s" % LAB_EXIT)
            e("%s:" % lab_busy)
            lds.pending = busy_pending
        if not CVTB:
            # ---------------------------------------------------------------- waves without a valid row (FLG bit 5; fewer than 97 rows in
            # the block, e.g. a 16- or 32-head model's decode step): they keep moving their eight rows of every tile and meet the
            # others at every barrier, and issue no MFMA, no fragment read and no softmax: a quarter of the matrix-core power for a
            # 32-head model, which the chip-wide clock gives back to the wave that computes
            lab_busy, lab_iloop, lab_inodma, lab_iw0, lab_iwd, lab_iend = (label(x) for x in ("busy", "iloop", "inodma", "iw0", "iwd", "iend"))
            lab_it1, lab_it1d = label("it1"), label("it1d")
            e("s_bitcmp1_b32 %s, 5" % s(FLG))
            e("s_cbranch_scc0 %s" % lab_busy)
            e("s_cmp_lt_u32 %s, 3" % s(NT))                 # as the first hand-over: tile 1 has landed
            e("s_cbranch_scc1 %s" % lab_it1)
            e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
            e("s_branch %s" % lab_it1d)
            e("%s:" % lab_it1)
            e("s_waitcnt vmcnt(0)")
            e("%s:" % lab_it1d)
            e("s_barrier")
            e("%s:" % lab_iloop)
            e("s_add_u32 %s, %s, 1" % (s(TMP), s(IT)))
            e("s_cmp_ge_u32 %s, %s" % (s(TMP), s(NT)))
            e("s_cbranch_scc1 %s" % lab_iend)               # the last tile has no successor to wait for
            e("s_mov_b32 %s, 0" % s(VMW))
            e("s_add_u32 %s, %s, 3" % (s(TMP), s(IT)))
            e("s_cmp_ge_u32 %s, %s" % (s(TMP), s(NT)))
            e("s_cbranch_scc1 %s" % lab_inodma)
            e("s_mov_b32 %s, 1" % s(VMW))
            for ln in dma_tile_lines(TMP, OFF3):
                e(ln)
            e("%s:" % lab_inodma)
            e("s_cmp_eq_u32 %s, 0" % s(VMW))
            e("s_cbranch_scc1 %s" % lab_iw0)
            e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
            e("s_branch %s" % lab_iwd)
            e("%s:" % lab_iw0)
            e("s_waitcnt vmcnt(0)")
            e("%s:" % lab_iwd)
            e("s_barrier")
            e("s_mov_b32 %s, %s" % (s(TMP), s(OFF0)))
            e("s_mov_b32 %s, %s" % (s(OFF0), s(OFF1)))
            e("s_mov_b32 %s, %s" % (s(OFF1), s(OFF2)))
            e("s_mov_b32 %s, %s" % (s(OFF2), s(OFF3)))
            e("s_mov_b32 %s, %s" % (s(OFF3), s(TMP)))
            e("s_add_u32 %s, %s, 1" % (s(IT), s(IT)))
            e("s_branch %s" % lab_iloop)
            e("%s:" % lab_iend)
            e("s_waitcnt vmcnt(0)")
            e("s_branch %s" % LAB_EXIT)
            e("%s:" % lab_busy)
    stamp(1)
    e("v_add_u32 %s, %s, %s" % (v(KADDR), s(OFF0), v(KADDR_LANE)))
    k_warm(KADDR)
    for slot in qk_slots(SA, KADDR):
        slot()
    # softmax of tile 0 (nothing to overlap it with); the accumulators are still zero, so no rescale
    e("s_sub_u32 %s, %s, %s" % (s(NVAL), s(KVE), s(KVB)))
    e("s_min_u32 %s, %s, 32" % (s(NVAL), s(NVAL)))
    e("s_nop 7")
    e("s_nop 7")
    if BIAS:
        bias_block(SA)
    mask_tail(SA)
    for ln in softmax_lines(SA):
        e(ln)
    # tile 1 has landed (tile 2 may still be in flight); first fragment reads of iteration 0
    def sync0():
        lab_t1, lab_t1d = label("t1"), label("t1d")
        if Q8 or CVTB:
            e("s_waitcnt vmcnt(0)")     # f16 tile 1 written (the hand-over waited for this wave's writes), raw tile 2 landed
            e("s_barrier")
            return
        e("s_cmp_lt_u32 %s, 3" % s(NT))
        e("s_cbranch_scc1 %s" % lab_t1)
        e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
        e("s_branch %s" % lab_t1d)
        e("%s:" % lab_t1)
        e("s_waitcnt vmcnt(0)")
        e("%s:" % lab_t1d)
        e("s_barrier")
    assert Q8 or CVTB or not lds.pending
    tile_handover(OFF1, OFF0, [], sync0)
    # ------------------------------------------------------------------ main loop (two copies: the register groups swap roles)
    lab_loop, lab_end = label("loop"), label("end")
    stamp(2)
    e("%s:" % lab_loop)
    r1 = iteration(SA, SB, "A")
    e("s_cmp_ge_u32 %s, %s" % (s(IT), s(NT)))
    e("s_cbranch_scc1 %s" % lab_end)
    r2 = iteration(SB, SA, "B")
    e("s_cmp_lt_u32 %s, %s" % (s(IT), s(NT)))
    e("s_cbranch_scc1 %s" % lab_loop)
    e("s_branch %s" % lab_end)
    # out-of-line rescale blocks
    for pairs in (r1, r2):
        for resc, back in pairs:
            e("%s:" % resc)
            rescale_block(back)
    e("%s:" % lab_end)
    stamp(3)
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
    if RELOAD_PTRS:
        # bytes 8..23 of this thread's hand-off record: the output pointer and the (m, l) pointer
        e("s_lshl_b32 %s, %s, 11" % (s(S0), s(WAVE)))
        e("v_lshlrev_b32 %s, 5, %s" % (v(X0), v(LANE)))
        e("v_add_u32 %s, %s, %s" % (v(X0), s(S0), v(X0)))
        e("v_add_u32 %s, %d, %s" % (v(X0), HOFF, v(X0)))
        e("ds_read_b64 %s, %s offset:8" % (v(OPTR, 2), v(X0)))
        e("ds_read_b64 %s, %s offset:16" % (v(MLPTR, 2), v(X0)))
        e("s_waitcnt lgkmcnt(0)")
    # rows past n_rows store nothing
    e("v_cmp_ne_u64 vcc, 0, %s" % v(OPTR, 2))
    e("s_mov_b64 %s, exec" % s(EXS, 2))
    e("s_nop 1")
    e("s_and_b64 exec, exec, vcc")
    # O^T block i, element 4j+c is column 32 i + 8 j + 4 g + c.
    # Final output (FLG bit 0): row-major rows of dst; the out pointer already includes the 4*g float offset.
    # Split-K partial: f16, layout [column/8][row][8] so that the 64 lanes of a wave write 512 contiguous bytes;
    # the out pointer already includes row*16 + g*8 bytes and every (i, j) step advances it by n_rows*16 bytes.
    lab_pstore, lab_sdone = label("pstore"), label("sdone")
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
    # partial: O / l of this split as f16, layout [column/8][row][8 halves]; T[2] holds 1/l here as well
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
            e("global_store_dwordx2 %s, %s, off%s" % (v(OPTR, 2), v(r, 2), PARTIAL_SCOPE))
            e("v_add_co_u32 %s, vcc, %s, %s" % (v(OPTR), s(OSTR), v(OPTR)))
            e("s_nop 1")
            e("v_addc_co_u32 %s, vcc, 0, %s, vcc" % (v(OPTR + 1), v(OPTR + 1)))
    e("%s:" % lab_sdone)
    stamp(4)
    # (m, l) of this split, written by the g == 0 lane of each row when a pointer was handed over
    e("v_cmp_ne_u64 vcc, 0, %s" % v(MLPTR, 2))
    e("s_nop 1")
    e("s_and_b64 exec, exec, vcc")
    e("v_mov_b32 %s, %s" % (v(T[0]), v(MRUN)))
    e("v_mov_b32 %s, %s" % (v(T[1]), v(LRUN)))
    e("s_nop 0")
    e("global_store_dwordx2 %s, %s, off%s" % (v(MLPTR, 2), v(T[0], 2), PARTIAL_SCOPE))
    e("s_mov_b64 exec, %s" % s(EXS, 2))
    e("s_waitcnt vmcnt(0)")
    stamp(5)
    if CLK:
        # every wave leaves its stamps and accumulators in the hand-off area: 64 bytes per wave
        e("s_lshl_b32 %s, %s, 6" % (s(S0), s(WAVE)))
        e("s_add_u32 %s, %s, %d" % (s(S0), s(S0), HOFF))
        e("v_mov_b32 %s, %s" % (v(X0), s(S0)))
        for k, reg in enumerate([80, 82, 84, 86, 88, 90, 92, 93, 100]):
            e("v_mov_b32 %s, %s" % (v(X1), s(reg)))
            e("ds_write_b32 %s, %s offset:%d" % (v(X0), v(X1), 4 * k))
        e("s_waitcnt lgkmcnt(0)")
        e("s_barrier")

    e("%s:" % LAB_EXIT)

    print("// generated by gen_decode_asm.py%s%s%s -- do not edit" % (" --q8" if Q8 else " --f16" if "--f16" in sys.argv else "", " --mask" if MASK else "", " --bias" if BIAS else ""))
    for ln in out:
        print('"%s\\n\\t"' % ln)
    # and nothing of the program is in flight when the compiled code goes on (the mirror image of the wait at the top: an LDS read
    # or a load requested ahead for a tile that never came would land in a register that code has taken since)
    print('"s_waitcnt vmcnt(0) lgkmcnt(0)\\n\\t"')


main()
