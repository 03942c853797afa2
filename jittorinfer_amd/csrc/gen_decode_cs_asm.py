#!/usr/bin/env python3
"""Generates mla_decode_cs_*.inc: the gfx950 instruction streams of the pipelined MLA decode kernel in its
"column-split" form (one inline-asm block each inside mla_decode_kernel.hip).
Usage: python gen_decode_cs_asm.py [--ks | --half] [--f16] [--mask [--bias | --stream]] > mla_decode_[cs|ks|csh]_[bf16|f16][_mask[_nt]|_bias].inc

Work of one wave w of a 4-wave workgroup (128 attention rows x one KV split), per 32-token tile `it`:
    part 1   S = K[it+1].Q^T for the wave's own 32 rows (36 MFMA, Q resident in 144 VGPRs, K fragments from LDS);
             in their shadow: the eight V^T fragments of tile `it` for the wave's own 128 output columns (transposing LDS
             reads), bf16 fragments converted to f16 in registers, and the LDS-DMA loads of tile it+3
    part 2   O^T[128 columns x 128 rows] += V[it]^T.P[it]^T (32 MFMA; the P^T fragments of all four waves come out of LDS),
             with softmax(S[it+1]) -> P[it+1] in their shadow
    end      barrier, P[it+1] -> LDS, barrier (tile it+2 has landed for every wave; P[it+1] is visible)
A wave thus owns 128 columns of all 128 rows of O (16 accumulator blocks of 32 x 32 in 256 AGPRs): a V^T fragment feeds
four MFMAs, so the transposing reads (the slow kind) drop to a quarter, and with 8 fragments per wave and tile the bf16 -> f16
conversion fits in registers: no pass over the tile in LDS, no tile buffer held for it, two tiles of loads in flight.
bf16 K is multiplied as bf16 (exact products either way); P and V meet as f16, which keeps 11 bits of P.
--mask: an additive f16 mask row per query token (ggml-cpu.c:12041-12057: s * scale + mask): the 16 mask values of a lane's 16
tokens of tile it+1 are loaded at the top of iteration `it` (four 8-byte loads) and enter the scores ahead of the softmax; the
eight registers they live in come out of the K and P^T fragment rings.
--mask --bias: the remaining terms of ggml-cpu.c:12041-12057, u = softcap * tanh(s * scale / softcap) + slope(head) * mask.  The slope
(ggml-cpu.c:11985-11989, :12006-12008; 1 without ALiBi) is a per-lane input that stays in a register the program never writes; the
soft cap runs as tanh(x) = 1 - 2 / (1 + 2^(2 x log2 e)) on v_exp_f32 / v_rcp_f32, and since a constant added to every logit of a
row changes neither the probabilities nor the split-K merge, the program keeps -2 softcap / (1 + e^(2x)) and drops the "+ softcap".
--half: 33 to 64 rows, i.e. two row blocks.  Waves 0 and 1 run the program above with two row blocks of P.V (16 MFMA); the waves
without rows (FLG bit 5) leave it behind the barrier that completes tile 0 for a loop of their own (iteration_rowless): their share
of the tile copies, the V^T fragments, their 128 columns of P.V, the same two barriers per tile -- no Q, no K.Q^T, no softmax.
--ks: see ks_main.
"""
import sys

ARGS = sys.argv[1:]
F16KV = "--f16" in ARGS                      # f16 KV rows: f16 MFMA for K.Q^T, V^T fragments used as they are
CLK = "--clk" in ARGS                        # timing builds: s_memtime stamps left in LDS at the end
MASK = "--mask" in ARGS                      # additive f16 mask rows (one per query token)
KS = "--ks" in ARGS                          # at most 32 rows: the four waves split the 576 columns of K.Q^T (see ks_main)
BIAS = "--bias" in ARGS                      # mask builds: ALiBi slope per head on the mask, tanh soft cap on the logits
STREAM = "--stream" in ARGS                  # mask builds: the tile copies carry the non-temporal hint (see NT_HINT)
HALF = "--half" in ARGS                      # 33 .. 64 rows: two row blocks; the waves without rows still copy tiles and take their columns of P.V
assert not (MASK and CLK) and (MASK or not BIAS) and (MASK or not STREAM) and not (BIAS and STREAM)
assert not (HALF and (MASK or KS or CLK))
NHB = 2 if HALF else 4                       # row blocks of 32 rows
NFRAG = 2 * NHB                              # P^T fragments of a tile
MF_QK = "v_mfma_f32_32x32x16_f16" if F16KV else "v_mfma_f32_32x32x16_bf16"
MF_PV = "v_mfma_f32_32x32x16_f16"


CONV_P1 = 8 if HALF else 5                   # V^T fragments converted in part 1; the rest in the first half of part 2

PITCH = 1168
TILE_BYTES = 32 * PITCH
NBUF = 4
PBUF = NBUF * TILE_BYTES                     # P^T exchange: [row block hb][k-step kk][lane][16 bytes] = 8 KB
HOFF = PBUF                                  # hand-off records of the C++ prologue (32 bytes per thread): read before P is first written
AOFF = PBUF + 8192                           # rescale factors: [lane][hb] f32 (64 x 16 bytes; lanes 32.. hold copies)
FOFF = AOFF + 1024                           # one word per wave: non-zero when its rows' running maxima moved
CPR = 73                                     # 16-byte chunks per padded row
WAVE_CHUNKS = 8 * CPR                        # each wave moves rows 8w .. 8w+7 of a tile
DMA_PER_TILE = 10
# Tile copies of the unmasked programs carry the non-temporal hint: a decode step reads every key once, and cells streamed through
# the L2s without the hint push out what is read again -- the operand image the workgroups of a sequence share, the partials the
# combine pass is about to read (config 3: step 92.4 -> 88.8 us; 128 sequences x 8192 keys, 16 heads: kernel 218 -> 199 us = 6.1 TB/s).
# The masked programs also run prompt chunks, whose row blocks read the same cells one after the other (config 4 with the hint:
# 174.8 -> 179.5 us): they come in two builds, and the launcher takes the one with the hint (--stream) when the cache is far larger
# than the L2s can hold -- the reference's decode batch, whose mask gives every token its own cells of one big cache (config 3 in
# that form: step 112.2 -> 109.1 us).
NT_HINT = " nt" if STREAM or not MASK else ""
# K fragment ring: five slots of its own, the sixth in T[4:7] (free while K.Q^T runs); mask builds give the last slot of each
# ring to the mask values
KRING, PRING = (5, 3) if MASK else (6, 4)
# The f16 partial rows and the (m, l) pairs are read by another kernel, on other XCDs: stored at device scope they go to memory as
# they are written, instead of waiting in this XCD's L2 for the write-back at the end of the kernel (config 3: step -1 %, a layer's
# decode step -1 us).  Not the f32 rows: final output written through loses the L2's merging of a row's pieces (a prompt chunk of
# 512 tokens from an empty cache: 97 -> 142 us with the same bit on those stores).
PARTIAL_SCOPE = " sc1"

# ---- VGPR map (v252..v255 are left to the compiler: the clobber list of the asm block ends at v251)
Q0 = 0
S = 144                 # scores of one tile; its P^T operands (f16 pairs) are built in place
VF = 160                # the eight V^T fragments of a tile, fragment f = 4 kk + cb in VF + 4 f
PR = 192                # ring of P^T fragments, fragment f = 4 kk + hb in slot f % 4
KF = 208                # ring of K fragments
T = list(range(228, 236))
KADDR_LANE, VADDR_LANE, MRUN, LRUN, KADDR, VADDR, PAGES = 236, 237, 238, 239, 240, 241, 242
PT = [243, 244, 245, 246, 247]   # per-lane byte offsets of the 10 LDS-DMA slots, two 16-bit values per register
PADDR = 248             # PBUF + lane * 16
X0 = 249
DT = [250, 251]         # address temporaries of the LDS-DMA slots; conversion temporaries in part 2
X1, X2 = 250, 251       # prologue / epilogue temporaries
NEGM, ALPHA, TMAX = T[5], T[6], T[7]   # live inside the softmax only
MKR = [204, 205, 206, 207, 224, 225, 226, 227]   # mask builds: the 16 f16 mask values of this lane's 16 tokens of a tile
MOFF = X0               # mask builds: byte offset of this lane's first mask element inside a tile's 64 mask bytes (from the end of the prologue on)
LANE = T[7]             # prologue only
SLOPE = 252             # bias builds: ALiBi slope of this lane's row (one register more than the other builds own)
N_VGPR = 253 if BIAS else 252
# ---- SGPR map (all inside the clobbered range s40..s99)
KV, BT, KVB, KVE, CL2, NPP, NB1, FLG = 40, 42, 44, 45, 46, 47, 48, 49
NT, IT, OFF0, OFF1, OFF2, OFF3, WAVE, TMP = 50, 51, 52, 53, 54, 55, 56, 57
TB, PMASK, VMW, EXS = 58, 60, 61, 62         # PMASK: 127 with a block table (token inside its page), all ones without
S0, S1, S2, S3, DMAB, NVAL, THR, PG0 = 64, 65, 66, 67, 68, 69, 70, 71
RSC, ONES, OSTR, QP, OB, MLB, RSTR, NRV = 72, 74, 75, 76, 78, 80, 82, 83
W4, WOFS, FADR, PGZ, SPITCH, SCLS = 84, 85, 86, 87, 88, 89
VM = [90, 92, 94, 96]   # epilogue: lanes whose row of row block hb exists
SB = 98                 # epilogue: running store base
# LDS-DMA loads (the epilogue's row masks take these registers afterwards): wave * bytes a wave copies per tile; the four clamp
# offsets of the current tile; the first of them for the last tile of the piece; number of tiles - 1
WDMA, CL, LAST0, NTM1 = 90, [91, 92, 93, 94], 95, 96
DMA_BIAS = 3072         # the k-th load behind an M0 update carries the instruction offset 1024 k, which moves both addresses: the
                        # table offsets are (true offset - 1024 k + 3072) and the tile base is taken 3072 bytes low
SCL, L2E, MSK = 98, 99, 76   # mask builds: scale, log2(e) (SB's registers until the epilogue), mask base (QP's registers once Q is requested)
K1, K2 = CL2, NPP            # bias builds: 2 log2(e) scale / softcap (the input that carries c_log2 elsewhere) and -2 softcap, 0 = no soft
                             # cap (NPP's register once the page ids are clamped)
TAU_BITS = 0x41000000   # 8.0f

out = []
uid = [0]


def e(s):
    out.append(s)


def label(prefix):
    uid[0] += 1
    return "L%s_%d_%%=" % (prefix, uid[0])


def v(i, n=1):
    assert 0 <= i and i + n - 1 < N_VGPR, (i, n)
    return "v%d" % i if n == 1 else "v[%d:%d]" % (i, i + n - 1)


def a(i, n=1):
    return "a%d" % i if n == 1 else "a[%d:%d]" % (i, i + n - 1)


def s(i, n=1):
    return "s%d" % i if n == 1 else "s[%d:%d]" % (i, i + n - 1)


class Lds:
    """Tracks outstanding LDS accesses so that each use waits for exactly the accesses that precede it."""

    def __init__(self):
        self.pending = []
        self.issued = set()      # since the last reset(): a use may only wait for an access that was issued

    def op(self, line, tag):
        e(line)
        self.pending.append(tag)
        self.issued.add(tag)

    def reset(self, pending):
        self.pending = list(pending)
        self.issued = set(pending)

    def need(self, tag):
        assert tag in self.issued, tag
        if tag in self.pending:
            after = min(len(self.pending) - 1 - self.pending.index(tag), 15)   # the counter field has 4 bits
            e("s_waitcnt lgkmcnt(%d)" % after)
            self.pending = self.pending[len(self.pending) - after:] if after else []

    def drain(self):
        if self.pending:
            e("s_waitcnt lgkmcnt(0)")
            self.pending = []


lds = Lds()


def emit_item(x):
    """A shadow item is a line, None, or a callable that emits lines (LDS accesses go through the tracker)."""
    if x is None:
        return
    if callable(x):
        x()
    else:
        e(x)


def spread(items, first, last):
    """Assigns the items of one stream to the MFMA slots first .. last, evenly and in order: [(slot, item)]."""
    n = len(items)
    span = last - first + 1
    return [(first + (k * span) // n, it) for k, it in enumerate(items)]


def run_slots(slots, first_index, streams, events=None):
    """Emits the MFMA slots; behind slot i the items the streams assign to slot first_index + i, and ahead of it events[i]."""
    by_slot = {}
    for st in streams:
        for idx, it in st:
            by_slot.setdefault(idx, []).append(it)
    for i, slot in enumerate(slots):
        for ev in (events or {}).get(first_index + i, []):
            emit_item(ev)
        slot()
        for it in by_slot.pop(first_index + i, []):
            emit_item(it)
    assert all(not (first_index <= k < first_index + len(slots)) for k in by_slot), sorted(by_slot)
    return by_slot


# ---------------------------------------------------------------------------------------------------------------
def tile_base_lines(tile_sreg, first_page_scalar=False):
    """Scalar lines: s[TB:TB+1] = address of the first row of tile s[tile_sreg], less DMA_BIAS (s[KV] is kept that much low).
    The page id comes from the lane of PAGES that holds the tile's page -- at most 64 pages per split, the launcher sees to that.
    A cache without a table has no such limit: its PAGES and s[PGZ] are 0 and s[PMASK] keeps all bits of the token, so the row is
    the token itself whatever lane the (wrapping) index picks.  first_page_scalar: a tile inside the split's first page takes the id from s[PGZ] (the
    prologue's tiles, issued while the vector load of the page ids may still be in flight)."""
    L = []
    L.append("s_lshl_b32 %s, %s, 5" % (s(S0), s(tile_sreg)))
    L.append("s_add_u32 %s, %s, %s" % (s(S0), s(S0), s(KVB)))                      # S0 = first token of the tile
    L.append("s_lshr_b32 %s, %s, 7" % (s(S1), s(S0)))                             # logical page
    L.append("s_sub_u32 %s, %s, %s" % (s(S1), s(S1), s(PG0)))                     # index into the preloaded lanes
    L.append("v_readlane_b32 %s, %s, %s" % (s(S2), v(PAGES), s(S1)))
    if first_page_scalar:
        L.append("s_cmp_eq_u32 %s, 0" % s(S1))
        L.append("s_cselect_b32 %s, %s, %s" % (s(S2), s(PGZ), s(S2)))
    L.append("s_lshl_b32 %s, %s, 7" % (s(S2), s(S2)))
    L.append("s_and_b32 %s, %s, %s" % (s(S3), s(S0), s(PMASK)))                 # token inside the page; the whole token without a table
    L.append("s_add_u32 %s, %s, %s" % (s(S2), s(S2), s(S3)))                      # row in the pool / in the cache
    L.append("s_mul_hi_u32 %s, %s, %s" % (s(S1), s(S2), s(NB1)))
    L.append("s_mul_i32 %s, %s, %s" % (s(S0), s(S2), s(NB1)))
    L.append("s_add_u32 %s, %s, %s" % (s(TB), s(KV), s(S0)))
    L.append("s_addc_u32 %s, %s, %s" % (s(TB + 1), s(KV + 1), s(S1)))
    return L


def dma_table_lines(lane, tmp):
    """Once per kernel: where the 16 bytes that lane l of LDS-DMA slot j copies sit inside a tile.  The LDS side of a slot
    is 64 consecutive 16-byte chunks of the padded tile (73 chunks per row, the 73rd is padding); the global side is
    row * nb1 + min(column chunk, 71) * 16 -- at most 31 * 1152 + 1136 -- stored with the bias the instruction offsets
    ask for (see DMA_BIAS), two 16-bit values per register."""
    L = []
    row, col, x0, x1, x2 = tmp
    L.append("v_mov_b32 %s, %s" % (v(col), v(lane)))
    L.append("s_lshl_b32 %s, %s, 3" % (s(S2), s(WAVE)))
    L.append("v_mov_b32 %s, %s" % (v(row), s(S2)))                     # a wave copies rows 8w .. 8w+7
    for j in range(10):
        L.append("v_min_u32 %s, 71, %s" % (v(x1), v(col)))
        L.append("v_lshlrev_b32 %s, 4, %s" % (v(x1), v(x1)))
        L.append("v_mad_u32_u24 %s, %s, %s, %s" % (v(x0), v(row), s(NB1), v(x1)))
        L.append("v_add_u32 %s, %d, %s" % (v(x0), DMA_BIAS - 1024 * (j % 4), v(x0)))
        if j % 2 == 0:
            L.append("v_mov_b32 %s, %s" % (v(PT[j // 2]), v(x0)))
        else:
            L.append("v_lshl_or_b32 %s, %s, 16, %s" % (v(PT[j // 2]), v(x0), v(PT[j // 2])))
        if j < 9:
            L.append("v_add_u32 %s, 64, %s" % (v(col), v(col)))
            L.append("v_cmp_le_u32 vcc, %d, %s" % (CPR, v(col)))
            L.append("v_subrev_u32 %s, %d, %s" % (v(x2), CPR, v(col)))
            L.append("v_add_u32 %s, 1, %s" % (v(x0), v(row)))
            L.append("s_nop 0")
            L.append("v_cndmask_b32 %s, %s, %s, vcc" % (v(col), v(col), v(x2)))
            L.append("v_cndmask_b32 %s, %s, %s, vcc" % (v(row), v(row), v(x0)))
    return L


def dma_tile_lines(tile_sreg, off_sreg, first_page_scalar=False):
    """Instruction list (to be interleaved) that issues the LDS-DMA loads of tile s[tile_sreg] into the buffer at LDS
    offset s[off_sreg].  In the last tile of the piece rows past the end of the sequence are replaced by the last 16 bytes
    of the last valid row (any finite data will do: their probabilities are exactly 0): the table offsets are clamped to
    that row's last chunk (one SDWA instruction unpacks and clamps); in every other tile the clamp is out of reach."""
    L = tile_base_lines(tile_sreg, first_page_scalar)
    L.append("s_cmp_eq_u32 %s, %s" % (s(tile_sreg), s(NTM1)))
    L.append("s_cselect_b32 %s, %s, 0xffff" % (s(CL[0]), s(LAST0)))
    for c in range(1, 4):
        L.append("s_sub_u32 %s, %s, %d" % (s(CL[c]), s(CL[0]), 1024 * c))
    L.append("s_add_u32 %s, %s, %s" % (s(DMAB), s(WDMA), s(off_sreg)))
    for j in range(10):
        t = DT[j & 1]
        c = j % 4
        unpack = "v_min_u32_sdwa %s, %s, %s dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_%d" % (v(t), s(CL[c]), v(PT[j // 2]), j % 2)
        if c == 0:
            L.append("s_add_u32 m0, %s, %d" % (s(DMAB), 4096 * (j // 4)))     # (the unpack below fills the wait state M0 needs)
        L.append(unpack)
        if j == 9:
            # 8 chunks left per wave: lanes 0..7 only.  One atomic group: nothing may be scheduled inside the exec window.
            L.append("\\n\\t".join(["s_mov_b64 %s, exec" % s(EXS, 2),
                                    "s_mov_b64 exec, 0xff",
                                    "global_load_lds_dwordx4 %s, %s offset:%d%s" % (v(t), s(TB, 2), 1024 * c, NT_HINT),
                                    "s_mov_b64 exec, %s" % s(EXS, 2)]))
        else:
            L.append("global_load_lds_dwordx4 %s, %s offset:%d%s" % (v(t), s(TB, 2), 1024 * c, NT_HINT))
    return L


# ---------------------------------------------------------------------------------------------------------------
def kf_reg(p):
    slot = p % KRING
    return KF + 4 * slot if slot < KRING - 1 else T[4]


def k_read(p):
    lds.op("ds_read_b128 %s, %s offset:%d" % (v(kf_reg(p), 4), v(KADDR), p * 32), ("k", p))


def k_warm():
    for p in range(KRING - 1):
        k_read(p)


def qk_slots():
    """36 MFMA slots of S = K.Q^T; K fragments come through a ring (k_warm first), one wait per two fragments."""
    depth = KRING - 1

    def mk(ks):
        def slot():
            lds.need(("k", ks + 1) if ks % 2 == 0 and ("k", ks + 1) in lds.pending else ("k", ks))   # fragments return in order
            c = "0" if ks == 0 else v(S, 16)
            e("%s %s, %s, %s, %s" % (MF_QK, v(S, 16), v(kf_reg(ks), 4), v(Q0 + 4 * ks, 4), c))
            if ks + depth < 36:
                k_read(ks + depth)
        return slot
    return [mk(ks) for ks in range(36)]


def v_read_items(f):
    """V^T fragment f = (kk, cb) of the tile at v[VADDR] -> VF + 4 f: two transposing reads."""
    kk, cb = f // 4, f % 4
    base = 16 * kk * PITCH + cb * 64
    r = VF + 4 * f
    return [lambda: lds.op("ds_read_b64_tr_b16 %s, %s offset:%d" % (v(r, 2), v(VADDR), base), ("v", f, 0)),
            lambda: lds.op("ds_read_b64_tr_b16 %s, %s offset:%d" % (v(r + 2, 2), v(VADDR), base + 8 * PITCH), ("v", f, 1))]


def v_conv_items(f, tmp):
    """bf16 -> f16 of fragment f in place: per 32-bit word both halves widened to f32, then v_cvt_pkrtz_f16_f32 (exact inside
    the f16 range; round-toward-zero turns larger magnitudes into 65504 instead of infinity)."""
    if F16KV:
        return []
    r = VF + 4 * f
    c0, c1 = tmp

    def first():
        lds.need(("v", f, 1))
        e("v_lshlrev_b32 %s, 16, %s" % (v(c0), v(r)))
    I = [first]
    for j in range(4):
        if j:
            I.append("v_lshlrev_b32 %s, 16, %s" % (v(c0), v(r + j)))
        I.append("v_and_b32 %s, 0xffff0000, %s" % (v(c1), v(r + j)))
        I.append("v_cvt_pkrtz_f16_f32 %s, %s, %s" % (v(r + j), v(c0), v(c1)))
    return I


def p_read(f):
    kk, hb = f // NHB, f % NHB
    lds.op("ds_read_b128 %s, %s offset:%d" % (v(PR + 4 * (f % PRING), 4), v(PADDR), (hb * 2 + kk) * 1024), ("p", f))


def pv_slots():
    """32 MFMA slots of O^T += V^T.P^T in the order [kk][hb][cb]: a P^T fragment serves four consecutive MFMAs, and
    MFMAs on the same accumulator block are 16 slots apart."""
    def mk(n):
        kk, hb, cb = n // (4 * NHB), (n // 4) % NHB, n % 4
        f = NHB * kk + hb
        acc = 16 * (4 * cb + hb)

        def slot():
            if cb == 0:
                lds.need(("p", f))
            lds.need(("v", 4 * kk + cb, 1))          # f16 KV: the fragment is used as read; bf16: converted long before (no-op)
            e("%s %s, %s, %s, %s" % (MF_PV, a(acc, 16), v(VF + 4 * (4 * kk + cb), 4), v(PR + 4 * (f % PRING), 4), a(acc, 16)))
            if cb == 0 and f + PRING - 1 < NFRAG:
                p_read(f + PRING - 1)                # into the slot of fragment f - 1 (for f = 0: the tile before's last), whose last MFMA has been issued
        return slot
    return [mk(n) for n in range(8 * NHB)]


def softmax_lines(first_tile=False):
    """Softmax of the scores in S as one list of VALU lines (no branches): tile max -> lazy max update (a new max only where
    it grew by more than TAU) -> ALPHA (rescale factor of O and l, 1 where the max stayed) and RSC (non-zero when some lane
    changed its max) -> p = 2^(s*c - m) -> P^T operands (f16 pairs) in S+0..3 (k-step 0) and S+8..11 (k-step 1) ->
    l += sum of the rounded p (the output stays an exact weighted mean of V rows)."""
    L = []
    m = [T[0], T[1], T[2], T[3], T[4]]
    if MASK:
        # u = s * scale + mask (the order of ggml-cpu.c:12048-12057); element k = token 8 (k / 4) + 4 g + k % 4, whose mask value is
        # half k % 2 of register 2 (k / 4) + (k % 4) / 2
        for k in range(16):
            h = k % 2
            if BIAS:   # the logits were scaled (and capped) by bias_block(): u += slope * mask
                L.append("v_fma_mix_f32 %s, %s, %s, %s op_sel:[%d,0,0] op_sel_hi:[1,0,0]" % (v(S + k), v(MKR[2 * (k // 4) + (k % 4) // 2]), v(SLOPE), v(S + k), h))
            else:
                L.append("v_fma_mix_f32 %s, %s, %s, %s op_sel:[0,0,%d] op_sel_hi:[0,0,1]" % (v(S + k), v(S + k), s(SCL), v(MKR[2 * (k // 4) + (k % 4) // 2]), h))
    CS = L2E if MASK else CL2           # factor from the values in S to log2 units
    L.append("v_max3_f32 %s, %s, %s, %s" % (v(m[0]), v(S + 0), v(S + 1), v(S + 2)))
    L.append("v_max3_f32 %s, %s, %s, %s" % (v(m[1]), v(S + 3), v(S + 4), v(S + 5)))
    L.append("v_max3_f32 %s, %s, %s, %s" % (v(m[2]), v(S + 6), v(S + 7), v(S + 8)))
    L.append("v_max3_f32 %s, %s, %s, %s" % (v(m[3]), v(S + 9), v(S + 10), v(S + 11)))
    L.append("v_max3_f32 %s, %s, %s, %s" % (v(m[4]), v(S + 12), v(S + 13), v(S + 14)))
    L.append("v_max3_f32 %s, %s, %s, %s" % (v(m[0]), v(m[0]), v(m[1]), v(S + 15)))
    L.append("v_max3_f32 %s, %s, %s, %s" % (v(m[0]), v(m[0]), v(m[2]), v(m[3])))
    L.append("v_max_f32 %s, %s, %s" % (v(m[0]), v(m[0]), v(m[4])))
    L.append("v_mov_b32 %s, %s" % (v(m[1]), v(m[0])))
    L.append("s_nop 1")
    L.append("v_permlane32_swap_b32 %s, %s" % (v(m[0]), v(m[1])))
    L.append("s_nop 1")
    L.append("v_max_f32 %s, %s, %s" % (v(TMAX), v(m[0]), v(m[1])))
    L.append("v_mul_f32 %s, %s, %s" % (v(TMAX), s(CS), v(TMAX)))            # log2 units (the factor is > 0)
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
    for k in range(16):
        L.append("v_fma_f32 %s, %s, %s, %s" % (v(S + k), v(S + k), s(CS), v(NEGM)))
    for k in range(16):
        L.append("v_exp_f32 %s, %s" % (v(S + k), v(S + k)))
    # P^T operands in place.  k-step kk owns registers b = S+8kk .. +7, holding p of tokens
    # (8(2kk)+4g+0..3, 8(2kk+1)+4g+0..3); pairs (b0,b1) (b2,b3) (b4,b5) (b6,b7) -> b0..b3.
    for kk in range(2):
        b = S + 8 * kk
        for j in range(4):
            L.append("v_cvt_pk_f16_f32 %s, %s, %s" % (v(b + j), v(b + 2 * j), v(b + 2 * j + 1)))
        for j in range(4):
            acc = T[j & 1]
            c = "0" if kk == 0 and j < 2 else v(acc)
            L.append("v_dot2_f32_f16 %s, %s, %s, %s" % (v(acc), v(b + j), s(ONES), c))
    L.append("s_nop 2")   # a dot product's result may be read by another kind of VALU instruction three wait states later
    L.append("v_add_f32 %s, %s, %s" % (v(T[0]), v(T[0]), v(T[1])))
    L.append("v_add_f32 %s, %s, %s" % (v(LRUN), v(LRUN), v(T[0])))
    if first_tile:
        L.append("s_mov_b64 %s, 0" % s(RSC, 2))     # the accumulators are still zero: nothing to rescale
    return L


def p_write_items():
    """P^T operands of the wave's 32 rows, the rescale factors of those rows and the wave's flag word -> LDS."""
    I = []
    I.append("v_add_u32 %s, %s, %s" % (v(T[2]), s(WOFS), v(PADDR)))
    I.append(lambda: lds.op("ds_write_b128 %s, %s" % (v(T[2]), v(S, 4)), ("w", 0)))
    I.append(lambda: lds.op("ds_write_b128 %s, %s offset:1024" % (v(T[2]), v(S + 8, 4)), ("w", 1)))
    I.append("v_add_u32 %s, %s, %s" % (v(T[3]), s(W4), v(PADDR)))
    I.append(lambda: lds.op("ds_write_b32 %s, %s offset:%d" % (v(T[3]), v(ALPHA), AOFF - PBUF), ("w", 2)))
    I.append("v_mov_b32 %s, %s" % (v(T[0]), s(RSC)))
    I.append("v_or_b32 %s, %s, %s" % (v(T[0]), s(RSC + 1), v(T[0])))
    I.append("v_mov_b32 %s, %s" % (v(T[1]), s(FADR)))
    I.append(lambda: lds.op("ds_write_b32 %s, %s" % (v(T[1]), v(T[0])), ("w", 3)))
    return I


def bias_block():
    """Bias builds, once the scores of a tile are complete: S <- s * scale, or, with a soft cap, -2 softcap / (1 + 2^(s K1))
    (= softcap * tanh(s * scale / softcap) - softcap).  Not in the shadow of MFMAs: the two forms are a branch apart.  Ahead of
    mask_tail(): the cap is bounded, so a key past the end of the sequence that was already at -inf would come back with a finite
    logit (and count, wherever the caller's mask says nothing about the cells past the end of a paged sequence)."""
    lab_plain, lab_done = label("nocap"), label("capd")
    e("s_cmp_eq_u32 %s, 0" % s(K2))
    e("s_cbranch_scc1 %s" % lab_plain)
    for k in range(16):
        e("v_mul_f32 %s, %s, %s" % (v(S + k), s(K1), v(S + k)))
    for k in range(16):
        e("v_exp_f32 %s, %s" % (v(S + k), v(S + k)))
    for k in range(16):
        e("v_add_f32 %s, 1.0, %s" % (v(S + k), v(S + k)))
    for k in range(16):
        e("v_rcp_f32 %s, %s" % (v(S + k), v(S + k)))
    for k in range(16):
        e("v_mul_f32 %s, %s, %s" % (v(S + k), s(K2), v(S + k)))
    e("s_branch %s" % lab_done)
    e("%s:" % lab_plain)
    for k in range(16):
        e("v_mul_f32 %s, %s, %s" % (v(S + k), s(SCL), v(S + k)))
    e("%s:" % lab_done)


def mask_tail():
    """Last tile of a sequence only: tokens >= n_valid get score -inf.  element k is token 8*(k/4) + 4g + k%4."""
    lab = label("full")
    e("s_cmp_ge_u32 %s, 32" % s(NVAL))
    e("s_cbranch_scc1 %s" % lab)
    e("v_mov_b32 %s, 0xff800000" % v(T[0]))
    e("v_mbcnt_lo_u32_b32 %s, -1, 0" % v(T[2]))
    e("v_mbcnt_hi_u32_b32 %s, -1, %s" % (v(T[2]), v(T[2])))
    e("v_lshrrev_b32 %s, 5, %s" % (v(T[2]), v(T[2])))
    e("v_lshlrev_b32 %s, 2, %s" % (v(T[2]), v(T[2])))                       # 4g
    for k in range(16):
        e("v_add_u32 %s, %d, %s" % (v(T[1]), 8 * (k // 4) + (k % 4), v(T[2])))
        e("v_cmp_gt_u32 vcc, %s, %s" % (s(NVAL), v(T[1])))                  # valid if n_valid > token
        e("s_nop 1")
        e("v_cndmask_b32 %s, %s, %s, vcc" % (v(S + k), v(T[0]), v(S + k)))
    e("%s:" % lab)


def mask_loads(tile_sreg):
    """Mask builds: the 64 mask bytes of tile s[tile_sreg] for this lane's query token -> MKR (four 8-byte loads)."""
    e("s_lshl_b32 %s, %s, 6" % (s(S0), s(tile_sreg)))
    e("s_add_u32 %s, %s, %s" % (s(S0), s(MSK), s(S0)))
    e("s_addc_u32 %s, %s, 0" % (s(S1), s(MSK + 1)))
    for j in range(4):
        e("global_load_dwordx2 %s, %s, %s offset:%d" % (v(MKR[2 * j], 2), v(MOFF), s(S0, 2), 16 * j))


def mask_wait():
    """Mask builds: the mask values requested at the top of the iteration are there (loads return in order: only the tile
    loads issued behind them, if any, may still be in flight)."""
    lab_m0, lab_md = label("m0"), label("md")
    e("s_cmp_eq_u32 %s, 0" % s(VMW))
    e("s_cbranch_scc1 %s" % lab_m0)
    e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
    e("s_branch %s" % lab_md)
    e("%s:" % lab_m0)
    e("s_waitcnt vmcnt(0)")
    e("%s:" % lab_md)


def canon_tags(rowless=False):
    """LDS reads in flight at the top of every iteration, in issue order (see handover)."""
    return ([] if rowless else [("k", p) for p in range(KRING - 1)]) + [("p", f) for f in range(PRING - 1)]


def handover(tail, resc, rowless=False):
    """Behind the barrier that ends a tile (tile IT is the one whose P.V comes next): the flag words of the four waves, the
    first K fragments of the next K.Q^T (tile IT+1, buffer at s[OFF1]) and the first P^T fragments of tile IT, around the
    last four P.V MFMAs of the tile that ends (they still use ring slot 3, which fragment 3 takes afterwards), with the
    scalars of the coming iteration in their shadow; then the accumulators take the new row maxima if some wave's flag is
    up (out of line, rare).  rowless (--half): a wave without rows multiplies no K.Q^T."""
    e("v_mov_b32 %s, 0x%x" % (v(T[4]), FOFF))
    lds.op("ds_read_b128 %s, %s" % (v(T[0], 4), v(T[4])), ("f",))
    if not rowless:
        e("v_add_u32 %s, %s, %s" % (v(KADDR), s(OFF1), v(KADDR_LANE)))
        k_warm()
    # the tile's last fragment, which the tail MFMAs still use, sits in ring slot (NFRAG - 1) % PRING: a fragment that shares it is
    # requested behind them
    early = [f for f in range(PRING - 1) if not tail or f % PRING != (NFRAG - 1) % PRING]
    for f in early:
        p_read(f)
    top = ["s_add_u32 %s, %s, 1" % (s(S0), s(IT)),
           "s_lshl_b32 %s, %s, 5" % (s(S0), s(S0)),
           "s_add_u32 %s, %s, %s" % (s(S0), s(S0), s(KVB)),
           "s_sub_u32 %s, %s, %s" % (s(NVAL), s(KVE), s(S0)),
           "s_min_u32 %s, %s, 32" % (s(NVAL), s(NVAL)),                    # valid tokens of tile IT+1
           "v_add_u32 %s, %s, %s" % (v(VADDR), s(OFF0), v(VADDR_LANE))]  # V^T fragments of tile IT
    if tail:
        run_slots(tail, 0, [spread(top, 0, len(tail) - 1)])
    else:
        for ln in top:
            e(ln)
    for f in range(PRING - 1):
        if f not in early:
            assert f > max(early)      # fragments return in order
            p_read(f)
    lds.need(("f",))
    if HALF:      # (the words of the waves without rows are never written)
        e("v_or_b32 %s, %s, %s" % (v(T[0]), v(T[0]), v(T[1])))
    else:
        e("v_or3_b32 %s, %s, %s, %s" % (v(T[0]), v(T[0]), v(T[1]), v(T[2])))
        e("v_or_b32 %s, %s, %s" % (v(T[0]), v(T[0]), v(T[3])))
    e("v_cmp_ne_u32 vcc, 0, %s" % v(T[0]))
    lab_resc, lab_back = label("resc"), label("back")
    e("s_cmp_lg_u64 vcc, 0")
    e("s_cbranch_scc1 %s" % lab_resc)
    e("%s:" % lab_back)
    resc.append((lab_resc, lab_back))
    assert lds.pending == canon_tags(rowless), (lds.pending, canon_tags(rowless))


def rescale_block(ret_label):
    """Rare path, entered when no MFMA is left to issue on the old maxima: acc[cb][hb] *= alpha[hb] (per lane = per row)."""
    e("s_nop 7")
    e("s_nop 7")
    e("s_nop 3")
    e("ds_read_b128 %s, %s offset:%d" % (v(T[4], 4), v(PADDR), AOFF - PBUF))
    e("s_waitcnt lgkmcnt(0)")
    for cb in range(4):
        for hb in range(NHB):
            base = 16 * (4 * cb + hb)
            for i in range(0, 16, 4):
                for j in range(4):
                    e("v_accvgpr_read_b32 %s, %s" % (v(T[j]), a(base + i + j)))
                for j in range(4):
                    e("v_mul_f32 %s, %s, %s" % (v(T[j]), v(T[j]), v(T[4 + hb])))
                for j in range(4):
                    e("v_accvgpr_write_b32 %s, %s" % (a(base + i + j), v(T[j])))
    e("s_nop 7")
    e("s_nop 7")
    e("s_branch %s" % ret_label)


CLK_PREV = 97                   # --clk builds: last time stamp
LAPS = ["prologue to Q + tile 0", "first tile", "parts 1 and 2", "barrier (P read by all)", "P write + 4 MFMA", "tile-load wait", "barrier (tile end)"]


def lap(k):
    """--clk builds: adds the shader cycles since the last lap to accumulator k of this wave in LDS (FOFF + 64 + 32 w + 4 k;
    lane 0 adds).  Only placed where no LDS access is in flight and X0 / DT are free."""
    if not CLK:
        return
    assert not lds.pending, lds.pending
    e("s_memtime %s" % s(S0, 2))
    e("s_waitcnt lgkmcnt(0)")
    if k >= 0:
        e("s_sub_u32 %s, %s, %s" % (s(S1), s(S0), s(CLK_PREV)))
        e("v_mov_b32 %s, %s" % (v(X0), s(S1)))
        e("s_lshl_b32 %s, %s, 5" % (s(S1), s(WAVE)))
        e("s_add_u32 %s, %s, 0x%x" % (s(S1), s(S1), FOFF + 64 + 4 * k))
        e("v_mov_b32 %s, %s" % (v(DT[0]), s(S1)))
        e("s_mov_b64 exec, 1")
        e("ds_add_u32 %s, %s" % (v(DT[0]), v(X0)))
        e("s_mov_b64 exec, -1")
        e("s_waitcnt lgkmcnt(0)")
    e("s_mov_b32 %s, %s" % (s(CLK_PREV), s(S0)))


def clk_init():
    if CLK:
        e("v_mov_b32 %s, 0" % v(X0))
        e("s_lshl_b32 %s, %s, 5" % (s(S1), s(WAVE)))
        e("s_add_u32 %s, %s, 0x%x" % (s(S1), s(S1), FOFF + 64))
        e("v_mov_b32 %s, %s" % (v(DT[0]), s(S1)))
        for k in range(8):
            e("ds_write_b32 %s, %s offset:%d" % (v(DT[0]), v(X0), 4 * k))
        e("s_waitcnt lgkmcnt(0)")


def clk_dump():
    pass


# P.V slot ahead of which the barrier "every wave has read P of this tile" sits: behind the request for the tile's last P^T fragment
# (a ring of four asks for fragment 7 at slot 16, a ring of three -- the mask builds -- at slot 20: with the barrier ahead of slot 20
# the other waves' reads of fragment 7, wave 3's rows, raced with wave 3's write of the next tile's P), with an MFMA or two between
# the request and the wait for it
B2_AT = 8 if HALF else 22 if PRING == 3 else 20
PW_AT = 12 if HALF else 24        # P.V slot ahead of which P of the next tile is written (the softmax is done by then)
TAIL_AT = 8 * NHB - 4             # the last four P.V MFMAs of a tile are issued behind the barrier that ends it (see handover)


def v_stream(n_conv, tmp):
    """Part 1: reads of all eight V^T fragments of tile IT (two fragments ahead of their conversion) and conversion of
    the first n_conv, as one ordered stream: the conversions share two temporaries."""
    items = v_read_items(0) + v_read_items(1)
    for f in range(8):
        if f < n_conv:
            items += v_conv_items(f, tmp)
        if f + 2 < 8:
            items += v_read_items(f + 2)
    return spread(items, 0, 35)


def tile_end_wait():
    """The loads of tile IT+2 have landed (those of tile IT+3, issued in this iteration, may still be in flight: loads complete in
    order)."""
    lab_w0, lab_wd = label("w0"), label("wd")
    e("s_cmp_eq_u32 %s, 0" % s(VMW))
    e("s_cbranch_scc1 %s" % lab_w0)
    e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
    e("s_branch %s" % lab_wd)
    e("%s:" % lab_w0)
    e("s_waitcnt vmcnt(0)")
    e("%s:" % lab_wd)


def rotate_buffers():
    e("s_mov_b32 %s, %s" % (s(TMP), s(OFF0)))
    e("s_mov_b32 %s, %s" % (s(OFF0), s(OFF1)))
    e("s_mov_b32 %s, %s" % (s(OFF1), s(OFF2)))
    e("s_mov_b32 %s, %s" % (s(OFF2), s(OFF3)))
    e("s_mov_b32 %s, %s" % (s(OFF3), s(TMP)))
    e("s_add_u32 %s, %s, 1" % (s(IT), s(IT)))


def p_read_by_all():
    # every P^T fragment of tile IT is in this wave's registers before any wave overwrites P
    assert all(("p", f) in lds.issued for f in range(NFRAG)), "barrier ahead of the request for a P^T fragment"
    lds.drain()
    e("s_barrier")


def iteration_rowless(resc, lab_loop):
    """--half, a wave without rows: tile IT's share of the tile copies and the V^T fragments, then its 128 columns of P.V of the
    two row blocks, through the same two barriers per tile as the waves with rows."""
    e("; ---- iteration of a wave without rows")
    e("s_mov_b32 %s, 0" % s(VMW))
    lab_last, lab_nodma, lab_p2 = label("last"), label("nodma"), label("p2")
    e("s_add_u32 %s, %s, 1" % (s(TMP), s(IT)))
    e("s_cmp_ge_u32 %s, %s" % (s(TMP), s(NT)))
    e("s_cbranch_scc1 %s" % lab_last)
    e("s_add_u32 %s, %s, 3" % (s(TMP), s(IT)))
    e("s_cmp_ge_u32 %s, %s" % (s(TMP), s(NT)))
    e("s_cbranch_scc1 %s" % lab_nodma)

    def part1(dma):
        lds.reset(canon_tags(True))
        run_slots([lambda: None] * 36, 0, [spread(dma, 0, 35), v_stream(8, (T[0], T[1]))])

    e("s_mov_b32 %s, 1" % s(VMW))
    dma = dma_tile_lines(TMP, OFF3)
    part1(dma)
    state_a = list(lds.pending)
    e("s_branch %s" % lab_p2)
    e("%s:" % lab_nodma)
    part1([None] * len(dma))
    assert lds.pending == state_a, (lds.pending, state_a)
    e("%s:" % lab_p2)
    pv = pv_slots()
    left = run_slots(pv[:TAIL_AT], 36, [], {36 + B2_AT: [p_read_by_all]})
    assert not left, left
    lds.drain()
    tile_end_wait()
    e("s_barrier")
    rotate_buffers()
    handover(pv[TAIL_AT:], resc, True)
    e("s_branch %s" % lab_loop)
    e("%s:" % lab_last)
    lds.reset(canon_tags(True))
    for f in range(8):
        for it_ in v_read_items(f):
            emit_item(it_)
    for f in range(8):
        for it_ in v_conv_items(f, (T[0], T[1])):
            emit_item(it_)
    for sl in pv_slots():
        sl()
    lds.drain()


def iteration(resc, lab_loop):
    """Tile IT: see the module docstring.  s[NVAL] and v[VADDR] were set by the hand-over before."""
    e("; ---- iteration")
    e("s_mov_b32 %s, 0" % s(VMW))
    lab_last, lab_nodma, lab_p2 = label("last"), label("nodma"), label("p2")
    e("s_add_u32 %s, %s, 1" % (s(TMP), s(IT)))
    e("s_cmp_ge_u32 %s, %s" % (s(TMP), s(NT)))
    e("s_cbranch_scc1 %s" % lab_last)
    if MASK:
        mask_loads(TMP)              # mask of tile IT+1: behind the loads of tile IT+2, ahead of those of tile IT+3
    e("s_add_u32 %s, %s, 3" % (s(TMP), s(IT)))
    e("s_cmp_ge_u32 %s, %s" % (s(TMP), s(NT)))
    e("s_cbranch_scc1 %s" % lab_nodma)

    def part1(dma):
        lds.reset(canon_tags())
        run_slots(qk_slots(), 0, [spread(dma, 0, 35), v_stream(CONV_P1, (T[0], T[1]))])

    # ---- part 1 with the LDS-DMA loads of tile IT+3
    e("s_mov_b32 %s, 1" % s(VMW))
    dma = dma_tile_lines(TMP, OFF3)
    part1(dma)
    state_a = list(lds.pending)
    e("s_branch %s" % lab_p2)
    e("%s:" % lab_nodma)
    part1([None] * len(dma))
    assert lds.pending == state_a, (lds.pending, state_a)
    # ---- part 2: P.V of tile IT, softmax of tile IT+1 in its shadow
    e("%s:" % lab_p2)
    if CLK:
        lds.drain()
        lap(0)
    pv = pv_slots()
    conv2 = []
    for f in range(CONV_P1, 8):
        conv2 += v_conv_items(f, (DT[0], DT[1]))
    conv2 = spread(conv2, 37, 48) if conv2 else []      # one ordered stream (shared temporaries), done before k-step 1 starts at slot 52

    def qk_done():
        e("s_nop 1")                    # the last K.Q^T MFMA has written S: two P.V MFMAs (8 passes each) were issued behind it
        if BIAS:
            bias_block()                # (ahead of mask_tail: the soft cap maps -inf to a finite value)
        mask_tail()
        if MASK:
            mask_wait()

    sm = softmax_lines()
    streams = [conv2, spread(sm, 38, 36 + PW_AT - 1)]
    left = run_slots(pv[:PW_AT], 36, streams, {38: [qk_done], 36 + B2_AT: [p_read_by_all]})
    assert not left, left
    for it_ in p_write_items():
        emit_item(it_)
    for sl in pv[PW_AT:TAIL_AT]:
        sl()
    lds.drain()
    # the loads of tile IT+2 have landed; every wave is done with the buffers of tiles IT (V) and IT+1 (K), and P[IT+1] is written
    tile_end_wait()
    if CLK:
        lap(1)
    e("s_barrier")
    rotate_buffers()
    handover(pv[TAIL_AT:], resc)
    e("s_branch %s" % lab_loop)          # (tile IT exists: the iteration before was not the last)
    # ---- last tile: P.V only
    e("%s:" % lab_last)
    lds.reset(canon_tags())
    for f in range(8):
        for it_ in v_read_items(f):
            emit_item(it_)
    for f in range(8):
        for it_ in v_conv_items(f, (T[0], T[1])):
            emit_item(it_)
    for sl in pv_slots():
        sl()
    lds.drain()


def prologue_head(early=None):
    """Inputs -> fixed registers, lane geometry, the page ids of the piece, running state, the tile loads' offset table; ends
    when tile 0 can be requested.  early: emitted once the wave and lane numbers are known (loads that should be on their way
    while the rest is set up; v[36:167] and the scalar temporaries are its own until the end of the prologue)."""
    # ------------------------------------------------------------------ entry: inputs -> fixed registers
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
    e("s_mov_b64 %s, %%[ob]" % s(OB, 2))
    e("s_mov_b64 %s, %%[mlb]" % s(MLB, 2))
    e("s_mov_b32 %s, %%[rstr]" % s(RSTR))
    e("s_mov_b32 %s, %%[nrv]" % s(NRV))
    e("v_mov_b32 %s, %%[tid]" % v(X0))
    if MASK:
        e("s_mov_b32 %s, %%[scl]" % s(SCL))
        e("s_mov_b32 %s, 0x3fb8aa3b" % s(L2E))
    e("s_mov_b32 %s, 0x%08x" % (s(THR), TAU_BITS))
    e("s_mov_b32 %s, 0x3c003c00" % s(ONES))
    e("v_and_b32 %s, 63, %s" % (v(LANE), v(X0)))
    e("v_lshrrev_b32 %s, 6, %s" % (v(X1), v(X0)))
    e("s_nop 0")
    e("v_readfirstlane_b32 %s, %s" % (s(WAVE), v(X1)))
    e("s_lshl_b32 %s, %s, 2" % (s(W4), s(WAVE)))
    e("s_lshl_b32 %s, %s, 11" % (s(WOFS), s(WAVE)))
    e("s_add_u32 %s, %s, 0x%x" % (s(FADR), s(W4), FOFF))
    clk_init()
    lap(-1)
    if early:
        early()
    # lane geometry
    e("v_and_b32 %s, 31, %s" % (v(X0), v(LANE)))                       # rl
    e("v_lshrrev_b32 %s, 5, %s" % (v(X1), v(LANE)))                    # g
    e("v_lshlrev_b32 %s, 2, %s" % (v(T[0]), v(X1)))                    # 4g
    e("v_lshlrev_b32 %s, 4, %s" % (v(X2), v(X1)))                      # 16g
    e("s_mov_b32 %s, %d" % (s(SPITCH), PITCH))
    e("v_mad_u32_u24 %s, %s, %s, %s" % (v(KADDR_LANE), v(X0), s(SPITCH), v(X2)))
    e("v_bfe_u32 %s, %s, 2, 2" % (v(X0), v(LANE)))                     # (lane & 15) >> 2
    e("v_add_u32 %s, %s, %s" % (v(X0), v(T[0]), v(X0)))                # 4g + ...
    e("v_bfe_u32 %s, %s, 4, 1" % (v(X1), v(LANE)))                     # (lane >> 4) & 1
    e("v_lshlrev_b32 %s, 5, %s" % (v(X1), v(X1)))                      # *16 elements *2 bytes
    e("v_and_b32 %s, 3, %s" % (v(X2), v(LANE)))
    e("v_lshlrev_b32 %s, 3, %s" % (v(X2), v(X2)))                      # *4 elements *2 bytes
    e("v_add_u32 %s, %s, %s" % (v(X1), v(X1), v(X2)))
    e("v_mad_u32_u24 %s, %s, %s, %s" % (v(VADDR_LANE), v(X0), s(SPITCH), v(X1)))
    # the wave's 128 output columns start at column 128 w (256 bytes into the rows); FLG bit 4: V is columns 64 .. 575 of
    # the rows instead of 0 .. 511 (second pass of a 576-wide V)
    e("s_lshl_b32 %s, %s, 8" % (s(S0), s(WAVE)))
    e("s_bitcmp1_b32 %s, 4" % s(FLG))
    e("s_cselect_b32 %s, 128, 0" % s(S1))
    e("s_add_u32 %s, %s, %s" % (s(S0), s(S0), s(S1)))
    e("v_add_u32 %s, %s, %s" % (v(VADDR_LANE), s(S0), v(VADDR_LANE)))
    e("v_lshlrev_b32 %s, 4, %s" % (v(PADDR), v(LANE)))
    e("v_add_u32 %s, 0x%x, %s" % (v(PADDR), PBUF, v(PADDR)))
    # ------------------------------------------------------------------ page ids of this split -> one lane each.  A cache without
    # a table: page 0 everywhere and the whole token as the offset inside it (and no clamp against a pool size)
    lab_nobt = label("nobt")
    e("s_lshr_b32 %s, %s, 7" % (s(PG0), s(KVB)))
    e("v_mov_b32 %s, 0" % v(PAGES))
    e("s_cmp_eq_u64 %s, 0" % s(BT, 2))
    e("s_cselect_b32 %s, 0x7fffffff, %s" % (s(NPP), s(NPP)))
    e("s_cselect_b32 %s, 0, %s" % (s(PGZ), s(PGZ)))
    e("s_cselect_b32 %s, -1, 127" % s(PMASK))
    e("s_cbranch_scc1 %s" % lab_nobt)
    e("v_add_u32 %s, %s, %s" % (v(PAGES), s(PG0), v(LANE)))
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
    # ------------------------------------------------------------------ state
    e("v_mov_b32 %s, 0xff800000" % v(MRUN))
    e("v_mov_b32 %s, 0" % v(LRUN))
    e("s_mov_b32 %s, 0" % s(OFF0))
    e("s_mov_b32 %s, %d" % (s(OFF1), TILE_BYTES))
    e("s_mov_b32 %s, %d" % (s(OFF2), 2 * TILE_BYTES))
    e("s_mov_b32 %s, %d" % (s(OFF3), 3 * TILE_BYTES))
    e("s_mov_b32 %s, 0" % s(IT))
    e("s_sub_u32 %s, %s, %d" % (s(KV), s(KV), DMA_BIAS))
    e("s_subb_u32 %s, %s, 0" % (s(KV + 1), s(KV + 1)))
    e("s_mul_i32 %s, %s, %d" % (s(WDMA), s(WAVE), WAVE_CHUNKS * 16))
    e("s_sub_u32 %s, %s, 1" % (s(NTM1), s(NT)))
    # clamp offset of the last tile: its last valid row's last chunk, (n_valid - 1) * nb1 + 71 * 16, with the bias
    e("s_sub_u32 %s, %s, %s" % (s(S0), s(KVE), s(KVB)))
    e("s_lshl_b32 %s, %s, 5" % (s(S1), s(NTM1)))
    e("s_sub_u32 %s, %s, %s" % (s(S0), s(S0), s(S1)))
    e("s_sub_u32 %s, %s, 1" % (s(S0), s(S0)))
    e("s_mul_i32 %s, %s, %s" % (s(S0), s(S0), s(NB1)))
    e("s_add_u32 %s, %s, %d" % (s(LAST0), s(S0), 71 * 16 + DMA_BIAS))
    for ln in dma_table_lines(LANE, (T[0], T[1], T[2], T[3], T[4])):
        e(ln)
    lap(3)
    # Tile 0 can be requested before the page ids are there when the split starts on a page boundary: it lies in the first
    # page, whose id came as a scalar.  Otherwise wait for the ids (the only load in flight).
    lab_al = label("aligned")
    e("s_and_b32 %s, %s, 127" % (s(S0), s(KVB)))
    e("s_cmp_eq_u32 %s, 0" % s(S0))
    e("s_cbranch_scc1 %s" % lab_al)
    e("s_waitcnt vmcnt(0)")
    e("v_max_i32 %s, 0, %s" % (v(PAGES), v(PAGES)))
    e("v_min_i32 %s, %s, %s" % (v(PAGES), s(NPP), v(PAGES)))
    e("%s:" % lab_al)


def q_image_issue():
    """The 36 coalesced 16-byte loads per lane of this wave's Q operands from the packed image, first thing in the program, so that
    they are on their way while the prologue sets up its tables (not when FLG bit 6 says the operands wait in LDS; --half: not
    for a wave without rows, FLG bit 5)."""
    lab = label("qlds")
    e("s_bitcmp1_b32 %s, %d" % (s(FLG), 5 if HALF else 6))
    e("s_cbranch_scc1 %s" % lab)
    e("v_lshlrev_b32 %s, 4, %s" % (v(X0), v(LANE)))
    e("s_mul_i32 %s, %s, %d" % (s(S0), s(WAVE), 36 * 1024))
    e("s_add_u32 %s, %s, %s" % (s(QP), s(QP), s(S0)))
    e("s_addc_u32 %s, %s, 0" % (s(QP + 1), s(QP + 1)))
    for ks in range(36):
        if ks and ks % 4 == 0:
            e("s_add_u32 %s, %s, 4096" % (s(QP), s(QP)))
            e("s_addc_u32 %s, %s, 0" % (s(QP + 1), s(QP + 1)))
        e("global_load_dwordx4 %s, %s, %s offset:%d" % (v(Q0 + 4 * ks, 4), v(X0), s(QP, 2), (ks % 4) * 1024))
    e("%s:" % lab)


def main():
    prologue_head(q_image_issue)
    # ------------------------------------------------------------------ the Q operands and tile 0.  FLG bit 6: the C++ prologue left this
    # wave's 32 rows, rounded to the KV type, in tile buffer `wave` in the layout of a KV tile, so an operand is read like a K
    # fragment, and once every wave has its operands the buffers are free for tile 0.  Otherwise the operands are on their way from
    # the packed image since the top of the program (q_image_issue): tile 0.  Tiles 1 and 2 follow; go on as soon as tile 0 and Q
    # are there
    lab_img, lab_qd = label("qimg"), label("qdone")
    if not HALF:          # (the launcher gives the two-row-block program an operand image)
        e("s_bitcmp1_b32 %s, 6" % s(FLG))
        e("s_cbranch_scc0 %s" % lab_img)
        e("s_mul_i32 %s, %s, %d" % (s(S0), s(WAVE), TILE_BYTES))
        e("v_add_u32 %s, %s, %s" % (v(X0), s(S0), v(KADDR_LANE)))
        for ks in range(36):
            e("ds_read_b128 %s, %s offset:%d" % (v(Q0 + 4 * ks, 4), v(X0), 32 * ks))
        e("s_waitcnt lgkmcnt(0)")
        e("s_barrier")
        e("s_mov_b32 %s, 0" % s(TMP))
        for ln in dma_tile_lines(TMP, OFF0, True):
            e(ln)
        e("s_branch %s" % lab_qd)
        e("%s:" % lab_img)
    e("s_mov_b32 %s, 0" % s(TMP))
    for ln in dma_tile_lines(TMP, OFF0, True):
        e(ln)
    e("%s:" % lab_qd)
    if MASK:
        # mask rows start at key kv_begin of this piece; QP's registers and X0 are free now
        e("s_mov_b64 %s, %%[msk]" % s(MSK, 2))
        e("s_lshl_b32 %s, %s, 1" % (s(S0), s(KVB)))
        e("s_add_u32 %s, %s, %s" % (s(MSK), s(MSK), s(S0)))
        e("s_addc_u32 %s, %s, 0" % (s(MSK + 1), s(MSK + 1)))
        if BIAS:   # (one vector input less: the offset is the first word of this thread's hand-off record)
            e("v_lshlrev_b32 %s, 5, %s" % (v(MOFF), v(LANE)))
            e("s_lshl_b32 %s, %s, 11" % (s(S0), s(WAVE)))
            e("s_add_u32 %s, %s, 0x%x" % (s(S0), s(S0), HOFF))
            e("v_add_u32 %s, %s, %s" % (v(MOFF), s(S0), v(MOFF)))
            e("ds_read_b32 %s, %s" % (v(MOFF), v(MOFF)))
            e("s_waitcnt lgkmcnt(0)")
        else:
            e("v_mov_b32 %s, %%[moff]" % v(MOFF))
        e("s_mov_b32 %s, 0" % s(TMP))
        mask_loads(TMP)
    lap(4)
    lab_w0, lab_w1, lab_wd = label("pw0"), label("pw1"), label("pwd")
    for i in range(256):
        e("v_accvgpr_write_b32 %s, 0" % a(i))
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
    lap(5)
    e("s_waitcnt vmcnt(%d)" % (2 * DMA_PER_TILE))
    e("s_branch %s" % lab_wd)
    e("%s:" % lab_w1)
    e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
    e("s_branch %s" % lab_wd)
    e("%s:" % lab_w0)
    e("s_waitcnt vmcnt(0)")
    e("%s:" % lab_wd)
    # page ids outside the pool can only come from table entries that are never used; clamped so that no address leaves the pool
    e("v_max_i32 %s, 0, %s" % (v(PAGES), v(PAGES)))
    e("v_min_i32 %s, %s, %s" % (v(PAGES), s(NPP), v(PAGES)))
    if BIAS:
        # the last 8 bytes of this thread's hand-off record: its row's slope, and -2 softcap
        e("v_lshlrev_b32 %s, 5, %s" % (v(DT[0]), v(LANE)))
        e("s_lshl_b32 %s, %s, 11" % (s(S0), s(WAVE)))
        e("s_add_u32 %s, %s, 0x%x" % (s(S0), s(S0), HOFF + 24))
        e("v_add_u32 %s, %s, %s" % (v(DT[0]), s(S0), v(DT[0])))
        e("ds_read_b64 %s, %s" % (v(DT[0], 2), v(DT[0])))
        e("s_waitcnt lgkmcnt(0)")
        e("v_mov_b32 %s, %s" % (v(SLOPE), v(DT[0])))
        e("v_readfirstlane_b32 %s, %s" % (s(K2), v(DT[1])))
    e("s_barrier")                      # tile 0 is complete; every wave has read its hand-off record
    if HALF:
        lab_rowless = label("rowless")
        e("s_bitcmp1_b32 %s, 5" % s(FLG))
        e("s_cbranch_scc1 %s" % lab_rowless)
    e("v_add_u32 %s, %s, %s" % (v(KADDR), s(OFF0), v(KADDR_LANE)))
    k_warm()
    for slot in qk_slots():
        slot()
    e("s_sub_u32 %s, %s, %s" % (s(NVAL), s(KVE), s(KVB)))
    e("s_min_u32 %s, %s, 32" % (s(NVAL), s(NVAL)))
    e("s_nop 7")
    e("s_nop 7")
    if BIAS:
        bias_block()
    mask_tail()
    for ln in softmax_lines(first_tile=True):
        e(ln)
    for it_ in p_write_items():
        emit_item(it_)
    lds.drain()

    def tile1_wait():
        # tile 1 has landed (tile 2 may still be in flight)
        lab_t1, lab_t1d = label("t1"), label("t1d")
        e("s_cmp_lt_u32 %s, 3" % s(NT))
        e("s_cbranch_scc1 %s" % lab_t1)
        e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
        e("s_branch %s" % lab_t1d)
        e("%s:" % lab_t1)
        e("s_waitcnt vmcnt(0)")
        e("%s:" % lab_t1d)
        e("s_barrier")
    tile1_wait()
    resc = []
    handover([], resc)
    # ------------------------------------------------------------------ main loop
    lab_loop, lab_end = label("loop"), label("end")
    e("%s:" % lab_loop)
    iteration(resc, lab_loop)
    e("s_branch %s" % lab_end)
    for lab, back in resc:
        e("%s:" % lab)
        rescale_block(back)
    if HALF:
        # ------------------------------------------------------------------ the waves without rows: the same barriers, no K.Q^T, no softmax
        e("%s:" % lab_rowless)
        lds.reset([])
        tile1_wait()
        resc = []
        handover([], resc, True)
        lab_loop = label("loop")
        e("%s:" % lab_loop)
        iteration_rowless(resc, lab_loop)
        e("s_branch %s" % lab_end)
        for lab, back in resc:
            e("%s:" % lab)
            rescale_block(back)
    e("%s:" % lab_end)
    clk_dump()
    epilogue(NHB)
    emit()


def epilogue(nhb):
    """1 / l of the rows, then the stores: nhb = 4 (2: --half): the wave's 128 columns of all 128 (64) rows, 1 / l exchanged through
    LDS; nhb = 1 (the k-split program): 32 rows, every wave has l itself."""
    # ------------------------------------------------------------------ epilogue
    if nhb > 1:
        e("s_barrier")                  # no wave is still reading rescale factors: their area carries 1 / l next
    e("s_nop 7")
    e("s_nop 7")
    e("s_nop 7")
    # l of the wave's own rows: l(lane) + l(lane ^ 32); 1 / l with one Newton step (l = 0 still gives inf / NaN)
    e("v_mov_b32 %s, %s" % (v(T[0]), v(LRUN)))
    e("v_mov_b32 %s, %s" % (v(T[1]), v(LRUN)))
    e("s_nop 1")
    e("v_permlane32_swap_b32 %s, %s" % (v(T[0]), v(T[1])))
    e("s_nop 1")
    e("v_add_f32 %s, %s, %s" % (v(LRUN), v(T[0]), v(T[1])))
    e("v_rcp_f32 %s, %s" % (v(T[2]), v(LRUN)))
    e("s_nop 0")
    e("v_fma_f32 %s, -%s, %s, 2.0" % (v(T[3]), v(LRUN), v(T[2])))
    e("v_mul_f32 %s, %s, %s" % (v(T[3]), v(T[2]), v(T[3])))
    e("s_mov_b32 %s, 0x1f8" % s(SCLS))
    e("v_cmp_class_f32 vcc, %s, %s" % (v(T[3]), s(SCLS)))   # finite?
    e("s_nop 1")
    e("v_cndmask_b32 %s, %s, %s, vcc" % (v(T[2]), v(T[2]), v(T[3])))
    if nhb > 1:
        # every wave needs 1 / l of all 128 rows: through the rescale-factor area, [lane][hb] (a wave without rows leaves a word nobody reads)
        e("v_add_u32 %s, %s, %s" % (v(T[3]), s(W4), v(PADDR)))
        e("ds_write_b32 %s, %s offset:%d" % (v(T[3]), v(T[2]), AOFF - PBUF))
        e("s_waitcnt lgkmcnt(0)")
        e("s_barrier")
        e("ds_read_b128 %s, %s offset:%d" % (v(T[4], 4), v(PADDR), AOFF - PBUF))   # T[4 + hb] = 1 / l of row 32 hb + lane % 32
    else:
        e("v_mov_b32 %s, %s" % (v(T[4]), v(T[2])))
    # lanes whose row exists, per row block: lane % 32 < n_rows_valid - 32 hb
    e("v_mbcnt_lo_u32_b32 %s, -1, 0" % v(X0))
    e("v_mbcnt_hi_u32_b32 %s, -1, %s" % (v(X0), v(X0)))               # lane
    e("v_and_b32 %s, 31, %s" % (v(X1), v(X0)))                         # rl
    for hb in range(nhb):
        e("s_sub_i32 %s, %s, %d" % (s(S0), s(NRV), 32 * hb))
        e("v_cmp_gt_i32 vcc, %s, %s" % (s(S0), v(X1)))
        e("s_mov_b64 %s, vcc" % s(VM[hb], 2))
    e("s_mov_b64 %s, exec" % s(EXS, 2))
    e("v_lshrrev_b32 %s, 5, %s" % (v(X2), v(X0)))                      # g
    e("s_waitcnt lgkmcnt(0)")
    lab_pstore, lab_sdone = label("pstore"), label("sdone")
    e("s_bitcmp1_b32 %s, 0" % s(FLG))
    e("s_cbranch_scc0 %s" % lab_pstore)
    # f32 rows (final output, or f32 partials): element (row, column) at OB + row * RSTR + column * 4.
    # acc[cb][hb] register 4 q + c of lane (rl, g) is row 32 hb + rl, column 128 w + 32 cb + 8 q + 4 g + c.
    e("v_mul_lo_u32 %s, %s, %s" % (v(T[0]), v(X1), s(RSTR)))
    e("v_lshlrev_b32 %s, 4, %s" % (v(T[1]), v(X2)))
    e("v_add_u32 %s, %s, %s" % (v(T[0]), v(T[0]), v(T[1])))
    e("s_lshl_b32 %s, %s, 9" % (s(S0), s(WAVE)))
    e("v_add_u32 %s, %s, %s" % (v(T[0]), s(S0), v(T[0])))              # rl * RSTR + 16 g + 512 w
    e("s_lshl_b32 %s, %s, 5" % (s(S1), s(RSTR)))                       # 32 rows
    e("s_mov_b64 %s, %s" % (s(SB, 2), s(OB, 2)))
    for hb in range(nhb):
        e("s_mov_b64 exec, %s" % s(VM[hb], 2))
        for cb in range(4):
            for q in range(4):
                r = S if (cb * 4 + q) % 2 == 0 else S + 4          # alternate two 4-register staging groups
                for c in range(4):
                    e("v_accvgpr_read_b32 %s, %s" % (v(r + c), a(16 * (4 * cb + hb) + 4 * q + c)))
                for c in range(4):
                    e("v_mul_f32 %s, %s, %s" % (v(r + c), v(r + c), v(T[4 + hb])))
                e("global_store_dwordx4 %s, %s, %s offset:%d" % (v(T[0]), v(r, 4), s(SB, 2), (32 * cb + 8 * q) * 4))
        e("s_add_u32 %s, %s, %s" % (s(SB), s(SB), s(S1)))
        e("s_addc_u32 %s, %s, 0" % (s(SB + 1), s(SB + 1)))
    e("s_branch %s" % lab_sdone)
    e("%s:" % lab_pstore)
    # f16 partials O / l, layout [column / 8][row][8 halves]: the 8 bytes of lane (rl, g) for column group 16 w + 4 cb + q
    # of row 32 hb + rl sit at OB + (16 w + 4 cb + q) * OSTR + (32 hb + rl) * 16 + 8 g  (OSTR = rows of a slot * 16)
    e("v_lshlrev_b32 %s, 4, %s" % (v(T[0]), v(X1)))
    e("v_lshlrev_b32 %s, 3, %s" % (v(T[1]), v(X2)))
    e("v_add_u32 %s, %s, %s" % (v(T[0]), v(T[0]), v(T[1])))            # rl * 16 + 8 g
    e("s_lshl_b32 %s, %s, 4" % (s(S0), s(WAVE)))
    e("s_mul_i32 %s, %s, %s" % (s(S0), s(S0), s(OSTR)))                # 16 w * OSTR  (< 2^31: OSTR <= 2^27 / 64 is checked on the host)
    e("s_add_u32 %s, %s, %s" % (s(S2), s(OB), s(S0)))
    e("s_addc_u32 %s, %s, 0" % (s(S3), s(OB + 1)))
    for hb in range(nhb):
        e("s_mov_b64 exec, %s" % s(VM[hb], 2))
        e("s_mov_b64 %s, %s" % (s(SB, 2), s(S2, 2)))
        for cb in range(4):
            for q in range(4):
                r = S if (cb * 4 + q) % 2 == 0 else S + 4
                for c in range(4):
                    e("v_accvgpr_read_b32 %s, %s" % (v(r + c), a(16 * (4 * cb + hb) + 4 * q + c)))
                for c in range(4):
                    e("v_mul_f32 %s, %s, %s" % (v(r + c), v(r + c), v(T[4 + hb])))
                e("v_cvt_pk_f16_f32 %s, %s, %s" % (v(r), v(r), v(r + 1)))
                e("v_cvt_pk_f16_f32 %s, %s, %s" % (v(r + 1), v(r + 2), v(r + 3)))
                e("s_nop 0")
                e("global_store_dwordx2 %s, %s, %s offset:%d%s" % (v(T[0]), v(r, 2), s(SB, 2), hb * 512, PARTIAL_SCOPE))
                e("s_add_u32 %s, %s, %s" % (s(SB), s(SB), s(OSTR)))
                e("s_addc_u32 %s, %s, 0" % (s(SB + 1), s(SB + 1)))
    e("%s:" % lab_sdone)
    # (m, l) of this split for the wave's own rows, written by the g == 0 lanes when a pointer was handed over
    lab_noml = label("noml")
    e("s_mov_b64 exec, %s" % s(EXS, 2))
    e("s_cmp_eq_u64 %s, 0" % s(MLB, 2))
    e("s_cbranch_scc1 %s" % lab_noml)
    if nhb == 1:
        e("s_cmp_lg_u32 %s, 0" % s(WAVE))      # every wave holds (m, l) of the 32 rows: the first one writes them
        e("s_cbranch_scc1 %s" % lab_noml)
    e("s_lshl_b32 %s, %s, 5" % (s(S0), s(WAVE)))
    e("s_sub_i32 %s, %s, %s" % (s(S0), s(NRV), s(S0)))                 # valid rows of this wave's block
    e("v_cmp_gt_i32 vcc, %s, %s" % (s(S0), v(X0)))                     # lane < that ...
    e("s_nop 1")
    e("s_and_b64 exec, exec, vcc")
    e("s_mov_b32 exec_hi, 0")                                          # ... and g == 0
    e("v_lshlrev_b32 %s, 3, %s" % (v(T[2]), v(X0)))
    e("s_lshl_b32 %s, %s, 8" % (s(S1), s(WAVE)))
    e("v_add_u32 %s, %s, %s" % (v(T[2]), s(S1), v(T[2])))              # (32 w + lane) * 8
    e("v_mov_b32 %s, %s" % (v(T[0]), v(MRUN)))
    e("v_mov_b32 %s, %s" % (v(T[1]), v(LRUN)))
    e("s_nop 0")
    e("global_store_dwordx2 %s, %s, %s%s" % (v(T[2]), v(T[0], 2), s(MLB, 2), PARTIAL_SCOPE))
    e("%s:" % lab_noml)
    e("s_mov_b64 exec, %s" % s(EXS, 2))
    e("s_waitcnt vmcnt(0)")


# ---------------------------------------------------------------------------------------------------------------
# --ks: the program for at most 32 rows per sequence (a decode step of a 16- or 32-head model).  One row block, so the column-split
# programs would leave K.Q^T to one wave; here the four waves split its 576 columns instead:
#   wave w:  S_w = K[it+1][:, 144 w .. 144 w + 143] . Q[:, the same columns]^T   (9 MFMA; the wave holds a quarter of Q, 36 VGPRs)
#            S_w -> LDS (4 KB per wave), barrier, every wave reads the four partial tiles and adds them in the same order, so all
#            four hold the same scores, run the same softmax and reach the same maxima, sums and rescale decisions: P^T never
#            goes through LDS, no flags, no factors
#            O^T[128 w .. 128 w + 127][32 rows] += V[it]^T . P[it]^T   (8 MFMA)
# 17 MFMAs per wave and tile instead of 68 / 100 on one wave.  Three tile buffers (loads two tiles ahead, requested as soon as every
# wave is done with the buffer); the exchange area takes the fourth one's place.
SQ, XR = 36, 52           # partial scores of this wave; the four waves' partial tiles as read back
XOFF = 3 * TILE_BYTES     # exchange area: [wave][quarter of the 16 registers][lane][16 bytes] = 16 KB


def ks_qk_slots():
    depth = KRING - 1

    def mk(ks):
        def slot():
            lds.need(("k", ks))
            e("%s %s, %s, %s, %s" % (MF_QK, v(SQ, 16), v(kf_reg(ks), 4), v(Q0 + 4 * ks, 4), "0" if ks == 0 else v(SQ, 16)))
            if ks + depth < 9:
                k_read(ks + depth)
        return slot
    return [mk(ks) for ks in range(9)]


def ks_scores():
    """The MFMA slots of K.Q^T of the tile at v[KADDR] for this wave's quarter of the columns; the first K fragments are requested here."""
    for p_ in range(min(KRING - 1, 9)):
        k_read(p_)
    return ks_qk_slots()


def ks_exchange_write():
    e("s_nop 7")                       # the last MFMA's result
    e("s_nop 7")
    e("s_nop 3")
    e("v_add_u32 %s, %s, %s" % (v(T[2]), s(WOFS), v(PADDR)))
    for q in range(4):
        lds.op("ds_write_b128 %s, %s offset:%d" % (v(T[2]), v(SQ + 4 * q, 4), 1024 * q), ("x", q))
    lds.drain()
    e("s_barrier")


def ks_exchange_read_items():
    return [(lambda w=w, q=q: lds.op("ds_read_b128 %s, %s offset:%d" % (v(XR + 16 * w + 4 * q, 4), v(PADDR), 4096 * w + 1024 * q), ("xr", w, q)))
            for w in range(4) for q in range(4)]


def ks_sum_lines():
    L = []
    for k in range(16):
        L.append("v_add_f32 %s, %s, %s" % (v(S + k), v(XR + k), v(XR + 16 + k)))
    for k in range(16):
        L.append("v_add_f32 %s, %s, %s" % (v(S + k), v(S + k), v(XR + 32 + k)))
    for k in range(16):
        L.append("v_add_f32 %s, %s, %s" % (v(S + k), v(S + k), v(XR + 48 + k)))
    return L


def ks_pv(n):
    """MFMA n of the 8 of O^T += V^T.P^T: the P^T operands are this wave's own registers (S+0..3, S+8..11)."""
    kk, cb = n // 4, n % 4
    e("%s %s, %s, %s, %s" % (MF_PV, a(64 * cb, 16), v(VF + 4 * (4 * kk + cb), 4), v(S + 8 * kk, 4), a(64 * cb, 16)))


def ks_v_items():
    items = []
    for f in range(8):
        items += v_read_items(f)
    for f in range(8):
        items += v_conv_items(f, (DT[0], DT[1]))
    return items


def ks_rescale_block(ret_label):
    """Rare path: the running maxima moved; acc[cb] *= alpha (per lane = per row).  Entered long after the last MFMA was issued."""
    e("s_nop 7")
    for cb in range(4):
        for i in range(0, 16, 4):
            for j in range(4):
                e("v_accvgpr_read_b32 %s, %s" % (v(T[j]), a(64 * cb + i + j)))
            for j in range(4):
                e("v_mul_f32 %s, %s, %s" % (v(T[j]), v(T[j]), v(ALPHA)))
            for j in range(4):
                e("v_accvgpr_write_b32 %s, %s" % (a(64 * cb + i + j), v(T[j])))
    e("s_nop 7")
    e("s_branch %s" % ret_label)


def ks_tail(first_tile, resc):
    """Once the four partial tiles are back: their sum -> S, the keys past the end masked, softmax -> P^T operands in S, the
    accumulators rescaled if some row's maximum moved."""
    for ln in ks_sum_lines():
        e(ln)
    if BIAS:
        bias_block()
    mask_tail()
    for ln in softmax_lines(first_tile=first_tile):
        e(ln)
    if not first_tile:
        lab_resc, lab_back = label("resc"), label("back")
        e("s_cmp_lg_u64 %s, 0" % s(RSC, 2))
        e("s_cbranch_scc1 %s" % lab_resc)
        e("%s:" % lab_back)
        resc.append((lab_resc, lab_back))


KS_RP, KS_LOFF, KS_WADDR, KS_BUF = 164, 166, 167, 36


def ks_q_issue():
    """The loads of this wave's quarter of Q (144 columns of the 32 rows, f32 in global memory), first thing in the program: their
    way to the MFMA operands is the longest (registers, rounding, LDS, registers).  Where each row's quarter starts comes from a
    table the C++ prologue left behind the exchange buffer (lane r of the table read holds row r's address); one 16-byte load per
    lane and row, lanes past the 36th repeat the 36th."""
    pairs = [S0, S2, RSC, EXS]         # (scalar temporaries of later phases: nothing of the prologue lives in them yet)
    e("v_and_b32 %s, 31, %s" % (v(X0), v(LANE)))
    e("v_lshlrev_b32 %s, 3, %s" % (v(X0), v(X0)))
    e("s_lshl_b32 %s, %s, 8" % (s(S0), s(WAVE)))
    e("s_add_u32 %s, %s, 0x%x" % (s(S0), s(S0), AOFF))
    e("v_add_u32 %s, %s, %s" % (v(X0), s(S0), v(X0)))
    e("ds_read_b64 %s, %s" % (v(KS_RP, 2), v(X0)))
    e("v_min_u32 %s, 35, %s" % (v(X1), v(LANE)))
    e("v_lshlrev_b32 %s, 4, %s" % (v(KS_LOFF), v(X1)))                 # byte offset of the lane's load inside the quarter row
    e("v_lshlrev_b32 %s, 3, %s" % (v(X1), v(X1)))
    e("s_mul_i32 %s, %s, 288" % (s(S0), s(WAVE)))
    e("s_add_u32 %s, %s, %d" % (s(S0), s(S0), 2 * TILE_BYTES))
    e("v_add_u32 %s, %s, %s" % (v(KS_WADDR), s(S0), v(X1)))            # where the lane's 8 bytes of row 0 go: tile buffer 2
    e("s_waitcnt lgkmcnt(0)")
    for batch in range(8):
        for j in range(4):
            r = 4 * batch + j
            e("v_readlane_b32 %s, %s, %d" % (s(pairs[j]), v(KS_RP), r))
            e("v_readlane_b32 %s, %s, %d" % (s(pairs[j] + 1), v(KS_RP + 1), r))
        e("s_nop 4")                                                   # a lane read's scalar result may not be an address for 5 cycles
        for j in range(4):
            r = 4 * batch + j
            e("global_load_dwordx4 %s, %s, %s" % (v(KS_BUF + 4 * r, 4), v(KS_LOFF), s(pairs[j], 2)))


def ks_q_round(behind):
    """The quarter of Q, as it arrives, -> tile buffer 2, rounded to the KV type (to nearest even, as ggml-cpu rounds Q:
    ggml-cpu.c:12034-12035) in the layout of a KV tile.  behind: loads issued after the last of Q's (None: wait for everything)."""
    cvt = "v_cvt_pk_f16_f32" if F16KV else "v_cvt_pk_bf16_f32"
    if behind is None:
        e("s_waitcnt vmcnt(0)")
    for r in range(32):
        b = KS_BUF + 4 * r
        if behind is not None:
            e("s_waitcnt vmcnt(%d)" % (31 - r + behind))
        e("%s %s, %s, %s" % (cvt, v(b), v(b), v(b + 1)))
        e("%s %s, %s, %s" % (cvt, v(b + 1), v(b + 2), v(b + 3)))
        e("ds_write_b64 %s, %s offset:%d" % (v(KS_WADDR), v(b, 2), r * PITCH))
    e("s_waitcnt lgkmcnt(0)")


def ks_main():
    assert not CLK and (MASK or not BIAS)
    prologue_head(ks_q_issue)
    e("s_mul_i32 %s, %s, 288" % (s(S0), s(WAVE)))                      # this wave's k-steps 9 w ..: 32 bytes each
    e("v_add_u32 %s, %s, %s" % (v(KADDR_LANE), s(S0), v(KADDR_LANE)))
    e("v_lshlrev_b32 %s, 4, %s" % (v(PADDR), v(LANE)))
    e("v_add_u32 %s, 0x%x, %s" % (v(PADDR), XOFF, v(PADDR)))
    e("s_lshl_b32 %s, %s, 12" % (s(WOFS), s(WAVE)))
    if MASK:
        # mask rows start at key kv_begin of this piece (the operand image's registers are free: this program has none)
        e("s_mov_b64 %s, %%[msk]" % s(MSK, 2))
        e("s_lshl_b32 %s, %s, 1" % (s(S0), s(KVB)))
        e("s_add_u32 %s, %s, %s" % (s(MSK), s(MSK), s(S0)))
        e("s_addc_u32 %s, %s, 0" % (s(MSK + 1), s(MSK + 1)))
    # ------------------------------------------------------------------ tiles 0 and 1 are requested; the wave's quarter of Q (on its way
    # since the top of the program) goes through tile buffer 2 (every wave its own columns of the 32 rows, in the layout of a KV
    # tile: an operand is read like a K fragment); tile 2 is requested once every wave has its operands
    e("s_mov_b32 %s, 0" % s(TMP))
    for ln in dma_tile_lines(TMP, OFF0, True):
        e(ln)
    # behind Q's loads: the page ids (when there is a table; counted as absent, which at worst waits for one load more) and the
    # 10 loads of each tile
    lab_w0, lab_wd, lab_qr = label("pw0"), label("pwd"), label("qr")
    e("s_cmp_lt_u32 %s, 2" % s(NT))
    e("s_cbranch_scc1 %s" % lab_w0)
    e("s_mov_b32 %s, 1" % s(TMP))
    for ln in dma_tile_lines(TMP, OFF1, True):
        e(ln)
    ks_q_round(2 * DMA_PER_TILE)
    e("s_branch %s" % lab_qr)
    e("%s:" % lab_w0)
    ks_q_round(None)
    e("%s:" % lab_qr)
    e("v_add_u32 %s, %d, %s" % (v(X0), 2 * TILE_BYTES, v(KADDR_LANE)))
    for ks in range(9):
        e("ds_read_b128 %s, %s offset:%d" % (v(Q0 + 4 * ks, 4), v(X0), 32 * ks))
    for cb in range(4):
        for i in range(16):
            e("v_accvgpr_write_b32 %s, 0" % a(64 * cb + i))
    lab_one = label("pone")
    e("s_cmp_lt_u32 %s, 2" % s(NT))
    e("s_cbranch_scc1 %s" % lab_one)
    e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
    e("s_branch %s" % lab_wd)
    e("%s:" % lab_one)
    e("s_waitcnt vmcnt(0)")
    e("%s:" % lab_wd)
    e("s_waitcnt lgkmcnt(0)")
    e("v_max_i32 %s, 0, %s" % (v(PAGES), v(PAGES)))
    e("v_min_i32 %s, %s, %s" % (v(PAGES), s(NPP), v(PAGES)))
    e("s_barrier")                      # tile 0 is complete; every wave has its Q operands
    if MASK:
        # the mask values of tile 0 (the byte offset of this lane's first one: its row's token, tokens 4 g .. of a tile, is the
        # first word of this thread's hand-off record), ahead of tile 2's request
        e("v_mbcnt_lo_u32_b32 %s, -1, 0" % v(MOFF))
        e("v_mbcnt_hi_u32_b32 %s, -1, %s" % (v(MOFF), v(MOFF)))
        e("v_lshlrev_b32 %s, 5, %s" % (v(MOFF), v(MOFF)))
        e("s_lshl_b32 %s, %s, 11" % (s(S0), s(WAVE)))
        e("s_add_u32 %s, %s, 0x%x" % (s(S0), s(S0), HOFF))
        e("v_add_u32 %s, %s, %s" % (v(MOFF), s(S0), v(MOFF)))
        if BIAS:
            # the last 8 bytes of the record: the row's slope, and -2 softcap (NPP's register: the page ids are clamped)
            e("ds_read_b64 %s, %s offset:24" % (v(DT[0], 2), v(MOFF)))
        e("ds_read_b32 %s, %s" % (v(MOFF), v(MOFF)))
        e("s_waitcnt lgkmcnt(0)")
        if BIAS:
            e("v_mov_b32 %s, %s" % (v(SLOPE), v(DT[0])))
            e("v_readfirstlane_b32 %s, %s" % (s(K2), v(DT[1])))
        e("s_mov_b32 %s, 0" % s(TMP))
        mask_loads(TMP)
    lab_no2 = label("no2")
    e("s_cmp_lt_u32 %s, 3" % s(NT))
    e("s_cbranch_scc1 %s" % lab_no2)
    e("s_mov_b32 %s, 2" % s(TMP))
    for ln in dma_tile_lines(TMP, OFF2, True):
        e(ln)
    e("%s:" % lab_no2)
    e("v_add_u32 %s, %s, %s" % (v(KADDR), s(OFF0), v(KADDR_LANE)))
    lds.reset([])
    for slot in ks_scores():
        slot()
    ks_exchange_write()
    for it_ in ks_exchange_read_items():
        it_()
    e("s_sub_u32 %s, %s, %s" % (s(NVAL), s(KVE), s(KVB)))
    e("s_min_u32 %s, %s, 32" % (s(NVAL), s(NVAL)))
    lds.drain()
    if MASK:
        # the mask values are there once at most tile 2's loads are in flight
        lab_m1, lab_m1d = label("mt1"), label("mt1d")
        e("s_cmp_lt_u32 %s, 3" % s(NT))
        e("s_cbranch_scc1 %s" % lab_m1)
        e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
        e("s_branch %s" % lab_m1d)
        e("%s:" % lab_m1)
        e("s_waitcnt vmcnt(0)")
        e("%s:" % lab_m1d)
    resc = []
    ks_tail(True, resc)
    lab_t1, lab_t1d = label("t1"), label("t1d")
    e("s_cmp_lt_u32 %s, 3" % s(NT))
    e("s_cbranch_scc1 %s" % lab_t1)
    e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
    e("s_branch %s" % lab_t1d)
    e("%s:" % lab_t1)
    e("s_waitcnt vmcnt(0)")
    e("%s:" % lab_t1d)
    e("s_barrier")                      # tile 1 is complete; every wave has read the partial tiles
    # ------------------------------------------------------------------ main loop: tile IT is the one whose P.V comes next
    lab_loop, lab_last, lab_nodma, lab_dd, lab_end = (label(x) for x in ("loop", "last", "nodma", "dd", "end"))
    e("%s:" % lab_loop)
    e("s_mov_b32 %s, 0" % s(VMW))
    e("v_add_u32 %s, %s, %s" % (v(VADDR), s(OFF0), v(VADDR_LANE)))
    e("s_add_u32 %s, %s, 1" % (s(TMP), s(IT)))
    e("s_cmp_ge_u32 %s, %s" % (s(TMP), s(NT)))
    e("s_cbranch_scc1 %s" % lab_last)
    e("v_add_u32 %s, %s, %s" % (v(KADDR), s(OFF1), v(KADDR_LANE)))
    e("s_lshl_b32 %s, %s, 5" % (s(S0), s(TMP)))
    e("s_add_u32 %s, %s, %s" % (s(S0), s(S0), s(KVB)))
    e("s_sub_u32 %s, %s, %s" % (s(NVAL), s(KVE), s(S0)))
    e("s_min_u32 %s, %s, 32" % (s(NVAL), s(NVAL)))                     # valid keys of tile IT+1
    if MASK:
        mask_loads(TMP)                 # mask of tile IT+1: behind the loads of tile IT+2, ahead of those of tile IT+3
    # part 1: the partial scores of tile IT+1, with the V^T fragments of tile IT (reads, conversion) in their shadow and behind
    lds.reset([])
    qk = ks_scores()
    vit = ks_v_items()
    n_in = 40 if not F16KV else len(vit)
    run_slots(qk, 0, [spread(vit[:n_in], 0, 8)])
    for it_ in vit[n_in:]:
        emit_item(it_)
    ks_exchange_write()                 # barrier: every wave is done with tile IT's V rows and tile IT+1's K rows
    # the buffer of tile IT takes tile IT+3
    e("s_add_u32 %s, %s, 3" % (s(TMP), s(IT)))
    e("s_cmp_ge_u32 %s, %s" % (s(TMP), s(NT)))
    e("s_cbranch_scc1 %s" % lab_nodma)
    e("s_mov_b32 %s, 1" % s(VMW))
    for ln in dma_tile_lines(TMP, OFF0):
        e(ln)
    e("%s:" % lab_nodma)
    # part 2: P.V of tile IT (P^T of tile IT is still in S) with the reads of the partial tiles in between; then S <- scores of tile IT+1
    # (the V^T fragments were waited for before the exchange barrier: ks_exchange_write drains)
    xr = ks_exchange_read_items()
    lds.reset([])
    for n in range(8):
        ks_pv(n)
        xr[2 * n]()
        xr[2 * n + 1]()
    lds.drain()
    if MASK:
        mask_wait()
    ks_tail(False, resc)
    lab_w0b, lab_wdb = label("w0"), label("wd")
    e("s_cmp_eq_u32 %s, 0" % s(VMW))
    e("s_cbranch_scc1 %s" % lab_w0b)
    e("s_waitcnt vmcnt(%d)" % DMA_PER_TILE)
    e("s_branch %s" % lab_wdb)
    e("%s:" % lab_w0b)
    e("s_waitcnt vmcnt(0)")
    e("%s:" % lab_wdb)
    e("s_barrier")                      # tile IT+2 is complete; every wave has read the partial tiles
    e("s_mov_b32 %s, %s" % (s(TMP), s(OFF0)))
    e("s_mov_b32 %s, %s" % (s(OFF0), s(OFF1)))
    e("s_mov_b32 %s, %s" % (s(OFF1), s(OFF2)))
    e("s_mov_b32 %s, %s" % (s(OFF2), s(TMP)))
    e("s_add_u32 %s, %s, 1" % (s(IT), s(IT)))
    e("s_branch %s" % lab_loop)
    # ---- last tile: P.V only
    e("%s:" % lab_last)
    lds.reset([])
    for it_ in ks_v_items():
        emit_item(it_)
    lds.drain()
    for n in range(8):
        ks_pv(n)
    e("s_branch %s" % lab_end)
    for lab, back in resc:
        e("%s:" % lab)
        ks_rescale_block(back)
    e("%s:" % lab_end)
    epilogue(1)
    emit()


def emit():
    print("// generated by gen_decode_cs_asm.py%s%s%s%s%s%s -- do not edit" % (" --ks" if KS else "", " --half" if HALF else "", " --f16" if F16KV else "", " --mask" if MASK else "", " --bias" if BIAS else "", " --stream" if STREAM else ""))
    for ln in out:
        print('"%s\\n\\t"' % ln)
    # and nothing of the program is in flight when the compiled code goes on (the mirror image of the wait at the top: an LDS read
    # or a load requested ahead for a tile that never came would land in a register that code has taken since)
    print('"s_waitcnt vmcnt(0) lgkmcnt(0)\\n\\t"')
    if CLK:
        sys.stderr.write("laps: %s\n" % "; ".join(LAPS))


if KS:
    ks_main()
else:
    main()
