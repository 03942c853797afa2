"""Test infrastructure: what the C++ prologue of mla_decode_kernel hands to a generated wave program, rebuilt on the host for the
emulator of tests/wave_emu.py -- one workgroup's piece of a paged (or contiguous) latent KV cache, the packed Q operand image, the
output area -- and the float64 attention its result is compared with."""
import os

import numpy as np

from tests import wave_emu as E

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "jittorinfer_amd", "csrc")
PITCH = 1168
TILE_BYTES = 32 * PITCH
PBUF = 4 * TILE_BYTES
SCALE = 1.0 / np.sqrt(192.0)


def program_text(name):
    with open(os.path.join(CSRC, name)) as f:
        return f.read()


def to_kv_type(x, f16):
    """f32 values -> the 16-bit encodings of the cache type, and the values those encodings stand for."""
    x = np.asarray(x, np.float32)
    if f16:
        bits = x.astype(np.float16).view(np.uint16)
        return bits, bits.view(np.float16).astype(np.float64)
    bits = E.f32_to_bf16_rne(x.reshape(-1)).reshape(x.shape)
    return bits, E.bf16_to_f32(bits).astype(np.float64)


class Piece:
    """One workgroup's work: rows [0, n_rows) of one sequence (at most 128), keys [kv_begin, kv_end) of it."""

    def __init__(self, rng, f16, n_rows=128, kv_begin=0, kv_end=128, seq_len=None, paged=True, mask=None, n_head=None, sigma=0.5,
                 q_scale=1.0, k_boost=None):
        self.f16, self.n_rows, self.kv_begin, self.kv_end, self.paged = f16, n_rows, kv_begin, kv_end, paged
        seq_len = kv_end if seq_len is None else seq_len
        n_pages = (seq_len + 127) // 128
        self.n_tiles = (kv_end - kv_begin + 31) // 32
        k = rng.standard_normal((n_pages * 128, 576)).astype(np.float32) * sigma
        if k_boost is not None:              # later keys much larger: the running maxima of the rows move (the rare rescale path)
            k *= k_boost(np.arange(n_pages * 128))[:, None]
        k[seq_len:] = 50.0                   # rows past the end of the sequence must never reach a result
        self.k_bits, self.k_val = to_kv_type(k, f16)
        q = rng.standard_normal((128, 576)).astype(np.float32) * q_scale
        self.q_f32 = q
        self.q_bits, self.q_val = to_kv_type(q, f16)
        self.gmem = E.GlobalMemory()
        if paged:
            n_pool = n_pages + 3
            perm = rng.permutation(n_pool)[:n_pages]
            pool = np.full((n_pool * 128, 576), 0x7bff if f16 else 0x4248, np.uint16)     # unused pages: large finite values
            for lp, pp in enumerate(perm):
                pool[pp * 128:(pp + 1) * 128] = self.k_bits[lp * 128:(lp + 1) * 128]
            self.bt = np.full(n_pages + 2, -7, np.int32)      # entries past the sequence are never used (and are not valid ids)
            self.bt[:n_pages] = perm
            self.kv_addr = self.gmem.add("kv", pool)
            self.bt_addr = self.gmem.add("bt", self.bt)
            self.npp = n_pool - 1
            self.pg0 = int(perm[kv_begin >> 7])
        else:
            self.kv_addr = self.gmem.add("kv", self.k_bits[:max(seq_len, 1)])
            self.bt_addr, self.npp, self.pg0 = 0, 0, 0
        # packed Q operand image of this (sequence, row block): [wave][k-step][lane][16 bytes], lane (rl, g) of wave w at k-step ks
        # holds Q[32 w + rl][16 ks + 8 g .. + 7] in the cache type
        img = np.zeros((4, 36, 64, 8), np.uint16)
        for w in range(4):
            for ks in range(36):
                for g in range(2):
                    img[w, ks, 32 * g:32 * g + 32] = self.q_bits[32 * w:32 * w + 32, 16 * ks + 8 * g:16 * ks + 8 * g + 8]
        self.qp_addr = self.gmem.add("q_image", img)
        self.mask = mask
        self.n_head = n_head or n_rows
        if mask is not None:                 # [query tokens][n_kv] f16 additive mask
            self.mask_addr = self.gmem.add("mask", mask.astype(np.float16))
            self.mask_nb1 = mask.shape[1] * 2

    def reference(self, scale=SCALE, softcap=0.0, slopes=None, v0=0):
        """float64: (O / l, m in log2 units, l) of the piece for every row, from the values the cache and the operand image hold."""
        ks = self.k_val[self.kv_begin:self.kv_end]
        s = self.q_val[:self.n_rows] @ ks.T * scale
        if softcap:
            s = softcap * np.tanh(s / softcap)
        if self.mask is not None:
            tok = np.minimum(np.arange(self.n_rows), self.n_rows - 1) // self.n_head
            mk = self.mask[tok][:, self.kv_begin:self.kv_end].astype(np.float64)
            s = s + (mk if slopes is None else mk * slopes[:self.n_rows, None])
        m = s.max(axis=1, keepdims=True)
        with np.errstate(invalid="ignore"):
            p = np.exp(s - m)
        l = p.sum(axis=1, keepdims=True)
        return (p @ ks[:, v0:v0 + 512]) / l, m[:, 0] * np.log2(np.e), l[:, 0]


def cs_inputs(piece, gmem_out, f32_rows=True, final=True, scale=SCALE, mask_build=False, bias_build=False):
    """Inputs of the column-split programs (MLA_DECODE_CS_INPUTS of mla_decode_kernel.hip) for every wave of the workgroup."""
    out_rows = np.zeros((128, 512), np.float32) if f32_rows else np.zeros((64, 128, 8), np.float16)
    ob = gmem_out.add("out", out_rows, writable=True)
    ml = gmem_out.add("ml", np.zeros((128, 2), np.float32), writable=True)
    common = dict(kv=piece.kv_addr, bt=piece.bt_addr, kvb=piece.kv_begin, kve=piece.kv_end,
                  cl2=int(np.array([scale * np.log2(np.e)], np.float32).view(np.uint32)[0]), npp=piece.npp, nb1=1152,
                  ntl=piece.n_tiles, ostr=128 * 16, qp=piece.qp_addr, pg0=piece.pg0, ob=ob, mlb=0 if final else ml,
                  rstr=512 * 4, nrv=piece.n_rows, scl=int(np.array([scale], np.float32).view(np.uint32)[0]))
    if mask_build:
        common["msk"] = piece.mask_addr

    def per_wave(w):
        d = dict(common)
        d["flg"] = (1 if f32_rows else 0) | (32 if 32 * w >= piece.n_rows else 0)
        d["tid"] = 64 * w + np.arange(64)
        if mask_build:
            row = np.minimum(32 * w + np.arange(64) % 32, piece.n_rows - 1)
            d["moff"] = (row // piece.n_head) * piece.mask_nb1 + 8 * (np.arange(64) // 32)
        return d
    return per_wave


def cs_handoff(piece, bias_build=False, slopes=None, softcap=0.0):
    """The hand-off records the C++ prologue leaves at PBUF (32 bytes per thread): first word the mask offset, last 8 bytes slope and
    -2 softcap (bias builds)."""
    rec = np.zeros((256, 8), np.uint32)
    for t in range(256):
        w, lane = t // 64, t % 64
        row = min(32 * w + lane % 32, piece.n_rows - 1)
        if piece.mask is not None:
            rec[t, 0] = (row // piece.n_head) * piece.mask_nb1 + 8 * (lane // 32)
        if bias_build:
            rec[t, 6] = np.array([1.0 if slopes is None else slopes[row]], np.float32).view(np.uint32)[0]
            rec[t, 7] = np.array([softcap], np.float32).view(np.uint32)[0]
    return [(PBUF, rec)]


AOFF = PBUF + 8192


def ks_inputs(piece, gmem_out, f32_rows=True, final=True, scale=SCALE, mask_build=False):
    """Inputs of the k-split programs (at most 32 rows): those of the column-split programs; Q comes as f32 rows in global memory."""
    base = cs_inputs(piece, gmem_out, f32_rows=f32_rows, final=final, scale=scale, mask_build=mask_build)

    def per_wave(w):
        d = base(w)
        d["flg"] = 1 if f32_rows else 0
        d["qp"] = 0
        d.pop("moff", None)
        return d
    return per_wave


def ks_lds_init(piece, bias_build=False, slopes=None, softcap=0.0):
    """Hand-off records (first word: the mask offset of the thread's row, rows counted inside the one block of 32; bias builds: last 8
    bytes the row's slope and -2 softcap) and, behind the exchange buffer, every wave's table of the addresses its quarter of the 32 Q
    rows starts at."""
    q_addr = piece.gmem.add("q_f32", piece.q_f32[:piece.n_rows])
    rec = np.zeros((256, 8), np.uint32)
    tab = np.zeros((4, 32), np.uint64)
    for t in range(256):
        w, lane = t // 64, t % 64
        row = min(lane % 32, piece.n_rows - 1)
        if piece.mask is not None:
            rec[t, 0] = (row // piece.n_head) * piece.mask_nb1 + 8 * (lane // 32)
        if bias_build:
            rec[t, 6] = np.array([1.0 if slopes is None else slopes[row]], np.float32).view(np.uint32)[0]
            rec[t, 7] = np.array([softcap], np.float32).view(np.uint32)[0]
    for w in range(4):
        for r in range(32):
            tab[w, r] = q_addr + min(r, piece.n_rows - 1) * 576 * 4 + w * 576
    return [(PBUF, rec), (AOFF, tab)]


Q8_ROW = 612


class PieceRS(Piece):
    """A piece for the row-split programs: kind "bf16" (hi + lo program), "f16", "cvt" (bf16 cache converted to f16 inside LDS) or
    "q8" (Q8_0 rows: 18 blocks of an f16 scale and 32 int8 values); the operand image holds what the launcher's pack kernels leave."""

    def __init__(self, rng, kind, **kw):
        self.kind = kind
        if kind != "q8":
            Piece.__init__(self, rng, kind == "f16", **kw)
            if kind == "cvt":       # Q rounded to bf16, handed over as the f16 numbers of the same values
                self._set_image(self.q_val.astype(np.float16).view(np.uint16))
            return
        n_rows, kv_begin, kv_end = kw.get("n_rows", 128), kw.get("kv_begin", 0), kw.get("kv_end", 128)
        seq_len, paged = kw.get("seq_len") or kv_end, kw.get("paged", True)
        self.f16, self.n_rows, self.kv_begin, self.kv_end, self.paged = True, n_rows, kv_begin, kv_end, paged
        self.n_tiles = (kv_end - kv_begin + 31) // 32
        n_pages = (seq_len + 127) // 128
        qi = np.clip(np.rint(rng.standard_normal((n_pages * 128, 18, 32)) * 40), -127, 127).astype(np.int8)
        d = (rng.uniform(0.5, 1.5, (n_pages * 128, 18)) / 80).astype(np.float16)
        if kw.get("k_boost") is not None:
            d = (d.astype(np.float32) * kw["k_boost"](np.arange(n_pages * 128))[:, None]).astype(np.float16)
        rows = np.zeros((n_pages * 128, Q8_ROW), np.uint8)
        blocks = rows.reshape(-1, 18, 34)
        blocks[:, :, 0:2] = d.view(np.uint8).reshape(-1, 18, 2)
        blocks[:, :, 2:] = qi.view(np.uint8)
        rows[seq_len:] = 0x7b                 # bytes past the end of the sequence: never part of a result
        # the value the program multiplies with: f16(q * d), one rounding of the exact product
        self.k_val = (qi.astype(np.float32) * d.astype(np.float32)[:, :, None]).astype(np.float16).astype(np.float64).reshape(-1, 576)
        q = rng.standard_normal((128, 576)).astype(np.float32)
        self.q_f32 = q
        self.q_bits, self.q_val = to_kv_type(q, True)
        self.gmem = E.GlobalMemory()
        if paged:
            n_pool = n_pages + 3
            perm = rng.permutation(n_pool)[:n_pages]
            pool = np.full((n_pool * 128, Q8_ROW), 0x7b, np.uint8)
            for lp, pp in enumerate(perm):
                pool[pp * 128:(pp + 1) * 128] = rows[lp * 128:(lp + 1) * 128]
            self.bt = np.full(n_pages + 2, -7, np.int32)
            self.bt[:n_pages] = perm
            self.kv_addr = self.gmem.add("kv", pool)
            self.bt_addr = self.gmem.add("bt", self.bt)
            self.npp, self.pg0 = n_pool - 1, int(perm[kv_begin >> 7])
        else:
            self.kv_addr = self.gmem.add("kv", rows[:(seq_len + 31) // 32 * 32])
            self.bt_addr, self.npp, self.pg0 = 0, 0, 0
        self.mask, self.n_head = kw.get("mask"), kw.get("n_head") or n_rows
        if self.mask is not None:
            self.mask_addr = self.gmem.add("mask", self.mask.astype(np.float16))
            self.mask_nb1 = self.mask.shape[1] * 2
        self._set_image(self.q_bits)

    def _set_image(self, bits):
        img = np.zeros((4, 36, 64, 8), np.uint16)
        for w in range(4):
            for ks in range(36):
                for g in range(2):
                    img[w, ks, 32 * g:32 * g + 32] = bits[32 * w:32 * w + 32, 16 * ks + 8 * g:16 * ks + 8 * g + 8]
        if any(b[2] == "q_image" for b in self.gmem.bufs):
            self.gmem.array("q_image")[:] = img.view(np.uint8).reshape(-1)
        else:
            self.qp_addr = self.gmem.add("q_image", img)


def rs_setup(piece, f32_rows=True, final=True, scale=SCALE, v_col0=False, bias_build=False, slopes=None, softcap=0.0):
    """Inputs (MLA_DECODE_INPUTS of mla_decode_kernel.hip) and hand-off records of the row-split programs: every thread finds the
    address of its row's output (0: the row does not exist) and, lanes of the lower half, of its (m, l) pair in its record; bias
    builds: in the last 8 bytes its row's slope and -2 softcap, and in the inputs what the launcher hands such a build."""
    q8 = piece.kind == "q8"
    hoff = (3 * TILE_BYTES + 2 * 32 * Q8_ROW) if q8 else 4 * TILE_BYTES
    out_rows = np.zeros((128, 512), np.float32) if f32_rows else np.zeros((64, 128, 8), np.float16)
    ob = piece.gmem.add("out", out_rows, writable=True)
    ml = piece.gmem.add("ml", np.zeros((128, 2), np.float32), writable=True)
    rec = np.zeros((256, 4), np.uint64)
    for t in range(256):
        w, lane = t // 64, t % 64
        rl, g = lane % 32, lane // 32
        row = 32 * w + rl
        if piece.mask is not None:
            rec[t, 0] = (min(row, piece.n_rows - 1) // piece.n_head) * piece.mask_nb1 + 8 * g
        if row < piece.n_rows:
            rec[t, 1] = ob + (row * 2048 + 16 * g if f32_rows else row * 16 + 8 * g)
            if not final and g == 0:
                rec[t, 2] = ml + row * 8
        if bias_build:
            sl = np.array([1.0 if slopes is None else slopes[min(row, piece.n_rows - 1)], -2.0 * softcap if softcap else 0.0], np.float32)
            rec[t, 3] = int(sl.view(np.uint32)[0]) | (int(sl.view(np.uint32)[1]) << 32)
    common = dict(kv=piece.kv_addr, bt=piece.bt_addr, kvb=piece.kv_begin, kve=piece.kv_end,
                  cl2=int(np.array([scale * np.log2(np.e)], np.float32).view(np.uint32)[0]), npp=piece.npp, nb1=Q8_ROW if q8 else 1152,
                  ntl=piece.n_tiles, ostr=128 * 16, qp=piece.qp_addr, pg0=piece.pg0, msk=getattr(piece, "mask_addr", 0),
                  scl=int(np.array([scale], np.float32).view(np.uint32)[0]))
    if bias_build and softcap:
        common["scl"] = int(np.array([scale / softcap], np.float32).view(np.uint32)[0])
        common["cl2"] = int(np.array([2.0 * np.log2(np.e) * scale / softcap], np.float32).view(np.uint32)[0])

    def per_wave(w):
        d = dict(common)
        d["flg"] = (1 if f32_rows else 0) | (32 if 32 * w >= piece.n_rows else 0) | (16 if v_col0 else 0)
        d["tid"] = 64 * w + np.arange(64)
        return d
    return per_wave, [(hoff, rec)]
