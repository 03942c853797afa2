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
