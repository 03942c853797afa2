"""Shared helpers of the parity tests: seeded inputs in the layouts of BASELINE.json's configs, the paged pool,
and the comparison against the oracle with the tolerances the target states (max-abs 2e-3, rel-L2 1e-3)."""
import numpy as np

from oracle import oracle as O

MAX_ABS_TOL = 2e-3
REL_L2_TOL = 1e-3
SCALE = float(1.0 / np.sqrt(192.0))  # kq_scale of DeepSeek-V2: 1/sqrt(n_embd_head_k = 192)
PAGE = 128


def f16_bits(x):
    return np.asarray(x, dtype=np.float16).view(np.uint16)


def encode_kv(kf, k_type, q8_scale=None, rng=None):
    """float32 rows -> storage rows (uint16 [..,576] or uint8 [..,612]) of the given ggml type."""
    if k_type == O.TYPE_BF16:
        return O.f32_to_bf16(kf)
    if k_type == O.TYPE_F16:
        return O.f32_to_f16(kf)
    if k_type == O.TYPE_Q8_0:
        if q8_scale is None:
            return O.quantize_q8_0(kf, 0)
        # BASELINE config 5: int8 = clip(round(N(0,1)/scale), +-127), one fp16 scale per block
        qs = np.clip(np.rint(kf / q8_scale), -127, 127).astype(np.int8)
        d = np.full(kf.shape[:-1] + (kf.shape[-1] // 32,), np.float16(q8_scale)).view(np.uint16)
        return O.make_q8_0(qs, d)
    raise ValueError(k_type)


def make_paged(rng, lens, k_type, n_pool_pages=None, sigma=1.0, q8_scale=None):
    """Page pool + shuffled block table for sequences of the given lengths.
    Returns pool [n_pool_pages*128, row], block_table int32 [B, max_blocks], per-sequence contiguous copies."""
    lens = np.asarray(lens, dtype=np.int64)
    nblk = (lens + PAGE - 1) // PAGE
    total = int(nblk.sum())
    if n_pool_pages is None:
        n_pool_pages = total
    assert n_pool_pages >= total
    perm = rng.permutation(n_pool_pages).astype(np.int32)
    max_blocks = max(int(nblk.max()), 1)
    bt = np.zeros((len(lens), max_blocks), dtype=np.int32)
    row = 576 if k_type != O.TYPE_Q8_0 else 612
    dt = np.uint16 if k_type != O.TYPE_Q8_0 else np.uint8
    # unused pool pages and the tail of every last page hold NaN-free but wild values: results must not depend on them
    pool = encode_kv((rng.standard_normal((n_pool_pages * PAGE, 576)) * 50.0).astype(np.float32), k_type, q8_scale)
    seqs = []
    pos = 0
    for b, L in enumerate(lens):
        ids = perm[pos:pos + nblk[b]]
        pos += int(nblk[b])
        bt[b, :nblk[b]] = ids
        kf = (rng.standard_normal((int(L), 576)) * sigma).astype(np.float32)
        enc = encode_kv(kf, k_type, q8_scale)
        seqs.append(enc)
        for j, pid in enumerate(ids):
            seg = enc[j * PAGE:(j + 1) * PAGE]
            pool[pid * PAGE: pid * PAGE + len(seg)] = seg
    assert pool.dtype == dt and pool.shape[1] == row
    return pool, bt, seqs


def oracle_per_seq(q, seqs, k_type, dv, mask=None, scale=SCALE, **kw):
    """Oracle output for sequences of different lengths: one oracle call per sequence (the op itself has one n_kv)."""
    outs = []
    for b, k in enumerate(seqs):
        m = None if mask is None else mask[:, :k.shape[0]]
        outs.append(O.flash_attn_ext(q[b:b + 1], k[None], k_type, dv=dv, mask=m, scale=scale, **kw)[0])
    return np.stack(outs)


def check(got, want, what="", max_abs=MAX_ABS_TOL, rel_l2=REL_L2_TOL):
    got = np.asarray(got)
    want = np.asarray(want)
    assert got.shape == want.shape, (got.shape, want.shape)
    nan_g, nan_w = np.isnan(got), np.isnan(want)
    assert np.array_equal(nan_g, nan_w), "%s: NaN pattern differs (%d vs %d)" % (what, nan_g.sum(), nan_w.sum())
    ma, rl = O.errors(np.where(nan_w, 0, got), np.where(nan_w, 0, want))
    assert ma <= max_abs and rl <= rel_l2, "%s: max-abs %.3e (tol %.1e), rel-L2 %.3e (tol %.1e)" % (what, ma, max_abs, rl, rel_l2)
    return ma, rl
