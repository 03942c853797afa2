"""The golden cases: small seeded instances of each BASELINE config.  Inputs are regenerated from the seed
(numpy default_rng); the fixture holds only a hash of the inputs and the reference's output."""
import hashlib

import numpy as np

from oracle import oracle as O
from tests import util as U

CASES = {
    # name: (k_type, n_seq, n_head, n_tok, n_kv, mask kind, seed)
    "config1_f16_h16_kv1024": (O.TYPE_F16, 1, 16, 1, 1024, None, 1234),
    "config2_bf16_h16_kv300": (O.TYPE_BF16, 2, 16, 1, 300, None, 2),
    "config3_bf16_h128_kv256_sigma05": (O.TYPE_BF16, 1, 128, 1, 256, None, 3),
    "config4_bf16_prefill_causal": (O.TYPE_BF16, 1, 16, 12, 76, "causal", 4),
    "config5_q8_0_h128_kv200": (O.TYPE_Q8_0, 1, 128, 1, 200, None, 5),
    "scattered_cells_mask": (O.TYPE_BF16, 1, 4, 3, 96, "random", 6),
    # shapes that take the other wave programs of the HIP path: two row blocks (64 heads), row blocks with idle waves under a mask
    "two_row_blocks_bf16_h64_kv300": (O.TYPE_BF16, 2, 64, 1, 300, None, 7),
    "idle_waves_bf16_h20x3_mask": (O.TYPE_BF16, 1, 20, 3, 160, "biased", 8),
    # ALiBi (max_bias) and the soft cap, BIAS below: on 48 heads (row-split), Q8_0 cells, 16 heads (k-split), 128 heads (column-split)
    "alibi_softcap_bf16_h48_mask": (O.TYPE_BF16, 1, 48, 1, 160, "biased", 9),
    "alibi_q8_0_h128x2_mask": (O.TYPE_Q8_0, 1, 128, 2, 160, "biased", 10),
    "softcap_bf16_h16x2_mask": (O.TYPE_BF16, 1, 16, 2, 160, "biased", 11),
    "alibi_softcap_bf16_h128_mask": (O.TYPE_BF16, 1, 128, 1, 160, "biased", 12),
}

# name: (max_bias, logit_softcap); absent: neither
BIAS = {
    "alibi_softcap_bf16_h48_mask": (8.0, 30.0),
    "alibi_q8_0_h128x2_mask": (8.0, 0.0),
    "softcap_bf16_h16x2_mask": (0.0, 20.0),
    "alibi_softcap_bf16_h128_mask": (4.0, 10.0),
}


def make_inputs(name):
    k_type, n_seq, n_head, n_tok, n_kv, mask_kind, seed = CASES[name]
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((n_seq, n_head, n_tok, 576)).astype(np.float32)
    sigma = 0.5 if "sigma05" in name else 1.0
    kf = (rng.standard_normal((n_seq, n_kv, 576)) * sigma).astype(np.float32)
    k = U.encode_kv(kf, k_type, q8_scale=(1.0 / 32 if k_type == O.TYPE_Q8_0 else None))
    mask = None
    if mask_kind == "causal":
        n_old = n_kv - n_tok
        mask = np.where(np.arange(n_kv)[None, :] > n_old + np.arange(n_tok)[:, None], -np.inf, 0.0).astype(np.float16).view(np.uint16)
    elif mask_kind == "random":
        m = np.where(rng.random((n_tok, n_kv)) < 0.5, -np.inf, 0.0).astype(np.float16)
        m[:, 0] = 0
        mask = m.view(np.uint16)
    elif mask_kind == "biased":     # finite biases (what an ALiBi slope multiplies) with holes
        m = rng.standard_normal((n_tok, n_kv)).astype(np.float32)
        m[rng.random((n_tok, n_kv)) < 0.3] = -np.inf
        m[:, 0] = 0
        mask = m.astype(np.float16).view(np.uint16)
    max_bias, softcap = BIAS.get(name, (0.0, 0.0))
    h = hashlib.sha256()
    h.update(q.tobytes())
    h.update(k.tobytes())
    if mask is not None:
        h.update(mask.tobytes())
    return dict(q=q, k=k, k_type=k_type, mask=mask, scale=U.SCALE, max_bias=max_bias, softcap=softcap, digest=h.hexdigest())


# The nodes either side of the attention node: (kind, weight type, n_head, n_tok, rope mode, freq_scale, ext_factor, attn_factor, seed)
FRONT_CASES = {
    "rope_norm_plain": ("rope", None, 3, 7, 0, 1.0, 0.0, 1.0, 11),
    "rope_norm_yarn_deepseek": ("rope", None, 3, 7, 0, 0.025, 1.0, 0.8, 12),
    "rope_neox_yarn_partial": ("rope", None, 2, 5, 2, 0.5, 0.25, 1.3, 13),
    "q_states_bf16": ("q_states", O.TYPE_BF16, 4, 5, 0, 0.025, 1.0, 0.8, 14),
    "q_states_f16": ("q_states", O.TYPE_F16, 4, 5, 0, 1.0, 0.0, 1.0, 15),
    "unabsorb_bf16": ("unabsorb", O.TYPE_BF16, 4, 5, 0, 1.0, 0.0, 1.0, 16),
    "unabsorb_f16": ("unabsorb", O.TYPE_F16, 4, 5, 0, 1.0, 0.0, 1.0, 17),
}


def make_front_inputs(name):
    kind, w_type, H, n_tok, mode, fs, ext, af, seed = FRONT_CASES[name]
    rng = np.random.default_rng(seed)
    p = O.rope_params(n_dims=64, mode=mode, freq_scale=fs, ext_factor=ext, attn_factor=af, n_ctx_orig=4096)
    pos = rng.integers(0, 160000, size=n_tok).astype(np.int32)
    d = dict(kind=kind, w_type=w_type, n_head=H, p=p, pos=pos)
    if kind == "rope":
        d["x"] = rng.standard_normal((n_tok, H, 64)).astype(np.float32)
        blobs = [d["x"], pos]
    else:
        w = (rng.standard_normal((H * 256, 512)) * 0.05).astype(np.float32)
        d["wkv_b"] = O.f32_to_f16(w) if w_type == O.TYPE_F16 else O.f32_to_bf16(w)
        d["x"] = rng.standard_normal((n_tok, H * 192) if kind == "q_states" else (H, n_tok, 512)).astype(np.float32)
        blobs = [d["x"], pos, d["wkv_b"]]
    h = hashlib.sha256()
    for b in blobs:
        h.update(b.tobytes())
    d["digest"] = h.hexdigest()
    return d
