"""Pins the CPU oracle (oracle/mla_oracle.c) without the GPU: exhaustive conversion checks, brute-force Q8_0,
closed forms and invariants of the attention function chosen so that a dropped term, a wrong index or a
transposed operand fails at least one of them, and a differential run against the reference's own compiled
ggml-cpu when oracle/_ref is built."""
import numpy as np
import pytest

from oracle import oracle as O
from tests import util as U


# ------------------------------------------------------------------ conversions (exhaustive over all 65536 encodings)

def test_f16_roundtrip_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    f = O.f16_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(np.isnan(f), np.isnan(want))
    assert np.array_equal(f[~np.isnan(f)].view(np.uint32), want[~np.isnan(want)].view(np.uint32))
    back = O.f32_to_f16(f)
    ok = ~np.isnan(f)
    assert np.array_equal(back[ok], bits[ok])


def test_f32_to_f16_rne_against_numpy():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 200000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 65536.0, 1e30, -1e30, np.inf, -np.inf, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25,
                  2.0 ** -14, 2.0 ** -14 - 2.0 ** -25, 5.9604645e-08, 6.1e-5], dtype=np.float32)])
    # every midpoint between adjacent f16 values and its float32 neighbours: ties must go to even
    h = np.arange(0, 0x7c00, dtype=np.uint16)
    lo, hi = O.f16_to_f32(h), O.f16_to_f32((h + 1).astype(np.uint16))
    mid = ((lo.astype(np.float64) + hi.astype(np.float64)) / 2).astype(np.float32)
    x = np.concatenate([x, mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(np.inf)), -mid])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(O.f32_to_f16(x), want)


def test_bf16_exhaustive_and_rne():
    bits = np.arange(65536, dtype=np.uint16)
    f = O.bf16_to_f32(bits)
    assert np.array_equal(f.view(np.uint32), bits.astype(np.uint32) << 16)
    ok = ~np.isnan(f)
    assert np.array_equal(O.f32_to_bf16(f)[ok], bits[ok])
    # round to nearest even on the dropped 16 bits, against integer arithmetic done a different way
    rng = np.random.default_rng(1)
    u = rng.integers(0, 0x7f800000, 300000, dtype=np.uint32) | (rng.integers(0, 2, 300000, dtype=np.uint32) << 31)
    x = u.view(np.float32)
    low, up = u & 0xffff, u >> 16
    want = np.where((low > 0x8000) | ((low == 0x8000) & ((up & 1) == 1)), up + 1, up).astype(np.uint16)
    assert np.array_equal(O.f32_to_bf16(x), want)
    nan = np.array([np.nan], dtype=np.float32)
    assert (O.f32_to_bf16(nan)[0] & 0x7fc0) == 0x7fc0  # quiet NaN


# ------------------------------------------------------------------ Q8_0

def test_q8_0_block_layout_and_textbook_formula():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((50, 576)).astype(np.float32) * 3
    y = O.quantize_q8_0(x, 0)
    assert y.shape == (50, 612)
    blk = y.reshape(50, 18, 34)
    d = blk[..., :2].copy().view(np.float16)[..., 0].astype(np.float32)
    qs = blk[..., 2:].view(np.int8).astype(np.float32)
    xb = x.reshape(50, 18, 32)
    amax = np.abs(xb).max(-1)
    assert np.array_equal(d, (amax / 127).astype(np.float16).astype(np.float32))
    # textbook: q = round(x / d) with d = amax / 127 (in float32); ties are measure-zero for random data
    dd = (amax / np.float32(127)).astype(np.float32)
    want = np.rint(xb * (np.float32(1) / dd)[..., None])
    assert np.abs(qs - want).max() <= 1 and (qs != want).mean() < 1e-3
    assert np.array_equal(O.dequantize_q8_0(y).reshape(50, 18, 32), qs * d[..., None])
    # the two quantizer variants agree except on rare one-step differences
    y1 = O.quantize_q8_0(x, 1).reshape(50, 18, 34)[..., 2:].view(np.int8).astype(np.int32)
    assert np.abs(y1 - qs.astype(np.int32)).max() <= 1
    # all-zero block
    z = O.quantize_q8_0(np.zeros((1, 32), np.float32), 1)
    assert not z.any()


def test_q8_0_rounding_modes_differ_on_ties():
    # amax = 127 makes id exactly 1: x = k + 0.5 is a tie; roundf goes away from zero, the x86 path to even
    x = np.zeros((1, 32), np.float32)
    x[0, 0], x[0, 1], x[0, 2], x[0, 3] = 127.0, 2.5, -2.5, 3.5
    q0 = O.quantize_q8_0(x, 0)[0, 2:].view(np.int8)
    q1 = O.quantize_q8_0(x, 1)[0, 2:].view(np.int8)
    assert list(q0[:4]) == [127, 3, -3, 4]
    assert list(q1[:4]) == [127, 2, -2, 4]


# ------------------------------------------------------------------ closed forms / invariants of the op

TYPES = [O.TYPE_BF16, O.TYPE_F16, O.TYPE_Q8_0]


def _rand(rng, n3, H, N, n_kv, k_type):
    q = rng.standard_normal((n3, H, N, 576)).astype(np.float32)
    k = U.encode_kv(rng.standard_normal((n3, n_kv, 576)).astype(np.float32), k_type)
    return q, k


@pytest.mark.parametrize("k_type", TYPES)
def test_single_key_returns_v_row(k_type):
    rng = np.random.default_rng(3)
    q, k = _rand(rng, 2, 3, 2, 1, k_type)
    out = O.flash_attn_ext(q, k, k_type, dv=512, scale=0.3)
    v = O.to_f32(k, k_type)[:, 0, :512]
    if k_type == O.TYPE_F16:
        v = v.astype(np.float16).astype(np.float32)
    for b in range(2):
        assert np.array_equal(out[b], np.broadcast_to(v[b], (2, 3, 512)))


@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_Q8_0])
def test_zero_query_gives_mean_of_v(k_type):
    rng = np.random.default_rng(4)
    q, k = _rand(rng, 1, 2, 1, 37, k_type)
    q[:] = 0
    out = O.flash_attn_ext(q, k, k_type, dv=576, scale=1.0)
    mean = O.to_f32(k, k_type)[0].astype(np.float64).mean(0)
    assert np.abs(out[0, 0, 0] - mean).max() < 2e-6 * 37


@pytest.mark.parametrize("k_type", TYPES)
def test_matches_f64_softmax_attention(k_type):
    """Independent numpy float64 evaluation (its own softmax, its own index order) of the same rounded inputs."""
    rng = np.random.default_rng(5)
    n3, H, N, n_kv = 2, 5, 3, 91
    q, k = _rand(rng, n3, H, N, n_kv, k_type)
    mask = np.where(rng.random((N, n_kv)) < 0.3, -np.inf, rng.standard_normal((N, n_kv))).astype(np.float16)
    mask[:, 0] = 0
    out = O.flash_attn_ext(q, k, k_type, dv=512, mask=mask.view(np.uint16), scale=U.SCALE)
    kf = O.to_f32(k, k_type).astype(np.float64)
    if k_type == O.TYPE_BF16:
        qr = O.bf16_to_f32(O.f32_to_bf16(q)).astype(np.float64)
    elif k_type == O.TYPE_F16:
        qr = O.f16_to_f32(O.f32_to_f16(q)).astype(np.float64)
    else:
        qr = O.dequantize_q8_0(O.quantize_q8_0(q, 1)).astype(np.float64)
    s = np.einsum("bhnd,bkd->bnhk", qr, kf) * U.SCALE + mask.astype(np.float64)[None, :, None, :]
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    want = np.einsum("bnhk,bkd->bnhd", p, kf[..., :512])
    ma, rl = O.errors(out, want)
    if k_type == O.TYPE_F16:  # the reference's f16 accumulator costs ~3 decimal digits (it is what is being restated)
        assert ma < 2e-2 and rl < 1e-2, (ma, rl)
    else:
        assert ma < 5e-6 and rl < 5e-6, (ma, rl)
    # the f64 companion entry point must agree with numpy much more tightly, for every type
    f64 = O.flash_attn_ext_f64(q, k, k_type, dv=512, mask=mask.view(np.uint16), scale=U.SCALE)
    assert O.errors(f64, want)[0] < 1e-6


def test_masked_keys_are_never_read():
    """-inf mask entries skip the key entirely: poisoning those K rows with NaN/Inf must change nothing."""
    rng = np.random.default_rng(6)
    q, k = _rand(rng, 1, 4, 2, 40, O.TYPE_BF16)
    mask = np.zeros((2, 40), np.float16)
    mask[0, 5:20] = -np.inf
    mask[1, 30:] = -np.inf
    base = O.flash_attn_ext(q, k, O.TYPE_BF16, dv=512, mask=mask.view(np.uint16), scale=U.SCALE)
    k2 = k.copy()
    k2[0, 30:] = 0x7fc0  # NaN rows, masked only for token 1
    out = O.flash_attn_ext(q, k2, O.TYPE_BF16, dv=512, mask=mask.view(np.uint16), scale=U.SCALE)
    assert np.array_equal(out[0, 1], base[0, 1])
    assert np.isnan(out[0, 0]).all()
    # a fully masked row divides by S = 0 like the reference: NaN
    mask[1, :] = -np.inf
    out = O.flash_attn_ext(q, k, O.TYPE_BF16, dv=512, mask=mask.view(np.uint16), scale=U.SCALE)
    assert np.isnan(out[0, 1]).all() and not np.isnan(out[0, 0]).any()


def test_head_broadcast_and_output_layout():
    """All heads read the single KV head; dst row index is (seq*n_tok + tok)*n_head + head."""
    rng = np.random.default_rng(7)
    q, k = _rand(rng, 2, 3, 4, 33, O.TYPE_BF16)
    out = O.flash_attn_ext(q, k, O.TYPE_BF16, dv=512, scale=U.SCALE)
    assert out.shape == (2, 4, 3, 512)
    for b in range(2):
        for h in range(3):
            for t in range(4):
                one = O.flash_attn_ext(q[b:b + 1, h:h + 1, t:t + 1], k[b:b + 1], O.TYPE_BF16, dv=512, scale=U.SCALE)
                assert np.array_equal(one[0, 0, 0], out[b, t, h])
    q2 = q.copy()
    q2[:, 1] = q2[:, 0]
    out2 = O.flash_attn_ext(q2, k, O.TYPE_BF16, dv=512, scale=U.SCALE)
    assert np.array_equal(out2[:, :, 0], out2[:, :, 1])


def test_dv_prefix_property():
    """Output columns are independent: the 512-wide result is the prefix of the 576-wide (V := K) one."""
    rng = np.random.default_rng(8)
    for k_type in (O.TYPE_BF16, O.TYPE_Q8_0, O.TYPE_F16):
        q, k = _rand(rng, 1, 2, 2, 50, k_type)
        a = O.flash_attn_ext(q, k, k_type, dv=512, scale=U.SCALE)
        b = O.flash_attn_ext(q, k, k_type, dv=576, scale=U.SCALE)
        assert np.array_equal(a, b[..., :512])


def test_alibi_and_softcap_against_numpy():
    rng = np.random.default_rng(9)
    n_head, n_kv = 6, 29  # 6 heads: n_head_log2 = 4, heads 4,5 use the second slope family
    q, k = _rand(rng, 1, n_head, 1, n_kv, O.TYPE_BF16)
    mask = (-np.arange(n_kv)[::-1].astype(np.float32))[None].astype(np.float16)
    max_bias, cap = 8.0, 5.0
    out = O.flash_attn_ext(q, k, O.TYPE_BF16, dv=512, mask=mask.view(np.uint16), scale=U.SCALE, max_bias=max_bias, softcap=cap)
    kf = O.bf16_to_f32(k).astype(np.float64)[0]
    qr = O.bf16_to_f32(O.f32_to_bf16(q)).astype(np.float64)[0, :, 0]
    m0, m1 = 2.0 ** (-max_bias / 4), 2.0 ** (-max_bias / 2 / 4)
    slopes = np.array([m0 ** (h + 1) if h < 4 else m1 ** (2 * (h - 4) + 1) for h in range(n_head)])
    s = cap * np.tanh(qr @ kf.T * (U.SCALE / cap)) + slopes[:, None] * mask.astype(np.float64)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    want = p @ kf[:, :512]
    assert O.errors(out[0, 0], want)[0] < 5e-6


def test_empty_and_tiny_inputs():
    rng = np.random.default_rng(10)
    q, k = _rand(rng, 1, 2, 1, 0, O.TYPE_BF16)
    out = O.flash_attn_ext(q, k, O.TYPE_BF16, dv=512, scale=1.0)
    assert np.isnan(out).all()  # S = 0 -> 0 * inf


# ------------------------------------------------------------------ differential against the compiled reference

needs_ref = pytest.mark.skipif(not O.ref_available(), reason="oracle/_ref (the reference's compiled ggml) is not built")


@needs_ref
@pytest.mark.parametrize("k_type", TYPES)
@pytest.mark.parametrize("masked", [False, True])
def test_oracle_vs_compiled_reference(k_type, masked):
    rng = np.random.default_rng(11 + k_type)
    n3, H, N, n_kv = 2, 4, 5, 160
    q, k = _rand(rng, n3, H, N, n_kv, k_type)
    mask = None
    if masked:
        mask = np.where(rng.random((N, n_kv)) < 0.4, -np.inf, 0.0).astype(np.float16)
        mask[:, 3] = 0
        mask = mask.view(np.uint16)
    got = O.flash_attn_ext(q, k, k_type, dv=576, mask=mask, scale=U.SCALE)
    want = O.ref_flash_attn_ext(q, k, k_type, mask=mask, scale=U.SCALE)
    ma, rl = O.errors(got, want)
    if k_type == O.TYPE_F16:  # f16 accumulator: a 1e-7 difference in a dot can flip a rounding
        assert ma < 2e-3 and rl < 3e-4, (ma, rl)
    else:
        assert ma < 3e-6 and rl < 2e-6, (ma, rl)


@needs_ref
def test_oracle_vs_compiled_reference_alibi_softcap():
    rng = np.random.default_rng(12)
    q, k = _rand(rng, 1, 6, 2, 64, O.TYPE_BF16)
    mask = (rng.standard_normal((2, 64)) * 2).astype(np.float16).view(np.uint16)
    got = O.flash_attn_ext(q, k, O.TYPE_BF16, dv=576, mask=mask, scale=U.SCALE, max_bias=4.0, softcap=30.0)
    want = O.ref_flash_attn_ext(q, k, O.TYPE_BF16, mask=mask, scale=U.SCALE, max_bias=4.0, softcap=30.0)
    assert O.errors(got, want)[0] < 3e-6


@needs_ref
def test_conversions_and_quantizers_vs_compiled_reference():
    import ctypes as C
    r = O.ref()
    rng = np.random.default_rng(13)
    x = (rng.standard_normal(1 << 16) * 10.0 ** rng.integers(-8, 5, 1 << 16)).astype(np.float32)
    y = np.empty(x.size, np.uint16)
    r.ref_f32_to_f16_row(x.ctypes.data, y.ctypes.data, x.size)
    assert np.array_equal(y, O.f32_to_f16(x))
    r.ref_f32_to_bf16_row(x.ctypes.data, y.ctypes.data, x.size)
    assert np.array_equal(y, O.f32_to_bf16(x))
    xq = rng.standard_normal((64, 576)).astype(np.float32)
    for mode, fn in ((0, r.ref_quantize_q8_0_ref), (1, r.ref_quantize_q8_0_cpu)):
        yq = np.empty((64, 612), np.uint8)
        fn(xq.ctypes.data, yq.ctypes.data, xq.size)
        assert np.array_equal(yq, O.quantize_q8_0(xq, mode)), mode
