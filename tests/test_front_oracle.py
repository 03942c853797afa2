"""The oracle of the nodes either side of the attention node (oracle/mla_front_oracle.c: rotary embedding with YaRN, the
absorb products), pinned without a GPU: closed forms in numpy float64, invariants of a rotation, special cases, and --
when oracle/_ref is built -- the reference's own compiled ggml-cpu, bit for bit for the rotary embedding."""
import ctypes as C
import os
import subprocess
import tempfile

import numpy as np
import pytest

from oracle import oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
needs_ref = pytest.mark.skipif(not O.ref_available(), reason="oracle/_ref (compiled reference) is not built")


def _rope_f64(x, pos, p, ff=None):
    """The published YaRN formula (Peng et al. 2023, as restated in ggml/src/ggml-cpu/ggml-cpu.c:10272-10307) in float64."""
    n_tok, n_head, ne0 = x.shape
    nd = p.n_dims
    i = np.arange(nd // 2, dtype=np.float64)
    inv = np.float64(p.freq_base) ** (-2.0 * i / nd)
    if ff is not None:
        inv = inv / ff[:nd // 2].astype(np.float64)
    extrap = pos.astype(np.float64)[:, None] * inv[None, :]
    interp = p.freq_scale * extrap
    theta, ms = interp, np.float64(p.attn_factor)
    if p.ext_factor != 0:
        lo, hi = O.rope_corr_dims(p)
        ramp = 1 - np.clip((i - lo) / max(0.001, hi - lo), 0, 1)
        mix = ramp * p.ext_factor
        theta = interp * (1 - mix) + extrap * mix
        ms = ms * (1 + 0.1 * np.log(1 / p.freq_scale))
    c, s = np.cos(theta)[:, None, :] * ms, np.sin(theta)[:, None, :] * ms
    out = x.astype(np.float64).copy()
    if p.mode == 2:
        a, b = x[..., :nd // 2].astype(np.float64), x[..., nd // 2:nd].astype(np.float64)
        out[..., :nd // 2], out[..., nd // 2:nd] = a * c - b * s, a * s + b * c
    else:
        a, b = x[..., 0:nd:2].astype(np.float64), x[..., 1:nd:2].astype(np.float64)
        out[..., 0:nd:2], out[..., 1:nd:2] = a * c - b * s, a * s + b * c
    return out


@pytest.mark.parametrize("mode", [0, 2])
@pytest.mark.parametrize("fs,ext,af", [(1.0, 0.0, 1.0), (0.025, 1.0, 0.8), (0.5, 0.25, 1.3)])
def test_rope_matches_float64_formula_at_small_positions(mode, fs, ext, af):
    """Positions below 2048 keep theta * eps_f32 under 2e-4 * ... : the f32 pipeline must agree with float64 to about
    (|theta| + 2) ulp; a wrong pairing, sign, ramp or magnitude scale is off by O(1)."""
    rng = np.random.default_rng(11)
    p = O.rope_params(n_dims=64, mode=mode, freq_scale=fs, ext_factor=ext, attn_factor=af, n_ctx_orig=4096)
    x = rng.standard_normal((50, 3, 64)).astype(np.float32)
    pos = rng.integers(0, 2048, size=50).astype(np.int32)
    got, want = O.rope(x, pos, p), _rope_f64(x, pos, p)
    assert np.max(np.abs(got - want)) < 2048 * 6e-8 * 8 * 2   # |theta| <= 2048, |x| <= ~5, mscale <= ~2
    assert O.errors(got, want)[1] < 2e-5


def test_rope_position_zero_is_a_pure_scaling():
    rng = np.random.default_rng(12)
    x = rng.standard_normal((4, 2, 64)).astype(np.float32)
    p = O.rope_params(freq_scale=0.1, ext_factor=1.0, attn_factor=0.9)
    ms = np.float32(0.9) * np.float32(1 + 0.1 * np.log(1 / 0.1))
    got = O.rope(x, np.zeros(4, np.int32), p)
    np.testing.assert_allclose(got, x * ms, rtol=3e-7)
    np.testing.assert_array_equal(O.rope(x, np.zeros(4, np.int32), O.rope_params()), x)


@pytest.mark.parametrize("mode", [0, 2])
def test_rope_preserves_pair_norms_and_relative_angle(mode):
    """A rotation keeps |(x0, x1)|; and <rope(q, m), rope(k, n)> depends on m - n only."""
    rng = np.random.default_rng(13)
    p = O.rope_params(mode=mode)
    q = rng.standard_normal((1, 1, 64)).astype(np.float32)
    k = rng.standard_normal((1, 1, 64)).astype(np.float32)
    out = O.rope(np.repeat(q, 5, 0), np.array([0, 1, 17, 300, 999], np.int32), p)
    pairs = (lambda t: t.reshape(-1, 2, 32).transpose(0, 2, 1)) if mode == 2 else (lambda t: t.reshape(-1, 32, 2))
    np.testing.assert_allclose(np.linalg.norm(pairs(out), axis=2), np.repeat(np.linalg.norm(pairs(q), axis=2), 5, 0), rtol=2e-6)
    dots = []
    for m, n in ((5, 2), (105, 102), (1003, 1000)):
        a = O.rope(q, np.array([m], np.int32), p).astype(np.float64).ravel()
        b = O.rope(k, np.array([n], np.int32), p).astype(np.float64).ravel()
        dots.append(a @ b)
    assert max(dots) - min(dots) < 2e-3 * np.linalg.norm(q) * np.linalg.norm(k) * 1e-1


def test_rope_neox_is_the_normal_form_on_permuted_channels():
    rng = np.random.default_rng(14)
    x = rng.standard_normal((6, 2, 64)).astype(np.float32)
    pos = rng.integers(0, 50000, 6).astype(np.int32)
    perm = np.concatenate([np.arange(0, 64, 2), np.arange(1, 64, 2)])   # neox channel i <-> normal channel perm[i]
    a = O.rope(x, pos, O.rope_params(mode=0, freq_scale=0.3, ext_factor=0.5))
    b = O.rope(np.ascontiguousarray(x[..., perm]), pos, O.rope_params(mode=2, freq_scale=0.3, ext_factor=0.5))
    np.testing.assert_array_equal(a[..., perm], b)


def test_rope_partial_dims_copy_the_tail_and_strided_rows():
    rng = np.random.default_rng(15)
    big = rng.standard_normal((5, 3, 192)).astype(np.float32)
    x = big[:, :, 128:]                      # the q_pe view of the reference: rows of 64 inside rows of 192
    pos = np.arange(5, dtype=np.int32) * 7
    p = O.rope_params(n_dims=32)
    got = O.rope(x, pos, p)
    np.testing.assert_array_equal(got[..., 32:], x[..., 32:])
    np.testing.assert_array_equal(got, O.rope(np.ascontiguousarray(x), pos, p))


def test_rope_freq_factors_divide_the_angle():
    rng = np.random.default_rng(16)
    x = rng.standard_normal((3, 1, 64)).astype(np.float32)
    pos = np.array([3, 50, 700], np.int32)
    ff = (1 + rng.random(32)).astype(np.float32)
    p = O.rope_params()
    got, want = O.rope(x, pos, p, ff), _rope_f64(x, pos, p, ff)
    assert np.max(np.abs(got - want)) < 1e-3 and O.errors(got, want)[1] < 2e-5


def test_corr_dims_deepseek_values():
    """DeepSeek-V2's YaRN: n_rot 64, original context 4096, base 10000, beta 32 / 1 -> dims [10, 23]
    (64 ln(4096 / (32 2 pi)) / (2 ln 10000) = 10.47, 64 ln(4096 / (2 pi)) / (2 ln 10000) = 22.5)."""
    assert O.rope_corr_dims(O.rope_params()) == (10.0, 23.0)
    assert O.rope_corr_dims(O.rope_params(beta_fast=1e9, beta_slow=1e-9)) == (0.0, 63.0)   # clamped to [0, n_dims - 1]


def _w(rng, shape, w_type, sigma=0.05):
    w = (rng.standard_normal(shape) * sigma).astype(np.float32)
    return {O.TYPE_F16: O.f32_to_f16, O.TYPE_BF16: O.f32_to_bf16, O.TYPE_F32: lambda t: t}[w_type](w)


def _w_f64(wb, w_type):
    return {O.TYPE_F16: O.f16_to_f32, O.TYPE_BF16: O.bf16_to_f32, O.TYPE_F32: lambda t: t}[w_type](wb).astype(np.float64)


def _round(x, w_type):
    if w_type == O.TYPE_F16:
        return O.f16_to_f32(O.f32_to_f16(x))
    if w_type == O.TYPE_BF16:
        return O.bf16_to_f32(O.f32_to_bf16(x))
    return x


@pytest.mark.parametrize("w_type", [O.TYPE_F16, O.TYPE_BF16, O.TYPE_F32])
def test_mul_mat_matches_numpy_on_rounded_operands(w_type):
    rng = np.random.default_rng(21)
    a = _w(rng, (3, 40, 64), w_type, 1.0)
    b = rng.standard_normal((6, 9, 64)).astype(np.float32)     # src0 broadcast over 2 consecutive batches (i2 / r2)
    got = O.mul_mat(a, w_type, b)
    want = np.einsum("bmk,bnk->bmn", _round(b, w_type).astype(np.float64), np.repeat(_w_f64(a, w_type), 2, axis=0))
    assert got.shape == (6, 9, 40)
    np.testing.assert_allclose(got, want, rtol=0, atol=1e-6 * 64)
    # rounding of src1 to the weight type is part of the contract: the unrounded product differs measurably for bf16
    if w_type == O.TYPE_BF16:
        raw = np.einsum("bmk,bnk->bmn", b.astype(np.float64), np.repeat(_w_f64(a, w_type), 2, axis=0))
        assert np.max(np.abs(raw - want)) > 1e-3


def test_mul_mat_strided_views_like_the_reference_graph():
    """q_nope is a permuted view of q (rows 768*H bytes apart per token, 768 per head), wk_b a view of wkv_b."""
    rng = np.random.default_rng(22)
    H, n_tok = 3, 5
    q = rng.standard_normal((n_tok, H, 192)).astype(np.float32)
    w = _w(rng, (H, 512, 128), O.TYPE_BF16)
    got = O.mul_mat(w, O.TYPE_BF16, q[:, :, :128].transpose(1, 0, 2))
    want = O.mul_mat(w, O.TYPE_BF16, np.ascontiguousarray(q[:, :, :128].transpose(1, 0, 2)))
    np.testing.assert_array_equal(got, want)
    one = np.einsum("k,nk->n", _round(q[2, 1, :128], O.TYPE_BF16).astype(np.float64), _w_f64(w[1], O.TYPE_BF16))
    np.testing.assert_allclose(got[1, 2], one, atol=1e-5)


def test_absorb_identity_qk_through_the_latent_equals_qk_through_k_nope():
    """What absorption rests on: (q_nope . wk_b_h) . c == q_nope . (wk_b_h . c) for a latent row c, and the un-absorb
    product of a one-hot attention result returns wv_b's row; checked in float64 on f32 weights."""
    rng = np.random.default_rng(23)
    H, n_tok = 2, 3
    wkv_b = _w(rng, (H * 256, 512), O.TYPE_F32, 0.1)
    q = rng.standard_normal((n_tok, H * 192)).astype(np.float32)
    pos = np.arange(n_tok, dtype=np.int32)
    qs = O.mla_q_states(q, wkv_b, O.TYPE_F32, pos, O.rope_params(), H)          # [H, n_tok, 576]
    c = rng.standard_normal(512).astype(np.float32)
    wk_b = wkv_b.reshape(-1)[:H * 512 * 128].reshape(H, 512, 128).astype(np.float64)
    for h in range(H):
        k_nope = c.astype(np.float64) @ wk_b[h]                                   # [128]
        for t in range(n_tok):
            want = q.reshape(n_tok, H, 192)[t, h, :128].astype(np.float64) @ k_nope
            assert abs(qs[h, t, :512].astype(np.float64) @ c - want) < 1e-4 * (1 + abs(want))
    kqv = np.zeros((H, n_tok, 512), np.float32)
    kqv[:, :, 7] = 1.0
    out = O.mla_unabsorb(kqv, wkv_b, O.TYPE_F32, H).reshape(n_tok, H, 128)
    wv_b = wkv_b.reshape(-1)[H * 512 * 128:].reshape(H, 128, 512)
    for h in range(H):
        np.testing.assert_array_equal(out[0, h], wv_b[h, :, 7])


@needs_ref
@pytest.mark.parametrize("mode", [0, 2])
def test_rope_bit_exact_against_compiled_reference(mode):
    rng = np.random.default_rng(31 + mode)
    x = rng.standard_normal((3, 2, 64)).astype(np.float32)
    pos = np.array([1, 77, 150000], dtype=np.int32)
    for _ in range(150):
        p = O.rope_params(mode=mode, freq_scale=float(np.float32(rng.uniform(0.01, 1.0))), ext_factor=float(np.float32(rng.uniform(0, 1.0))),
                          attn_factor=float(np.float32(rng.uniform(0.5, 1.5))), n_ctx_orig=int(rng.integers(1000, 10000)),
                          freq_base=float(rng.choice([10000.0, 500000.0, 1e6])))
        np.testing.assert_array_equal(O.rope(x, pos, p), O.ref_rope(x, pos, p))
    p = O.rope_params(n_dims=32, mode=mode, freq_scale=0.25, ext_factor=1.0)
    x = rng.standard_normal((9, 3, 80)).astype(np.float32)
    ff = (1 + rng.random(16)).astype(np.float32)
    np.testing.assert_array_equal(O.rope(x, np.arange(9, dtype=np.int32) * 1000, p, ff), O.ref_rope(x, np.arange(9, dtype=np.int32) * 1000, p, ff))


@needs_ref
@pytest.mark.parametrize("w_type", [O.TYPE_F16, O.TYPE_BF16, O.TYPE_F32])
def test_mul_mat_and_absorb_graphs_against_compiled_reference(w_type):
    """The reference sums products in f32 lanes (ggml-cpu.c:1586-1698); the oracle in double: the difference is bounded by
    a few f32 roundings of sum |a||b|."""
    rng = np.random.default_rng(41)
    H, n_tok = 6, 11
    wkv_b = _w(rng, (H * 256, 512), w_type)
    a = wkv_b.reshape(-1)[:H * 512 * 128].reshape(H, 512, 128)
    b = rng.standard_normal((H, 7, 128)).astype(np.float32)
    o, ab = O.mul_mat(a, w_type, b, with_abs=True)
    assert np.max(np.abs(o - O.ref_mul_mat(a, w_type, b)) / ab) < 1e-6
    q = rng.standard_normal((n_tok, H * 192)).astype(np.float32)
    pos = rng.integers(0, 100000, size=n_tok).astype(np.int32)
    p = O.rope_params(freq_scale=0.025, ext_factor=1.0, attn_factor=0.8)
    mine, theirs = O.mla_q_states(q, wkv_b, w_type, pos, p, H), O.ref_mla_q_states(q, wkv_b, w_type, pos, p, H)
    np.testing.assert_array_equal(mine[:, :, 512:], theirs[:, :, 512:])     # cont + rope + permute + concat: exact
    assert O.errors(mine, theirs)[1] < 1e-6
    kqv = rng.standard_normal((H, n_tok, 512)).astype(np.float32)
    assert O.errors(O.mla_unabsorb(kqv, wkv_b, w_type, H), O.ref_mla_unabsorb(kqv, wkv_b, w_type, H))[1] < 1e-6


def test_oracle_against_golden_vectors_of_the_compiled_reference():
    """tests/golden/front_golden.npz: outputs of the reference's compiled ggml-cpu (made by tests/golden/gen_golden.py)."""
    from tests.golden import cases
    gold = np.load(os.path.join(ROOT, "tests", "golden", "front_golden.npz"))
    for name in cases.FRONT_CASES:
        inp = cases.make_front_inputs(name)
        assert bytes(gold[name + "/digest"]).decode() == inp["digest"], "inputs of %s are not the ones the fixture was made from" % name
        if inp["kind"] == "rope":
            np.testing.assert_array_equal(O.rope(inp["x"], inp["pos"], inp["p"]), gold[name])
        elif inp["kind"] == "q_states":
            got = O.mla_q_states(inp["x"], inp["wkv_b"], inp["w_type"], inp["pos"], inp["p"], inp["n_head"])
            np.testing.assert_array_equal(got[:, :, 512:], gold[name][:, :, 512:])
            assert O.errors(got, gold[name])[1] < 1e-6
        else:
            assert O.errors(O.mla_unabsorb(inp["x"], inp["wkv_b"], inp["w_type"], inp["n_head"]), gold[name])[1] < 1e-6


def _header_offsets(struct, fields):
    src = '#include <stdio.h>\n#include <stddef.h>\n#include "mla_front.h"\nint main(void){\n'
    src += 'printf("%%zu\\n", sizeof(%s));\n' % struct
    for f in fields:
        src += 'printf("%%zu\\n", offsetof(%s, %s));\n' % (struct, f)
    src += "return 0;}\n"
    with tempfile.TemporaryDirectory() as d:
        with open(os.path.join(d, "t.c"), "w") as f:
            f.write(src)
        subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), os.path.join(d, "t.c"), "-o", os.path.join(d, "t")], check=True)
        return [int(v) for v in subprocess.run([os.path.join(d, "t")], check=True, stdout=subprocess.PIPE, text=True).stdout.split()]


def test_ctypes_mirrors_match_the_header():
    import jittorinfer_amd as J
    for cls, name in ((J.MlaRopeArgs, "mla_rope_args"), (J.MlaMulMatArgs, "mla_mul_mat_args"), (J.MlaCopyArgs, "mla_copy_args")):
        fields = [f[0] for f in cls._fields_]
        vals = _header_offsets(name, fields)
        assert vals[0] == C.sizeof(cls)
        assert vals[1:] == [getattr(cls, f).offset for f in fields]
