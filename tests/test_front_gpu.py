"""GPU parity of the nodes either side of the attention node (include/mla_front.h) against the oracle on the same seeded
inputs.  Tolerances (floating point, stated here):
  rotary embedding   max-abs 4e-6 * max|x| * mscale (the oracle's arithmetic is replayed operation by operation; only
                     cosf / sinf come from a different libm, about 1 ulp apart), channels past n_dims bit-exact
  absorb products    |got - want| <= 4e-6 * sum |a||b| per element (f32 accumulation order; inputs rounded identically)
  copies             bit-exact
"""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def _t(gpu, a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a.view(np.int16) if a.dtype == np.uint16 else a)).to(gpu)


def _rope_gpu(gpu, x, pos, p, ff=None, inplace=False):
    import torch
    import jittorinfer_amd as J
    tx = _t(gpu, x)
    out = tx if inplace else torch.full(x.shape, float("nan"), dtype=torch.float32, device=gpu)
    J.ggml_rope_ext(tx, _t(gpu, pos), n_dims=p.n_dims, mode=p.mode, n_ctx_orig=p.n_ctx_orig, freq_base=p.freq_base,
                    freq_scale=p.freq_scale, ext_factor=p.ext_factor, attn_factor=p.attn_factor, beta_fast=p.beta_fast,
                    beta_slow=p.beta_slow, freq_factors=None if ff is None else _t(gpu, ff), out=out)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def _check_rope(got, want, x, p):
    ms = abs(p.attn_factor) * (1 + 0.1 * np.log(1 / p.freq_scale) if p.ext_factor else 1.0)
    err = float(np.max(np.abs(got - want)))
    tol = 4e-6 * float(np.max(np.abs(x))) * ms
    assert err <= tol, "rope max-abs %.3g > %.3g" % (err, tol)
    return err


@pytest.mark.parametrize("mode", [0, 2])
@pytest.mark.parametrize("fs,ext,af", [(1.0, 0.0, 1.0), (0.025, 1.0, 0.8), (0.5, 0.25, 1.3)])
def test_rope_q_pe_shape(gpu, mode, fs, ext, af):
    """q_pe of a decode step: 32 tokens x 128 heads x 64, positions up to 160 k (DeepSeek's YaRN range)."""
    rng = np.random.default_rng(100 + mode)
    p = O.rope_params(n_dims=64, mode=mode, freq_scale=fs, ext_factor=ext, attn_factor=af, n_ctx_orig=4096)
    x = rng.standard_normal((32, 128, 64)).astype(np.float32)
    pos = rng.integers(0, 163840, size=32).astype(np.int32)
    print(_check_rope(_rope_gpu(gpu, x, pos, p), O.rope(x, pos, p), x, p))


def test_rope_k_pe_shape_in_place_and_many_tokens(gpu):
    """k_pe: one head, a prefill chunk of 2048 tokens; also rotated in place."""
    rng = np.random.default_rng(101)
    p = O.rope_params(freq_scale=0.025, ext_factor=1.0, attn_factor=0.8)
    x = rng.standard_normal((2048, 1, 64)).astype(np.float32)
    pos = (np.arange(2048) + 7000).astype(np.int32)
    want = O.rope(x, pos, p)
    _check_rope(_rope_gpu(gpu, x, pos, p), want, x, p)
    _check_rope(_rope_gpu(gpu, x, pos, p, inplace=True), want, x, p)


@pytest.mark.parametrize("mode", [0, 2])
def test_rope_partial_dims_freq_factors_odd_sizes(gpu, mode):
    rng = np.random.default_rng(102)
    p = O.rope_params(n_dims=32, mode=mode, freq_scale=0.25, ext_factor=1.0)
    x = rng.standard_normal((9, 3, 81)).astype(np.float32)     # odd row length: scalar path, 4-byte alignment only
    pos = (np.arange(9) * 1000).astype(np.int32)
    ff = (1 + rng.random(16)).astype(np.float32)
    got, want = _rope_gpu(gpu, x, pos, p, ff), O.rope(x, pos, p, ff)
    _check_rope(got, want, x, p)
    np.testing.assert_array_equal(got[..., 32:], x[..., 32:])


def test_rope_strided_source_view(gpu):
    """The q_pe view itself (rows of 64 inside rows of 192) without the ggml_cont in front of it."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(103)
    big = rng.standard_normal((17, 16, 192)).astype(np.float32)
    pos = rng.integers(0, 5000, size=17).astype(np.int32)
    p = O.rope_params()
    tb = _t(gpu, big)
    out = J.ggml_rope_ext(tb[:, :, 128:], _t(gpu, pos), n_dims=64, n_ctx_orig=4096)
    torch.cuda.synchronize()
    _check_rope(out.cpu().numpy(), O.rope(big[:, :, 128:], pos, p), big, p)


def _w(rng, shape, w_type, sigma=0.05):
    w = (rng.standard_normal(shape) * sigma).astype(np.float32)
    return O.f32_to_f16(w) if w_type == O.TYPE_F16 else O.f32_to_bf16(w)


def _check_mm(got, want, ab, what):
    err = float(np.max(np.abs(got - want) / np.maximum(ab, 1e-30)))
    assert err <= 4e-6, "%s: |err| / sum|a||b| = %.3g" % (what, err)
    return err


@pytest.mark.parametrize("w_type", [O.TYPE_BF16, O.TYPE_F16])
@pytest.mark.parametrize("K,N,M,H", [(128, 512, 32, 16), (512, 128, 32, 16), (128, 512, 1, 4), (512, 128, 33, 3),
                                     (128, 512, 130, 2), (64, 100, 70, 5), (16, 32, 5, 1), (528, 40, 64, 2), (256, 96, 100, 3), (512, 128, 321, 2)])
def test_mul_mat_shapes(gpu, w_type, K, N, M, H):
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(200 + K + N + M)
    w = _w(rng, (H, N, K), w_type, 0.3)
    x = rng.standard_normal((H, M, K)).astype(np.float32)
    out = torch.full((H, M, N), float("nan"), dtype=torch.float32, device=gpu)
    J.ggml_mul_mat(_t(gpu, w), w_type, _t(gpu, x), out=out)
    torch.cuda.synchronize()
    want, ab = O.mul_mat(w, w_type, x, with_abs=True)
    print(_check_mm(out.cpu().numpy(), want, ab, "mul_mat"))


def test_mul_mat_broadcast_weights_and_strided_rows(gpu):
    """src0 shared by groups of batches (r2 = 3), src1 a permuted view (q_nope of the reference's graph)."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(210)
    w = _w(rng, (2, 96, 128), O.TYPE_BF16, 0.3)
    q = rng.standard_normal((37, 6, 192)).astype(np.float32)
    tq = _t(gpu, q)
    out = J.ggml_mul_mat(_t(gpu, w), O.TYPE_BF16, tq[:, :, :128].permute(1, 0, 2))
    torch.cuda.synchronize()
    want, ab = O.mul_mat(w, O.TYPE_BF16, q[:, :, :128].transpose(1, 0, 2), with_abs=True)
    _check_mm(out.cpu().numpy(), want, ab, "broadcast / strided")


@pytest.mark.parametrize("w_type", [O.TYPE_BF16, O.TYPE_F16])
@pytest.mark.parametrize("n_tok", [1, 32, 200])
def test_query_side_and_output_side_of_the_attention_node(gpu, w_type, n_tok):
    """cont(q_pe) -> rope -> permute; permute(q_nope) x wk_b; concat; and wv_b x kqv -> permute -> cont, composed from
    the library's entry points the way the reference's graph composes the nodes (src/llama-graph-attn.cpp:264-277,
    :303-323), against the oracle's composition."""
    import torch
    import jittorinfer_amd as J
    H = 16
    rng = np.random.default_rng(300 + n_tok)
    wkv_b = _w(rng, (H * 256, 512), w_type)
    q = rng.standard_normal((n_tok, H * 192)).astype(np.float32)
    pos = rng.integers(0, 100000, size=n_tok).astype(np.int32)
    p = O.rope_params(freq_scale=0.025, ext_factor=1.0, attn_factor=0.8)
    tw, tq = _t(gpu, wkv_b).reshape(-1), _t(gpu, q).reshape(n_tok, H, 192)
    q_pe = torch.empty((n_tok, H, 64), dtype=torch.float32, device=gpu)
    J.copy_f32(tq[:, :, 128:], q_pe)                                                      # ggml_cont
    J.ggml_rope_ext(q_pe, _t(gpu, pos), n_dims=64, n_ctx_orig=4096, freq_scale=0.025, ext_factor=1.0, attn_factor=0.8, out=q_pe)
    q_states = torch.full((H, n_tok, 576), float("nan"), dtype=torch.float32, device=gpu)
    J.ggml_mul_mat(tw[:H * 512 * 128].reshape(H, 512, 128), w_type, tq[:, :, :128].permute(1, 0, 2), out=q_states[:, :, :512])
    J.copy_f32(q_pe.permute(1, 0, 2), q_states[:, :, 512:])                               # second half of ggml_concat
    torch.cuda.synchronize()
    want = O.mla_q_states(q, wkv_b, w_type, pos, p, H)
    got = q_states.cpu().numpy()
    assert float(np.max(np.abs(got[:, :, 512:] - want[:, :, 512:]))) <= 4e-6 * 6
    assert O.errors(got[:, :, :512], want[:, :, :512])[1] < 2e-6

    kqv = rng.standard_normal((H, n_tok, 512)).astype(np.float32)
    o = J.ggml_mul_mat(tw[H * 512 * 128:].reshape(H, 128, 512), w_type, _t(gpu, kqv))      # [H, n_tok, 128]
    cur = torch.full((n_tok, H, 128), float("nan"), dtype=torch.float32, device=gpu)
    J.copy_f32(o.permute(1, 0, 2), cur)                                                   # permute + ggml_cont_2d
    torch.cuda.synchronize()
    assert O.errors(cur.cpu().numpy().reshape(n_tok, H * 128), O.mla_unabsorb(kqv, wkv_b, w_type, H))[1] < 2e-6


def test_copy_f32_strided_both_sides_and_unaligned(gpu):
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(400)
    a = rng.standard_normal((3, 5, 7, 66)).astype(np.float32)
    ta = _t(gpu, a)
    dst = torch.zeros((3, 7, 5, 70), dtype=torch.float32, device=gpu)
    J.copy_f32(ta.permute(0, 2, 1, 3)[..., 1:64], dst[..., 3:66])     # 63 columns at odd offsets: scalar path
    J.copy_f32(ta.permute(0, 2, 1, 3)[..., :64], dst[..., :64].clone())  # aligned vector path, result discarded
    torch.cuda.synchronize()
    want = np.zeros((3, 7, 5, 70), np.float32)
    want[..., 3:66] = a.transpose(0, 2, 1, 3)[..., 1:64]
    np.testing.assert_array_equal(dst.cpu().numpy(), want)
    big = rng.standard_normal((64, 128, 576)).astype(np.float32)
    tb = _t(gpu, big)
    out = torch.empty((128, 64, 512), dtype=torch.float32, device=gpu)
    J.copy_f32(tb.permute(1, 0, 2)[..., :512], out)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), big.transpose(1, 0, 2)[..., :512])


def test_rejected_arguments(gpu):
    import ctypes as C
    import torch
    import jittorinfer_amd as J
    lib = J.library()
    x = torch.zeros((2, 2, 64), dtype=torch.float32, device=gpu)
    pos = torch.zeros(2, dtype=torch.int32, device=gpu)
    with pytest.raises(RuntimeError):
        J.ggml_rope_ext(x, pos, n_dims=63)                # odd
    with pytest.raises(RuntimeError):
        J.ggml_rope_ext(x, pos, n_dims=64, mode=8)        # mrope: not taken
    w = torch.zeros((1, 32, 24), dtype=torch.int16, device=gpu)
    with pytest.raises(RuntimeError):
        J.ggml_mul_mat(w, O.TYPE_BF16, torch.zeros((1, 4, 24), dtype=torch.float32, device=gpu))   # K % 16 != 0
    assert lib.mla_rope_launch(None, None) == -5 and lib.mla_mul_mat_launch(None, None) == -5 and lib.mla_copy_f32_launch(None, None) == -5


def test_query_side_in_two_launches_through_the_strides(gpu):
    """The byte strides of both entry points take the reference's views as they are: rope reads the q_pe view inside q and
    writes the last 64 columns of q_states, the product reads the permuted q_nope view and writes the first 512: two
    launches produce what cont + rope + permute + mul_mat + concat produce."""
    import torch
    import jittorinfer_amd as J
    H, n_tok = 16, 40
    rng = np.random.default_rng(600)
    wkv_b = _w(rng, (H * 256, 512), O.TYPE_BF16)
    q = rng.standard_normal((n_tok, H * 192)).astype(np.float32)
    pos = rng.integers(0, 100000, size=n_tok).astype(np.int32)
    p = O.rope_params(freq_scale=0.025, ext_factor=1.0, attn_factor=0.8)
    tw, tq = _t(gpu, wkv_b).reshape(-1), _t(gpu, q).reshape(n_tok, H, 192)
    q_states = torch.full((H, n_tok, 576), float("nan"), dtype=torch.float32, device=gpu)
    J.ggml_rope_ext(tq[:, :, 128:], _t(gpu, pos), n_dims=64, n_ctx_orig=4096, freq_scale=0.025, ext_factor=1.0, attn_factor=0.8,
                    out=q_states[:, :, 512:].permute(1, 0, 2))
    J.ggml_mul_mat(tw[:H * 512 * 128].reshape(H, 512, 128), O.TYPE_BF16, tq[:, :, :128].permute(1, 0, 2), out=q_states[:, :, :512])
    torch.cuda.synchronize()
    want = O.mla_q_states(q, wkv_b, O.TYPE_BF16, pos, p, H)
    got = q_states.cpu().numpy()
    assert float(np.max(np.abs(got[:, :, 512:] - want[:, :, 512:]))) <= 4e-6 * 6
    assert O.errors(got[:, :, :512], want[:, :, :512])[1] < 2e-6
