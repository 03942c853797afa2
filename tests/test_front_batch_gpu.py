"""GPU tests of the batched launch (mla_front_batch_launch, include/mla_front.h) and of the cache write with the rotary
embedding folded in (mla_kv_write_rope_launch, include/mla_kv_write.h).  Both restate work the library already does
launch by launch, with the same device code: the bar is bit-exact equality with the separate launches, which the tests of
the separate launches hold to the oracle; the folded cache write is also compared with the oracle's rope + cache write
directly (the rope to its stated tolerance before rounding means a cache value may differ by one unit in the last place
of the storage type, so that comparison counts mismatching bytes instead)."""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu
TYPES = [O.TYPE_BF16, O.TYPE_F16, O.TYPE_Q8_0]
ROPE = dict(n_dims=64, n_ctx_orig=4096, freq_scale=0.025, ext_factor=1.0, attn_factor=0.8)


def _t(gpu, a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a.view(np.int16) if a.dtype == np.uint16 else a)).to(gpu)


def _cache(rng, n_rows, kv_type):
    if kv_type == O.TYPE_Q8_0:
        return rng.integers(0, 256, size=(n_rows, 612), dtype=np.uint8)
    return rng.integers(0, 65536, size=(n_rows, 576), dtype=np.uint16)


def _layer_inputs(gpu, rng, B, H, kv_type):
    import torch
    n_pages = B * 3 + 2
    w = _t(gpu, O.f32_to_bf16(rng.standard_normal((H, 512, 128)).astype(np.float32) * 0.05))
    q = _t(gpu, rng.standard_normal((B, H, 192)).astype(np.float32))
    kv_new = _t(gpu, (rng.standard_normal((B, 576)) * 0.5).astype(np.float32))
    pos = _t(gpu, rng.integers(0, 128 * 3, size=B).astype(np.int32))
    bt = _t(gpu, rng.permutation(n_pages)[:B * 3].reshape(B, 3).astype(np.int32))
    seq_ids = torch.arange(B, dtype=torch.int32, device=gpu)
    cache = _t(gpu, _cache(rng, n_pages * 128, kv_type))
    return w, q, kv_new, pos, bt, seq_ids, cache


@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("B,H", [(32, 128), (5, 16), (1, 3)])
def test_the_nodes_ahead_of_the_attention_node_in_one_dispatch(gpu, kv_type, B, H):
    """rope(q_pe) into the Q rows, the absorb product into the Q rows, rope(k_pe) + cache write through the block table: one
    dispatch against four launches, every output bit for bit."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(7 + B)
    w, q, kv_new, pos, bt, seq_ids, cache = _layer_inputs(gpu, rng, B, H, kv_type)

    def run(batched):
        qs = torch.full((H, B, 576), float("nan"), dtype=torch.float32, device=gpu)
        c = cache.clone()
        kv = kv_new.clone()
        b = J.FrontBatch() if batched else None
        J.ggml_rope_ext(q[:, :, 128:], pos, out=qs[:, :, 512:].permute(1, 0, 2), batch=b, **ROPE)
        J.ggml_mul_mat(w, J.MLA_TYPE_BF16, q[:, :, :128].permute(1, 0, 2), out=qs[:, :, :512], batch=b)
        if batched:
            J.kv_write(kv, c, kv_type, block_table=bt, seq_ids=seq_ids, positions=pos, k_pe=kv[:, 512:], rope=dict(pos=pos, **ROPE), batch=b)
            b.launch(device=gpu)
        else:
            k_pe = kv[:, 512:].unsqueeze(1)
            J.ggml_rope_ext(k_pe, pos, out=k_pe, **ROPE)
            J.kv_write(kv, c, kv_type, block_table=bt, seq_ids=seq_ids, positions=pos)
        torch.cuda.synchronize()
        return qs.cpu().numpy(), c.cpu().numpy()

    q1, c1 = run(False)
    q2, c2 = run(True)
    assert not np.isnan(q1).any()
    assert np.array_equal(q1.view(np.uint32), q2.view(np.uint32))
    assert np.array_equal(c1, c2)
    assert not np.array_equal(c1, cache.cpu().numpy())


@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("mode", ["row0", "rows", "paged"])
def test_cache_write_with_the_rope_folded_in(gpu, kv_type, mode):
    """mla_kv_write_rope_launch on its own: equal to rope in place + cache write bit for bit, in every addressing mode, with
    frequency factors, from latent rows that hold only their 512 values, and close to the oracle's own rope + write."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(31)
    n_tok, n_rows = 77, 1024
    lat = (rng.standard_normal((n_tok, 512)) * 0.7).astype(np.float32)
    kpe = (rng.standard_normal((n_tok, 64)) * 2.0).astype(np.float32)
    pos = rng.integers(0, 160000, size=n_tok).astype(np.int32)
    ff = (1 + rng.random(32)).astype(np.float32)
    cache = _cache(rng, n_rows, kv_type)
    kw = {}
    if mode == "row0":
        kw["row0"], dest = 200, np.arange(200, 200 + n_tok)
    elif mode == "rows":
        dest = rng.permutation(n_rows)[:n_tok].astype(np.int64)
        kw["rows"] = _t(gpu, dest)
    else:
        bt = rng.permutation(8)[:8].reshape(2, 4).astype(np.int32)
        seq = rng.integers(0, 2, size=n_tok).astype(np.int32)
        p_in = np.concatenate([rng.permutation(512)[:(seq == s).sum()] for s in (0, 1)])   # distinct positions per sequence
        wpos = np.zeros(n_tok, dtype=np.int32)
        wpos[np.argsort(seq, kind="stable")] = p_in
        dest = bt[seq, wpos // 128] * 128 + wpos % 128
        kw.update(block_table=_t(gpu, bt), seq_ids=_t(gpu, seq), positions=_t(gpu, wpos))
    tpos, tff = _t(gpu, pos), _t(gpu, ff)
    rope = dict(ROPE, freq_factors=tff)
    # separate launches on rows of 576
    rows = _t(gpu, np.concatenate([lat, kpe], axis=1))
    c1 = _t(gpu, cache)
    k = rows[:, 512:].unsqueeze(1)
    J.ggml_rope_ext(k, tpos, out=k, **rope)
    J.kv_write(rows, c1, kv_type, **kw)
    # folded: latent rows of 512 values, k_pe a tensor of its own
    c2 = _t(gpu, cache)
    J.kv_write(_t(gpu, lat), c2, kv_type, k_pe=_t(gpu, kpe), rope=dict(pos=tpos, **rope), **kw)
    torch.cuda.synchronize()
    assert np.array_equal(c1.cpu().numpy(), c2.cpu().numpy())
    # against the oracle: the rotated values may sit one ulp of f32 away before they are rounded to the cache type
    p = O.rope_params(n_dims=64, mode=0, n_ctx_orig=4096, freq_scale=0.025, ext_factor=1.0, attn_factor=0.8)
    want_rows = np.concatenate([lat, O.rope(kpe[:, None, :], pos, p, ff)[:, 0, :]], axis=1)
    want = O.kv_write(want_rows, cache.copy(), kv_type, dest)
    got = c2.cpu().numpy()
    got = got.view(np.uint16) if cache.dtype == np.uint16 else got
    untouched = np.setdiff1d(np.arange(n_rows), dest)
    assert np.array_equal(got[untouched], cache[untouched])
    assert np.array_equal(got[dest][:, :(512 if cache.dtype == np.uint16 else 16 * 34)], want[dest][:, :(512 if cache.dtype == np.uint16 else 16 * 34)])
    frac = float(np.mean(got[dest] != want[dest]))
    assert frac < 2e-3, frac


def test_more_ops_than_one_dispatch_holds_and_shapes_without_a_batch_form(gpu):
    """Eleven independent ops (two dispatches) of every kind, among them a product of 100 rows per head, which has no form in
    the batch kernel and is launched on its own by the same call, an empty op, and copies with and without 16-byte
    alignment; every result equals that of the op launched alone."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(5)

    def inputs():
        d = {}
        d["w1"] = _t(gpu, O.f32_to_bf16(rng.standard_normal((16, 512, 128)).astype(np.float32) * 0.05))
        d["x1"] = _t(gpu, rng.standard_normal((16, 7, 128)).astype(np.float32))
        d["w2"] = _t(gpu, O.f32_to_f16(rng.standard_normal((16, 128, 512)).astype(np.float32) * 0.05))
        d["x2"] = _t(gpu, rng.standard_normal((16, 20, 512)).astype(np.float32))
        d["w3"] = _t(gpu, O.f32_to_bf16(rng.standard_normal((4, 512, 128)).astype(np.float32) * 0.05))
        d["x3"] = _t(gpu, rng.standard_normal((4, 100, 128)).astype(np.float32))
        d["r1"] = _t(gpu, rng.standard_normal((9, 3, 81)).astype(np.float32))
        d["p1"] = _t(gpu, (np.arange(9) * 1000).astype(np.int32))
        d["r2"] = _t(gpu, rng.standard_normal((40, 16, 64)).astype(np.float32))
        d["p2"] = _t(gpu, rng.integers(0, 9000, size=40).astype(np.int32))
        d["c1"] = _t(gpu, rng.standard_normal((6, 5, 48)).astype(np.float32))
        d["c2"] = _t(gpu, rng.standard_normal((3, 7, 33)).astype(np.float32))
        d["k1"] = _t(gpu, rng.standard_normal((50, 576)).astype(np.float32))
        d["k2"] = _t(gpu, _cache(rng, 20, O.TYPE_Q8_0))
        d["idx"] = _t(gpu, rng.permutation(256)[:50].astype(np.int32))
        d["idx2"] = _t(gpu, rng.permutation(256)[:20].astype(np.int64))
        d["cache_bf16"] = _t(gpu, _cache(rng, 256, O.TYPE_BF16))
        d["cache_f16"] = _t(gpu, _cache(rng, 256, O.TYPE_F16))
        d["cache_q8"] = _t(gpu, _cache(rng, 256, O.TYPE_Q8_0))
        d["cache_q8b"] = _t(gpu, _cache(rng, 256, O.TYPE_Q8_0))
        return d

    d = inputs()

    def run(b):
        o = {k: v.clone() for k, v in d.items() if k.startswith("cache")}
        o["m1"] = J.ggml_mul_mat(d["w1"], J.MLA_TYPE_BF16, d["x1"], batch=b)          # 128-wide tiles
        o["m2"] = J.ggml_mul_mat(d["w2"], J.MLA_TYPE_F16, d["x2"], batch=b)           # the K-split form
        o["m3"] = J.ggml_mul_mat(d["w3"], J.MLA_TYPE_BF16, d["x3"], batch=b)          # 100 rows: the streaming kernel, launched alone
        o["r1"] = J.ggml_rope_ext(d["r1"], d["p1"], n_dims=32, mode=2, freq_scale=0.25, ext_factor=1.0, batch=b)
        o["r2"] = J.ggml_rope_ext(d["r2"], d["p2"], n_dims=64, batch=b)
        o["c1"] = torch.zeros((6, 5, 64), dtype=torch.float32, device=gpu)
        J.copy_f32(d["c1"], o["c1"][:, :, 16:], batch=b)
        o["c2"] = torch.zeros((3, 7, 40), dtype=torch.float32, device=gpu)
        J.copy_f32(d["c2"], o["c2"][:, :, 3:36], batch=b)
        J.copy_f32(d["c2"][:0], o["c2"][:0, :, 3:36], batch=b)                        # nothing to do
        J.kv_write(d["k1"], o["cache_bf16"], J.MLA_TYPE_BF16, rows=d["idx"], batch=b)
        J.kv_write(d["k1"], o["cache_f16"], J.MLA_TYPE_F16, row0=100, batch=b)
        J.kv_write(d["k1"], o["cache_q8"], J.MLA_TYPE_Q8_0, rows=d["idx"], batch=b)
        J.kv_write(d["k2"], o["cache_q8b"], J.MLA_TYPE_Q8_0, rows=d["idx2"], batch=b)  # rows already Q8_0: copied
        if b is not None:
            assert len(b.ops) == 12
            b.launch(device=gpu)
        torch.cuda.synchronize()
        return {k: v.cpu().numpy() for k, v in o.items()}

    alone, batched = run(None), run(J.FrontBatch())
    for k in alone:
        assert np.array_equal(alone[k].view(np.uint8), batched[k].view(np.uint8)), k
    assert np.abs(alone["m3"]).max() > 0 and np.abs(alone["c2"]).max() > 0


def test_a_bad_op_stops_the_whole_batch(gpu):
    """Every op is checked before the first is launched: a batch with one refused op changes nothing."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(9)
    src = _t(gpu, rng.standard_normal((4, 8)).astype(np.float32))
    dst = torch.zeros((4, 8), dtype=torch.float32, device=gpu)
    b = J.FrontBatch()
    J.copy_f32(src, dst, batch=b)
    x = _t(gpu, rng.standard_normal((2, 1, 64)).astype(np.float32))
    J.ggml_rope_ext(x, _t(gpu, np.zeros(2, dtype=np.int32)), n_dims=64, mode=1, batch=b)   # mode 1 does not exist
    with pytest.raises(RuntimeError, match="-6"):
        b.launch(device=gpu)
    torch.cuda.synchronize()
    assert float(dst.abs().max()) == 0.0
