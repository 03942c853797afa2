"""GPU parity of the KV cache write (include/mla_kv_write.h) against the oracle: bit-exact cache contents."""
import os

import numpy as np
import pytest

from oracle import oracle as O
from tests import util as U

pytestmark = pytest.mark.gpu
TYPES = [O.TYPE_BF16, O.TYPE_F16, O.TYPE_Q8_0]


def _cache(rng, n_rows, kv_type):
    if kv_type == O.TYPE_Q8_0:
        return rng.integers(0, 256, size=(n_rows, 612), dtype=np.uint8)
    return rng.integers(0, 65536, size=(n_rows, 576), dtype=np.uint16)


def _to_gpu(gpu, a):
    import torch
    return torch.from_numpy(a.view(np.int16) if a.dtype == np.uint16 else a).to(gpu)


def _back(t, like):
    a = t.cpu().numpy()
    return a.view(np.uint16) if like.dtype == np.uint16 else a


@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("n_tok,row0", [(1, 0), (3, 125), (700, 11)])
def test_consecutive_rows(gpu, kv_type, n_tok, row0):
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(100 + n_tok)
    cache = _cache(rng, 1024, kv_type)
    x = (rng.standard_normal((n_tok, 576)) * rng.choice([1e-4, 1.0, 300.0], size=(n_tok, 1))).astype(np.float32)
    x[0, 32:64] = 0.0
    tc = _to_gpu(gpu, cache)
    J.kv_write(torch.from_numpy(x).to(gpu), tc, kv_type, row0=row0)
    torch.cuda.synchronize()
    want = O.kv_write(x, cache.copy(), kv_type, np.arange(row0, row0 + n_tok))
    assert np.array_equal(_back(tc, cache), want)


@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("idx_dtype", ["int32", "int64"])
def test_scatter_rows_converting_and_raw(gpu, kv_type, idx_dtype):
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(200)
    cache = _cache(rng, 512, kv_type)
    dest = rng.permutation(512)[:90].astype(idx_dtype)
    x = rng.standard_normal((90, 576)).astype(np.float32)
    tc = _to_gpu(gpu, cache)
    J.kv_write(torch.from_numpy(x).to(gpu), tc, kv_type, rows=torch.from_numpy(dest).to(gpu))
    torch.cuda.synchronize()
    want = O.kv_write(x, cache.copy(), kv_type, dest)
    assert np.array_equal(_back(tc, cache), want)
    # rows already in the cache type: ggml_scatter_update's plain row copy
    raw = _cache(rng, 90, kv_type)
    J.kv_write(_to_gpu(gpu, raw), tc, kv_type, rows=torch.from_numpy(dest).to(gpu))
    torch.cuda.synchronize()
    want = O.kv_write(raw, want, kv_type, dest, src_type=kv_type)
    assert np.array_equal(_back(tc, cache), want)


@pytest.mark.parametrize("kv_type", TYPES)
def test_paged_write_then_attention(gpu, kv_type):
    """Tokens of 3 sequences written through the block table in arrival order, then read back by the attention kernel:
    the cache bytes equal the oracle's, and attention over the written cache equals attention over the same rows."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(300)
    lens = [200, 77, 131]
    n_pages = 8
    bt = rng.permutation(n_pages)[:6].astype(np.int32).reshape(3, 2)
    seq_ids = np.concatenate([np.full(l, b, dtype=np.int32) for b, l in enumerate(lens)])
    positions = np.concatenate([np.arange(l, dtype=np.int32) for l in lens])
    order = rng.permutation(len(seq_ids))
    seq_ids, positions = seq_ids[order], positions[order]
    x = rng.standard_normal((len(seq_ids), 576)).astype(np.float32)
    cache = _cache(rng, n_pages * 128, kv_type)
    if kv_type == O.TYPE_Q8_0:
        cache[:] = O.quantize_q8_0((rng.standard_normal((n_pages * 128, 576)) * 50).astype(np.float32), 1)   # finite garbage
    else:
        cache[:] = U.encode_kv((rng.standard_normal((n_pages * 128, 576)) * 50).astype(np.float32), kv_type)
    tc = _to_gpu(gpu, cache)
    J.kv_write(torch.from_numpy(x).to(gpu), tc, kv_type, block_table=torch.from_numpy(bt).to(gpu),
               seq_ids=torch.from_numpy(seq_ids).to(gpu), positions=torch.from_numpy(positions).to(gpu))
    torch.cuda.synchronize()
    dest = bt[seq_ids, positions // 128].astype(np.int64) * 128 + positions % 128
    want = O.kv_write(x, cache.copy(), kv_type, dest)
    got = _back(tc, cache)
    assert np.array_equal(got, want)
    # attention over the written pages
    q = rng.standard_normal((3, 16, 1, 576)).astype(np.float32)
    out = torch.full((3, 1, 16, 576), float("nan"), dtype=torch.float32, device=gpu)
    J.ggml_flash_attn_ext(torch.from_numpy(q).to(gpu), tc, kv_type, dv=512, scale=U.SCALE, block_table=torch.from_numpy(bt).to(gpu),
                          seq_lens=torch.tensor(lens, dtype=torch.int32, device=gpu), out=out)
    torch.cuda.synchronize()
    seqs = []
    for b, l in enumerate(lens):
        rows = bt[b, np.arange(l) // 128].astype(np.int64) * 128 + np.arange(l) % 128
        seqs.append(want[rows])
    if kv_type == O.TYPE_F16:
        ref = np.stack([O.flash_attn_ext_f64(q[b:b + 1], k[None], kv_type, dv=512, scale=U.SCALE)[0] for b, k in enumerate(seqs)])
    else:
        ref = U.oracle_per_seq(q, seqs, kv_type, 512)
    print(U.check(out.cpu().numpy()[..., :512], ref, "attention over written pages"))


@pytest.mark.skipif(not O.ref_available(), reason="oracle/_ref is not built")
@pytest.mark.parametrize("kv_type", TYPES)
def test_reference_ggml_drives_the_cpy_node(gpu, kv_type):
    """The reference's own compiled ggml loads the plugin (ggml_backend_load) and computes llm_attn_mla's cache write
    (ggml_cpy into a view of the cache) on it; the cache bytes equal what ggml-cpu writes for the same node."""
    import jittorinfer_amd as J
    rng = np.random.default_rng(400)
    cache = _cache(rng, 256, kv_type)
    x = rng.standard_normal((33, 576)).astype(np.float32)
    want = O.ref_kv_cpy(x, cache.copy(), kv_type, 70)
    got, info = O.ref_backend_kv_cpy(J.library_path(), x, cache.copy(), kv_type, 70)
    assert "HIP-MLA" in info
    assert np.array_equal(got, want)
