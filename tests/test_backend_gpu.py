"""The ggml backend plugin driven the way the reference drives a backend: loaded with ggml_backend_load by the
reference's own compiled ggml (oracle/_ref), buffers from its buffer type, the node built by ggml_flash_attn_ext,
computed with ggml_backend_graph_compute and through ggml_backend_sched next to the CPU backend.  Results are
compared with the oracle.  Needs oracle/_ref (built in the build container; it travels with the tree)."""
import numpy as np
import pytest

from oracle import oracle as O
from tests import util as U

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not O.ref_available(), reason="oracle/_ref is not built")]


def _so():
    import jittorinfer_amd as J
    return J.library_path()


@pytest.mark.parametrize("use_sched", [False, True])
@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_Q8_0])
def test_node_as_ggml_cpu_accepts_it(gpu, k_type, use_sched):
    """V := K (576 wide): the same node runs on ggml-cpu and on the plugin; outputs agree in every column."""
    rng = np.random.default_rng(21)
    q = rng.standard_normal((2, 16, 2, 576)).astype(np.float32)
    k = U.encode_kv(rng.standard_normal((2, 200, 576)).astype(np.float32), k_type)
    mask = np.where(rng.random((2, 200)) < 0.2, -np.inf, 0.0).astype(np.float16)
    mask[:, 0] = 0
    mask = mask.view(np.uint16)
    got, info = O.ref_backend_flash_attn_ext(_so(), q, k, k_type, dv=576, mask=mask, scale=U.SCALE, use_sched=use_sched)
    assert "HIP-MLA" in info and "HIPMLA0" in info
    cpu = O.ref_flash_attn_ext(q, k, k_type, mask=mask, scale=U.SCALE)
    print(info, U.check(got, cpu, "plugin vs ggml-cpu"))


def test_latent_prefix_view_and_block_table(gpu):
    """The MLA form: V is a 512-wide view of K, K is the page pool, src[4]/src[5] carry the block table and lengths."""
    rng = np.random.default_rng(22)
    lens = [300, 1, 128, 515]
    pool, bt, seqs = U.make_paged(rng, lens, O.TYPE_BF16, n_pool_pages=16)
    q = rng.standard_normal((4, 128, 1, 576)).astype(np.float32)
    got, info = O.ref_backend_flash_attn_ext(_so(), q, pool, O.TYPE_BF16, dv=512, block_table=bt, seq_lens=lens, scale=U.SCALE, use_sched=True)
    want = U.oracle_per_seq(q, seqs, O.TYPE_BF16, 512)
    print(U.check(got[..., :512], want, "paged node through the scheduler"))


@pytest.mark.parametrize("use_sched", [False, True])
def test_batched_decode_through_the_mask_as_llama_builds_it(gpu, use_sched):
    """The reference's decode batch: one shared cache, one query token per sequence, the f16 mask padded to 64 rows selects
    each token's own cells (src/llama-context.cpp:364-404); V is the 512-wide latent prefix view of K.  The reference's
    compiled ggml drives the plugin; the pipelined masked kernel computes the node."""
    rng = np.random.default_rng(23)
    n_kv, lens = 1024, [200, 256, 31, 300]
    k = U.encode_kv(rng.standard_normal((1, n_kv, 576)).astype(np.float32), O.TYPE_BF16)
    m = np.full((len(lens), n_kv), -np.inf, dtype=np.float32)
    pos = 0
    for s, l in enumerate(lens):
        m[s, pos:pos + l] = 0.0
        pos += l + 20
    mask = m.astype(np.float16).view(np.uint16)
    q = rng.standard_normal((1, 128, len(lens), 576)).astype(np.float32)
    got, info = O.ref_backend_flash_attn_ext(_so(), q, k, O.TYPE_BF16, dv=512, mask=mask, scale=U.SCALE, use_sched=use_sched)
    want = O.flash_attn_ext(q, k, O.TYPE_BF16, dv=512, mask=mask, scale=U.SCALE)
    print(U.check(got[..., :512], want, "masked batched decode through the reference's ggml"))
