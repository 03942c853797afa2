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


@pytest.mark.parametrize("n_head,n_tok", [(48, 1), (16, 2), (128, 1)])
@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_Q8_0])
def test_node_with_alibi_and_soft_cap(gpu, k_type, n_head, n_tok):
    """max_bias and logit_softcap travel in the node's op_params (ggml.c:4024-4030): the same node, with a mask of finite biases, on
    ggml-cpu and on the plugin -- 48 heads (a row block with idle waves), 16 heads x 2 tokens, 128 heads; bf16 and Q8_0 cells (block
    scale 1/32: the f16 operands of the fast Q8_0 path are exact there)."""
    rng = np.random.default_rng(23)
    q = rng.standard_normal((2, n_head, n_tok, 576)).astype(np.float32)
    k = U.encode_kv(rng.standard_normal((2, 224, 576)).astype(np.float32), k_type, q8_scale=1.0 / 32 if k_type == O.TYPE_Q8_0 else None)
    m = rng.standard_normal((n_tok, 224)).astype(np.float32)
    m[rng.random((n_tok, 224)) < 0.3] = -np.inf
    m[:, 0] = 0
    mask = m.astype(np.float16).view(np.uint16)
    for max_bias, softcap in ((8.0, 0.0), (0.0, 30.0), (4.0, 12.0)):
        got, info = O.ref_backend_flash_attn_ext(_so(), q, k, k_type, dv=576, mask=mask, scale=U.SCALE, max_bias=max_bias, softcap=softcap, use_sched=True)
        assert "HIP-MLA" in info and "HIPMLA0" in info
        cpu = O.ref_flash_attn_ext(q, k, k_type, mask=mask, scale=U.SCALE, max_bias=max_bias, softcap=softcap)
        print(max_bias, softcap, U.check(got, cpu, "plugin vs ggml-cpu, max_bias %g softcap %g" % (max_bias, softcap)))


def test_latent_prefix_view_and_block_table(gpu):
    """The MLA form: V is a 512-wide view of K, K is the page pool, src[4]/src[5] carry the block table and lengths."""
    rng = np.random.default_rng(22)
    lens = [300, 1, 128, 515]
    pool, bt, seqs = U.make_paged(rng, lens, O.TYPE_BF16, n_pool_pages=16)
    q = rng.standard_normal((4, 128, 1, 576)).astype(np.float32)
    got, info = O.ref_backend_flash_attn_ext(_so(), q, pool, O.TYPE_BF16, dv=512, block_table=bt, seq_lens=lens, scale=U.SCALE, use_sched=True)
    want = U.oracle_per_seq(q, seqs, O.TYPE_BF16, 512)
    print(U.check(got[..., :512], want, "paged node through the scheduler"))


def test_f16_cache_with_the_reference_accumulator_on_request(gpu, monkeypatch):
    """F16 KV: ggml-cpu accumulates V in f16 and lands 4e-3 from the exact value; the plugin accumulates in f32 unless
    the backend is initialised with f16_acc=strict (here through the environment), and then replays the reference's
    accumulator: only that mode agrees with ggml-cpu to the tolerance."""
    rng = np.random.default_rng(31)
    q = rng.standard_normal((1, 16, 1, 576)).astype(np.float32)
    k = U.encode_kv(rng.standard_normal((1, 1024, 576)).astype(np.float32), O.TYPE_F16)
    cpu = O.ref_flash_attn_ext(q, k, O.TYPE_F16, scale=U.SCALE)
    fast, _ = O.ref_backend_flash_attn_ext(_so(), q, k, O.TYPE_F16, dv=576, scale=U.SCALE)
    monkeypatch.setenv("GGML_HIP_MLA_F16_ACC", "strict")
    strict, _ = O.ref_backend_flash_attn_ext(_so(), q, k, O.TYPE_F16, dv=576, scale=U.SCALE)
    e_fast, e_strict = O.errors(fast, cpu), O.errors(strict, cpu)
    print("vs ggml-cpu: f32 accumulation", e_fast, "replay", e_strict)
    U.check(strict, cpu, "strict replay vs ggml-cpu")
    # the numbers include/ggml_mla_backend.h states for the default: outside the tolerance against ggml-cpu's fused node
    # because that node is 3.9e-3 from the exact value of the same rounded inputs, and the default is 2e-4 from it (the probabilities meet V as f16)
    exact = O.flash_attn_ext_f64(q, k, O.TYPE_F16, dv=576, scale=U.SCALE)
    e_cpu_exact, e_fast_exact = O.errors(cpu, exact), O.errors(fast, exact)
    print("vs the exact value: ggml-cpu", e_cpu_exact, "default", e_fast_exact)
    assert 2e-3 < e_fast[1] < 6e-3 and 2e-3 < e_cpu_exact[1] < 6e-3 and e_fast_exact[1] < 3e-4
    assert e_strict[1] < 0.5 * e_fast[1]


def test_q8_0_cache_with_the_reference_arithmetic_on_request(gpu, monkeypatch):
    """Q8_0 KV with block scales of their own (a real quantization of N(0, 3) rows) and a mask that leaves every query token three
    keys: the matrix-core operands (q * d rounded to f16) show in single elements, the documented deviation of the default path; a
    backend initialised with q8=exact (here through the environment) runs ggml-cpu's own arithmetic and agrees with the reference's
    compiled node to 1e-5.  Both against ggml-cpu itself (oracle/_ref), through the plugin interface."""
    rng = np.random.default_rng(33)
    n_tok, n_kv = 4, 1024
    q = (rng.standard_normal((1, 16, n_tok, 576)) * 2).astype(np.float32)
    k = U.encode_kv((rng.standard_normal((1, n_kv, 576)) * 3).astype(np.float32), O.TYPE_Q8_0)
    m = np.full((n_tok, n_kv), -np.inf, np.float32)
    for t in range(n_tok):
        m[t, rng.choice(n_kv, 3, replace=False)] = 0.0
    mask = m.astype(np.float16).view(np.uint16)
    cpu = O.ref_flash_attn_ext(q, k, O.TYPE_Q8_0, mask=mask, scale=U.SCALE)
    fast, _ = O.ref_backend_flash_attn_ext(_so(), q, k, O.TYPE_Q8_0, dv=576, mask=mask, scale=U.SCALE)
    monkeypatch.setenv("GGML_HIP_MLA_Q8", "exact")
    exact, _ = O.ref_backend_flash_attn_ext(_so(), q, k, O.TYPE_Q8_0, dv=576, mask=mask, scale=U.SCALE)
    e_fast, e_exact = O.errors(fast, cpu), O.errors(exact, cpu)
    print("vs ggml-cpu: matrix-core operands", e_fast, "reference arithmetic", e_exact)
    # (the default path on this input: queries of N(0, 2) against rows of N(0, 3) put the logits of the three open keys tens of units
    # apart, and a logit moved by 1e-3 of its size moves the probabilities of keys whose V values differ by up to 20: 3e-2 in single
    # elements at 7e-4 rel-L2 -- the deviation include/ggml_mla_backend.h documents, at its worst)
    U.check(fast, cpu, "Q8_0 default vs ggml-cpu", max_abs=0.1)
    U.check(exact, cpu, "Q8_0 exact vs ggml-cpu", max_abs=2e-5, rel_l2=1e-5)
    assert e_exact[0] < 0.05 * e_fast[0]


@pytest.mark.parametrize("paged", [False, True])
def test_scheduler_set_up_as_llama_sets_it_up(gpu, paged):
    """The scheduler as the reference's context builds it (src/llama-context-load-utils.cpp:108-131): the CPU backend's
    compute buffer in the device's pinned host buffer type, pipeline parallelism on (four copies of the inputs ordered
    by the plugin's events), Q produced by a CPU op and the result consumed by one.  Three asynchronous computes in a row
    (Q, then 2Q with half the softmax scale, which the driver checks to be bit-identical, then Q again)."""
    rng = np.random.default_rng(29)
    if paged:
        lens = [300, 1, 128, 515]
        pool, bt, seqs = U.make_paged(rng, lens, O.TYPE_BF16, n_pool_pages=16)
        q = rng.standard_normal((4, 128, 1, 576)).astype(np.float32)
        got, info = O.ref_backend_flash_attn_ext(_so(), q, pool, O.TYPE_BF16, dv=512, block_table=bt, seq_lens=lens, scale=U.SCALE, use_sched=2)
        want = U.oracle_per_seq(q, seqs, O.TYPE_BF16, 512)
    else:
        q = rng.standard_normal((2, 16, 2, 576)).astype(np.float32)
        k = U.encode_kv(rng.standard_normal((2, 200, 576)).astype(np.float32), O.TYPE_BF16)
        mask = np.where(rng.random((2, 200)) < 0.2, -np.inf, 0.0).astype(np.float16)
        mask[:, 0] = 0
        mask = mask.view(np.uint16)
        got, info = O.ref_backend_flash_attn_ext(_so(), q, k, O.TYPE_BF16, dv=512, mask=mask, scale=U.SCALE, use_sched=2)
        want = O.flash_attn_ext(q, k, O.TYPE_BF16, dv=512, mask=mask, scale=U.SCALE)
    assert "host_buft=HIPMLA0_Host" in info
    print(info, U.check(got[..., :512], want[..., :512], "llama-style scheduler"))


@pytest.mark.parametrize("use_sched", [False, True])
@pytest.mark.parametrize("n_head", [128, 16])
def test_batched_decode_through_the_mask_as_llama_builds_it(gpu, use_sched, n_head):
    """The reference's decode batch: one shared cache, one query token per sequence, the f16 mask padded to 64 rows selects
    each token's own cells (src/llama-context.cpp:364-404); V is the 512-wide latent prefix view of K.  The reference's
    compiled ggml drives the plugin; the pipelined masked kernel computes the node (16 heads: issued as row blocks and token
    by token, the device runs the token form)."""
    rng = np.random.default_rng(23 + n_head)
    n_kv, lens = 1024, [200, 256, 31, 300]
    k = U.encode_kv(rng.standard_normal((1, n_kv, 576)).astype(np.float32), O.TYPE_BF16)
    m = np.full((len(lens), n_kv), -np.inf, dtype=np.float32)
    pos = 0
    for s, l in enumerate(lens):
        m[s, pos:pos + l] = 0.0
        pos += l + 20
    mask = m.astype(np.float16).view(np.uint16)
    q = rng.standard_normal((1, n_head, len(lens), 576)).astype(np.float32)
    got, info = O.ref_backend_flash_attn_ext(_so(), q, k, O.TYPE_BF16, dv=512, mask=mask, scale=U.SCALE, use_sched=use_sched)
    want = O.flash_attn_ext(q, k, O.TYPE_BF16, dv=512, mask=mask, scale=U.SCALE)
    print(U.check(got[..., :512], want, "masked batched decode through the reference's ggml"))


@pytest.mark.parametrize("n_head", [128, 16])
@pytest.mark.parametrize("rescan", [False, True])
def test_two_attention_nodes_of_one_graph_share_the_mask(gpu, monkeypatch, n_head, rescan):
    """The layers of one llama graph share their mask tensor: the second attention node of a graph finds the key extents of the
    mask in the plugin's workspace, left there by the first, and leaves out the scan (GGML_HIP_MLA_MASK_EXTENTS=rescan: every
    node scans for itself).  Two nodes over one cache and one mask with different queries, both against the oracle; then the
    same graph with another mask -- the extents of the first graph must not survive into the second call."""
    if rescan:
        monkeypatch.setenv("GGML_HIP_MLA_MASK_EXTENTS", "rescan")
    import ctypes
    lib = ctypes.CDLL(_so())
    lib.mla_ggml_mask_extent_reuses.restype = ctypes.c_int64
    before = lib.mla_ggml_mask_extent_reuses()
    rng = np.random.default_rng(61 + n_head)
    n_kv, lens = 1536, [300, 512, 77, 400]
    k = U.encode_kv(rng.standard_normal((1, n_kv, 576)).astype(np.float32), O.TYPE_BF16)
    qa = rng.standard_normal((1, n_head, len(lens), 576)).astype(np.float32)
    qb = rng.standard_normal((1, n_head, len(lens), 576)).astype(np.float32)
    for shift in (0, 40):                       # the second graph: every sequence sits 40 cells further on
        m = np.full((len(lens), n_kv), -np.inf, dtype=np.float32)
        pos = shift
        for s, l in enumerate(lens):
            m[s, pos:pos + l] = 0.0
            pos += l + 20
        mask = m.astype(np.float16).view(np.uint16)
        got_a, got_b, info = O.ref_backend_flash_attn_ext(_so(), qa, k, O.TYPE_BF16, dv=512, mask=mask, scale=U.SCALE, q_second=qb)
        print(U.check(got_a[..., :512], O.flash_attn_ext(qa, k, O.TYPE_BF16, dv=512, mask=mask, scale=U.SCALE), "first node, shift %d" % shift))
        print(U.check(got_b[..., :512], O.flash_attn_ext(qb, k, O.TYPE_BF16, dv=512, mask=mask, scale=U.SCALE), "second node, shift %d" % shift))
    assert lib.mla_ggml_mask_extent_reuses() - before == (0 if rescan else 2)    # the second node of each of the two graphs


@pytest.mark.parametrize("w_type", [O.TYPE_BF16, O.TYPE_F16])
@pytest.mark.parametrize("n_tok", [1, 32, 150])
def test_query_side_and_output_side_graphs_through_the_plugin(gpu, w_type, n_tok):
    """The sub-graphs llm_attn_mla builds before and after the attention node (views of q, CONT, ROPE, PERMUTE, MUL_MAT
    with the wk_b / wv_b views of wkv_b, CONCAT, CONT_2D), built by the reference's own ggml and computed node by node
    by the plugin; the same graphs on the reference's ggml-cpu are the expected values.
    Tolerances: the rope columns 4e-6 * max|x| * mscale, the products 2e-6 relative L2 (f32 accumulation order)."""
    H = 16
    rng = np.random.default_rng(500 + n_tok)
    w = (rng.standard_normal((H * 256, 512)) * 0.05).astype(np.float32)
    wkv_b = O.f32_to_f16(w) if w_type == O.TYPE_F16 else O.f32_to_bf16(w)
    q = rng.standard_normal((n_tok, H * 192)).astype(np.float32)
    pos = rng.integers(0, 100000, size=n_tok).astype(np.int32)
    p = O.rope_params(freq_scale=0.025, ext_factor=1.0, attn_factor=0.8)
    got = O.ref_mla_q_states(q, wkv_b, w_type, pos, p, H, so_path=_so())
    cpu = O.ref_mla_q_states(q, wkv_b, w_type, pos, p, H)
    assert not np.isnan(got).any()
    assert float(np.max(np.abs(got[:, :, 512:] - cpu[:, :, 512:]))) <= 4e-6 * 6
    assert O.errors(got[:, :, :512], cpu[:, :, :512])[1] < 2e-6
    assert O.errors(got, O.mla_q_states(q, wkv_b, w_type, pos, p, H))[1] < 2e-6
    kqv = rng.standard_normal((H, n_tok, 512)).astype(np.float32)
    got = O.ref_mla_unabsorb(kqv, wkv_b, w_type, H, so_path=_so())
    assert O.errors(got, O.ref_mla_unabsorb(kqv, wkv_b, w_type, H))[1] < 2e-6


@pytest.mark.parametrize("mode", [0, 2])
def test_rope_node_through_the_plugin(gpu, mode):
    rng = np.random.default_rng(510)
    p = O.rope_params(n_dims=32, mode=mode, freq_scale=0.25, ext_factor=1.0)
    x = rng.standard_normal((9, 3, 80)).astype(np.float32)
    pos = (np.arange(9) * 1000).astype(np.int32)
    ff = (1 + rng.random(16)).astype(np.float32)
    got = O.ref_rope(x, pos, p, ff, so_path=_so())
    assert float(np.max(np.abs(got - O.ref_rope(x, pos, p, ff)))) <= 4e-6 * 6 * 1.2
    np.testing.assert_array_equal(got[..., 32:], x[..., 32:])


def test_mul_mat_node_the_plugin_leaves_to_other_backends(gpu):
    """An F32 src0, or a BF16 product that is not one of the layer's two per-head products, is not taken (supports_op false
    -> the driver reports the node index); nothing is computed wrongly."""
    rng = np.random.default_rng(520)
    a = rng.standard_normal((2, 512, 128)).astype(np.float32)
    b = rng.standard_normal((2, 5, 128)).astype(np.float32)
    with pytest.raises(RuntimeError, match="-100"):
        O.ref_mul_mat(a, O.TYPE_F32, b, so_path=_so())
    with pytest.raises(RuntimeError, match="-100"):
        O.ref_mul_mat(O.f32_to_bf16(a[:, :32, :64].copy()), O.TYPE_BF16, b[:, :, :64].copy(), so_path=_so())
    w = O.f32_to_bf16(a)
    got = O.ref_mul_mat(w, O.TYPE_BF16, b, so_path=_so())
    assert O.errors(got, O.ref_mul_mat(w, O.TYPE_BF16, b))[1] < 2e-6
