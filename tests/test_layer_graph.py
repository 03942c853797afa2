"""The one-node form of the MLA attention layer against the graph the reference really emits.

llm_attn_mla (src/llama-graph-attn.cpp:233-323) does not build a FLASH_ATTN_EXT node: it copies the new rows into a K cache
and, transposed, into a V cache, and runs mul_mat(k, q) -> soft_max_ext(mask, kq_scale) -> mul_mat(v, kq) -> wv_b.  The plugin
accelerates the one-node form (q_states -> cache write -> flash_attn_ext over ONE latent cache -> wv_b).  oracle/ref_driver.c
builds both with the reference's own ggml: the unfused graph runs on its ggml-cpu, the one-node graph on the plugin under
ggml_backend_sched; the same seeded steps (a prefill, two decode tokens, a chunk of five) go through both.

What the comparison has to allow for, from the reference's side: its mul_mat rounds the f32 operand to the cache's
vec_dot type (ggml-cpu.c:7467-7545), so the probabilities are rounded to f16 before they meet the F16 V cache (2^-11
relative, inside the tolerance), and with a BF16 V cache they would be rounded to bf16 (2^-9, outside it) -- the V cache
of the unfused side is therefore F16 in every case, which is also what a Q8_0 K cache forces there (a transposed cache
cannot hold 32-value blocks).  The new rows are drawn so that both caches hold the same V values: bf16-exact values for
BF16 / F16 caches, and for Q8_0 latents on a power-of-two grid with a full-scale value in every block, which Q8_0 and
F16 both store exactly.  The 64 rope columns are unrestricted.  kv_b is an F16 weight: mul_mat rounds the attention
result to the weight's type before the un-absorb product, and with a BF16 weight a result that differs in the last f32
bits can round to the neighbouring bf16 value (2^-8), which would measure the weight format and not the node.
"""
import numpy as np
import pytest

from oracle import oracle as O
from tests import util as U

needs_ref = pytest.mark.skipif(not O.ref_available(), reason="oracle/_ref (the reference's compiled ggml) is not built")
STEPS = (70, 1, 1, 5)
N_CTX = 256
W_TYPE = O.TYPE_F16   # kv_b as an F16 weight: the un-absorb product rounds the node's output to the weight's type on both sides


def _so():
    import jittorinfer_amd as J
    return J.library_path()


def _inputs(seed, k_type, n_head, steps=STEPS):
    rng = np.random.default_rng(seed)
    wkv_b = O.f32_to_f16((rng.standard_normal((n_head * 256, 512)) * 0.03).astype(np.float32))
    out = []
    for n in steps:
        q = rng.standard_normal((n, n_head, 192)).astype(np.float32)
        kv = rng.standard_normal((n, 576)).astype(np.float32)
        if k_type == O.TYPE_Q8_0:
            ints = rng.integers(-127, 128, size=(n, 16, 32))
            ints[np.arange(n)[:, None], np.arange(16)[None, :], rng.integers(0, 32, size=(n, 16))] = 127
            kv[:, :512] = (ints * 2.0 ** -6).reshape(n, 512)
        else:
            kv = O.bf16_to_f32(O.f32_to_bf16(kv))
        out.append((q, kv))
    return wkv_b, out


def _oracle_one_node(k_type, n_head, wkv_b, steps, node=O.flash_attn_ext):
    """The one-node form from the oracle's own pieces (cache write, absorb product, attention node, un-absorb product)."""
    cache = np.zeros((N_CTX, 612), np.uint8) if k_type == O.TYPE_Q8_0 else np.zeros((N_CTX, 576), np.uint16)
    wk_b = wkv_b.reshape(-1)[:n_head * 512 * 128].reshape(n_head, 512, 128)
    head, outs = 0, []
    for q, kv in steps:
        n = q.shape[0]
        O.kv_write(kv, cache, k_type, np.arange(head, head + n))
        q_abs = O.mul_mat(wk_b, W_TYPE, q[:, :, :128].transpose(1, 0, 2))
        q_states = np.concatenate([q_abs, q[:, :, 128:].transpose(1, 0, 2)], axis=2)          # [H, n, 576]; the node returns [n, H, 512]
        n_kv = min((head + n + 31) // 32 * 32, N_CTX)
        mask = np.where(np.arange(n_kv)[None, :] <= head + np.arange(n)[:, None], 0.0, -np.inf).astype(np.float16).view(np.uint16)
        kqv = node(q_states[None], cache[None, :n_kv], k_type, dv=512, mask=mask, scale=U.SCALE)[0]
        outs.append(O.mla_unabsorb(np.ascontiguousarray(kqv.transpose(1, 0, 2)), wkv_b, W_TYPE, n_head))
        head += n
    return outs, cache


@needs_ref
@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_F16, O.TYPE_Q8_0])
def test_oracle_one_node_form_equals_the_reference_s_unfused_graph(k_type):
    """On the CPU alone: the graph llm_attn_mla emits, run by the reference's ggml-cpu, against the one-node form
    evaluated by the oracle -- the equivalence the plugin's node rests on, independent of any GPU."""
    n_head = 16
    wkv_b, steps = _inputs(5, k_type, n_head)
    ref, _, ref_cache = O.ref_mla_layer(0, k_type, W_TYPE, n_head, N_CTX, steps, wkv_b, U.SCALE)
    got, cache = _oracle_one_node(k_type, n_head, wkv_b, steps)
    np.testing.assert_array_equal(cache.view(np.uint8).reshape(N_CTX, -1), ref_cache)         # same K / latent cache bytes
    if k_type == O.TYPE_F16:
        # ggml-cpu's fused node keeps its V accumulator in f16 for an F16 cache (ggml-cpu.c:12003-12100); the unfused graph's
        # mul_mat sums in f32.  The fused node as ggml-cpu computes it is therefore the one that is off, by more than the
        # tolerance on the decode steps; the node with an f32 accumulator (what the plugin does by default) is not.
        worst = max(O.errors(g, r)[1] for g, r in zip(got, ref))
        print("F16 cache, ggml-cpu's f16 accumulator vs the unfused graph: worst rel-L2 %.2e" % worst)
        assert worst > U.REL_L2_TOL
        got, _ = _oracle_one_node(k_type, n_head, wkv_b, steps, node=O.flash_attn_ext_f64)
    for s, (g, r) in enumerate(zip(got, ref)):
        print("step %d (%d tokens):" % (s, g.shape[0]), U.check(g, r, "one-node form vs unfused graph, step %d" % s))


@needs_ref
@pytest.mark.gpu
@pytest.mark.parametrize("mode", [1, 2])
@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_F16, O.TYPE_Q8_0])
def test_plugin_layer_graph_equals_the_reference_s_unfused_graph(gpu, k_type, mode):
    """mode 1: contiguous cache written by CPY, masked node; mode 2: page pool written by SCATTER_UPDATE, node with block
    table and length.  Every node between the q projection and wo runs on the plugin."""
    n_head = 16
    wkv_b, steps = _inputs(6, k_type, n_head)
    ref, _, ref_cache = O.ref_mla_layer(0, k_type, W_TYPE, n_head, N_CTX, steps, wkv_b, U.SCALE)
    bt = np.array([[5, 2, 7, 0]], np.int32) if mode == 2 else None
    n_ctx = 8 * 128 if mode == 2 else N_CTX
    got, where, cache = O.ref_mla_layer(mode, k_type, W_TYPE, n_head, n_ctx, steps, wkv_b, U.SCALE, so_path=_so(), block_table=bt)
    assert (where == 0x1f).all(), where          # cache write, attention node, MUL_MATs, CONCAT, CONT: all on the plugin
    if mode == 1:
        np.testing.assert_array_equal(cache, ref_cache)
    else:                                        # positions 0..76 live in pages 5 and then 2... of the pool
        n = sum(STEPS)
        np.testing.assert_array_equal(cache[5 * 128:5 * 128 + n], ref_cache[:n])
        assert not cache[:5 * 128].any() and not cache[6 * 128:].any()
    for s, (g, r) in enumerate(zip(got, ref)):
        print("step %d (%d tokens):" % (s, g.shape[0]), U.check(g, r, "plugin layer graph vs unfused graph, step %d" % s))


@needs_ref
@pytest.mark.gpu
@pytest.mark.parametrize("n_head", [128, 64, 48])
def test_plugin_layer_graph_at_128_heads_across_pages(gpu, n_head):
    """DeepSeek-V2's head count (and what a device holds of it at tensor-parallel degree 2; 48 heads: a row block with idle waves), a
    prefill that crosses a page boundary and decode steps behind it, paged form."""
    k_type, steps_n = O.TYPE_BF16, (200, 1, 1)
    wkv_b, steps = _inputs(8, k_type, n_head, steps_n)
    ref, _, _ = O.ref_mla_layer(0, k_type, W_TYPE, n_head, 256, steps, wkv_b, U.SCALE)
    got, where, _ = O.ref_mla_layer(2, k_type, W_TYPE, n_head, 4 * 128, steps, wkv_b, U.SCALE, so_path=_so(),
                                    block_table=np.array([[3, 1]], np.int32))
    assert (where == 0x1f).all(), where
    for s, (g, r) in enumerate(zip(got, ref)):
        print("step %d:" % s, U.check(g, r, "%d heads, step %d" % (n_head, s)))


@needs_ref
@pytest.mark.gpu
@pytest.mark.parametrize("mode", [1, 2])
@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_F16, O.TYPE_Q8_0])
def test_plugin_layer_graph_with_the_model_s_rope_nodes(gpu, k_type, mode, monkeypatch):
    """The front of the layer as the DeepSeek-V2 graph spells it (src/llama-graph-deepseek2.cpp:216-236): cont and rope_ext of
    q_pe and k_pe, view, concat into kv_states, then the cache write -- against the same graph in its unfused form on the
    reference's ggml-cpu.  The plugin issues these nodes as dispatches of several nodes each, reads the rope sources through the
    cont nodes and rotates k_pe on its way into the cache; with GGML_HIP_MLA_BATCH=off it launches node by node.  Both ways must
    agree bit for bit, the first in at most 7 dispatches per step for its 10 nodes."""
    import jittorinfer_amd as J
    lib = J.library()
    lib.mla_ggml_front_dispatches.restype = lib.mla_ggml_front_nodes.restype = __import__("ctypes").c_int64
    n_head = 16
    wkv_b, steps = _inputs(16, k_type, n_head)
    ref, _, ref_cache = O.ref_mla_layer(0, k_type, W_TYPE, n_head, N_CTX, steps, wkv_b, U.SCALE, rope_in_graph=True)
    bt = np.array([[5, 2, 7, 0]], np.int32) if mode == 2 else None
    n_ctx = 8 * 128 if mode == 2 else N_CTX
    d0, n0 = lib.mla_ggml_front_dispatches(), lib.mla_ggml_front_nodes()
    got, where, cache = O.ref_mla_layer(mode, k_type, W_TYPE, n_head, n_ctx, steps, wkv_b, U.SCALE, so_path=_so(), block_table=bt, rope_in_graph=True)
    assert (where == 0x3f).all(), where          # cache write, attention node, MUL_MATs, CONCATs, CONTs, ROPEs: all on the plugin
    assert lib.mla_ggml_front_nodes() - n0 == 10 * len(STEPS)
    # (13 launches per step node by node: a CONCAT is two.  How far below that the dispatches get is up to the graph allocator,
    # which reuses the memory of tensors that are dead in node order and so makes later nodes wait for their readers.)
    assert lib.mla_ggml_front_dispatches() - d0 <= 7 * len(STEPS)
    monkeypatch.setenv("GGML_HIP_MLA_BATCH", "off")
    got1, where1, cache1 = O.ref_mla_layer(mode, k_type, W_TYPE, n_head, n_ctx, steps, wkv_b, U.SCALE, so_path=_so(), block_table=bt, rope_in_graph=True)
    monkeypatch.delenv("GGML_HIP_MLA_BATCH")
    assert (where1 == 0x3f).all() and lib.mla_ggml_front_nodes() - n0 == 10 * len(STEPS)
    np.testing.assert_array_equal(cache, cache1)
    for g, g1 in zip(got, got1):
        np.testing.assert_array_equal(g.view(np.uint32), g1.view(np.uint32))
    n = sum(STEPS)
    rows = cache[5 * 128:5 * 128 + n] if mode == 2 else cache[:n]
    lat = 16 * 34 if k_type == O.TYPE_Q8_0 else 1024    # bytes of a row that hold the latent part
    np.testing.assert_array_equal(rows[:, :lat], ref_cache[:n, :lat])
    # the rope part: cosf / sinf of another libm, so a value may land on the neighbouring code of the cache type
    assert np.mean(rows[:, lat:] != ref_cache[:n, lat:]) < 5e-3
    assert rows[:, lat:].any()
    for s, (g, r) in enumerate(zip(got, ref)):
        print("step %d (%d tokens):" % (s, g.shape[0]), U.check(g, r, "plugin layer graph with rope nodes vs unfused graph, step %d" % s))


@needs_ref
def test_reference_graph_with_rope_nodes_equals_the_rotation_applied_outside_the_graph():
    """Pins the rope front of the driver's graphs: the unfused reference graph with cont / rope_ext / concat nodes on unrotated
    inputs gives, bit for bit, what the same graph gives on inputs rotated beforehand by the oracle's rope (itself bit-exact
    against the compiled reference)."""
    k_type, n_head = O.TYPE_F16, 16
    wkv_b, steps = _inputs(21, k_type, n_head)
    p = O.rope_params(n_dims=64, mode=0, n_ctx_orig=4096, freq_base=10000.0, freq_scale=0.025, ext_factor=1.0, attn_factor=0.8)
    rotated, head = [], 0
    for q, kv in steps:
        pos = (head + np.arange(q.shape[0])).astype(np.int32)
        q2, kv2 = q.copy(), kv.copy()
        q2[:, :, 128:] = O.rope(np.ascontiguousarray(q[:, :, 128:]), pos, p)
        kv2[:, 512:] = O.rope(np.ascontiguousarray(kv[:, None, 512:]), pos, p)[:, 0]
        rotated.append((q2, kv2))
        head += q.shape[0]
    a, _, cache_a = O.ref_mla_layer(0, k_type, W_TYPE, n_head, N_CTX, steps, wkv_b, U.SCALE, rope_in_graph=True)
    b, _, cache_b = O.ref_mla_layer(0, k_type, W_TYPE, n_head, N_CTX, rotated, wkv_b, U.SCALE)
    np.testing.assert_array_equal(cache_a, cache_b)
    for x, y in zip(a, b):
        np.testing.assert_array_equal(x.view(np.uint32), y.view(np.uint32))


@needs_ref
@pytest.mark.gpu
@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_Q8_0])
def test_generated_graphs_of_front_nodes_scheduled_by_levels(gpu, k_type, monkeypatch):
    """Graphs of cont / rope_ext / concat nodes (with the model's cont -> rope pairs, ropes of strided views, and the k side's
    rope -> view -> concat -> cpy) drawn from a seed and laid out by ggml's graph allocator, which reuses dead tensors' memory:
    the plugin's level schedule (dispatches of several nodes, reads through CONT nodes, the rope folded into the cache write) must
    give, bit for bit, what it gives node by node, and both what the reference's ggml-cpu gives for the same graph (rope: cosf /
    sinf of another libm, 4e-6 relative to the largest value per rope a value went through)."""
    import ctypes
    import jittorinfer_amd as J
    lib = J.library()
    lib.mla_ggml_front_dispatches.restype = lib.mla_ggml_front_nodes.restype = ctypes.c_int64
    rng = np.random.default_rng(77)
    saved = 0
    for seed in range(40):
        n_head, n_tok, n_ops = int(rng.integers(1, 20)), int(rng.integers(1, 40)), int(rng.integers(4, 40))
        a = rng.standard_normal((n_tok, n_head, 192)).astype(np.float32)
        b = rng.standard_normal((n_tok, 576)).astype(np.float32)
        pos = rng.integers(0, 100000, size=n_tok).astype(np.int32)
        ref, ref_cache, n_nodes = O.ref_random_front(seed, n_head, n_tok, n_ops, k_type, a, b, pos)
        d0, n0 = lib.mla_ggml_front_dispatches(), lib.mla_ggml_front_nodes()
        got, cache, _ = O.ref_random_front(seed, n_head, n_tok, n_ops, k_type, a, b, pos, so_path=_so())
        d1, n1 = lib.mla_ggml_front_dispatches(), lib.mla_ggml_front_nodes()
        monkeypatch.setenv("GGML_HIP_MLA_BATCH", "off")
        got1, cache1, _ = O.ref_random_front(seed, n_head, n_tok, n_ops, k_type, a, b, pos, so_path=_so())
        monkeypatch.delenv("GGML_HIP_MLA_BATCH")
        assert lib.mla_ggml_front_nodes() == n1            # node by node: the scheduler is not in the way
        np.testing.assert_array_equal(got.view(np.uint32), got1.view(np.uint32), err_msg="seed %d" % seed)
        np.testing.assert_array_equal(cache, cache1, err_msg="seed %d" % seed)
        assert not np.isnan(got).any()
        tol = 4e-6 * n_ops * max(1.0, float(np.abs(ref).max()))
        assert float(np.abs(got - ref).max()) <= tol, (seed, float(np.abs(got - ref).max()), tol)
        lat = 16 * 34 if k_type == O.TYPE_Q8_0 else 1024
        np.testing.assert_array_equal(cache[:, :lat], ref_cache[:, :lat])
        assert np.mean(cache[:, lat:] != ref_cache[:, lat:]) < 2e-2
        saved += (n1 - n0) - (d1 - d0)
    assert saved > 40, saved      # dispatches saved over the 40 graphs
