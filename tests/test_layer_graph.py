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
def test_plugin_layer_graph_at_128_heads_across_pages(gpu):
    """DeepSeek-V2's head count, a prefill that crosses a page boundary and decode steps behind it, paged form."""
    n_head, k_type, steps_n = 128, O.TYPE_BF16, (200, 1, 1)
    wkv_b, steps = _inputs(8, k_type, n_head, steps_n)
    ref, _, _ = O.ref_mla_layer(0, k_type, W_TYPE, n_head, 256, steps, wkv_b, U.SCALE)
    got, where, _ = O.ref_mla_layer(2, k_type, W_TYPE, n_head, 4 * 128, steps, wkv_b, U.SCALE, so_path=_so(),
                                    block_table=np.array([[3, 1]], np.int32))
    assert (where == 0x1f).all(), where
    for s, (g, r) in enumerate(zip(got, ref)):
        print("step %d:" % s, U.check(g, r, "128 heads, step %d" % s))
