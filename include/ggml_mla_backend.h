/*
 * C ABI of the "HIP-MLA" ggml backend plugin (libggml-hip-mla.so).
 *
 * The plugin is loaded by the reference exactly like any other dynamic ggml backend:
 *   ggml_backend_load(path)            ggml/src/ggml-backend-reg.cpp:401-403 -> load_backend :225-271
 *   GGML_BACKEND_PATH=<path>           ggml/src/ggml-backend-reg.cpp:583-587
 *   ggml_backend_load_all()            finds "libggml-hip-*.so" next to the executable, :488-558, :574
 * After that the reference talks to it only through the vtables of ggml/src/ggml-backend-impl.h, whose layouts
 * are mirrored in jittorinfer_amd/csrc/ggml_abi.h.  All handles are passed as void* here so that this header needs
 * no ggml header; they are ggml_backend_reg_t / ggml_tensor* of the reference.
 *
 * Node contract of the attention op it accepts, GGML_OP_FLASH_ATTN_EXT built by ggml_flash_attn_ext
 * (ggml/src/ggml.c:3988-4022), with the operands llm_attn_mla defines (src/llama-graph-attn.cpp:259-315):
 *   src[0] q     F32  [576, n_tok, n_head, n_seq]
 *   src[1] k     F16 | BF16 | Q8_0  [576, n_kv, 1, n_seq or 1]   the latent KV rows
 *   src[2] v     k itself (V := K, 576 wide) or a 512-wide view of k at offset 0 (the latent prefix)
 *   src[3] mask  F16 [>= n_kv, >= n_tok] or NULL, additive, -inf removes a key (src/llama-context.cpp:364-404)
 *   src[4], src[5]  optional, both or none: I32 block table [max_blocks, n_seq] of 128-token page ids into k
 *                (k is then the page pool [576, n_pages*128, 1, 1]) and I32 [n_seq] sequence lengths -- the same
 *                slot convention ggml_flash_attn_prompt uses for its length tensors (ggml/src/ggml.c:2707-2710)
 *   op_params    {scale, max_bias, logit_softcap} f32, [3] = precision (ggml/src/ggml.c:4012-4013, :4024-4030)
 *   dst          F32 [576, n_head, n_tok, n_seq]; the first v->ne[0] floats of every row are written
 * The cache write that precedes it (kernels behind include/mla_kv_write.h):
 *   GGML_OP_CPY             src[0] F32 [576, n_tok] with dense rows -> dst, a contiguous BF16 | F16 | Q8_0 view with as many
 *                           elements (ggml_cpy(kv_cur, k_cache_view), src/llama-graph-attn.cpp:236-241)
 *   GGML_OP_SCATTER_UPDATE  src[0] cache BF16 | F16 | Q8_0 [576, n_rows], src[1] I32 | I64 [n_tok] row indices,
 *                           src[2] updates [576, n_tok] of the cache type (copied) or F32 (converted)
 *                           (ggml_scatter_update, ggml/src/ggml.c:3203-3223; src/llama-graph-attn.cpp:380-383)
 * The nodes either side of it in llm_attn_mla and the DeepSeek-V2 graph (kernels behind include/mla_front.h):
 *   GGML_OP_CONT            src[0] F32 with dense rows (any other strides) -> contiguous F32 dst with as many elements
 *                           (ggml_cont of the q_pe / k_pe views, src/llama-graph-deepseek2.cpp:216-226; ggml_cont_2d of
 *                           the permuted result, src/llama-graph-attn.cpp:322)
 *   GGML_OP_ROPE            src[0] F32 [ne0, heads, n_tok, *], src[1] I32 [n_tok] positions, src[2] optional F32 frequency
 *                           factors; op_params of ggml_rope_ext (ggml/src/ggml.c:3413-3449), mode 0 or 2
 *   GGML_OP_MUL_MAT         src[0] F16 | BF16 [K, N, H] (K % 16 == 0, rows 16-byte aligned), src[1] F32 [K, M, H, *],
 *                           dst F32 [N, M, H, *], one matrix per head with K = 512 >= N or N = 512 >= K: the absorb
 *                           products q_nope x wk_b and wv_b x kqv (src/llama-graph-attn.cpp:264-275, :303-317) and
 *                           nothing else -- a model's other F16 / BF16 products stay with the backend that owns them
 * For every one of these ops supports_op runs the argument checks of the launch itself (shapes, strides, 16-byte
 * alignment of rows and of view offsets), so a node it accepts is one graph_compute runs; a node it refuses is placed on
 * another backend by the scheduler.
 *   GGML_OP_CONCAT          F32 operands with dense rows along any dimension (q_states = concat(q_nope_absorbed, q_pe),
 *                           src/llama-graph-attn.cpp:277; kv_states, src/llama-graph-deepseek2.cpp:235)
 * Every other op except the no-op view ops (NONE, RESHAPE, VIEW, PERMUTE, TRANSPOSE) is reported unsupported, so
 * the reference's scheduler keeps it on another backend (ggml/src/ggml-backend.cpp:820-846).
 *
 * Besides the device buffer type ("HIPMLA<i>") every device offers, like the reference's own accelerator backend
 * (ggml/src/ggml-cann/ggml-cann.cpp:1252-1365, :2192-2219, :2365-2410):
 *   get_host_buffer_type   "HIPMLA<i>_Host": pinned host memory, is_host, which the reference asks for to hold the CPU
 *                          backend's compute buffer and the logits (src/llama-context-load-utils.cpp:116-123,
 *                          src/llama-context.cpp:181); pageable memory when pinning fails
 *   event_new / event_free / event_synchronize and the backend's event_record / event_wait: HIP events on the
 *                          backend's stream, which ggml_backend_sched uses to keep several copies of a graph's inputs in
 *                          flight (ggml/src/ggml-backend.cpp:1508-1530, :1576-1580, :1630-1634)
 * F16 KV: the node accumulates V in f32 by default.  That is what the graph the reference emits for MLA does -- llm_attn_mla
 * builds mul_mat(v, softmax(..)) (src/llama-graph-attn.cpp:287-317), whose F16 dot product sums in f32 -- and the default
 * agrees with that graph to 4e-4 rel-L2 (tests/test_layer_graph.py).  ggml-cpu's fused FLASH_ATTN_EXT node is the odd one:
 * it keeps the V accumulator in f16 (ggml-cpu.c:12066-12080) and lands 1.4e-3 (77 keys) to 3.9e-3 (1024 keys) rel-L2 from
 * the exact value of the same rounded inputs, where the default lands 2e-4 away -- so against ggml-cpu's fused node the
 * default is outside the 1e-3 tolerance by that much (tests/test_backend_gpu.py states both numbers).  A backend
 * initialised with params containing "f16_acc=strict" (ggml_backend_dev_init(dev, params)), or with
 * GGML_HIP_MLA_F16_ACC=strict in the environment, replays ggml-cpu's f16 accumulator step for step instead (1.1e-4 from
 * ggml-cpu's node; contiguous and paged caches; 4 times slower on a decode step): for bit-for-bit comparisons with ggml-cpu's
 * fused node, not for serving.
 * Q8_0 KV: the matrix cores are fed q * d rounded to f16 (K, V and the Q8_0-quantized Q alike) where ggml-cpu multiplies integers and
 * scales (ggml-cpu-quants.c:3814-4241) and dequantises V to f32 (ggml-quants.c:357-373).  Over many keys the rounding averages out
 * (4.5e-4 rel-L2 at any block scale); when two or three keys carry a row it shows in single elements, up to 4e-3 max-abs against
 * the stated 2e-3 for values of unit variance (the largest of 4 000 random small cases: 3.9e-3; rel-L2 stays below 5e-4), and more for larger ones, since both the logits' and V's
 * rounding scale with the values: 3e-2 in single elements for rows of N(0, 3) under queries of N(0, 2) (tests/test_backend_gpu.py).  A cache of at most one page per sequence takes the exact path by itself (while rows x keys stay within 16 384 x 128); params containing
 * "q8=exact", or GGML_HIP_MLA_Q8=exact in the environment, make every Q8_0 node take it (the reference's own arithmetic, keys in
 * order: within 1e-5 of ggml-cpu's node at any shape, 10 to 100 times slower): for comparisons, not for serving.
 * BF16 KV, more than 32 attention rows per sequence: the decode kernel converts the cache tiles to f16 on the way (exact for magnitudes in [2^-14, 65504], which a
 * latent cache holds; see MLA_FLAG_BF16_DIRECT in mla_attn.h); params containing "bf16=direct", or GGML_HIP_MLA_BF16=direct
 * in the environment, keep the tiles in bf16 for caches with values outside that range.
 * and reports caps {async, host_buffer, events} (struct ggml_backend_dev_caps, ggml/include/ggml-backend.h:145-154).
 */
#ifndef GGML_MLA_BACKEND_H
#define GGML_MLA_BACKEND_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* replaces: the ggml_backend_init symbol every dynamic backend exports (GGML_BACKEND_DL_IMPL,
 * ggml/src/ggml-backend-impl.h:227-243; CANN's is ggml_backend_cann_reg, ggml/src/ggml-cann/ggml-cann.cpp:2506-2550).
 * Returns the process-lifetime ggml_backend_reg_t (api_version 1); one device per gfx950 GPU. */
void * ggml_backend_init(void);

/* replaces: the optional ggml_backend_score symbol (ggml/src/ggml-backend-impl.h:244-258, used at
 * ggml/src/ggml-backend-reg.cpp:520-535).  100 when a gfx950 device is present, 0 otherwise. */
int ggml_backend_score(void);

/* replaces: the static-registration accessor each in-tree backend has (ggml_backend_cann_reg, ggml-cann.cpp:2506),
 * for hosts that call ggml_backend_register(reg) (ggml/src/ggml-backend-reg.cpp:305-307) instead of dlopen. */
void * ggml_backend_hip_mla_reg(void);

/* no counterpart in the reference: entry i of the sizeof/offsetof/ordinal table this build assumes for the
 * reference's structs; returns the table length.  Lets a maintainer (and tests/test_abi.py) check the mirror
 * against the real headers without running anything on a GPU. */
int mla_ggml_abi_table(int i, const char ** name, int64_t * value);

/* no counterpart: supports_op's verdict for one node (any op) plus the violated clause (for diagnostics). */
int mla_ggml_supports_node(const void * ggml_tensor_node, const char ** why);

/* no counterpart: the argument block graph_compute builds for this node, handed to its launcher's check (mla_attn_plan,
 * mla_kv_write_check, mla_copy_f32_check, mla_rope_check, mla_mul_mat_check): 0 when the launch would accept it.  The node
 * must have the sources its op needs; nothing is read from the device.  supports_op makes the same call, so for every
 * node it accepts this returns 0 -- tests/test_supports_op.py checks that over generated nodes. */
int mla_ggml_node_launch_check(const void * ggml_tensor_node);

/* no counterpart: how many FLASH_ATTN_EXT nodes this process has launched with the key extents of their mask taken from the
 * node before them in the same graph (the layers of one llama graph share their mask tensor,
 * src/llama-graph-deepseek2.cpp:99-103) instead of scanning the mask again; GGML_HIP_MLA_MASK_EXTENTS=rescan, or
 * "mask_extents=rescan" in the params of init_backend, turns that off.  For tests and diagnostics. */
int64_t mla_ggml_mask_extent_reuses(void);

/* no counterpart: the CPY / SCATTER_UPDATE / CONT / CONCAT / ROPE / MUL_MAT nodes this process has computed through
 * graph_compute, and the dispatches (mla_front_batch_launch calls) they took: graph_compute issues the nodes between
 * two attention nodes level by level of their dependencies, the independent ones of a level in one dispatch, where the
 * reference's executors take a pass per node (ggml-cpu.c:15230-15268, ggml-cann.cpp:1761-1800).
 * GGML_HIP_MLA_BATCH=off, or "batch=off" in the params of init_backend, gives every node a launch of its own.  For
 * tests and diagnostics. */
int64_t mla_ggml_front_dispatches(void);
int64_t mla_ggml_front_nodes(void);

/* no counterpart: frees a buffer obtained from this backend's buffer type when no ggml is present in the process
 * to do it (what ggml_backend_buffer_free does, ggml/src/ggml-backend.cpp). */
void mla_ggml_buffer_free(void * ggml_backend_buffer);

#ifdef __cplusplus
}
#endif
#endif
