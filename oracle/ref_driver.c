/*
 * Driver around the REFERENCE's own compiled ggml (oracle/_ref/libggml_ref.so).  TEST INFRASTRUCTURE ONLY.
 *
 * This file is ours; it includes the reference's public headers at build time (from /root/reference, never
 * copied) and exports a few plain-C entry points for the Python tests:
 *   ref_flash_attn_ext            run ggml_flash_attn_ext (ggml/src/ggml.c:3988-4022) on the ggml-cpu backend
 *   ref_backend_flash_attn_ext    load a backend .so with ggml_backend_load (ggml-backend-reg.cpp:401-403) and
 *                                 run the same node on it through the reference's ggml-backend API, i.e. the
 *                                 way the reference's scheduler would drive a drop-in backend
 *   ref_quantize_q8_0_ref / _cpu  the two Q8_0 quantizers (ggml-quants.c:202-226, ggml-cpu-quants.c:767-900)
 *   ref_f32_to_f16_row / bf16     the reference's conversions
 *   ref_rope / ref_mul_mat        one ROPE / MUL_MAT node on ggml-cpu, or on a loaded backend
 *   ref_mla_q_states / _unabsorb  the query side and the output side of llm_attn_mla around the attention node
 *                                 (src/llama-graph-attn.cpp:264-277, :303-323), on ggml-cpu or on a loaded backend
 *   ref_mla_layer                 whole steps of llm_attn_mla on one KV cache: the graph the reference emits (unfused,
 *                                 src/llama-graph-attn.cpp:233-323) on ggml-cpu, or the one-node form on a loaded backend
 *                                 through ggml_backend_sched
 *   ref_abi_table                 sizeof/offsetof/enum facts of the structs a backend must mirror
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "ggml.h"
#include "ggml-alloc.h"
#include "ggml-backend.h"
#include "ggml-cpu.h"
#include "ggml-backend-impl.h"
#include "ggml-impl.h"
#define GGML_COMMON_DECL_C
#include "ggml-common.h"
#include "ggml-quants.h"

void quantize_row_q8_0(const float * x, void * y, int64_t k); /* ggml-cpu-quants.c:767 */

static size_t row_bytes(enum ggml_type t, int64_t n) { return ggml_row_size(t, n); }

static struct ggml_tensor * make_mask(struct ggml_context * ctx, int64_t n_kv, int64_t n_tok) {
    return ggml_new_tensor_2d(ctx, GGML_TYPE_F16, n_kv, GGML_PAD(n_tok, GGML_KQ_MASK_PAD));
}

/*
 * q:    f32, contiguous [n3][n_head][n_tok][DK]        (ggml ne = {DK, n_tok, n_head, n3})
 * k:    k_type rows, contiguous [n3][n_kv][row_bytes]  (ggml ne = {DK, n_kv, 1, n3});  V := K
 * mask: f16 [n_tok][n_kv] or NULL (rows n_tok..pad64 are filled with -inf here)
 * dst:  f32 [n3][n_tok][n_head][DK]
 */
int ref_flash_attn_ext(int k_type, int64_t DK, int64_t n_tok, int64_t n_head, int64_t n3, int64_t n_kv,
                       const float * q, const void * k, const uint16_t * mask, float scale, float max_bias,
                       float softcap, float * dst, int n_threads) {
    const enum ggml_type kt = (enum ggml_type) k_type;
    size_t mem = (size_t) DK * n_tok * n_head * n3 * 4 * 2 + row_bytes(kt, DK) * n_kv * n3 +
                 (size_t) n_kv * GGML_PAD(n_tok, GGML_KQ_MASK_PAD) * 2 + (64u << 20);
    mem += (size_t) n_threads * (3 * DK + 64) * 4 + (16u << 20);
    struct ggml_init_params ip = { mem, NULL, false };
    struct ggml_context *   ctx = ggml_init(ip);
    if (!ctx) return -1;
    struct ggml_tensor * tq = ggml_new_tensor_4d(ctx, GGML_TYPE_F32, DK, n_tok, n_head, n3);
    struct ggml_tensor * tk = ggml_new_tensor_4d(ctx, kt, DK, n_kv, 1, n3);
    memcpy(tq->data, q, ggml_nbytes(tq));
    memcpy(tk->data, k, ggml_nbytes(tk));
    struct ggml_tensor * tm = NULL;
    if (mask) {
        tm = make_mask(ctx, n_kv, n_tok);
        uint16_t * md = (uint16_t *) tm->data;
        for (int64_t i = 0; i < tm->ne[1]; i++)
            for (int64_t j = 0; j < n_kv; j++) md[i * n_kv + j] = i < n_tok ? mask[i * n_kv + j] : 0xfc00; /* -inf */
    }
    struct ggml_tensor * o = ggml_flash_attn_ext(ctx, tq, tk, tk, tm, scale, max_bias, softcap);
    ggml_flash_attn_ext_set_prec(o, GGML_PREC_F32);
    struct ggml_cgraph * gf = ggml_new_graph(ctx);
    ggml_build_forward_expand(gf, o);
    enum ggml_status st = ggml_graph_compute_with_ctx(ctx, gf, n_threads);
    if (st == GGML_STATUS_SUCCESS) memcpy(dst, o->data, ggml_nbytes(o));
    ggml_free(ctx);
    return (int) st;
}

/*
 * Same node, computed by a backend loaded from `so_path`, driven only through the reference's ggml-backend API.
 * Optional paged extension: block_table (i32 [n3][max_blocks]) and seq_lens (i32 [n3]) become src[4]/src[5] of
 * the node; k is then the page pool, contiguous [n_kv][row_bytes] with n_kv = pool tokens (ggml ne = {DK, n_kv, 1, 1}).
 * mask (optional) is f16 [n_tok][mask_ne0]; rows n_tok..pad64 are filled with -inf here.
 * dv: DK passes V := K; 512 passes a 512-wide view of K as V (which ggml-cpu itself asserts on, ggml-cpu.c:11943).
 * use_sched != 0 runs the graph through ggml_backend_sched with {loaded backend, CPU} the way llama_decode does
 * (ggml-backend.cpp:1493-1587, :1727-1739) instead of calling ggml_backend_graph_compute directly.
 * use_sched == 2 sets the scheduler up the way llama's context does (src/llama-context-load-utils.cpp:108-131): the CPU
 * backend's compute buffer comes from the device's host buffer type, pipeline parallelism is on (several copies of the
 * inputs, ordered by the backends' events), Q reaches the node through an op the CPU backend runs (ggml_scale by 1) and
 * the result leaves through another; the graph is computed three times with Q, 2Q (softmax scale halved) and Q again.
 * Returns 0 on success; negative for set-up failures; the ggml_status otherwise.
 */
struct fa_graph {
    struct ggml_context * ctx;
    struct ggml_tensor *  tq, *tm, *tb, *tl, *q_in, *fa, *o;
    struct ggml_tensor *  tq_b, *fa_b;   /* second_node: another query tensor and another node over the same cache and mask */
    struct ggml_cgraph *  gf;
};

/* The node and its operands in a fresh context (llama rebuilds its graph for every decode too: the scheduler rewires the
 * sources of the nodes it splits, so a graph is computed once).  tk may be NULL: K is then part of this context. */
static int fa_graph_build(struct fa_graph * g, struct ggml_tensor * tk_in, struct ggml_tensor ** tk_out, enum ggml_type kt,
                          int64_t DK, int64_t dv, int64_t n_tok, int64_t n_head, int64_t n3, int64_t n_kv, int paged,
                          int with_mask, int64_t mask_ne0, int64_t max_blocks, float scale, float max_bias, float softcap,
                          int cpu_ops, int second_node) {
    struct ggml_init_params ip = { ggml_tensor_overhead() * 32 + ggml_graph_overhead() + 4096, NULL, true };
    memset(g, 0, sizeof(*g));
    g->ctx = ggml_init(ip);
    if (!g->ctx) return -13;
    struct ggml_context * ctx = g->ctx;
    g->tq = ggml_new_tensor_4d(ctx, GGML_TYPE_F32, DK, n_tok, n_head, n3);
    struct ggml_tensor * tk = tk_in ? tk_in : ggml_new_tensor_4d(ctx, kt, DK, n_kv, 1, paged ? 1 : n3);
    struct ggml_tensor * tv = tk;
    if (dv != DK) tv = ggml_view_4d(ctx, tk, dv, tk->ne[1], tk->ne[2], tk->ne[3], tk->nb[1], tk->nb[2], tk->nb[3], 0);
    g->tm = with_mask ? make_mask(ctx, mask_ne0, n_tok) : NULL;
    g->tb = paged ? ggml_new_tensor_2d(ctx, GGML_TYPE_I32, max_blocks, n3) : NULL;
    g->tl = paged ? ggml_new_tensor_1d(ctx, GGML_TYPE_I32, n3) : NULL;
    ggml_set_input(g->tq);
    if (g->tm) ggml_set_input(g->tm);
    if (g->tb) { ggml_set_input(g->tb); ggml_set_input(g->tl); }
    g->q_in = cpu_ops ? ggml_scale(ctx, g->tq, 1.0f) : g->tq;
    g->fa = g->o = ggml_flash_attn_ext(ctx, g->q_in, tk, tv, g->tm, scale, max_bias, softcap);
    ggml_flash_attn_ext_set_prec(g->fa, GGML_PREC_F32);
    g->fa->src[4] = g->tb; /* same slot convention as ggml_flash_attn_prompt's length tensors, ggml.c:2707-2710 */
    g->fa->src[5] = g->tl;
    if (cpu_ops) g->o = ggml_scale(ctx, g->fa, 1.0f);
    ggml_set_output(g->o);
    g->gf = ggml_new_graph(ctx);
    ggml_build_forward_expand(g->gf, g->o);
    if (second_node) {
        /* the attention nodes of the layers of one llama graph share one mask tensor (src/llama-graph-deepseek2.cpp:99-103) */
        g->tq_b = ggml_new_tensor_4d(ctx, GGML_TYPE_F32, DK, n_tok, n_head, n3);
        ggml_set_input(g->tq_b);
        g->fa_b = ggml_flash_attn_ext(ctx, g->tq_b, tk, tv, g->tm, scale, max_bias, softcap);
        ggml_flash_attn_ext_set_prec(g->fa_b, GGML_PREC_F32);
        g->fa_b->src[4] = g->tb;
        g->fa_b->src[5] = g->tl;
        ggml_set_output(g->fa_b);
        ggml_build_forward_expand(g->gf, g->fa_b);
    }
    if (tk_out) *tk_out = tk;
    return 0;
}

int ref_backend_flash_attn_ext(const char * so_path, int k_type, int64_t DK, int64_t dv, int64_t n_tok, int64_t n_head,
                               int64_t n3, int64_t n_kv, const float * q, const void * k, const uint16_t * mask,
                               int64_t mask_ne0, const int32_t * block_table, int64_t max_blocks,
                               const int32_t * seq_lens, float scale, float max_bias, float softcap, int use_sched,
                               float * dst, char * info, size_t info_len, const float * q_b, float * dst_b) {
    static ggml_backend_reg_t reg = NULL;
    static char               loaded_path[4096];
    if (!reg || strcmp(loaded_path, so_path) != 0) {
        reg = ggml_backend_load(so_path);
        if (!reg) return -10;
        snprintf(loaded_path, sizeof(loaded_path), "%s", so_path);
    }
    if (ggml_backend_reg_dev_count(reg) < 1) return -11;
    ggml_backend_dev_t dev = ggml_backend_reg_dev_get(reg, 0);
    ggml_backend_t     be  = ggml_backend_dev_init(dev, NULL);
    if (!be) return -12;
    if (info) snprintf(info, info_len, "reg=%s dev=%s (%s) type=%d backend=%s buft=%s", ggml_backend_reg_name(reg),
                       ggml_backend_dev_name(dev), ggml_backend_dev_description(dev), (int) ggml_backend_dev_type(dev),
                       ggml_backend_name(be), ggml_backend_buft_name(ggml_backend_dev_buffer_type(dev)));

    const enum ggml_type  kt     = (enum ggml_type) k_type;
    const int             paged  = block_table != NULL;
    const int             n_runs = use_sched == 2 ? 3 : 1;
    int                   rc     = 0;
    ggml_backend_buffer_t buf    = NULL;
    ggml_backend_buffer_t buf_kv = NULL;
    ggml_backend_sched_t  sched  = NULL;
    ggml_backend_t        cpu    = NULL;
    struct ggml_tensor *  tk     = NULL;
    struct fa_graph       g;
    memset(&g, 0, sizeof(g));
    /* with a scheduler the KV rows live in their own context, allocated up front in the backend's buffer the way
     * llama_kv_cache_init allocates k_l[il] (src/llama-kv-cache.cpp:82-90,153-158) */
    struct ggml_init_params ipk    = { ggml_tensor_overhead() * 4, NULL, true };
    struct ggml_context *   ctx_kv = ggml_init(ipk);
    if (!ctx_kv) { ggml_backend_free(be); return -13; }
    const size_t nq = (size_t) (DK * n_tok * n_head * n3);
    float *      q2 = (float *) malloc(nq * sizeof(float));
    float *      d2 = NULL;
    for (size_t i = 0; i < nq; i++) q2[i] = 2.0f * q[i];

    if (use_sched) {
        tk     = ggml_new_tensor_4d(ctx_kv, kt, DK, n_kv, 1, paged ? 1 : n3);
        buf_kv = ggml_backend_alloc_ctx_tensors(ctx_kv, be);
        if (!buf_kv) { rc = -18; goto done; }
        ggml_backend_buffer_clear(buf_kv, 0); /* src/llama-kv-cache.cpp:158 */
        ggml_backend_tensor_set(tk, k, 0, ggml_nbytes(tk));
        cpu = ggml_backend_init_by_type(GGML_BACKEND_DEVICE_TYPE_CPU, NULL);
        if (!cpu) { rc = -15; goto done; }
        ggml_backend_t             backends[2] = { be, cpu };
        ggml_backend_buffer_type_t bufts[2]    = { ggml_backend_get_default_buffer_type(be), ggml_backend_get_default_buffer_type(cpu) };
        if (use_sched == 2) {
            ggml_backend_buffer_type_t   host = ggml_backend_dev_host_buffer_type(dev);
            struct ggml_backend_dev_props props;
            ggml_backend_dev_get_props(dev, &props);
            if (!host || !ggml_backend_buft_is_host(host) || !props.caps.host_buffer || !props.caps.events) { rc = -20; goto done; }
            if (info) snprintf(info + strlen(info), info_len - strlen(info), " host_buft=%s", ggml_backend_buft_name(host));
            bufts[1] = host;
        }
        sched = ggml_backend_sched_new(backends, bufts, 2, GGML_DEFAULT_GRAPH_SIZE, use_sched == 2);
        if (!sched) { rc = -16; goto done; }
    }

    /* use_sched == 2: three asynchronous computes, as consecutive llama_decode calls issue them: every one takes the next
     * copy of the inputs, and the events keep a copy from being overwritten while the device still reads it */
    for (int run = 0; run < n_runs; run++) {
        const float run_scale = run == 1 ? 0.5f * scale : scale;
        rc = fa_graph_build(&g, tk, use_sched ? NULL : &tk, kt, DK, dv, n_tok, n_head, n3, n_kv, paged, mask != NULL, mask_ne0,
                            max_blocks, run_scale, max_bias, softcap, use_sched == 2, q_b != NULL);
        if (rc) goto done;
        if (!ggml_backend_dev_supports_op(dev, g.fa)) { rc = -14; goto done; }
        if (use_sched) {
            if (run > 0) ggml_backend_sched_reset(sched);
            /* llama's graph callback pins attention nodes to the layer's device the same way */
            ggml_backend_sched_set_tensor_backend(sched, g.fa, be);
            if (!ggml_backend_sched_alloc_graph(sched, g.gf)) { rc = -16; goto done; }
            if (ggml_backend_sched_get_tensor_backend(sched, g.fa) != be) { rc = -17; goto done; }
            if (use_sched == 2 && (ggml_backend_sched_get_tensor_backend(sched, g.q_in) != cpu || ggml_backend_sched_get_n_splits(sched) < 3)) { rc = -21; goto done; }
        } else {
            ggml_set_input(tk);
            buf = ggml_backend_alloc_ctx_tensors(g.ctx, be);
            if (!buf) { rc = -18; goto done; }
            ggml_backend_tensor_set(tk, k, 0, ggml_nbytes(tk));
        }
        ggml_backend_tensor_set(g.tq, run == 1 ? q2 : q, 0, ggml_nbytes(g.tq));
        if (g.tq_b) ggml_backend_tensor_set(g.tq_b, q_b, 0, ggml_nbytes(g.tq_b));
        if (g.tm) {
            const size_t nrow = (size_t) g.tm->ne[1];
            uint16_t *   md   = (uint16_t *) malloc(nrow * mask_ne0 * 2);
            for (size_t i = 0; i < nrow; i++)
                for (int64_t j = 0; j < mask_ne0; j++) md[i * mask_ne0 + j] = (int64_t) i < n_tok ? mask[i * mask_ne0 + j] : 0xfc00;
            ggml_backend_tensor_set(g.tm, md, 0, ggml_nbytes(g.tm));
            free(md);
        }
        if (g.tb) {
            ggml_backend_tensor_set(g.tb, block_table, 0, ggml_nbytes(g.tb));
            ggml_backend_tensor_set(g.tl, seq_lens, 0, ggml_nbytes(g.tl));
        }
        enum ggml_status st;
        if (use_sched == 2) {
            st = ggml_backend_sched_graph_compute_async(sched, g.gf);
            ggml_backend_sched_synchronize(sched);
        } else {
            st = use_sched ? ggml_backend_sched_graph_compute(sched, g.gf) : ggml_backend_graph_compute(be, g.gf);
        }
        if (st != GGML_STATUS_SUCCESS) { rc = (int) st ? (int) st : -19; goto done; }
        const size_t nb = ggml_nbytes(g.o);
        if (g.fa_b && run == 0) ggml_backend_tensor_get(g.fa_b, dst_b, 0, ggml_nbytes(g.fa_b));
        if (run == 1) {
            /* softmax(0.5 * scale * (2Q).K) is softmax(scale * Q.K) bit for bit: doubling is exact in every rounding step */
            d2 = (float *) malloc(nb);
            ggml_backend_tensor_get(g.o, d2, 0, nb);
            if (memcmp(d2, dst, nb) != 0) { rc = -22; goto done; }
        } else {
            if (run == 2) memset(dst, 0xff, nb);
            ggml_backend_tensor_get(g.o, dst, 0, nb);
            if (run == 2 && memcmp(d2, dst, nb) != 0) { rc = -23; goto done; }
        }
        ggml_free(g.ctx);
        g.ctx = NULL;
    }
done:
    if (sched) ggml_backend_sched_free(sched);
    if (buf) ggml_backend_buffer_free(buf);
    if (buf_kv) ggml_backend_buffer_free(buf_kv);
    if (cpu) ggml_backend_free(cpu);
    if (g.ctx) ggml_free(g.ctx);
    ggml_free(ctx_kv);
    ggml_backend_free(be);
    free(q2);
    free(d2);
    return rc;
}

/* ------------------------------------------------------------------ small pinning helpers */

/*
 * The KV cache write of llm_attn_mla (src/llama-graph-attn.cpp:236-241) on the reference's ggml-cpu:
 * cache = typed tensor of n_cache rows of 576 (filled from `cache` first), kv_cur = f32 [576, n_tok],
 * ggml_cpy(kv_cur, ggml_view_1d(cache, n_tok*576, row_size*kv_head)); the whole cache is copied back into `cache`.
 */
int ref_kv_cpy(int k_type, int64_t n_cache, int64_t kv_head, int64_t n_tok, const float * kv_cur, void * cache, int n_threads) {
    const enum ggml_type kt = (enum ggml_type) k_type;
    const int64_t D = 576;
    size_t mem = row_bytes(kt, D) * n_cache + (size_t) D * n_tok * 4 + (32u << 20);
    struct ggml_init_params ip = { mem, NULL, false };
    struct ggml_context *   ctx = ggml_init(ip);
    if (!ctx) return -1;
    struct ggml_tensor * tc = ggml_new_tensor_1d(ctx, kt, D * n_cache);
    struct ggml_tensor * tx = ggml_new_tensor_2d(ctx, GGML_TYPE_F32, D, n_tok);
    memcpy(tc->data, cache, ggml_nbytes(tc));
    memcpy(tx->data, kv_cur, ggml_nbytes(tx));
    struct ggml_tensor * view = ggml_view_1d(ctx, tc, n_tok * D, ggml_row_size(kt, D) * kv_head);
    struct ggml_tensor * o    = ggml_cpy(ctx, tx, view);
    struct ggml_cgraph * gf   = ggml_new_graph(ctx);
    ggml_build_forward_expand(gf, o);
    enum ggml_status st = ggml_graph_compute_with_ctx(ctx, gf, n_threads);
    if (st == GGML_STATUS_SUCCESS) memcpy(cache, tc->data, ggml_nbytes(tc));
    ggml_free(ctx);
    return (int) st;
}

/*
 * The same write through a backend loaded from `so_path` (cache and kv_cur live in that backend's buffer, the node is
 * computed by ggml_backend_graph_compute), followed by nothing else: the cache bytes come back in `cache`.
 */
int ref_backend_kv_cpy(const char * so_path, int k_type, int64_t n_cache, int64_t kv_head, int64_t n_tok, const float * kv_cur,
                       void * cache, char * info, size_t info_len) {
    const enum ggml_type kt = (enum ggml_type) k_type;
    const int64_t D = 576;
    ggml_backend_reg_t reg = ggml_backend_load(so_path);
    if (!reg) return -10;
    if (ggml_backend_reg_dev_count(reg) < 1) return -11;
    ggml_backend_dev_t dev = ggml_backend_reg_dev_get(reg, 0);
    ggml_backend_t     be  = ggml_backend_dev_init(dev, NULL);
    if (!be) return -12;
    if (info) snprintf(info, info_len, "%s / %s", ggml_backend_reg_name(reg), ggml_backend_dev_name(dev));
    struct ggml_init_params ip = { ggml_tensor_overhead() * 16 + ggml_graph_overhead(), NULL, true };
    struct ggml_context *   ctx = ggml_init(ip);
    struct ggml_tensor * tc = ggml_new_tensor_1d(ctx, kt, D * n_cache);
    struct ggml_tensor * tx = ggml_new_tensor_2d(ctx, GGML_TYPE_F32, D, n_tok);
    struct ggml_tensor * view = ggml_view_1d(ctx, tc, n_tok * D, ggml_row_size(kt, D) * kv_head);
    struct ggml_tensor * o    = ggml_cpy(ctx, tx, view);
    struct ggml_cgraph * gf   = ggml_new_graph(ctx);
    ggml_build_forward_expand(gf, o);
    int rc = 0;
    ggml_backend_buffer_t buf = ggml_backend_alloc_ctx_tensors(ctx, be);
    if (!buf) rc = -13;
    if (!rc && !ggml_backend_supports_op(be, o)) rc = -14;
    if (!rc) {
        ggml_backend_tensor_set(tc, cache, 0, ggml_nbytes(tc));
        ggml_backend_tensor_set(tx, kv_cur, 0, ggml_nbytes(tx));
        enum ggml_status st = ggml_backend_graph_compute(be, gf);
        if (st != GGML_STATUS_SUCCESS) rc = (int) st ? (int) st : -15;
        else ggml_backend_tensor_get(tc, cache, 0, ggml_nbytes(tc));
    }
    if (buf) ggml_backend_buffer_free(buf);
    ggml_free(ctx);
    ggml_backend_free(be);
    return rc;
}

/* ------------------------------------------------------------------ the nodes either side of the attention node
 * One code path for both executors: `so_path` == NULL runs the graph on the reference's ggml-cpu backend, otherwise on
 * the backend loaded from that file; tensors live in the executor's buffer. */
struct front_rt {
    ggml_backend_t        be;
    struct ggml_context * ctx;
    struct ggml_cgraph *  gf;
    ggml_backend_buffer_t buf;
};

static int front_open(struct front_rt * rt, const char * so_path, int n_threads) {
    memset(rt, 0, sizeof(*rt));
    if (so_path) {
        ggml_backend_reg_t reg = ggml_backend_load(so_path);
        if (!reg) return -10;
        if (ggml_backend_reg_dev_count(reg) < 1) return -11;
        rt->be = ggml_backend_dev_init(ggml_backend_reg_dev_get(reg, 0), NULL);
    } else {
        rt->be = ggml_backend_cpu_init();
        if (rt->be) ggml_backend_cpu_set_n_threads(rt->be, n_threads);
    }
    if (!rt->be) return -12;
    struct ggml_init_params ip = { ggml_tensor_overhead() * 64 + ggml_graph_overhead(), NULL, true };
    rt->ctx = ggml_init(ip);
    rt->gf  = ggml_new_graph(rt->ctx);
    return 0;
}
/* allocate every tensor of the context, check that the executor takes every node */
static int front_alloc(struct front_rt * rt) {
    rt->buf = ggml_backend_alloc_ctx_tensors(rt->ctx, rt->be);
    if (!rt->buf) return -13;
    for (int i = 0; i < ggml_graph_n_nodes(rt->gf); i++)
        if (!ggml_backend_supports_op(rt->be, ggml_graph_node(rt->gf, i))) return -100 - i;
    return 0;
}
static int front_run(struct front_rt * rt) {
    enum ggml_status st = ggml_backend_graph_compute(rt->be, rt->gf);
    return st == GGML_STATUS_SUCCESS ? 0 : ((int) st ? (int) st : -15);
}
static void front_close(struct front_rt * rt) {
    if (rt->buf) ggml_backend_buffer_free(rt->buf);
    if (rt->ctx) ggml_free(rt->ctx);
    if (rt->be) ggml_backend_free(rt->be);
}

struct ref_rope_params {
    int32_t n_dims, mode, n_ctx_orig;
    float   freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow;
};

/* ggml_rope_ext (ggml.c:3495-3501) of x = f32 [ne0, ne1, ne2] with pos[ne2] and optional freq_factors[n_dims/2] */
int ref_rope(const char * so_path, int64_t ne0, int64_t ne1, int64_t ne2, const float * x, const int32_t * pos,
             const float * freq_factors, const struct ref_rope_params * p, float * out, int n_threads) {
    struct front_rt rt;
    int rc = front_open(&rt, so_path, n_threads);
    if (rc) return rc;
    struct ggml_tensor * tx = ggml_new_tensor_3d(rt.ctx, GGML_TYPE_F32, ne0, ne1, ne2);
    struct ggml_tensor * tp = ggml_new_tensor_1d(rt.ctx, GGML_TYPE_I32, ne2);
    struct ggml_tensor * tf = freq_factors ? ggml_new_tensor_1d(rt.ctx, GGML_TYPE_F32, p->n_dims / 2) : NULL;
    struct ggml_tensor * o  = ggml_rope_ext(rt.ctx, tx, tp, tf, p->n_dims, p->mode, p->n_ctx_orig, p->freq_base, p->freq_scale,
                                            p->ext_factor, p->attn_factor, p->beta_fast, p->beta_slow);
    ggml_build_forward_expand(rt.gf, o);
    rc = front_alloc(&rt);
    if (!rc) {
        ggml_backend_tensor_set(tx, x, 0, ggml_nbytes(tx));
        ggml_backend_tensor_set(tp, pos, 0, ggml_nbytes(tp));
        if (tf) ggml_backend_tensor_set(tf, freq_factors, 0, ggml_nbytes(tf));
        rc = front_run(&rt);
        if (!rc) ggml_backend_tensor_get(o, out, 0, ggml_nbytes(o));
    }
    front_close(&rt);
    return rc;
}

/* ggml_mul_mat of a contiguous src0 = type0 [K, N, ne02] and a contiguous f32 src1 = [K, M, ne12]; out f32 [N, M, ne12] */
int ref_mul_mat(const char * so_path, int type0, int64_t K, int64_t N, int64_t ne02, int64_t M, int64_t ne12,
                const void * a, const float * b, float * out, int n_threads) {
    struct front_rt rt;
    int rc = front_open(&rt, so_path, n_threads);
    if (rc) return rc;
    struct ggml_tensor * ta = ggml_new_tensor_3d(rt.ctx, (enum ggml_type) type0, K, N, ne02);
    struct ggml_tensor * tb = ggml_new_tensor_3d(rt.ctx, GGML_TYPE_F32, K, M, ne12);
    struct ggml_tensor * o  = ggml_mul_mat(rt.ctx, ta, tb);
    ggml_build_forward_expand(rt.gf, o);
    rc = front_alloc(&rt);
    if (!rc) {
        ggml_backend_tensor_set(ta, a, 0, ggml_nbytes(ta));
        ggml_backend_tensor_set(tb, b, 0, ggml_nbytes(tb));
        rc = front_run(&rt);
        if (!rc) ggml_backend_tensor_get(o, out, 0, ggml_nbytes(o));
    }
    front_close(&rt);
    return rc;
}

/*
 * The query side of llm_attn_mla as the reference's graph builds it (src/llama-graph-deepseek2.cpp:183-194, :216-222,
 * src/llama-graph-attn.cpp:264-277): q = f32 [192*H, n_tok]; q_nope / q_pe strided views; q_pe -> cont -> rope;
 * q_nope permuted -> mul_mat with wk_b (view of wkv_b: [128, 512, H]); concat with the permuted q_pe along dim 0.
 * out = q_states f32 [576, n_tok, H].  wkv_b = w_type [512, H*(128+128)] as the model stores it.
 */
int ref_mla_q_states(const char * so_path, int w_type, int64_t H, int64_t n_tok, const float * q, const void * wkv_b,
                     const int32_t * pos, const struct ref_rope_params * p, float * out, int n_threads) {
    const int64_t NOPE = 128, ROPE = 64, LORA = 512, DV = 128;
    const enum ggml_type wt = (enum ggml_type) w_type;
    struct front_rt rt;
    int rc = front_open(&rt, so_path, n_threads);
    if (rc) return rc;
    struct ggml_context * c = rt.ctx;
    struct ggml_tensor * tq = ggml_new_tensor_2d(c, GGML_TYPE_F32, (NOPE + ROPE) * H, n_tok);
    struct ggml_tensor * tw = ggml_new_tensor_2d(c, wt, LORA, H * (NOPE + DV));
    struct ggml_tensor * tp = ggml_new_tensor_1d(c, GGML_TYPE_I32, n_tok);
    struct ggml_tensor * q_nope = ggml_view_3d(c, tq, NOPE, H, n_tok, ggml_row_size(tq->type, NOPE + ROPE),
                                               ggml_row_size(tq->type, (NOPE + ROPE) * H), 0);
    struct ggml_tensor * q_pe = ggml_view_3d(c, tq, ROPE, H, n_tok, ggml_row_size(tq->type, NOPE + ROPE),
                                             ggml_row_size(tq->type, (NOPE + ROPE) * H), ggml_row_size(tq->type, NOPE));
    q_pe = ggml_cont(c, q_pe);
    q_pe = ggml_rope_ext(c, q_pe, tp, NULL, p->n_dims, p->mode, p->n_ctx_orig, p->freq_base, p->freq_scale, p->ext_factor,
                         p->attn_factor, p->beta_fast, p->beta_slow);
    struct ggml_tensor * wk_b = ggml_view_3d(c, tw, NOPE, LORA, H, ggml_row_size(wt, NOPE), ggml_row_size(wt, NOPE * LORA), 0);
    q_nope = ggml_permute(c, q_nope, 0, 2, 1, 3);
    q_nope = ggml_mul_mat(c, wk_b, q_nope);
    q_pe   = ggml_permute(c, q_pe, 0, 2, 1, 3);
    struct ggml_tensor * o = ggml_concat(c, q_nope, q_pe, 0);
    ggml_build_forward_expand(rt.gf, o);
    rc = front_alloc(&rt);
    if (!rc) {
        ggml_backend_tensor_set(tq, q, 0, ggml_nbytes(tq));
        ggml_backend_tensor_set(tw, wkv_b, 0, ggml_nbytes(tw));
        ggml_backend_tensor_set(tp, pos, 0, ggml_nbytes(tp));
        rc = front_run(&rt);
        if (!rc) ggml_backend_tensor_get(o, out, 0, ggml_nbytes(o));
    }
    front_close(&rt);
    return rc;
}

/*
 * The output side (src/llama-graph-attn.cpp:303-323): kqv = f32 [512, n_tok, H] (the attention result per head),
 * wv_b = view of wkv_b [512, 128, H] behind the wk_b part; mul_mat, permute(0,2,1,3), cont_2d -> out f32 [128*H, n_tok].
 */
int ref_mla_unabsorb(const char * so_path, int w_type, int64_t H, int64_t n_tok, const float * kqv, const void * wkv_b,
                     float * out, int n_threads) {
    const int64_t NOPE = 128, LORA = 512, DV = 128;
    const enum ggml_type wt = (enum ggml_type) w_type;
    struct front_rt rt;
    int rc = front_open(&rt, so_path, n_threads);
    if (rc) return rc;
    struct ggml_context * c = rt.ctx;
    struct ggml_tensor * tk = ggml_new_tensor_3d(c, GGML_TYPE_F32, LORA, n_tok, H);
    struct ggml_tensor * tw = ggml_new_tensor_2d(c, wt, LORA, H * (NOPE + DV));
    struct ggml_tensor * wv_b = ggml_view_3d(c, tw, LORA, DV, H, ggml_row_size(wt, LORA), ggml_row_size(wt, LORA * DV),
                                             ggml_row_size(wt, LORA * NOPE * H));
    struct ggml_tensor * o = ggml_mul_mat(c, wv_b, tk);
    o = ggml_permute(c, o, 0, 2, 1, 3);
    o = ggml_cont_2d(c, o, DV * H, n_tok);
    ggml_build_forward_expand(rt.gf, o);
    rc = front_alloc(&rt);
    if (!rc) {
        ggml_backend_tensor_set(tk, kqv, 0, ggml_nbytes(tk));
        ggml_backend_tensor_set(tw, wkv_b, 0, ggml_nbytes(tw));
        rc = front_run(&rt);
        if (!rc) ggml_backend_tensor_get(o, out, 0, ggml_nbytes(o));
    }
    front_close(&rt);
    return rc;
}

/* ------------------------------------------------------------------ one attention layer, several steps on one cache
 *
 * mode 0  the graph llm_attn_mla builds today (src/llama-graph-attn.cpp:233-323), on the reference's ggml-cpu: the new
 *         rows copied into the K cache (k_type, [576, n_ctx]) and, transposed, into the V cache (v_type, [n_ctx, 512]);
 *         q_states = concat(q_nope . wk_b, q_pe); kq = mul_mat(k, q) at f32 precision; soft_max_ext with the f32 mask
 *         and kq_scale; kqv = mul_mat(v, kq); mul_mat with wv_b; permute; cont_2d.
 * mode 1  the one-node form on the backend loaded from so_path, scheduled by ggml_backend_sched over {that backend, CPU}
 *         as llama_decode schedules its graphs (ggml-backend.cpp:1493-1587): ONE latent cache (k_type, [576, n_ctx]) in
 *         the backend's buffer written by the same ggml_cpy; q_states as above; ggml_flash_attn_ext(q_states, k,
 *         v = the first 512 columns of k, f16 mask) at f32 precision; the first 512 floats of its rows -> wv_b -> permute
 *         -> cont_2d.
 * mode 2  as mode 1 with the cache as a pool of 128-row pages: the new rows go in by ggml_scatter_update (ggml.c:3203-3223)
 *         at rows block_table[pos / 128] * 128 + pos % 128, the node carries the block table and the sequence length in
 *         src[4] / src[5], and only a step of several tokens carries a (causal) mask.
 *
 * One sequence; step s appends n_tok[s] tokens at positions kv_head[s] .. (every step's kv_head is the number of tokens
 * before it).  q: per step f32 [n_tok][H][128 + 64] (q_nope | q_pe, q_pe already rotated), kv_cur: per step f32
 * [n_tok][576], both concatenated over the steps; wkv_b = w_type [512, H * (128 + 128)] as the model stores it.
 * out: per step f32 [n_tok][128 * H], concatenated.  on_backend[s] (modes 1, 2): bit 0 = the cache write ran on the
 * loaded backend, bit 1 = the attention node, bit 2 = every MUL_MAT, bit 3 = CONCAT, bit 4 = CONT.
 * cache_out (may be NULL): the K / latent cache bytes after the last step.
 */
struct layer_io {
    struct ggml_tensor *q, *kv_cur, *mask, *idx, *bt, *lens, *out, *write, *fa, *pos;
};

/* the rotary embedding as the DeepSeek-V2 graph applies it to q_pe and k_pe (src/llama-graph-deepseek2.cpp:216-233): cont of
 * the view, rope_ext with YaRN parameters (DeepSeek-V2's: n_rot 64, normal pairing, n_ctx_orig 4096, factor 40) */
static struct ggml_tensor * layer_rope(struct ggml_context * c, struct ggml_tensor * pe, struct ggml_tensor * pos) {
    pe = ggml_cont(c, pe);
    return ggml_rope_ext(c, pe, pos, NULL, 64, 0, 4096, 10000.0f, 0.025f, 1.0f, 0.8f, 32.0f, 1.0f);
}

static struct ggml_tensor * layer_q_states(struct ggml_context * c, struct ggml_tensor * tq, struct ggml_tensor * tw, int64_t H, int64_t n_tok, struct ggml_tensor * pos) {
    const int64_t NOPE = 128, ROPE = 64, LORA = 512;
    struct ggml_tensor * q_nope = ggml_view_3d(c, tq, NOPE, H, n_tok, ggml_row_size(tq->type, NOPE + ROPE), ggml_row_size(tq->type, (NOPE + ROPE) * H), 0);
    struct ggml_tensor * q_pe   = ggml_view_3d(c, tq, ROPE, H, n_tok, ggml_row_size(tq->type, NOPE + ROPE), ggml_row_size(tq->type, (NOPE + ROPE) * H),
                                               ggml_row_size(tq->type, NOPE));
    struct ggml_tensor * wk_b   = ggml_view_3d(c, tw, NOPE, LORA, H, ggml_row_size(tw->type, NOPE), ggml_row_size(tw->type, NOPE * LORA), 0);
    if (pos) q_pe = layer_rope(c, q_pe, pos);
    q_nope = ggml_mul_mat(c, wk_b, ggml_permute(c, q_nope, 0, 2, 1, 3));
    return ggml_concat(c, q_nope, ggml_permute(c, q_pe, 0, 2, 1, 3), 0); /* [576, n_tok, H] */
}

static struct ggml_tensor * layer_unabsorb(struct ggml_context * c, struct ggml_tensor * kqv /* [512, n_tok, H] */, struct ggml_tensor * tw, int64_t H, int64_t n_tok) {
    const int64_t NOPE = 128, LORA = 512, DV = 128;
    struct ggml_tensor * wv_b = ggml_view_3d(c, tw, LORA, DV, H, ggml_row_size(tw->type, LORA), ggml_row_size(tw->type, LORA * DV),
                                             ggml_row_size(tw->type, LORA * NOPE * H));
    struct ggml_tensor * o = ggml_mul_mat(c, wv_b, kqv);
    return ggml_cont_2d(c, ggml_permute(c, o, 0, 2, 1, 3), DV * H, n_tok);
}

int ref_mla_layer(const char * so_path, int mode, int k_type, int v_type, int w_type, int64_t H, int64_t n_ctx, int n_steps,
                  const int32_t * n_tok_s, const int32_t * kv_head_s, const float * q, const float * kv_cur, const void * wkv_b,
                  float kq_scale, const int32_t * block_table, int64_t max_blocks, float * out, int32_t * on_backend,
                  void * cache_out, int n_threads) {
    const int64_t D = 576, LORA = 512, QW = 192, DV = 128;
    const enum ggml_type kt = (enum ggml_type) k_type, vt = (enum ggml_type) v_type, wt = (enum ggml_type) w_type;
    /* mode | 8: the rotary embedding is part of the graph, as in the model's graph: q_pe and the last 64 values of the kv_cur
     * rows arrive unrotated, positions kv_head .. in an I32 tensor, q_pe = rope(cont(view)), k_pe = rope(cont(view)),
     * kv_states = concat(view of the 512 latent values, view_2d(k_pe)) is what goes into the K / latent cache
     * (src/llama-graph-deepseek2.cpp:216-236); on_backend bit 5 = every ROPE ran on the loaded backend */
    const int rope_in_graph = (mode & 8) != 0;
    mode &= 7;
    if (mode < 0 || mode > 2 || (mode == 2 && (!block_table || n_ctx % 128))) return -1;
    ggml_backend_t be = NULL, cpu = NULL;
    if (mode == 0) {
        be = ggml_backend_cpu_init();
        if (be) ggml_backend_cpu_set_n_threads(be, n_threads);
    } else {
        ggml_backend_reg_t reg = ggml_backend_load(so_path);
        if (!reg) return -10;
        if (ggml_backend_reg_dev_count(reg) < 1) return -11;
        be  = ggml_backend_dev_init(ggml_backend_reg_dev_get(reg, 0), NULL);
        cpu = ggml_backend_init_by_type(GGML_BACKEND_DEVICE_TYPE_CPU, NULL);
        if (!cpu) { if (be) ggml_backend_free(be); return -15; }
    }
    if (!be) return -12;
    int                   rc = 0;
    ggml_backend_sched_t  sched = NULL;
    struct ggml_context * g = NULL;
    /* the cache(s) and the weight live in the executor's buffer for the whole run (src/llama-kv-cache.cpp:82-90, :153-158) */
    struct ggml_init_params ipk = { ggml_tensor_overhead() * 8, NULL, true };
    struct ggml_context *   ck  = ggml_init(ipk);
    struct ggml_tensor *    k_l = ggml_new_tensor_1d(ck, kt, D * n_ctx);
    struct ggml_tensor *    v_l = mode == 0 ? ggml_new_tensor_1d(ck, vt, LORA * n_ctx) : NULL;
    struct ggml_tensor *    tw  = ggml_new_tensor_2d(ck, wt, LORA, H * (128 + DV));
    ggml_backend_buffer_t   bufk = ggml_backend_alloc_ctx_tensors(ck, be);
    if (!bufk) { rc = -18; goto done; }
    ggml_backend_buffer_clear(bufk, 0);
    ggml_backend_tensor_set(tw, wkv_b, 0, ggml_nbytes(tw));
    if (mode != 0) {
        ggml_backend_t             backends[2] = { be, cpu };
        ggml_backend_buffer_type_t bufts[2]    = { ggml_backend_get_default_buffer_type(be), ggml_backend_get_default_buffer_type(cpu) };
        sched = ggml_backend_sched_new(backends, bufts, 2, GGML_DEFAULT_GRAPH_SIZE, false);
        if (!sched) { rc = -16; goto done; }
    }

    for (int s = 0; s < n_steps; s++) {
        const int64_t n_tok = n_tok_s[s], kv_head = kv_head_s[s];
        int64_t       n_kv  = GGML_PAD(kv_head + n_tok, 32); /* llama_kv_cache_get_padding without flash attention */
        if (n_kv > n_ctx) n_kv = n_ctx;
        if (kv_head + n_tok > n_ctx || (mode == 2 && kv_head + n_tok > max_blocks * 128)) { rc = -2; goto done; }
        struct ggml_init_params ip = { ggml_tensor_overhead() * 128 + ggml_graph_overhead(), NULL, true };
        g = ggml_init(ip);
        struct ggml_cgraph * gf = ggml_new_graph(g);
        struct layer_io io;
        memset(&io, 0, sizeof(io));
        io.q      = ggml_new_tensor_2d(g, GGML_TYPE_F32, QW * H, n_tok);
        io.kv_cur = ggml_new_tensor_2d(g, GGML_TYPE_F32, D, n_tok);
        ggml_set_input(io.q);
        ggml_set_input(io.kv_cur);
        const int64_t mask_w = mode == 2 ? max_blocks * 128 : n_kv;
        if (mode != 2 || n_tok > 1) {
            io.mask = ggml_new_tensor_2d(g, mode == 0 ? GGML_TYPE_F32 : GGML_TYPE_F16, mask_w, GGML_PAD(n_tok, GGML_KQ_MASK_PAD));
            ggml_set_input(io.mask);
        }
        struct ggml_tensor * kv_states = io.kv_cur;
        if (rope_in_graph) {
            io.pos = ggml_new_tensor_1d(g, GGML_TYPE_I32, n_tok);
            ggml_set_input(io.pos);
            struct ggml_tensor * k_pe = ggml_view_3d(g, io.kv_cur, 64, 1, n_tok, io.kv_cur->nb[1], io.kv_cur->nb[1], ggml_row_size(GGML_TYPE_F32, LORA));
            k_pe = layer_rope(g, k_pe, io.pos);
            k_pe = ggml_view_2d(g, k_pe, 64, n_tok, ggml_row_size(k_pe->type, 64), 0);
            kv_states = ggml_concat(g, ggml_view_2d(g, io.kv_cur, LORA, n_tok, io.kv_cur->nb[1], 0), k_pe, 0);
        }
        struct ggml_tensor * k;
        if (mode == 2) {
            io.idx  = ggml_new_tensor_1d(g, GGML_TYPE_I32, n_tok);
            io.bt   = ggml_new_tensor_2d(g, GGML_TYPE_I32, max_blocks, 1);
            io.lens = ggml_new_tensor_1d(g, GGML_TYPE_I32, 1);
            ggml_set_input(io.idx); ggml_set_input(io.bt); ggml_set_input(io.lens);
            k = io.write = ggml_scatter_update(g, ggml_reshape_2d(g, k_l, D, n_ctx), io.idx, kv_states);
        } else {
            io.write = ggml_cpy(g, kv_states, ggml_view_1d(g, k_l, n_tok * D, ggml_row_size(kt, D) * kv_head));
            ggml_build_forward_expand(gf, io.write);
            k = ggml_view_2d(g, k_l, D, n_kv, ggml_row_size(kt, D), 0);
        }
        struct ggml_tensor * q_states = layer_q_states(g, io.q, tw, H, n_tok, io.pos);
        if (mode == 0) {
            struct ggml_tensor * v_cache_view = ggml_view_2d(g, v_l, n_tok, LORA, n_ctx * ggml_element_size(v_l), kv_head * ggml_element_size(v_l));
            struct ggml_tensor * v_cur        = ggml_transpose(g, ggml_view_2d(g, io.kv_cur, LORA, n_tok, ggml_row_size(GGML_TYPE_F32, D), 0));
            ggml_build_forward_expand(gf, ggml_cpy(g, v_cur, v_cache_view));
            struct ggml_tensor * v  = ggml_view_2d(g, v_l, n_kv, LORA, ggml_element_size(v_l) * n_ctx, 0);
            struct ggml_tensor * q2 = ggml_view_2d(g, q_states, D, H * n_tok, ggml_row_size(GGML_TYPE_F32, D), 0);
            struct ggml_tensor * kq = ggml_mul_mat(g, k, q2);
            ggml_mul_mat_set_prec(kq, GGML_PREC_F32);
            kq = ggml_view_3d(g, kq, n_kv, n_tok, H, ggml_row_size(GGML_TYPE_F32, n_kv), ggml_row_size(GGML_TYPE_F32, n_kv * n_tok), 0);
            kq = ggml_soft_max_ext(g, kq, io.mask, kq_scale, 0.0f);
            kq = ggml_view_2d(g, kq, n_kv, n_tok * H, ggml_row_size(GGML_TYPE_F32, n_kv), 0);
            struct ggml_tensor * kqv = ggml_mul_mat(g, v, kq);
            kqv    = ggml_view_3d(g, kqv, LORA, n_tok, H, ggml_row_size(GGML_TYPE_F32, LORA), ggml_row_size(GGML_TYPE_F32, LORA * n_tok), 0);
            io.out = layer_unabsorb(g, kqv, tw, H, n_tok);
        } else {
            struct ggml_tensor * v = ggml_view_2d(g, k, LORA, k->ne[1], k->nb[1], 0);
            io.fa = ggml_flash_attn_ext(g, q_states, k, v, io.mask, kq_scale, 0.0f, 0.0f);
            ggml_flash_attn_ext_set_prec(io.fa, GGML_PREC_F32);
            io.fa->src[4] = io.bt;
            io.fa->src[5] = io.lens;
            /* [576, H, n_tok]: the first 512 floats of every row, seen as [512, n_tok, H] */
            struct ggml_tensor * kqv = ggml_view_3d(g, io.fa, LORA, H, n_tok, io.fa->nb[1], io.fa->nb[2], 0);
            io.out = layer_unabsorb(g, ggml_permute(g, kqv, 0, 2, 1, 3), tw, H, n_tok);
        }
        ggml_set_output(io.out);
        ggml_build_forward_expand(gf, io.out);

        ggml_backend_buffer_t bufg = NULL;
        if (mode == 0) {
            bufg = ggml_backend_alloc_ctx_tensors(g, be);
            if (!bufg) { rc = -18; goto done; }
        } else {
            ggml_backend_sched_reset(sched);
            if (!ggml_backend_sched_alloc_graph(sched, gf)) { rc = -16; goto done; }
            int32_t where = rope_in_graph ? 0x3c : 0x1c;
            for (int i = 0; i < ggml_graph_n_nodes(gf); i++) {
                struct ggml_tensor * n  = ggml_graph_node(gf, i);
                const int            on = ggml_backend_sched_get_tensor_backend(sched, n) == be;
                if (n == io.write && on) where |= 1;
                if (n == io.fa && on) where |= 2;
                if (n->op == GGML_OP_MUL_MAT && !on) where &= ~4;
                if (n->op == GGML_OP_CONCAT && !on) where &= ~8;
                if (n->op == GGML_OP_CONT && !on) where &= ~16;
                if (n->op == GGML_OP_ROPE && !on) where &= ~32;
            }
            if (on_backend) on_backend[s] = where;
        }
        ggml_backend_tensor_set(io.q, q, 0, ggml_nbytes(io.q));
        ggml_backend_tensor_set(io.kv_cur, kv_cur, 0, ggml_nbytes(io.kv_cur));
        if (io.mask) { /* causal over the cells of this one sequence: cell j holds position j (src/llama-context.cpp:364-404) */
            const int64_t rows = io.mask->ne[1];
            void *        md   = malloc((size_t) rows * mask_w * 4);
            for (int64_t i = 0; i < rows; i++)
                for (int64_t j = 0; j < mask_w; j++) {
                    const int open = i < n_tok && j <= kv_head + i;
                    if (mode == 0) ((float *) md)[i * mask_w + j] = open ? 0.0f : -INFINITY;
                    else ((uint16_t *) md)[i * mask_w + j] = open ? 0 : 0xfc00;
                }
            ggml_backend_tensor_set(io.mask, md, 0, ggml_nbytes(io.mask));
            free(md);
        }
        if (io.pos) {
            int32_t * pp = (int32_t *) malloc(sizeof(int32_t) * n_tok);
            for (int64_t i = 0; i < n_tok; i++) pp[i] = (int32_t) (kv_head + i);
            ggml_backend_tensor_set(io.pos, pp, 0, ggml_nbytes(io.pos));
            free(pp);
        }
        if (mode == 2) {
            int32_t * rows = (int32_t *) malloc(sizeof(int32_t) * n_tok);
            for (int64_t i = 0; i < n_tok; i++) rows[i] = block_table[(kv_head + i) / 128] * 128 + (int32_t) ((kv_head + i) % 128);
            const int32_t len = (int32_t) (kv_head + n_tok);
            ggml_backend_tensor_set(io.idx, rows, 0, ggml_nbytes(io.idx));
            ggml_backend_tensor_set(io.bt, block_table, 0, ggml_nbytes(io.bt));
            ggml_backend_tensor_set(io.lens, &len, 0, sizeof(len));
            free(rows);
        }
        const enum ggml_status st = mode == 0 ? ggml_backend_graph_compute(be, gf) : ggml_backend_sched_graph_compute(sched, gf);
        if (st != GGML_STATUS_SUCCESS) rc = (int) st ? (int) st : -19;
        else ggml_backend_tensor_get(io.out, out, 0, ggml_nbytes(io.out));
        if (bufg) ggml_backend_buffer_free(bufg);
        ggml_free(g);
        g = NULL;
        if (rc) goto done;
        q      += QW * H * n_tok;
        kv_cur += D * n_tok;
        out    += DV * H * n_tok;
    }
    if (cache_out) ggml_backend_tensor_get(k_l, cache_out, 0, ggml_nbytes(k_l));
done:
    if (g) ggml_free(g);
    if (sched) ggml_backend_sched_free(sched);
    if (bufk) ggml_backend_buffer_free(bufk);
    ggml_free(ck);
    if (cpu) ggml_backend_free(cpu);
    ggml_backend_free(be);
    return rc;
}

/* ------------------------------------------------------------------ generated graphs of the nodes around the attention node
 *
 * A graph drawn from `seed` out of the node kinds the model's front uses -- cont of strided views, rope_ext, concat, and the
 * k side's cont -> rope_ext -> view_2d -> concat -> cpy into a cache of kv_type -- over inputs a = f32 [192, H, T], b = f32
 * [576, T], pos = i32 [T]; allocated with the graph allocator (ggml_gallocr: a tensor's memory goes to a later node once
 * its last consumer in node order has run, ggml-alloc.c:553-679), run on the reference's ggml-cpu (so_path NULL) or on the
 * loaded backend.  out: the final f32 [192, H, T] tensor; cache_out: the T cache rows; n_nodes_out: nodes in the graph.
 * Deterministic in (seed, H, T, n_ops, kv_type): two calls build the same graph, whichever executor runs it. */
static uint32_t rg_next(uint32_t * st) { *st = *st * 1664525u + 1013904223u; return *st >> 8; }

int ref_random_front(const char * so_path, uint32_t seed, int64_t H, int64_t T, int n_ops, int kv_type, const float * a_in,
                     const float * b_in, const int32_t * pos_in, float * out, void * cache_out, int32_t * n_nodes_out, int n_threads) {
    ggml_backend_t be = NULL;
    if (so_path) {
        ggml_backend_reg_t reg = ggml_backend_load(so_path);
        if (!reg) return -10;
        if (ggml_backend_reg_dev_count(reg) < 1) return -11;
        be = ggml_backend_dev_init(ggml_backend_reg_dev_get(reg, 0), NULL);
    } else {
        be = ggml_backend_cpu_init();
        if (be) ggml_backend_cpu_set_n_threads(be, n_threads);
    }
    if (!be) return -12;
    int rc = 0;
    const enum ggml_type kt = (enum ggml_type) kv_type;
    struct ggml_init_params ipk = { ggml_tensor_overhead() * 4, NULL, true };
    struct ggml_context *   ck  = ggml_init(ipk);
    struct ggml_tensor *    cache = ggml_new_tensor_1d(ck, kt, 576 * T);
    ggml_backend_buffer_t   bufk = ggml_backend_alloc_ctx_tensors(ck, be);
    struct ggml_init_params ip = { ggml_tensor_overhead() * (size_t) (8 * n_ops + 64) + ggml_graph_overhead(), NULL, true };
    struct ggml_context *   c  = ggml_init(ip);
    struct ggml_cgraph *    gf = ggml_new_graph(c);
    ggml_gallocr_t          ga = NULL;
    if (!bufk) { rc = -13; goto done; }
    ggml_backend_buffer_clear(bufk, 0);
    {
        struct ggml_tensor * ta = ggml_new_tensor_3d(c, GGML_TYPE_F32, 192, H, T);
        struct ggml_tensor * tb = ggml_new_tensor_2d(c, GGML_TYPE_F32, 576, T);
        struct ggml_tensor * tp = ggml_new_tensor_1d(c, GGML_TYPE_I32, T);
        ggml_set_input(ta); ggml_set_input(tb); ggml_set_input(tp);
#define RG_ROPE(x) ggml_rope_ext(c, (x), tp, NULL, 64, 0, 4096, 10000.0f, 0.025f, 1.0f, 0.8f, 32.0f, 1.0f)
#define RG_VIEW(src, w, off) ggml_view_3d(c, (src), (w), H, T, (src)->nb[1], (src)->nb[2], (size_t) (off) * 4)
        enum { CAP = 256 };
        struct ggml_tensor * w64[CAP], * w128[CAP], * w192[CAP];
        int n64 = 0, n128 = 0, n192 = 0;
        uint32_t st = seed * 2654435761u + 12345u;
        w192[n192++] = ta;
        for (int i = 0; i < n_ops && n64 < CAP - 2 && n128 < CAP - 2 && n192 < CAP - 2; i++) {
            int kind = (int) (rg_next(&st) % 8);
            if ((kind == 1 || kind == 3) && n64 == 0) kind = 0;
            if (kind == 4 && (n128 == 0 || n64 == 0)) kind = n64 ? 3 : 0;
            if (kind == 6 && n128 == 0) kind = 5;
            if (n64 >= CAP - 4) break;
            switch (kind) {
                case 0: {   /* cont of a 64-wide view of a wider tensor */
                    const int wide = n128 && (rg_next(&st) & 1);
                    struct ggml_tensor * src = wide ? w128[rg_next(&st) % n128] : w192[rg_next(&st) % n192];
                    const int slots = wide ? 2 : 3;
                    w64[n64++] = ggml_cont(c, RG_VIEW(src, 64, 64 * (rg_next(&st) % slots)));
                    break;
                }
                case 1: w64[n64++] = RG_ROPE(w64[rg_next(&st) % n64]); break;
                case 2: {   /* the model's pair: rope of the cont of a view */
                    struct ggml_tensor * src = w192[rg_next(&st) % n192];
                    w64[n64++] = RG_ROPE(ggml_cont(c, RG_VIEW(src, 64, 64 * (rg_next(&st) % 3))));
                    break;
                }
                case 3: w128[n128++] = ggml_concat(c, w64[rg_next(&st) % n64], w64[rg_next(&st) % n64], 0); break;
                case 4:
                    if (rg_next(&st) & 1) w192[n192++] = ggml_concat(c, w128[rg_next(&st) % n128], w64[rg_next(&st) % n64], 0);
                    else                  w192[n192++] = ggml_concat(c, w64[rg_next(&st) % n64], w128[rg_next(&st) % n128], 0);
                    break;
                case 5: w128[n128++] = ggml_cont(c, RG_VIEW(w192[rg_next(&st) % n192], 128, 64 * (rg_next(&st) % 2))); break;
                case 6: w64[n64++] = RG_ROPE(RG_VIEW(w128[rg_next(&st) % n128], 64, 64 * (rg_next(&st) % 2))); break;   /* rope of a strided view */
                default: {  /* one cont with two consumers, one of which rotates it in place: whichever comes later in node order sees the other's work */
                    struct ggml_tensor * t = ggml_cont(c, RG_VIEW(w192[rg_next(&st) % n192], 64, 64 * (rg_next(&st) % 3)));
                    w64[n64++] = ggml_rope_ext_inplace(c, t, tp, NULL, 64, 0, 4096, 10000.0f, 0.025f, 1.0f, 0.8f, 32.0f, 1.0f);
                    w64[n64++] = RG_ROPE(t);
                    break;
                }
            }
        }
        /* the k side, written into the cache the way llm_attn_mla does it, ahead of the rest (src/llama-graph-attn.cpp:236-241) */
        struct ggml_tensor * k_pe = ggml_view_3d(c, tb, 64, 1, T, tb->nb[1], tb->nb[1], 512 * 4);
        k_pe = RG_ROPE(ggml_cont(c, k_pe));
        k_pe = ggml_view_2d(c, k_pe, 64, T, ggml_row_size(GGML_TYPE_F32, 64), 0);
        struct ggml_tensor * kv_states = ggml_concat(c, ggml_view_2d(c, tb, 512, T, tb->nb[1], 0), k_pe, 0);
        ggml_build_forward_expand(gf, ggml_cpy(c, kv_states, ggml_view_1d(c, cache, 576 * T, 0)));
        /* the result: the three newest tensors of each width, folded into one of 192 */
        struct ggml_tensor * p64  = n64 ? w64[n64 - 1] : ggml_cont(c, RG_VIEW(ta, 64, 128));
        struct ggml_tensor * p128 = n128 ? w128[n128 - 1] : ggml_cont(c, RG_VIEW(ta, 128, 0));
        struct ggml_tensor * res  = ggml_concat(c, p128, p64, 0);
        if (n192 > 1) res = ggml_concat(c, ggml_cont(c, RG_VIEW(w192[n192 - 1], 128, 64)), ggml_cont(c, RG_VIEW(res, 64, 64 * (rg_next(&st) % 3))), 0);
        ggml_set_output(res);
        ggml_build_forward_expand(gf, res);
#undef RG_ROPE
#undef RG_VIEW
        if (n_nodes_out) *n_nodes_out = ggml_graph_n_nodes(gf);
        for (int i = 0; i < ggml_graph_n_nodes(gf); i++)
            if (!ggml_backend_supports_op(be, ggml_graph_node(gf, i))) { rc = -100 - i; goto done; }
        ga = ggml_gallocr_new(ggml_backend_get_default_buffer_type(be));
        if (!ga || !ggml_gallocr_alloc_graph(ga, gf)) { rc = -14; goto done; }
        ggml_backend_tensor_set(ta, a_in, 0, ggml_nbytes(ta));
        ggml_backend_tensor_set(tb, b_in, 0, ggml_nbytes(tb));
        ggml_backend_tensor_set(tp, pos_in, 0, ggml_nbytes(tp));
        const enum ggml_status gs = ggml_backend_graph_compute(be, gf);
        if (gs != GGML_STATUS_SUCCESS) { rc = (int) gs ? (int) gs : -15; goto done; }
        ggml_backend_tensor_get(res, out, 0, ggml_nbytes(res));
        if (cache_out) ggml_backend_tensor_get(cache, cache_out, 0, ggml_nbytes(cache));
    }
done:
    if (ga) ggml_gallocr_free(ga);
    ggml_free(c);
    if (bufk) ggml_backend_buffer_free(bufk);
    ggml_free(ck);
    ggml_backend_free(be);
    return rc;
}

void ref_quantize_q8_0_ref(const float * x, void * y, int64_t k) { quantize_row_q8_0_ref(x, (block_q8_0 *) y, k); }
void ref_quantize_q8_0_cpu(const float * x, void * y, int64_t k) { quantize_row_q8_0(x, y, k); }
void ref_dequantize_q8_0(const void * x, float * y, int64_t k) { dequantize_row_q8_0((const block_q8_0 *) x, y, k); }
void ref_f32_to_f16_row(const float * x, uint16_t * y, int64_t n) { ggml_fp32_to_fp16_row(x, y, n); }
void ref_f32_to_bf16_row(const float * x, uint16_t * y, int64_t n) { ggml_fp32_to_bf16_row(x, (ggml_bf16_t *) y, n); }
void ref_f16_to_f32_row(const uint16_t * x, float * y, int64_t n) { ggml_fp16_to_fp32_row(x, y, n); }

/* sizeof / offsetof / ordinals a drop-in backend has to agree with (ggml.h:597-631, :360-401, :438-549,
 * ggml-backend-impl.h, ggml-impl.h:287-304).  Names are matched by tests/test_abi.py against the mirror. */
struct ref_abi_entry { const char * name; int64_t value; };
#define E(n, v) { n, (int64_t) (v) }
static const struct ref_abi_entry abi_table[] = {
    E("sizeof(ggml_tensor)", sizeof(struct ggml_tensor)),
    E("offsetof(ggml_tensor,type)", offsetof(struct ggml_tensor, type)),
    E("offsetof(ggml_tensor,buffer)", offsetof(struct ggml_tensor, buffer)),
    E("offsetof(ggml_tensor,ne)", offsetof(struct ggml_tensor, ne)),
    E("offsetof(ggml_tensor,nb)", offsetof(struct ggml_tensor, nb)),
    E("offsetof(ggml_tensor,op)", offsetof(struct ggml_tensor, op)),
    E("offsetof(ggml_tensor,op_params)", offsetof(struct ggml_tensor, op_params)),
    E("offsetof(ggml_tensor,flags)", offsetof(struct ggml_tensor, flags)),
    E("offsetof(ggml_tensor,src)", offsetof(struct ggml_tensor, src)),
    E("offsetof(ggml_tensor,view_src)", offsetof(struct ggml_tensor, view_src)),
    E("offsetof(ggml_tensor,view_offs)", offsetof(struct ggml_tensor, view_offs)),
    E("offsetof(ggml_tensor,data)", offsetof(struct ggml_tensor, data)),
    E("offsetof(ggml_tensor,name)", offsetof(struct ggml_tensor, name)),
    E("offsetof(ggml_tensor,extra)", offsetof(struct ggml_tensor, extra)),
    E("GGML_MAX_DIMS", GGML_MAX_DIMS), E("GGML_MAX_SRC", GGML_MAX_SRC), E("GGML_MAX_OP_PARAMS", GGML_MAX_OP_PARAMS),
    E("GGML_MAX_NAME", GGML_MAX_NAME), E("GGML_KQ_MASK_PAD", GGML_KQ_MASK_PAD),
    E("sizeof(ggml_cgraph)", sizeof(struct ggml_cgraph)),
    E("offsetof(ggml_cgraph,n_nodes)", offsetof(struct ggml_cgraph, n_nodes)),
    E("offsetof(ggml_cgraph,nodes)", offsetof(struct ggml_cgraph, nodes)),
    E("sizeof(ggml_backend_buffer_type_i)", sizeof(struct ggml_backend_buffer_type_i)),
    E("sizeof(ggml_backend_buffer_type)", sizeof(struct ggml_backend_buffer_type)),
    E("offsetof(ggml_backend_buffer_type,device)", offsetof(struct ggml_backend_buffer_type, device)),
    E("offsetof(ggml_backend_buffer_type,context)", offsetof(struct ggml_backend_buffer_type, context)),
    E("sizeof(ggml_backend_buffer_i)", sizeof(struct ggml_backend_buffer_i)),
    E("sizeof(ggml_backend_buffer)", sizeof(struct ggml_backend_buffer)),
    E("offsetof(ggml_backend_buffer,buft)", offsetof(struct ggml_backend_buffer, buft)),
    E("offsetof(ggml_backend_buffer,context)", offsetof(struct ggml_backend_buffer, context)),
    E("offsetof(ggml_backend_buffer,size)", offsetof(struct ggml_backend_buffer, size)),
    E("offsetof(ggml_backend_buffer,usage)", offsetof(struct ggml_backend_buffer, usage)),
    E("sizeof(ggml_backend_i)", sizeof(struct ggml_backend_i)),
    E("offsetof(ggml_backend_i,graph_compute)", offsetof(struct ggml_backend_i, graph_compute)),
    E("offsetof(ggml_backend_i,synchronize)", offsetof(struct ggml_backend_i, synchronize)),
    E("sizeof(ggml_backend)", sizeof(struct ggml_backend)),
    E("offsetof(ggml_backend,iface)", offsetof(struct ggml_backend, iface)),
    E("offsetof(ggml_backend,device)", offsetof(struct ggml_backend, device)),
    E("offsetof(ggml_backend,context)", offsetof(struct ggml_backend, context)),
    E("sizeof(ggml_backend_device_i)", sizeof(struct ggml_backend_device_i)),
    E("offsetof(ggml_backend_device_i,supports_op)", offsetof(struct ggml_backend_device_i, supports_op)),
    E("sizeof(ggml_backend_device)", sizeof(struct ggml_backend_device)),
    E("offsetof(ggml_backend_device,reg)", offsetof(struct ggml_backend_device, reg)),
    E("offsetof(ggml_backend_device,context)", offsetof(struct ggml_backend_device, context)),
    E("sizeof(ggml_backend_reg_i)", sizeof(struct ggml_backend_reg_i)),
    E("sizeof(ggml_backend_reg)", sizeof(struct ggml_backend_reg)),
    E("offsetof(ggml_backend_reg,iface)", offsetof(struct ggml_backend_reg, iface)),
    E("offsetof(ggml_backend_reg,context)", offsetof(struct ggml_backend_reg, context)),
    E("sizeof(ggml_backend_dev_props)", sizeof(struct ggml_backend_dev_props)),
    E("offsetof(ggml_backend_dev_props,type)", offsetof(struct ggml_backend_dev_props, type)),
    E("offsetof(ggml_backend_dev_props,caps)", offsetof(struct ggml_backend_dev_props, caps)),
    E("sizeof(ggml_backend_event)", sizeof(struct ggml_backend_event)),
    E("GGML_BACKEND_API_VERSION", GGML_BACKEND_API_VERSION),
    E("GGML_TYPE_F32", GGML_TYPE_F32), E("GGML_TYPE_F16", GGML_TYPE_F16), E("GGML_TYPE_Q8_0", GGML_TYPE_Q8_0),
    E("GGML_TYPE_I8", GGML_TYPE_I8), E("GGML_TYPE_I32", GGML_TYPE_I32), E("GGML_TYPE_BF16", GGML_TYPE_BF16),
    E("GGML_TYPE_COUNT", GGML_TYPE_COUNT),
    E("GGML_OP_NONE", GGML_OP_NONE), E("GGML_OP_CPY", GGML_OP_CPY), E("GGML_OP_CONT", GGML_OP_CONT),
    E("GGML_OP_RESHAPE", GGML_OP_RESHAPE), E("GGML_OP_VIEW", GGML_OP_VIEW), E("GGML_OP_PERMUTE", GGML_OP_PERMUTE),
    E("GGML_OP_TRANSPOSE", GGML_OP_TRANSPOSE), E("GGML_OP_FLASH_ATTN_EXT", GGML_OP_FLASH_ATTN_EXT),
    E("GGML_OP_SCATTER_UPDATE", GGML_OP_SCATTER_UPDATE),
    E("GGML_OP_ROPE", GGML_OP_ROPE), E("GGML_OP_MUL_MAT", GGML_OP_MUL_MAT), E("GGML_OP_CONCAT", GGML_OP_CONCAT), E("GGML_OP_COUNT", GGML_OP_COUNT),
    E("GGML_STATUS_ALLOC_FAILED", GGML_STATUS_ALLOC_FAILED), E("GGML_STATUS_FAILED", GGML_STATUS_FAILED),
    E("GGML_STATUS_SUCCESS", GGML_STATUS_SUCCESS), E("GGML_STATUS_ABORTED", GGML_STATUS_ABORTED),
    E("GGML_BACKEND_DEVICE_TYPE_CPU", GGML_BACKEND_DEVICE_TYPE_CPU), E("GGML_BACKEND_DEVICE_TYPE_GPU", GGML_BACKEND_DEVICE_TYPE_GPU),
    E("GGML_BACKEND_BUFFER_USAGE_ANY", GGML_BACKEND_BUFFER_USAGE_ANY), E("GGML_BACKEND_BUFFER_USAGE_COMPUTE", GGML_BACKEND_BUFFER_USAGE_COMPUTE),
    E("GGML_PREC_DEFAULT", GGML_PREC_DEFAULT), E("GGML_PREC_F32", GGML_PREC_F32),
    E("GGML_TENSOR_FLAG_INPUT", GGML_TENSOR_FLAG_INPUT), E("GGML_TENSOR_FLAG_OUTPUT", GGML_TENSOR_FLAG_OUTPUT),
    E("sizeof(block_q8_0)", sizeof(block_q8_0)),
};
int ref_abi_table(int i, const char ** name, int64_t * value) {
    const int n = (int) (sizeof(abi_table) / sizeof(abi_table[0]));
    if (i < 0 || i >= n) return n;
    *name = abi_table[i].name; *value = abi_table[i].value;
    return n;
}
