/*
 * C ABI of the nodes either side of the MLA attention node: the rotary embedding of q_pe / k_pe, the batched "absorb"
 * products (q_nope x wk_b before the node, wv_b x kqv after it) and the strided copies that ggml_cont / ggml_concat
 * stand for.  Plain pointers and sizes only; all pointers are DEVICE pointers; strides are in BYTES and follow ggml's
 * ne/nb order (index 0 = the contiguous dimension); `stream` is a hipStream_t passed as void* (NULL = the default
 * stream); returns 0, a negative MLA_ERR_* code (include/mla_attn.h) or a positive hipError_t value.  Nothing here
 * allocates.
 *
 * What it replaces in the reference (paths relative to the JittorInfer tree):
 *   mla_rope_launch
 *       ggml_rope_ext(q_pe | k_pe, inp_pos, NULL, n_rot, rope_type, n_ctx_orig, freq_base, freq_scale, ext_factor,
 *       attn_factor, beta_fast, beta_slow), src/llama-graph-deepseek2.cpp:218-233; constructor ggml/src/ggml.c:3413-3449;
 *       on ggml-cpu ggml_compute_forward_rope_f32, ggml/src/ggml-cpu/ggml-cpu.c:10361-10552 (cos/sin cache :10295-10307,
 *       YaRN :10272-10293, correction dims ggml/src/ggml.c:3529-3541).  Modes 0 (adjacent pairs, what DeepSeek-V2/V3 use:
 *       LLAMA_ROPE_TYPE_NORM, src/llama-model.cpp:1345-1350) and 2 (NeoX halves); not mrope / vision.
 *   mla_mul_mat_launch
 *       ggml_mul_mat(wk_b, permute(q_nope)) and ggml_mul_mat(wv_b, kqv) of llm_attn_mla,
 *       src/llama-graph-attn.cpp:264-275, :303-317; on ggml-cpu ggml_compute_forward_mul_mat,
 *       ggml/src/ggml-cpu/ggml-cpu.c:8431-8700: the f32 rows of src1 are rounded to src0's type (vec_dot_type, table
 *       :269-434), products are summed in f32.
 *   mla_copy_f32_launch
 *       ggml_cont (ggml-cpu.c:9441-9445 -> ggml_compute_forward_dup, :4465-4510) of the q_pe / k_pe views and of the
 *       permuted result (ggml_cont_2d, src/llama-graph-attn.cpp:322), and each half of ggml_concat
 *       (src/llama-graph-attn.cpp:277; ggml-cpu.c:6822-6862): f32 elements from a strided source to a strided
 *       destination.
 */
#ifndef MLA_FRONT_H
#define MLA_FRONT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MLA_ROPE_MODE_NORM 0 /* pairs (x[2i], x[2i+1]) */
#define MLA_ROPE_MODE_NEOX 2 /* pairs (x[i], x[i + n_dims/2]) */

typedef struct mla_rope_args {
    const void * src;     /* f32 [ne0, ne1 (heads), ne2 (tokens), ne3] */
    int64_t      ne[4];
    int64_t      src_nb[4]; /* src_nb[0] must be 4 */
    void *       dst;     /* f32, same shape; may be the source itself (in place) */
    int64_t      dst_nb[4]; /* dst_nb[0] must be 4 */
    const int32_t * pos;  /* [ne2] position of every token */
    const float * freq_factors; /* [n_dims/2] or NULL */
    int32_t n_dims;       /* rotated channels (even, <= ne0); the rest is copied */
    int32_t mode;         /* MLA_ROPE_MODE_* */
    int32_t n_ctx_orig;
    float   freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow;
} mla_rope_args;

int mla_rope_launch(const mla_rope_args * args, void * stream);
/* The argument checks of the launch alone (the value the launch would return before it touches the device): what the
 * plugin's supports_op asks, in the place of ggml_backend_cann_supports_op's per-op clauses
 * (ggml/src/ggml-cann/ggml-cann.cpp:1994-2145).  Only the low bits of the addresses are looked at. */
int mla_rope_check(const mla_rope_args * args);

typedef struct mla_mul_mat_args {
    int32_t      w_type;  /* type of src0: MLA_TYPE_F16 | MLA_TYPE_BF16 */
    int32_t      _pad;
    const void * w;       /* src0 [K, N, w_ne2, w_ne3], rows of K contiguous values */
    int64_t      K, N, w_ne2, w_ne3;
    int64_t      w_nb1, w_nb2, w_nb3;
    const void * x;       /* src1 f32 [K, M, ne2, ne3], rows of K contiguous values; ne2 % w_ne2 == 0, ne3 % w_ne3 == 0 */
    int64_t      M, ne2, ne3;
    int64_t      x_nb1, x_nb2, x_nb3;
    void *       dst;     /* f32 [N, M, ne2, ne3] */
    int64_t      d_nb1, d_nb2, d_nb3;
} mla_mul_mat_args;

int mla_mul_mat_launch(const mla_mul_mat_args * args, void * stream);
int mla_mul_mat_check(const mla_mul_mat_args * args);   /* as mla_rope_check */

typedef struct mla_copy_args {
    const void * src;
    void *       dst;
    int64_t      ne[4];
    int64_t      src_nb[4]; /* src_nb[0] and dst_nb[0] must be 4 */
    int64_t      dst_nb[4];
} mla_copy_args;

int mla_copy_f32_launch(const mla_copy_args * args, void * stream);
int mla_copy_f32_check(const mla_copy_args * args);     /* as mla_rope_check */

/* Several independent launches of this header and of include/mla_kv_write.h in one dispatch.  The nodes llm_attn_mla and
 * the DeepSeek-V2 graph put ahead of the attention node of a decode step (src/llama-graph-deepseek2.cpp:216-236,
 * src/llama-graph-attn.cpp:236-277) move a few MB each; as launches of their own each costs 4 - 5 us however little it
 * does, and the reference's graph executor has no counterpart to take that away (ggml_backend_sched hands a backend its
 * nodes as one graph, ggml/src/ggml-backend.cpp:1493-1587; what the backend makes of consecutive nodes is its own
 * business).  The ops of a batch must be independent: none reads or writes memory that another one writes.  The result
 * is that of launching them one after the other, in any order.  Ops whose shape has no form inside the batch kernel (a
 * product with more than 32 rows per matrix: a prefill chunk) are launched on their own by the same call.  All ops are
 * checked before the first is launched: a refused argument block (a negative MLA_ERR_* return) means nothing ran. */
#define MLA_FRONT_ROPE          0 /* args: const mla_rope_args * */
#define MLA_FRONT_MUL_MAT       1 /* const mla_mul_mat_args * */
#define MLA_FRONT_COPY          2 /* const mla_copy_args * */
#define MLA_FRONT_KV_WRITE      3 /* const mla_kv_write_args *      (include/mla_kv_write.h) */
#define MLA_FRONT_KV_WRITE_ROPE 4 /* const mla_kv_write_rope_args * (include/mla_kv_write.h) */
#define MLA_FRONT_BATCH_MAX     8 /* ops per dispatch; a longer list takes several */

typedef struct mla_front_op {
    int32_t      kind;  /* MLA_FRONT_* */
    int32_t      _pad;
    const void * args;
} mla_front_op;

int mla_front_batch_launch(const mla_front_op * ops, int32_t n_ops, void * stream);
int mla_front_batch_check(const mla_front_op * ops, int32_t n_ops);   /* as mla_rope_check, for every op */

#ifdef __cplusplus
}
#endif
#endif
