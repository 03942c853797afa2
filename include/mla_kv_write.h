/*
 * C ABI of the latent-KV cache write: rows of 576 values (512 latent + 64 rope) of the new tokens are converted to the
 * cache's storage type and written into their cache rows.  Plain pointers and sizes only; all pointers are DEVICE
 * pointers; `stream` is a hipStream_t passed as void* (NULL = the default stream); returns 0, a negative MLA_ERR_*
 * code (include/mla_attn.h) or a positive hipError_t value.  Nothing here allocates.
 *
 * What it replaces in the reference (paths relative to the JittorInfer tree):
 *   mla_kv_write_launch, rows == NULL, block_table == NULL
 *       ggml_cpy(kv_cur, k_cache_view) of llm_attn_mla, src/llama-graph-attn.cpp:236-241: n_tok consecutive cache rows
 *       starting at `row0` (kv_head); on ggml-cpu ggml_compute_forward_dup_f32, ggml/src/ggml-cpu/ggml-cpu.c:3965-4040,
 *       with from_float of the cache type (type_traits_cpu, ggml-cpu.c:269-434): ggml_fp32_to_fp16_row,
 *       ggml_fp32_to_bf16_row (ggml/src/ggml-impl.h:553-568) or quantize_row_q8_0 (ggml-cpu-quants.c:767-900).
 *   mla_kv_write_launch, rows != NULL
 *       ggml_scatter_update(k, indices, k_cur), src/llama-graph-attn.cpp:380-383, constructor ggml/src/ggml.c:3203-3223,
 *       CANN implementation ggml/src/ggml-cann/aclnn_ops.cpp:6052-6129: cache row rows[i] := new row i.
 *   mla_kv_write_launch, block_table != NULL
 *       no counterpart (the reference has no block table): token i of sequence seq_ids[i] at position positions[i] goes
 *       to cache row block_table[seq_ids[i]][positions[i] / 128] * 128 + positions[i] % 128, the addressing the
 *       attention kernels of include/mla_attn.h read with.
 */
#ifndef MLA_KV_WRITE_H
#define MLA_KV_WRITE_H

#include <stddef.h>
#include <stdint.h>

#include "mla_front.h" /* mla_rope_args */

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mla_kv_write_args {
    int32_t n_tok;      /* new rows */
    int32_t src_type;   /* MLA_TYPE_F32 (converted on write), or the cache type itself (rows are copied as they are,
                           what ggml_scatter_update does) */
    int32_t kv_type;    /* MLA_TYPE_BF16 | MLA_TYPE_F16 | MLA_TYPE_Q8_0 */
    int32_t rows_type;  /* type of `rows`: 0 = int32, 1 = int64 (ggml.c:3211 accepts both) */
    const void * src;   /* [n_tok] rows of 576 values */
    int64_t src_nb1;    /* bytes between source rows */
    void *  kv;         /* cache: rows of 576 (1152 bytes bf16/f16, 612 bytes Q8_0 = 18 blocks of fp16 d + 32 int8) */
    int64_t kv_nb1;     /* bytes between cache rows */
    int64_t n_kv_rows;  /* rows in the cache; a destination outside [0, n_kv_rows) is skipped */
    int64_t row0;       /* consecutive mode: first destination row */
    const void * rows;  /* scatter mode: [n_tok] destination rows, or NULL */
    /* paged mode (block_table != NULL): */
    const int32_t * block_table; /* [n_seq][bt_stride] page ids */
    int64_t bt_stride;
    const int32_t * seq_ids;     /* [n_tok] sequence of every new token */
    const int32_t * positions;   /* [n_tok] its position in that sequence */
} mla_kv_write_args;

int mla_kv_write_launch(const mla_kv_write_args * args, void * stream);
/* The argument checks of the launch alone (the value the launch would return before it touches the device), for the
 * plugin's supports_op (the reference's counterpart: ggml_backend_cann_supports_op, ggml/src/ggml-cann/ggml-cann.cpp:1994-2145).
 * Only the low bits of the addresses are looked at. */
int mla_kv_write_check(const mla_kv_write_args * args);

/* The cache write with the rotary embedding of the row's last 64 values folded in: what the DeepSeek-V2 graph spells
 * k_pe = ggml_rope_ext(ggml_cont(k_pe), ...); kv_states = ggml_concat(kv_compressed, k_pe, 0)
 * (src/llama-graph-deepseek2.cpp:226-236) followed by the copy into the cache (src/llama-graph-attn.cpp:236-241), as one
 * pass over the new rows: values 0 .. 511 of row t come from `w.src` (f32 rows; only their first 512 values are read),
 * values 512 .. 575 are rope.src row t ([64, 1, n_tok, 1], f32, 16-byte aligned rows) rotated at rope.pos[t] with the
 * arithmetic of mla_rope_launch (bit-identical to it), then the row is converted and written as mla_kv_write_launch
 * writes it.  rope.n_dims must be 64, rope.mode MLA_ROPE_MODE_NORM (the pairing DeepSeek-V2/V3 use), w.src_type
 * MLA_TYPE_F32; rope.dst is not used: the rotated k_pe exists only in the cache. */
typedef struct mla_kv_write_rope_args {
    mla_kv_write_args w;
    mla_rope_args     rope;
} mla_kv_write_rope_args;

int mla_kv_write_rope_launch(const mla_kv_write_rope_args * args, void * stream);
int mla_kv_write_rope_check(const mla_kv_write_rope_args * args);   /* as mla_kv_write_check */

#ifdef __cplusplus
}
#endif
#endif
