/*
 * Thin C ABI over the hand-written gfx950 kernels for absorbed-MLA attention
 * (GGML_OP_FLASH_ATTN_EXT with 576-d Q.K, a 512- or 576-wide V that is a prefix of the same latent K row,
 * one KV stream shared by all heads).
 *
 * Plain pointers and sizes only: no ggml, torch or HIP types.  All pointers are DEVICE pointers unless said
 * otherwise; `stream` is a hipStream_t passed as void* (NULL = the default stream).  Every function returns 0 on
 * success, a negative MLA_ERR_* code for a rejected argument, or a positive hipError_t value.
 * Nothing here allocates device memory: scratch space comes from the caller (`workspace`).
 *
 * What each entry point replaces in the reference (paths relative to the JittorInfer tree):
 *   mla_attn_launch            the per-node compute of GGML_OP_FLASH_ATTN_EXT,
 *                              ggml/src/ggml-cpu/ggml-cpu.c:11914-12142 (dispatch :14267-14272), i.e. what
 *                              iface.graph_compute (ggml/src/ggml-backend-impl.h:116) runs for that node; the
 *                              operands are those llm_attn_mla defines, src/llama-graph-attn.cpp:259-315.
 *   mla_attn_workspace_size    the per-thread scratch sizing of the same op, ggml-cpu.c:15175-15180.
 *   mla_attn_plan              no counterpart: reports which kernel variant / split the launch will use.
 *   mla_hbm_copy_launch        no counterpart: a plain 16-byte-per-lane copy kernel used to calibrate the
 *                              rocprofv3 FETCH_SIZE / WRITE_SIZE counters against a known byte count.
 */
#ifndef MLA_ATTN_H
#define MLA_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types: the ggml_type ordinals of the reference (ggml/include/ggml.h:360-401) */
#define MLA_TYPE_F32  0
#define MLA_TYPE_F16  1
#define MLA_TYPE_Q8_0 8
#define MLA_TYPE_BF16 30

/* flags */
#define MLA_FLAG_F16_ACC_STRICT 1u /* F16 KV only: replay ggml-cpu's per-key f16 accumulator (ggml-cpu.c:12066-12080)
                                      instead of accumulating in f32; sequential over keys, a correctness mode; over a
                                      contiguous cache or through the block table */
#define MLA_FLAG_Q8_EXACT 16u      /* Q8_0 KV only: the reference's own arithmetic -- Q quantized to Q8_0, integer block dots times
                                      d_q * d_k (ggml-cpu-quants.c:3814-4241), V dequantised to f32 (ggml-quants.c:357-373), f32
                                      accumulator, keys in order -- instead of the matrix-core path, whose operands are q * d rounded to
                                      f16 (q * d has 19 significant bits, f16 keeps 11).  That rounding averages out over many keys
                                      (4.5e-4 relative L2 error at any block scale) but shows in single elements when two or three
                                      keys carry a row: up to 4e-3 against the stated 2e-3 for values of unit variance, more for larger ones.  A correctness mode like the one above,
                                      10 to 100 times slower; without the flag it is taken by itself when no sequence can hold more
                                      than one page of keys, where it costs nothing to speak of. */
#define MLA_FLAG_UNIFORM_SPLITS 2u /* paged decode: give every sequence the same number of equal KV splits (sized for the longest
                                      sequence the block table can hold) instead of the balanced schedule that deals equal
                                      runs of the batch's whole page list to the workgroups, and the sequences of a batch of
                                      more than 256 in batch order instead of longest first; for comparing the two */
#define MLA_FLAG_MASK_EXTENTS_VALID 8u /* masked launch: the workspace still holds the key extents of this mask, left there by the
                                      launch before it, which had the same arguments except q, kv and dst (the attention nodes of
                                      the layers of one graph share their mask, src/llama-graph-deepseek2.cpp:99-103): the scan of
                                      the mask is left out.  The caller vouches for it; nothing else may have used the workspace
                                      in between. */
#define MLA_FLAG_BF16_DIRECT 4u    /* BF16 KV, pipelined kernel: multiply the bf16 tiles as they are, with the probabilities fed as
                                      hi + lo bf16 halves (100 MFMAs per 32 keys).  Without the flag, and with more than 32
                                      attention rows (heads x query tokens) per sequence, the tiles are converted
                                      to f16 inside LDS and the f16 path runs (68 MFMAs): exact for values whose magnitude is
                                      0 or in [2^-14, 65504] (bf16 has fewer mantissa bits than f16), larger ones become
                                      +-65504, smaller ones lose bits below 2^-24; probabilities are rounded to f16.  Set it
                                      for a cache that holds values outside that range. */

/* errors */
#define MLA_ERR_BAD_SHAPE     (-1)
#define MLA_ERR_BAD_TYPE      (-2)
#define MLA_ERR_BAD_ALIGNMENT (-3)
#define MLA_ERR_WORKSPACE     (-4)
#define MLA_ERR_NULL          (-5)
#define MLA_ERR_UNSUPPORTED   (-6)
#define MLA_ERR_TOO_LARGE     (-7) /* mla_attn_launch_static: the call needs more scratch than MLA_ATTN_STATIC_WORKSPACE_MAX */

#define MLA_PAGE_TOKENS 128

typedef struct mla_attn_args {
    /* ---- shapes (ggml names: q ne = {dk, n_tok, n_head, n_seq}) */
    int32_t n_seq;   /* q->ne[3]: sequences in the batch */
    int32_t n_head;  /* q->ne[2]: query heads; all of them read the same K/V rows (MQA broadcast, ggml-cpu.c:11955) */
    int32_t n_tok;   /* q->ne[1]: query tokens per sequence (1 = decode) */
    int32_t dk;      /* q->ne[0] = k->ne[0]: must be 576 */
    int32_t dv;      /* v->ne[0]: 512 (latent prefix) or 576 (V := K, what ggml-cpu requires, ggml-cpu.c:11943) */
    int32_t q_type;  /* MLA_TYPE_F32 (what ggml graphs carry); rounded to K's dot type as ggml-cpu does (:12034-12035) */
    int32_t kv_type; /* MLA_TYPE_BF16 | MLA_TYPE_F16 | MLA_TYPE_Q8_0 */
    uint32_t flags;

    /* ---- op_params of the node (ggml/src/ggml.c:4012-4013) */
    float scale;
    float max_bias;
    float logit_softcap;

    /* ---- Q, byte strides as in ggml (nb0 == 4) */
    const void * q;
    int64_t q_nb1, q_nb2, q_nb3;

    /* ---- latent KV.  V is the first dv columns of the same rows.
     * Without a block table: row `ic` of sequence `b` is at kv + ic*kv_nb1 + b*kv_nb3 and every sequence has n_kv rows.
     * With a block table: kv is the page pool; logical row ic of sequence b is pool row
     *   block_table[b*bt_stride + ic/128]*128 + ic%128 (at kv + row*kv_nb1) and sequence b has seq_lens[b] rows. */
    const void * kv;
    int64_t kv_nb1; /* row stride in bytes: 1152 for f16/bf16, 612 for Q8_0 (18 x 34-byte blocks) when packed */
    int64_t kv_nb3;
    int64_t n_kv;   /* rows per sequence (no block table); with a block table: number of rows in the pool (bounds check) */

    /* ---- optional additive mask, f16 [mask_ne0 >= keys, >= n_tok rows], shared by heads and sequences
     * (src/llama-context.cpp:364-404; ggml-cpu.c:12024,12041-12044: -inf skips the key) */
    const void * mask;
    int64_t mask_nb1;
    int64_t mask_ne0;

    /* ---- optional paged extension (src[4]/src[5] of the node) */
    const int32_t * block_table; /* [n_seq][bt_stride] page ids */
    int64_t bt_stride;           /* ints per sequence (= max pages per sequence) */
    const int32_t * seq_lens;    /* [n_seq] */

    /* ---- output, f32: row (b*n_tok + t)*n_head + h starts at dst + row*dst_nb1 bytes (ggml-cpu.c:12122);
     * dv floats of each row are written */
    float * dst;
    int64_t dst_nb1;

    /* ---- scratch, at least mla_attn_workspace_size() bytes, 256-byte aligned */
    void * workspace;
    size_t workspace_size;

    /* ---- tuning: 0 = choose.  n_splits: KV splits per sequence; rows_per_wg: 32, 64 or 128 rows per workgroup */
    int32_t n_splits;
    int32_t rows_per_wg;
} mla_attn_args;

typedef struct mla_attn_plan_info {
    int32_t variant;      /* 0 = general tiled MFMA kernel, 1 = strict f16-accumulator replay, 2 = pipelined decode kernel */
    int32_t rows_per_wg;  /* (token, head) rows one workgroup owns */
    int32_t n_row_blocks; /* workgroups along rows, per sequence */
    int32_t n_splits;     /* KV splits per sequence (1 = no combine pass) */
    int32_t split_tokens; /* tokens per split */
    int32_t n_passes;     /* passes over d (2 for dv = 576) */
    int64_t lds_bytes;
    int32_t balanced;     /* 1 = paged decode with the balanced schedule: n_workgroups workgroups take equal runs of the batch's
                             page list (n_splits / split_tokens then describe the uniform plan it replaces); 2 = a masked launch
                             over one cache, equal runs of the 32-key tiles its blocks of 128 rows may attend to; 4 = such a
                             launch with few heads (up to 32; 33 to 64 that do not divide 128, or of Q8_0 cells) and at most 256
                             query tokens: issued both in that form and token by token
                             (every query token's rows a workgroup's rows), the device runs the one with fewer tiles to visit */
    int32_t n_workgroups;
} mla_attn_plan_info;

size_t mla_attn_workspace_size(const mla_attn_args * args);
int    mla_attn_plan(const mla_attn_args * args, mla_attn_plan_info * out);
int    mla_attn_launch(const mla_attn_args * args, void * stream);

/* The two halves of mla_attn_launch, for callers that time or schedule them separately: the attention kernel(s)
 * that read the KV rows (writing split-K partials into the workspace, or the final output when the plan has one
 * split), and the log-sum-exp combine pass over the partials (a no-op for one split).  No counterpart in the
 * reference, whose CPU op has no split-K. */
int    mla_attn_launch_partials(const mla_attn_args * args, void * stream);
int    mla_attn_launch_combine(const mla_attn_args * args, void * stream);

/* mla_attn_launch_partials without the small passes that run ahead of the pipelined kernel (the Q operand image and,
 * with a mask, its key extents; the order of the sequences of a large batch): the one kernel that reads the KV rows, alone, for timing it.  Valid only after
 * mla_attn_launch or mla_attn_launch_partials has run with the same arguments and workspace.  No counterpart in
 * the reference. */
int    mla_attn_launch_kernel(const mla_attn_args * args, void * stream);

/* mla_attn_launch with the library's own scratch instead of `workspace` (args->workspace and workspace_size are ignored).
 * No counterpart in the reference.  For callers that cannot allocate device memory around the call: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The scratch is a fixed array of
 * MLA_ATTN_STATIC_WORKSPACE_MAX bytes that every device the library runs on holds until the process ends; a call whose
 * mla_attn_workspace_size() exceeds it returns MLA_ERR_TOO_LARGE (the headline decode step, 32 sequences x 128 heads x 8192
 * keys, needs 43 MB).  Allocates nothing.  All calls on one device share the array: calls that overlap in time on the same
 * device (different streams or threads) race; calls on one stream, or otherwise ordered, do not. */
#define MLA_ATTN_STATIC_WORKSPACE_MAX ((size_t) 48 << 20)
int    mla_attn_launch_static(const mla_attn_args * args, void * stream);

/* dst[i] = src[i] for n_bytes (multiple of 16) */
int mla_hbm_copy_launch(const void * src, void * dst, size_t n_bytes, void * stream);

/* library identification: "gfx950" and a build string; never NULL */
const char * mla_attn_target_arch(void);

#ifdef __cplusplus
}
#endif
#endif /* MLA_ATTN_H */
