/*
 * Host-side C ABI of the page allocator / block-table builder for the paged latent-KV cache: the bookkeeping the
 * reference does per cell, done per 128-token page, producing the src[4]/src[5] operands of the attention node
 * (include/ggml_mla_backend.h) and the destination rows of the cache write (include/mla_kv_write.h).
 * Plain pointers and sizes; all pointers are HOST pointers; nothing here touches the GPU.
 *
 * What each entry point replaces in the reference (paths relative to the JittorInfer tree):
 *   mla_page_table_create / _free   the cell array of llama_kv_cache_init, src/llama-kv-cache.cpp:25-165 (cells.resize(kv_size))
 *   mla_page_table_clear            llama_kv_cache_clear, src/llama-kv-cache.cpp:167-180
 *   mla_page_table_find_slot        llama_kv_cache_find_slot / llama_kv_cache_find_scatter_slot, src/llama-kv-cache.cpp:347-459:
 *                                   place the tokens of a batch; here a token's cell is fixed by (sequence, position): row =
 *                                   page_of(sequence, position / 128) * 128 + position % 128, pages taken from a free list
 *   mla_page_table_seq_rm           llama_kv_cache_seq_rm, src/llama-kv-cache.cpp:182-240
 *   mla_page_table_seq_cp           llama_kv_cache_seq_cp, :242-283 (whole pages are shared by reference count; a partly
 *                                   filled last page is given to the destination as a fresh page whose rows must be copied:
 *                                   the copy is reported to the caller)
 *   mla_page_table_seq_unshare      no call of its own in the reference: its cells carry a set of sequence ids each
 *                                   (llama_kv_cell::seq_id, src/llama-kv-cache.h:12-27), so removing a suffix of one sequence
 *                                   (:182-240) leaves the other's cells in place and the next find_slot takes other cells; with
 *                                   pages the same sequence of calls -- copy, roll the copy or the source back into the
 *                                   shared prefix, append -- needs the partly used shared page copied first
 *   mla_page_table_seq_keep         llama_kv_cache_seq_keep, :285-313
 *   mla_page_table_seq_add          llama_kv_cache_seq_add, :285-345: the reference marks the cache has_shift, and its next
 *                                   update aborts on that (GGML_ASSERT(!lctx.kv_self.has_shift), "we do not support shift",
 *                                   src/llama-execute-kvupdate.cpp:151-155: the keys in the cache were rotated for their old
 *                                   positions and nothing re-rotates them).  Here the call itself is refused and nothing
 *                                   changes; like the reference's it succeeds when the range holds no cell or delta is 0
 *   mla_page_table_defrag           llama_kv_cache_defrag, :470-475, and the row moves of build_defrag,
 *                                   src/llama-graph-defrag.cpp:23-84 (ggml_cpy of cell runs into the holes that seq_rm left).
 *                                   With pages there is nothing to move: what seq_rm frees are whole pages, which go back to the
 *                                   free list, and any free page serves any sequence through the block table; the only slack
 *                                   is the unused tail of a sequence's last page (under 128 cells per sequence)
 *   mla_page_table_used_cells       llama_get_kv_cache_used_cells, :480-482 (tokens held, shared pages counted once)
 *   mla_page_table_fill_inputs      the mask builder of llama_set_inputs, src/llama-context.cpp:326-447: instead of the
 *                                   O(n_tokens x n_kv) f16 mask it fills the I32 block table [n_seqs][max_blocks] and the I32
 *                                   lengths [n_seqs] that ride in src[4]/src[5] of the FLASH_ATTN_EXT node
 * Return values: 0 on success; MLA_PT_ERR_* (negative) otherwise, and then nothing was changed (the reference restores
 * its cache after a failed find_slot with llama_kv_slot_restorer, src/llama-kv-cache.h:128-170).
 */
#ifndef MLA_PAGE_TABLE_H
#define MLA_PAGE_TABLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MLA_PT_ERR_NO_SPACE   (-1) /* not enough free pages, or a sequence would exceed max_blocks pages */
#define MLA_PT_ERR_BAD_ARG    (-2) /* sequence id out of range, negative position, null pointer */
#define MLA_PT_ERR_NOT_CONTIG (-3) /* a position that neither extends its sequence by one nor overwrites an existing cell */
#define MLA_PT_ERR_UNSUPPORTED (-4) /* seq_rm of a range that is neither a suffix nor the whole sequence; find_slot: overwriting a row of
                                       a page that another sequence maps too, or appending into one (see mla_page_table_seq_unshare);
                                       seq_add that would move a cached position */

typedef struct mla_page_table mla_page_table;

mla_page_table * mla_page_table_create(int32_t n_pages, int32_t n_seq_max, int32_t max_blocks);
void             mla_page_table_free(mla_page_table * t);
void             mla_page_table_clear(mla_page_table * t);

/* Places n_tokens tokens: token i is position pos[i] of sequence seq_id[i].  Tokens of a sequence must come in increasing
 * position order and either overwrite existing positions or extend the sequence without a gap.  rows_out[i] receives the
 * cache row of token i (the `rows` operand of mla_kv_write_launch). */
int mla_page_table_find_slot(mla_page_table * t, int32_t n_tokens, const int32_t * seq_id, const int32_t * pos, int32_t * rows_out);

/* Removes positions [p0, p1) of a sequence (p0 < 0: from 0; p1 < 0: to the end; seq_id < 0: every sequence). */
int mla_page_table_seq_rm(mla_page_table * t, int32_t seq_id, int32_t p0, int32_t p1);

/* Makes positions [0, p1) of src also the content of dst (dst is emptied first; p0 must be <= 0, p1 < 0: to the end).
 * copy_src_row / copy_dst_row / copy_n_rows (each may be NULL) receive the one row run the caller has to copy on the
 * device when the last page is only partly filled (copy_n_rows = 0 when there is none). */
int mla_page_table_seq_cp(mla_page_table * t, int32_t seq_src, int32_t seq_dst, int32_t p0, int32_t p1,
                          int32_t * copy_src_row, int32_t * copy_dst_row, int32_t * copy_n_rows);

/* Gives the sequence a private copy of its last page when that page is only partly used by it (length not a multiple of 128)
 * and other sequences map it too -- the state a seq_cp followed by seq_rm(seq, p0 inside the shared pages) leaves.  Until then
 * find_slot refuses to append to the sequence (MLA_PT_ERR_UNSUPPORTED): the new rows would overwrite the other sequences'.
 * copy_src_row / copy_dst_row / copy_n_rows (each may be NULL) receive the row run the caller copies on the device
 * (copy_n_rows = 0: nothing to do).  MLA_PT_ERR_NO_SPACE when no page is free. */
int mla_page_table_seq_unshare(mla_page_table * t, int32_t seq_id, int32_t * copy_src_row, int32_t * copy_dst_row, int32_t * copy_n_rows);

/* Adds delta to positions [p0, p1) of a sequence: 0 when the range holds no cell or delta == 0, else MLA_PT_ERR_UNSUPPORTED
 * (nothing changed). */
int mla_page_table_seq_add(mla_page_table * t, int32_t seq_id, int32_t p0, int32_t p1, int32_t delta);

/* Compacts the cache: *n_moves (may be NULL) receives the number of row runs the caller has to copy on the device, always 0. */
int mla_page_table_defrag(mla_page_table * t, int32_t * n_moves);

/* Removes every sequence but seq_id. */
int mla_page_table_seq_keep(mla_page_table * t, int32_t seq_id);

int32_t mla_page_table_seq_len(const mla_page_table * t, int32_t seq_id);      /* tokens of a sequence, < 0 on a bad id */
int32_t mla_page_table_free_pages(const mla_page_table * t);
int32_t mla_page_table_used_cells(const mla_page_table * t);

/* Fills block_table[n_seqs][max_blocks] (unused entries 0) and seq_lens[n_seqs] for the given sequences, in order. */
int mla_page_table_fill_inputs(const mla_page_table * t, int32_t n_seqs, const int32_t * seq_ids, int32_t * block_table, int32_t * seq_lens);

#ifdef __cplusplus
}
#endif
#endif
