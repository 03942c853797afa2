// Page allocator and block-table builder of the paged latent-KV cache (host only).  The reference keeps one record per
// cache cell (llama_kv_cell, src/llama-kv-cache.h:12-27) and scans them per step (find_slot, the mask builder); here the
// unit is a page of 128 cells with a reference count, a sequence is a list of pages plus a length, and every operation
// is O(pages touched).

#include "../../include/mla_page_table.h"

#include <algorithm>
#include <vector>

namespace {
constexpr int PAGE = 128;
}

struct mla_page_table {
    int32_t n_pages, n_seq_max, max_blocks;
    std::vector<int32_t> free_list;               // stack of free page ids
    std::vector<int32_t> refcount;                // per page
    std::vector<std::vector<int32_t>> pages;      // per sequence
    std::vector<int32_t> len;                     // per sequence, tokens
};

namespace {

void release_page(mla_page_table * t, int32_t p) {
    if (--t->refcount[p] == 0) t->free_list.push_back(p);
}

// drop the pages of `seq` beyond what `new_len` tokens need
void truncate(mla_page_table * t, int32_t seq, int32_t new_len) {
    const size_t need = (size_t) (new_len + PAGE - 1) / PAGE;
    auto & pg = t->pages[seq];
    while (pg.size() > need) { release_page(t, pg.back()); pg.pop_back(); }
    t->len[seq] = new_len;
}

bool seq_ok(const mla_page_table * t, int32_t s) { return t && s >= 0 && s < t->n_seq_max; }

}  // namespace

extern "C" {

mla_page_table * mla_page_table_create(int32_t n_pages, int32_t n_seq_max, int32_t max_blocks) {
    if (n_pages < 1 || n_seq_max < 1 || max_blocks < 1) return nullptr;
    mla_page_table * t = new mla_page_table;
    t->n_pages = n_pages; t->n_seq_max = n_seq_max; t->max_blocks = max_blocks;
    t->refcount.assign(n_pages, 0);
    t->pages.assign(n_seq_max, {});
    t->len.assign(n_seq_max, 0);
    mla_page_table_clear(t);
    return t;
}

void mla_page_table_free(mla_page_table * t) { delete t; }

void mla_page_table_clear(mla_page_table * t) {
    if (!t) return;
    std::fill(t->refcount.begin(), t->refcount.end(), 0);
    for (auto & p : t->pages) p.clear();
    std::fill(t->len.begin(), t->len.end(), 0);
    t->free_list.clear();
    for (int32_t p = t->n_pages - 1; p >= 0; p--) t->free_list.push_back(p);   // page 0 is handed out first
}

int mla_page_table_find_slot(mla_page_table * t, int32_t n_tokens, const int32_t * seq_id, const int32_t * pos, int32_t * rows_out) {
    if (!t || n_tokens < 0 || (n_tokens > 0 && (!seq_id || !pos || !rows_out))) return MLA_PT_ERR_BAD_ARG;
    // first pass: validate and count the pages needed, without changing anything
    std::vector<int32_t> new_len(t->len);
    for (int32_t i = 0; i < n_tokens; i++) {
        const int32_t s = seq_id[i];
        if (!seq_ok(t, s) || pos[i] < 0) return MLA_PT_ERR_BAD_ARG;
        if (pos[i] > new_len[s]) return MLA_PT_ERR_NOT_CONTIG;
        if (pos[i] == new_len[s]) {
            // appending into a page another sequence also maps (a copy that was rolled back into its shared prefix) would
            // overwrite that sequence's rows: the caller gives the sequence a private tail first (mla_page_table_seq_unshare)
            if (pos[i] == t->len[s] && pos[i] % PAGE != 0 && t->refcount[t->pages[s][pos[i] / PAGE]] > 1) return MLA_PT_ERR_UNSUPPORTED;
            new_len[s]++;
        }
        // pages shared after seq_cp are read-only: overwriting a position inside one is not supported
        else if (pos[i] < t->len[s] && t->refcount[t->pages[s][pos[i] / PAGE]] > 1) return MLA_PT_ERR_UNSUPPORTED;
    }
    int64_t need = 0;
    for (int32_t s = 0; s < t->n_seq_max; s++) {
        const int64_t blocks = (new_len[s] + PAGE - 1) / PAGE;
        if (blocks > t->max_blocks) return MLA_PT_ERR_NO_SPACE;
        need += blocks - (int64_t) t->pages[s].size();
    }
    if (need > (int64_t) t->free_list.size()) return MLA_PT_ERR_NO_SPACE;
    // second pass: commit
    for (int32_t i = 0; i < n_tokens; i++) {
        const int32_t s = seq_id[i];
        if (pos[i] == t->len[s]) {
            if (t->len[s] % PAGE == 0) {
                const int32_t p = t->free_list.back();
                t->free_list.pop_back();
                t->refcount[p] = 1;
                t->pages[s].push_back(p);
            }
            t->len[s]++;
        }
        rows_out[i] = t->pages[s][pos[i] / PAGE] * PAGE + pos[i] % PAGE;
    }
    return 0;
}

int mla_page_table_seq_rm(mla_page_table * t, int32_t seq_id, int32_t p0, int32_t p1) {
    if (!t || seq_id >= t->n_seq_max) return MLA_PT_ERR_BAD_ARG;
    if (p0 < 0) p0 = 0;
    if (seq_id < 0) {
        if (p0 != 0 || p1 >= 0) {
            for (int32_t s = 0; s < t->n_seq_max; s++) if (p1 >= 0 && p1 < t->len[s]) return MLA_PT_ERR_UNSUPPORTED;
        }
        for (int32_t s = 0; s < t->n_seq_max; s++) truncate(t, s, std::min(t->len[s], p0));
        return 0;
    }
    const int32_t n = t->len[seq_id];
    if (p1 < 0 || p1 > n) p1 = n;
    if (p0 >= p1) return 0;
    if (p1 < n) return MLA_PT_ERR_UNSUPPORTED;   // a hole in the middle: positions are implicit in the paged layout
    truncate(t, seq_id, p0);
    return 0;
}

int mla_page_table_seq_cp(mla_page_table * t, int32_t seq_src, int32_t seq_dst, int32_t p0, int32_t p1,
                          int32_t * copy_src_row, int32_t * copy_dst_row, int32_t * copy_n_rows) {
    if (!seq_ok(t, seq_src) || !seq_ok(t, seq_dst) || p0 > 0) return MLA_PT_ERR_BAD_ARG;
    if (copy_n_rows) *copy_n_rows = 0;
    if (seq_src == seq_dst) return 0;
    int32_t n = t->len[seq_src];
    if (p1 >= 0 && p1 < n) n = p1;
    const int32_t full = n / PAGE, tail = n % PAGE;
    if (full + (tail ? 1 : 0) > t->max_blocks) return MLA_PT_ERR_NO_SPACE;
    // pages the destination gives back count as free for this check
    int64_t freed = 0;
    for (int32_t p : t->pages[seq_dst]) if (t->refcount[p] == 1) freed++;
    if (tail && freed + (int64_t) t->free_list.size() < 1) return MLA_PT_ERR_NO_SPACE;
    truncate(t, seq_dst, 0);
    for (int32_t b = 0; b < full; b++) {
        const int32_t p = t->pages[seq_src][b];
        t->refcount[p]++;
        t->pages[seq_dst].push_back(p);
    }
    if (tail) {
        const int32_t p = t->free_list.back();
        t->free_list.pop_back();
        t->refcount[p] = 1;
        t->pages[seq_dst].push_back(p);
        if (copy_src_row) *copy_src_row = t->pages[seq_src][full] * PAGE;
        if (copy_dst_row) *copy_dst_row = p * PAGE;
        if (copy_n_rows) *copy_n_rows = tail;
    }
    t->len[seq_dst] = n;
    return 0;
}

int mla_page_table_seq_unshare(mla_page_table * t, int32_t seq_id, int32_t * copy_src_row, int32_t * copy_dst_row, int32_t * copy_n_rows) {
    if (!seq_ok(t, seq_id)) return MLA_PT_ERR_BAD_ARG;
    if (copy_n_rows) *copy_n_rows = 0;
    const int32_t tail = t->len[seq_id] % PAGE;
    if (tail == 0 || t->pages[seq_id].empty()) return 0;          // the next token opens a fresh page anyway
    const int32_t old = t->pages[seq_id].back();
    if (t->refcount[old] == 1) return 0;                          // already private
    if (t->free_list.empty()) return MLA_PT_ERR_NO_SPACE;
    const int32_t p = t->free_list.back();
    t->free_list.pop_back();
    t->refcount[p] = 1;
    t->refcount[old]--;                                           // (> 0: the other sequences keep it)
    t->pages[seq_id].back() = p;
    if (copy_src_row) *copy_src_row = old * PAGE;
    if (copy_dst_row) *copy_dst_row = p * PAGE;
    if (copy_n_rows) *copy_n_rows = tail;
    return 0;
}

int mla_page_table_seq_add(mla_page_table * t, int32_t seq_id, int32_t p0, int32_t p1, int32_t delta) {
    if (!seq_ok(t, seq_id)) return MLA_PT_ERR_BAD_ARG;
    if (p0 < 0) p0 = 0;
    const int32_t n = t->len[seq_id];
    if (p1 < 0 || p1 > n) p1 = n;
    if (p0 >= p1 || delta == 0) return 0;   // no cell in the range, or nothing to add: the reference returns early too
    return MLA_PT_ERR_UNSUPPORTED;          // a shift of cached positions: the rows hold keys rotated for their old positions
}

int mla_page_table_defrag(mla_page_table * t, int32_t * n_moves) {
    if (!t) return MLA_PT_ERR_BAD_ARG;
    if (n_moves) *n_moves = 0;   // freed cells are whole pages on the free list, and any free page serves any sequence
    return 0;
}

int mla_page_table_seq_keep(mla_page_table * t, int32_t seq_id) {
    if (!seq_ok(t, seq_id)) return MLA_PT_ERR_BAD_ARG;
    for (int32_t s = 0; s < t->n_seq_max; s++) if (s != seq_id) truncate(t, s, 0);
    return 0;
}

int32_t mla_page_table_seq_len(const mla_page_table * t, int32_t seq_id) { return seq_ok(t, seq_id) ? t->len[seq_id] : MLA_PT_ERR_BAD_ARG; }

int32_t mla_page_table_free_pages(const mla_page_table * t) { return t ? (int32_t) t->free_list.size() : MLA_PT_ERR_BAD_ARG; }

int32_t mla_page_table_used_cells(const mla_page_table * t) {
    if (!t) return MLA_PT_ERR_BAD_ARG;
    // tokens held, a page shared by several sequences counted once, by the sequence that uses most of it
    std::vector<int32_t> used(t->n_pages, 0);
    for (int32_t s = 0; s < t->n_seq_max; s++)
        for (size_t b = 0; b < t->pages[s].size(); b++) {
            const int32_t p = t->pages[s][b];
            used[p] = std::max(used[p], std::min<int32_t>(PAGE, t->len[s] - (int32_t) b * PAGE));
        }
    int64_t cells = 0;
    for (int32_t c : used) cells += c;
    return (int32_t) cells;
}

int mla_page_table_fill_inputs(const mla_page_table * t, int32_t n_seqs, const int32_t * seq_ids, int32_t * block_table, int32_t * seq_lens) {
    if (!t || n_seqs < 0 || (n_seqs > 0 && (!seq_ids || !block_table || !seq_lens))) return MLA_PT_ERR_BAD_ARG;
    for (int32_t i = 0; i < n_seqs; i++) if (!seq_ok(t, seq_ids[i])) return MLA_PT_ERR_BAD_ARG;
    for (int32_t i = 0; i < n_seqs; i++) {
        const auto & pg = t->pages[seq_ids[i]];
        int32_t * row = block_table + (int64_t) i * t->max_blocks;
        for (int32_t b = 0; b < t->max_blocks; b++) row[b] = b < (int32_t) pg.size() ? pg[b] : 0;
        seq_lens[i] = t->len[seq_ids[i]];
    }
    return 0;
}

}  // extern "C"
