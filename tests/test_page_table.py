"""The host-side page allocator / block-table builder (include/mla_page_table.h) against a plain Python model of the same
bookkeeping, under random operation sequences, plus its error paths.  No GPU involved."""
import numpy as np
import pytest

import jittorinfer_amd as J

PAGE = 128


class Model:
    """Sequences as lists of (page id) with lengths; pages with reference counts.  Mirrors the documented semantics only."""

    def __init__(self, n_pages, n_seq, max_blocks):
        self.n_pages, self.max_blocks = n_pages, max_blocks
        self.free = list(range(n_pages - 1, -1, -1))
        self.ref = [0] * n_pages
        self.pages = [[] for _ in range(n_seq)]
        self.len = [0] * n_seq

    def _truncate(self, s, n):
        need = (n + PAGE - 1) // PAGE
        while len(self.pages[s]) > need:
            p = self.pages[s].pop()
            self.ref[p] -= 1
            if self.ref[p] == 0:
                self.free.append(p)
        self.len[s] = n

    def find_slot(self, seq_id, pos):
        new_len = list(self.len)
        for s, p in zip(seq_id, pos):
            assert p <= new_len[s]
            if p == new_len[s]:
                new_len[s] += 1
        need = 0
        for s in range(len(self.len)):
            blocks = (new_len[s] + PAGE - 1) // PAGE
            if blocks > self.max_blocks:
                return None
            need += blocks - len(self.pages[s])
        if need > len(self.free):
            return None
        rows = []
        for s, p in zip(seq_id, pos):
            if p == self.len[s]:
                if self.len[s] % PAGE == 0:
                    pg = self.free.pop()
                    self.ref[pg] = 1
                    self.pages[s].append(pg)
                self.len[s] += 1
            rows.append(self.pages[s][p // PAGE] * PAGE + p % PAGE)
        return rows


def _check_same(t, m, n_seq):
    assert t.free_pages == len(m.free)
    bt, sl = t.fill_inputs(np.arange(n_seq))
    for s in range(n_seq):
        assert sl[s] == m.len[s] == t.seq_len(s)
        assert list(bt[s, :len(m.pages[s])]) == m.pages[s]
        assert (bt[s, len(m.pages[s]):] == 0).all()
    owned = [p for s in range(n_seq) for p in m.pages[s]]
    assert len(set(owned)) + len(m.free) == m.n_pages          # every page is free or owned
    assert not (set(owned) & set(m.free))


def test_random_batches_against_the_model():
    rng = np.random.default_rng(1)
    n_pages, n_seq, max_blocks = 40, 6, 12
    t, m = J.PageTable(n_pages, n_seq, max_blocks), Model(n_pages, n_seq, max_blocks)
    for step in range(400):
        op = rng.random()
        if op < 0.75:     # a batch: a few sequences each get a run of new tokens (prefill chunk or decode token)
            seqs = rng.choice(n_seq, size=int(rng.integers(1, 4)), replace=False)
            seq_id, pos = [], []
            for s in seqs:
                n = int(rng.choice([1, 1, 1, 5, 130, 300]))
                seq_id += [int(s)] * n
                pos += list(range(m.len[s], m.len[s] + n))
            order = np.argsort(np.array(seq_id) * 100000 + np.array(pos), kind="stable")
            if rng.random() < 0.5:   # interleave the sequences' tokens, keeping each sequence's order
                order = np.argsort(np.array(pos) * 100 + np.array(seq_id), kind="stable")
            seq_id, pos = [seq_id[i] for i in order], [pos[i] for i in order]
            free_before = t.free_pages
            got, want = t.find_slot(seq_id, pos), m.find_slot(seq_id, pos)
            if want is None:
                assert got is None and t.free_pages == free_before
            else:
                assert list(got) == want
        elif op < 0.9:    # drop a suffix or a whole sequence
            s = int(rng.integers(0, n_seq))
            p0 = int(rng.integers(0, m.len[s] + 1)) if rng.random() < 0.6 else -1
            assert t.seq_rm(s, p0, -1)
            m._truncate(s, max(p0, 0) if p0 >= 0 else 0)
        else:             # overwrite the last token of a sequence (llama re-decodes a position): same row again
            s = int(rng.integers(0, n_seq))
            if m.len[s]:
                r1 = t.find_slot([s], [m.len[s] - 1])
                assert list(r1) == m.find_slot([s], [m.len[s] - 1])
        _check_same(t, m, n_seq)
    assert t.used_cells == sum(m.len)


def test_rows_follow_the_attention_kernels_addressing():
    t = J.PageTable(8, 2, 4)
    rows = t.find_slot([0] * 300 + [1] * 3, list(range(300)) + [0, 1, 2])
    bt, sl = t.fill_inputs([0, 1])
    assert list(sl) == [300, 3]
    pos = np.arange(300)
    assert np.array_equal(rows[:300], bt[0, pos // 128] * 128 + pos % 128)
    assert np.array_equal(rows[300:], bt[1, 0] * 128 + np.arange(3))
    assert len(set(rows.tolist())) == 303


def test_error_paths_leave_the_table_unchanged():
    t = J.PageTable(2, 2, 2)
    assert t.find_slot([0] * 200, list(range(200))) is not None
    free = t.free_pages
    assert t.find_slot([1] * 10, list(range(10))) is None                      # no free page
    assert t.find_slot([0] * 100, list(range(200, 300))) is None               # would need a third block
    assert t.free_pages == free and t.seq_len(0) == 200 and t.seq_len(1) == 0
    with pytest.raises(ValueError):
        t.find_slot([0], [500])                                                 # gap
    with pytest.raises(ValueError):
        t.find_slot([5], [0])                                                   # sequence id out of range
    assert not t.seq_rm(0, 10, 20)                                              # a hole in the middle
    assert t.seq_len(0) == 200
    assert t.seq_rm(-1, -1, -1) and t.free_pages == 2                           # everything


def test_seq_cp_shares_full_pages_and_reports_the_tail_copy():
    t = J.PageTable(10, 3, 5)
    t.find_slot([0] * 300, list(range(300)))
    src_row, dst_row, n = t.seq_cp(0, 1)
    bt, sl = t.fill_inputs([0, 1])
    assert list(sl) == [300, 300]
    assert list(bt[0, :2]) == list(bt[1, :2]) and bt[0, 2] != bt[1, 2]          # two full pages shared, tail page private
    assert (src_row, dst_row, n) == (bt[0, 2] * 128, bt[1, 2] * 128, 44)
    assert t.free_pages == 10 - 4 and t.used_cells == 300 + 44
    with pytest.raises(ValueError):
        t.find_slot([1], [5])                                                   # a shared page is read-only
    assert t.find_slot([1], [300]) is not None                                  # extending the copy goes to its own tail page
    assert t.seq_rm(0) and t.seq_len(0) == 0
    assert t.free_pages == 10 - 3                                               # the shared pages live on with sequence 1
    assert t.seq_keep(2) and t.free_pages == 10


def test_append_after_rolling_back_into_a_shared_page_needs_a_private_copy():
    """seq_cp shares full pages; rolling one of the two sequences back into a shared page and appending again must not
    write into rows the other sequence still maps: find_slot refuses until seq_unshare has given the sequence its own page
    (the reference's per-cell sequence sets make the same sequence of calls safe, src/llama-kv-cache.cpp:182-240, :347-404)."""
    t = J.PageTable(8, 2, 4)
    t.find_slot([0] * 200, list(range(200)))
    t.seq_cp(0, 1)
    bt, sl = t.fill_inputs([0, 1])
    assert bt[0, 0] == bt[1, 0] and list(sl) == [200, 200]
    assert t.seq_rm(0, 100, -1) and t.seq_len(0) == 100          # sequence 0 keeps 100 tokens of the shared page
    free = t.free_pages
    with pytest.raises(ValueError):
        t.find_slot([0], [100])                                   # row 100 of the shared page is sequence 1's position 100
    assert t.free_pages == free and t.seq_len(0) == 100
    src, dst, n = t.seq_unshare(0)
    bt2, sl2 = t.fill_inputs([0, 1])
    assert n == 100 and src == bt[1, 0] * 128 and dst == bt2[0, 0] * 128 and bt2[0, 0] != bt2[1, 0]
    assert t.free_pages == free - 1
    rows = t.find_slot([0], [100])
    assert rows[0] == bt2[0, 0] * 128 + 100
    assert list(t.fill_inputs([1])[0][0, :2]) == list(bt[1, :2])  # sequence 1 is untouched
    assert t.seq_unshare(0) == (0, 0, 0) and t.seq_unshare(1) == (0, 0, 0)   # nothing shared and partly used any more
    # the copy rolled back instead of the source: same rule
    t2 = J.PageTable(8, 2, 4)
    t2.find_slot([0] * 130, list(range(130)))
    t2.seq_cp(0, 1)
    assert t2.seq_rm(1, 64, -1)
    with pytest.raises(ValueError):
        t2.find_slot([1], [64])
    assert t2.seq_unshare(1)[2] == 64 and t2.find_slot([1], [64]) is not None
    # a roll-back to a page boundary needs nothing: the next token opens a fresh page
    t3 = J.PageTable(8, 2, 4)
    t3.find_slot([0] * 300, list(range(300)))
    t3.seq_cp(0, 1)
    assert t3.seq_rm(1, 128, -1) and t3.seq_unshare(1) == (0, 0, 0) and t3.find_slot([1], [128]) is not None


def test_random_copies_and_roll_backs_never_alias_rows():
    """Contents model: every find_slot row gets a fresh value written, seq_cp / seq_unshare copy the row runs they report, and
    after every operation each sequence must still read back exactly what was written at its own positions -- a page shared
    by mistake, or a tail copy left out, shows up as a foreign value."""
    rng = np.random.default_rng(7)
    n_pages, n_seq, max_blocks = 48, 5, 8
    t = J.PageTable(n_pages, n_seq, max_blocks)
    store = np.full(n_pages * PAGE, -1, np.int64)
    want = [[] for _ in range(n_seq)]
    stamp = 0
    refused = 0
    for step in range(600):
        op = rng.random()
        s = int(rng.integers(0, n_seq))
        if op < 0.55:
            n = int(rng.choice([1, 1, 7, 100, 129]))
            if rng.random() < 0.2 and want[s]:
                pos = [len(want[s]) - 1]                      # re-decode the last position
            else:
                pos = list(range(len(want[s]), len(want[s]) + n))
            try:
                rows = t.find_slot([s] * len(pos), pos)
            except ValueError:
                refused += 1                                  # a shared page in the way: take a private copy and try again
                cp = t.seq_unshare(s)
                if cp is None:
                    continue
                a, b, k = cp
                store[b:b + k] = store[a:a + k]
                try:
                    rows = t.find_slot([s] * len(pos), pos)
                except ValueError:                            # an overwrite inside a shared full page stays unsupported
                    assert pos[0] < len(want[s])
                    continue
            if rows is None:
                continue
            for r, p_ in zip(rows, pos):
                stamp += 1
                store[r] = stamp
                if p_ == len(want[s]):
                    want[s].append(stamp)
                else:
                    want[s][p_] = stamp
        elif op < 0.75:
            d = int(rng.integers(0, n_seq))
            cp = None
            try:
                cp = t.seq_cp(s, d)
            except ValueError:
                continue
            if cp is None:
                continue
            a, b, k = cp
            store[b:b + k] = store[a:a + k]
            if d != s:
                want[d] = list(want[s])
        else:
            p0 = int(rng.integers(0, len(want[s]) + 1))
            assert t.seq_rm(s, p0, -1)
            del want[s][p0:]
        bt, sl = t.fill_inputs(np.arange(n_seq))
        for q in range(n_seq):
            assert sl[q] == len(want[q])
            if want[q]:
                pos = np.arange(len(want[q]))
                assert (store[bt[q, pos // PAGE] * PAGE + pos % PAGE] == np.array(want[q])).all(), (step, q)
    assert refused > 0     # the case this test is for did occur


def test_seq_add_and_defrag_counterparts():
    """llama_kv_cache_seq_add (src/llama-kv-cache.cpp:285-345) succeeds without effect when the range holds no cell, and a real
    shift is what the reference aborts on at its next cache update (src/llama-execute-kvupdate.cpp:151-155): refused here, table
    unchanged.  llama_kv_cache_defrag (:470-475): holes are whole pages on the free list, so there is never a row to move."""
    t = J.PageTable(8, 2, 6)
    assert t.find_slot([0] * 300, list(range(300))) is not None
    bt0, lens0 = t.fill_inputs([0, 1])
    assert t.seq_add(0, 300, -1, -7)          # no cell at or past position 300
    assert t.seq_add(0, 50, 50, -7)           # empty range
    assert t.seq_add(0, 0, -1, 0)             # nothing to add
    assert t.seq_add(1, 0, -1, 5)             # an empty sequence
    assert not t.seq_add(0, 100, -1, -50)     # a context shift
    assert not t.seq_add(0, 0, -1, 3)
    bt1, lens1 = t.fill_inputs([0, 1])
    assert np.array_equal(bt0, bt1) and np.array_equal(lens0, lens1) and t.seq_len(0) == 300
    # holes come back as whole pages and are reused as they are: nothing to compact, before or after
    assert t.defrag() == 0
    assert t.seq_rm(0, 130, -1) and t.free_pages == 6
    assert t.find_slot([1] * 700, list(range(700))) is not None and t.free_pages == 0
    assert t.defrag() == 0 and t.seq_len(0) == 130 and t.seq_len(1) == 700
    rows0 = set(t.find_slot([0] * 130, list(range(130))))
    rows1 = set(t.find_slot([1] * 700, list(range(700))))
    assert len(rows0) == 130 and len(rows1) == 700 and not (rows0 & rows1)
