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
