"""A small serving loop over the three pieces of the paged path: the host page table decides where tokens go
(include/mla_page_table.h), the cache write puts their latent rows there (include/mla_kv_write.h), the attention node
reads them back through the block table (include/mla_attn.h).  Sequences are prefetched, decoded, forked and dropped;
after every step each sequence's attention output equals the oracle's over that sequence's whole history."""
import numpy as np
import pytest

from oracle import oracle as O
from tests import util as U

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kv_type", [O.TYPE_BF16, O.TYPE_Q8_0])
def test_prefill_decode_fork_drop(gpu, kv_type):
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(77)
    n_pages, n_seq_max, max_blocks, H = 24, 4, 8, 16
    table = J.PageTable(n_pages, n_seq_max, max_blocks)
    row_bytes = 612 if kv_type == O.TYPE_Q8_0 else 1152
    wild = U.encode_kv((rng.standard_normal((n_pages * 128, 576)) * 40).astype(np.float32), kv_type)   # stale finite data everywhere
    cache = torch.from_numpy(wild.view(np.uint8).reshape(n_pages * 128, row_bytes).copy()).to(gpu)
    history = {s: np.zeros((0, 576), np.float32) for s in range(n_seq_max)}    # f32 rows as the model produced them

    def append(batch):
        """batch: {seq: n_new_tokens}; writes their latent rows; returns nothing."""
        seq_id = np.concatenate([np.full(n, s, np.int32) for s, n in batch.items()])
        pos = np.concatenate([np.arange(len(history[s]), len(history[s]) + n, dtype=np.int32) for s, n in batch.items()])
        rows = table.find_slot(seq_id, pos)
        assert rows is not None
        x = rng.standard_normal((len(seq_id), 576)).astype(np.float32)
        J.kv_write(torch.from_numpy(x).to(gpu), cache, kv_type, rows=torch.from_numpy(rows).to(gpu))
        off = 0
        for s, n in batch.items():
            history[s] = np.concatenate([history[s], x[off:off + n]])
            off += n

    def decode_and_check(seqs, what):
        bt, sl = table.fill_inputs(seqs)
        assert list(sl) == [len(history[s]) for s in seqs]
        q = rng.standard_normal((len(seqs), H, 1, 576)).astype(np.float32)
        out = J.ggml_flash_attn_ext(torch.from_numpy(q).to(gpu), cache, kv_type, dv=512, scale=U.SCALE,
                                    block_table=torch.from_numpy(bt).to(gpu), seq_lens=torch.from_numpy(sl).to(gpu))
        torch.cuda.synchronize()
        stored = [O.kv_write(history[s], np.zeros((len(history[s]), row_bytes // (1 if kv_type == O.TYPE_Q8_0 else 2)),
                                                  np.uint8 if kv_type == O.TYPE_Q8_0 else np.uint16), kv_type, np.arange(len(history[s]))) for s in seqs]
        want = U.oracle_per_seq(q, stored, kv_type, 512)
        print(what, U.check(out.cpu().numpy()[..., :512], want, what))

    append({0: 150, 1: 260})                       # two prompts
    decode_and_check([0, 1], "after prefill")
    for step in range(3):                          # decode steps, one token each
        append({0: 1, 1: 1})
        decode_and_check([1, 0], "decode step %d" % step)
    append({2: 100})                               # a third sequence joins
    src_row, dst_row, n = table.seq_cp(1, 3)       # fork sequence 1: full pages shared, the tail rows copied on the device
    assert n == (260 + 3) % 128
    J.kv_write(cache[src_row:src_row + n], cache, kv_type, row0=dst_row)
    history[3] = history[1].copy()
    assert table.seq_rm(0)                         # sequence 0 finishes
    history[0] = np.zeros((0, 576), np.float32)
    for step in range(130):                        # long enough for the fork's tail page to fill and a new page to start
        append({1: 1, 2: 1, 3: 1})
    decode_and_check([3, 2, 1], "after the fork diverged")
    assert table.used_cells == sum(len(h) for h in history.values()) - 256   # the two shared pages count once
