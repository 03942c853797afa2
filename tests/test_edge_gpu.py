"""Edge cases of the attention paths on the GPU (ragged, empty and boundary-length sequences, partial row blocks,
strided Q, garbage in unused table entries) against the oracle, and size-independent properties at BASELINE's full
sizes (page-permutation invariance, split invariance, causal independence)."""
import numpy as np
import pytest

from oracle import oracle as O
from tests import util as U
from tests.test_parity_gpu import _run

pytestmark = pytest.mark.gpu


def _want(q, seqs, k_type, mask=None):
    if k_type == O.TYPE_F16:   # f32 accumulation against ggml-cpu's f16 accumulator: held to the f64 value
        return np.stack([O.flash_attn_ext_f64(q[b:b + 1], k[None], k_type, dv=512, scale=U.SCALE,
                                              mask=None if mask is None else mask[:, :k.shape[0]])[0] if len(k) else
                         np.full((q.shape[2], q.shape[1], 512), np.nan, np.float32) for b, k in enumerate(seqs)])
    outs = []
    for b, k in enumerate(seqs):
        if len(k) == 0:        # no key at all: 0 * (1/0), the reference's NaN row
            outs.append(np.full((q.shape[2], q.shape[1], 512), np.nan, np.float32))
        else:
            outs.append(O.flash_attn_ext(q[b:b + 1], k[None], k_type, dv=512, scale=U.SCALE,
                                         mask=None if mask is None else mask[:, :k.shape[0]])[0])
    return np.stack(outs)


@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_F16, O.TYPE_Q8_0])
@pytest.mark.parametrize("n_splits", [0, 3])
def test_boundary_lengths_and_an_empty_sequence(gpu, k_type, n_splits):
    rng = np.random.default_rng(11)
    lens = [0, 1, 31, 32, 33, 127, 128, 129, 300]
    pool, bt, seqs = U.make_paged(rng, np.maximum(lens, 1), k_type, n_pool_pages=16)
    seqs = [s[:l] for s, l in zip(seqs, lens)]
    bt = np.concatenate([bt, np.full((len(lens), 2), 2 ** 30, np.int32)], axis=1)   # table entries past every sequence: never read
    q = rng.standard_normal((len(lens), 128, 1, 576)).astype(np.float32)
    got = _run(gpu, q, pool, k_type, bt=bt, lens=lens, scale=U.SCALE, n_splits=n_splits)
    print(U.check(got[..., :512], _want(q, seqs, k_type), "boundary lengths"))


@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_Q8_0])
def test_partial_row_blocks(gpu, k_type):
    """48 heads x 5 query tokens = 240 rows: one full block of 128 and one of 112, rows of one token split over blocks."""
    rng = np.random.default_rng(12)
    lens = [260, 200]
    pool, bt, seqs = U.make_paged(rng, lens, k_type)
    q = rng.standard_normal((2, 48, 5, 576)).astype(np.float32)
    got = _run(gpu, q, pool, k_type, bt=bt, lens=lens, scale=U.SCALE)
    print(U.check(got[..., :512], _want(q, seqs, k_type), "partial row blocks"))


def test_partial_row_blocks_masked(gpu):
    rng = np.random.default_rng(13)
    n_tok, n_kv = 5, 384
    q = rng.standard_normal((2, 48, n_tok, 576)).astype(np.float32)
    k = U.encode_kv(rng.standard_normal((2, n_kv, 576)).astype(np.float32), O.TYPE_BF16)
    m = np.where(np.arange(n_kv)[None, :] > 300 + 17 * np.arange(n_tok)[:, None], -np.inf, 0.0).astype(np.float32)
    m[:, ::7] += 0.5
    mask = m.astype(np.float16).view(np.uint16)
    got = _run(gpu, q, k, O.TYPE_BF16, mask=mask, scale=U.SCALE)
    want = O.flash_attn_ext(q, k, O.TYPE_BF16, dv=512, mask=mask, scale=U.SCALE)
    print(U.check(got[..., :512], want, "partial row blocks, masked"))


@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_F16, O.TYPE_Q8_0])
def test_fewer_than_sixteen_rows(gpu, k_type):
    """1, 2, 5, 8 and 15 attention rows per sequence (a model with few heads per device, single-head probes): the pipelined
    kernel takes them too -- the k-split programs without a mask over 16-bit rows, the row-split programs with a mask or over
    Q8_0 rows.  Paged with ragged lengths (an empty sequence among them) and contiguous with a mask that has holes and a
    fully masked row."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(21 + k_type)
    lens = [0, 1, 33, 129, 700, 2048]
    pool, bt, seqs = U.make_paged(rng, np.maximum(lens, 1), k_type)
    seqs = [s[:l] for s, l in zip(seqs, lens)]
    kt = {O.TYPE_BF16: J.MLA_TYPE_BF16, O.TYPE_F16: J.MLA_TYPE_F16, O.TYPE_Q8_0: J.MLA_TYPE_Q8_0}[k_type]
    for n_head, n_tok in ((1, 1), (2, 1), (5, 1), (8, 1), (5, 3), (1, 2)):
        q = rng.standard_normal((len(lens), n_head, n_tok, 576)).astype(np.float32)
        for n_splits in (0, 2):
            got = _run(gpu, q, pool, k_type, bt=bt, lens=lens, scale=U.SCALE, n_splits=n_splits)
            print(n_head, n_tok, n_splits, U.check(got[..., :512], _want(q, seqs, k_type), "fewer than 16 rows, paged"))
        n_kv = 320
        k = U.encode_kv(rng.standard_normal((2, n_kv, 576)).astype(np.float32), k_type)
        m = (rng.standard_normal((n_tok, n_kv)) * 1.5).astype(np.float32)
        m[rng.random((n_tok, n_kv)) < 0.4] = -np.inf
        m[:, 290:] = -np.inf
        if n_tok > 1:
            m[1, :] = -np.inf                                 # a query token that may attend to nothing: NaN rows, like the reference's
        mask = m.astype(np.float16).view(np.uint16)
        q2 = q[:2]
        tq = torch.from_numpy(q2).to(gpu)
        tk = torch.from_numpy(k.view(np.int16) if k.dtype == np.uint16 else k).to(gpu)
        out = torch.empty((2, n_tok, n_head, 576), dtype=torch.float32, device=gpu)
        info = J.plan(tq, tk, kt, dv=512, mask=torch.from_numpy(mask.view(np.float16)).to(gpu), scale=U.SCALE, out=out)
        assert info["variant"] == 2, info                     # the pipelined kernel
        got = _run(gpu, q2, k, k_type, mask=mask, scale=U.SCALE)
        fn = O.flash_attn_ext_f64 if k_type == O.TYPE_F16 else O.flash_attn_ext
        want = fn(q2, k, k_type, dv=512, mask=mask, scale=U.SCALE)
        # (Q8_0 on the matrix cores: the documented 3e-3 of the default path where a few keys carry a row; the same launch with the
        # reference's own arithmetic, MLA_FLAG_Q8_EXACT, meets a hundredth of the stated tolerance)
        print(n_head, n_tok, U.check(got[..., :512], want, "fewer than 16 rows, masked", max_abs=3e-3 if k_type == O.TYPE_Q8_0 else U.MAX_ABS_TOL))
        if k_type == O.TYPE_Q8_0:
            exact = _run(gpu, q2, k, k_type, mask=mask, scale=U.SCALE, flags=J.MLA_FLAG_Q8_EXACT)
            print(U.check(exact[..., :512], want, "fewer than 16 rows, masked, exact", max_abs=2e-5, rel_l2=1e-5))


def test_strided_q(gpu):
    """Q handed over as a permuted view ([seq, tok, head, 576] storage), the layout a fused Q projection would leave."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(14)
    q_store = rng.standard_normal((2, 3, 128, 576)).astype(np.float32)
    k = U.encode_kv(rng.standard_normal((2, 256, 576)).astype(np.float32), O.TYPE_BF16)
    tq = torch.from_numpy(q_store).to(gpu).permute(0, 2, 1, 3)   # [seq, head, tok, 576], non-contiguous
    out = J.ggml_flash_attn_ext(tq, torch.from_numpy(k.view(np.int16)).to(gpu), O.TYPE_BF16, dv=512, scale=U.SCALE)
    torch.cuda.synchronize()
    want = O.flash_attn_ext(np.ascontiguousarray(q_store.transpose(0, 2, 1, 3)), k, O.TYPE_BF16, dv=512, scale=U.SCALE)
    print(U.check(out.cpu().numpy()[..., :512], want, "strided q"))


@pytest.mark.parametrize("H", [128, 64])
def test_full_size_config3_properties(gpu, H):
    """BASELINE configs[2] at full size (B=32, H=128, ctx 8192, bf16 pages; and the same batch at 64 heads, which the two-row-block
    program takes): the output does not depend on where the pages sit in the pool (bit-exact under a permutation of pages + table),
    nor on the number of KV splits (within the f16-partial rounding), and one sequence equals the oracle."""
    import torch
    import jittorinfer_amd as J
    g = torch.Generator(device=gpu)
    g.manual_seed(5)
    B, L = 32, 8192
    pages = B * L // 128
    pool = (torch.randn((pages * 128, 576), generator=g, device=gpu) * 0.5).to(torch.bfloat16).view(torch.int16)
    bt = torch.randperm(pages, generator=g, device=gpu).to(torch.int32).reshape(B, L // 128).contiguous()
    sl = torch.full((B,), L, dtype=torch.int32, device=gpu)
    q = torch.randn((B, H, 1, 576), generator=g, device=gpu)
    base = J.ggml_flash_attn_ext(q, pool, J.MLA_TYPE_BF16, dv=512, scale=U.SCALE, block_table=bt, seq_lens=sl)[..., :512].clone()
    # (a) move every page: new_pool[perm[p]] = pool[p], table entries mapped through perm
    perm = torch.randperm(pages, generator=g, device=gpu)
    pool2 = torch.empty_like(pool)
    pool2.view(pages, 128, 576)[perm] = pool.view(pages, 128, 576)
    bt2 = perm[bt.long()].to(torch.int32).contiguous()
    moved = J.ggml_flash_attn_ext(q, pool2, J.MLA_TYPE_BF16, dv=512, scale=U.SCALE, block_table=bt2, seq_lens=sl)[..., :512]
    assert torch.equal(base, moved)
    # (b) 16 splits instead of the planned 8
    s16 = J.ggml_flash_attn_ext(q, pool, J.MLA_TYPE_BF16, dv=512, scale=U.SCALE, block_table=bt, seq_lens=sl, n_splits=16)[..., :512]
    ma, rl = O.errors(s16.cpu().numpy(), base.cpu().numpy())
    assert ma <= 5e-4 and rl <= 3e-4, (ma, rl)
    # (c) sequence 7 against the oracle
    b = 7
    rows = (bt[b].long()[:, None] * 128 + torch.arange(128, device=gpu)[None, :]).reshape(-1)
    k7 = pool[rows].cpu().numpy().view(np.uint16)[None]
    want = O.flash_attn_ext(q[b:b + 1].cpu().numpy(), k7, O.TYPE_BF16, dv=512, scale=U.SCALE)
    print(U.check(base[b:b + 1].cpu().numpy(), want, "config 3 full size, sequence 7"))


def test_full_size_config5_properties(gpu):
    """BASELINE configs[4] at full size (B=64, H=128, lengths uniform in [2048, 8192], Q8_0 pages with the block scale
    1/32): bit-exact under a permutation of the pages, the balanced page schedule agrees with uniform splits, the
    garbage after every sequence's last token is never read, and one sequence equals the oracle."""
    import torch
    import jittorinfer_amd as J
    g = torch.Generator(device=gpu)
    g.manual_seed(55)
    B, H = 64, 128
    lens = torch.randint(2048, 8193, (B,), generator=g, device=gpu).to(torch.int32)
    nblk = (lens.long() + 127) // 128
    pages, max_blocks = int(nblk.sum()), int(nblk.max())
    qs = torch.clamp(torch.round(torch.randn((pages * 128, 18, 32), generator=g, device=gpu) * 16), -127, 127).to(torch.int8)
    pool = torch.empty((pages * 128, 18, 34), dtype=torch.uint8, device=gpu)
    pool[..., 0], pool[..., 1] = 0x00, 0x28          # f16 1/32, little endian
    pool[..., 2:] = qs.view(torch.uint8)
    pool = pool.reshape(pages * 128, 612)
    ids = torch.randperm(pages, generator=g, device=gpu).to(torch.int32)
    bt = torch.full((B, max_blocks), 2 ** 30, dtype=torch.int32, device=gpu)   # entries past a sequence: never read
    start = torch.cumsum(nblk, 0) - nblk
    for b in range(B):
        bt[b, :int(nblk[b])] = ids[int(start[b]):int(start[b]) + int(nblk[b])]
    q = torch.randn((B, H, 1, 576), generator=g, device=gpu)
    kw = dict(dv=512, scale=U.SCALE)
    info = J.plan(q, pool, J.MLA_TYPE_Q8_0, block_table=bt, seq_lens=lens, **kw)
    assert info["variant"] == 2 and info["balanced"] == 1
    base = J.ggml_flash_attn_ext(q, pool, J.MLA_TYPE_Q8_0, block_table=bt, seq_lens=lens, **kw)[..., :512].clone()
    assert not torch.isnan(base).any()
    # (a) move every page
    perm = torch.randperm(pages, generator=g, device=gpu)
    pool2 = torch.empty_like(pool)
    pool2.view(pages, 128, 612)[perm] = pool.view(pages, 128, 612)
    bt2 = torch.where(bt < pages, perm[bt.clamp(max=pages - 1).long()].to(torch.int32), bt).contiguous()
    moved = J.ggml_flash_attn_ext(q, pool2, J.MLA_TYPE_Q8_0, block_table=bt2, seq_lens=lens, **kw)[..., :512]
    assert torch.equal(base, moved)
    # (b) the rows after every sequence's last token hold other values: same bits
    pool3 = pool.clone().view(pages, 128, 612)
    for b in range(B):
        tail = int(lens[b]) % 128
        if tail:
            pool3[int(bt[b, int(nblk[b]) - 1]), tail:] = 0x7b
    same = J.ggml_flash_attn_ext(q, pool3.view(pages * 128, 612), J.MLA_TYPE_Q8_0, block_table=bt, seq_lens=lens, **kw)[..., :512]
    assert torch.equal(base, same)
    # (c) uniform splits per sequence instead of the balanced page schedule
    uni = J.ggml_flash_attn_ext(q, pool, J.MLA_TYPE_Q8_0, block_table=bt, seq_lens=lens, flags=J.MLA_FLAG_UNIFORM_SPLITS, **kw)[..., :512]
    ma, rl = O.errors(uni.cpu().numpy(), base.cpu().numpy())
    assert ma <= 5e-4 and rl <= 3e-4, (ma, rl)
    # (d) the shortest sequence against the oracle
    b = int(torch.argmin(lens))
    rows = (bt[b, :int(nblk[b])].long()[:, None] * 128 + torch.arange(128, device=gpu)[None, :]).reshape(-1)[:int(lens[b])]
    kb = pool[rows].cpu().numpy()[None]
    want = O.flash_attn_ext(q[b:b + 1].cpu().numpy(), kb, O.TYPE_Q8_0, dv=512, scale=U.SCALE)
    print(U.check(base[b:b + 1].cpu().numpy(), want, "config 5 full size, sequence %d (%d keys)" % (b, int(lens[b]))))


@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_Q8_0])
def test_long_sequences_in_a_pool_beyond_4_gib(gpu, k_type):
    """Sequences of up to 131 072 tokens (1024 pages: sixteen times what one workgroup's page list holds) whose pages lie
    anywhere in a pool of more than 4 GiB, the top page included: byte offsets need 64 bits.  The result equals, bit for
    bit, the same sequences gathered into a compact pool, and the short one equals the oracle."""
    import torch
    import jittorinfer_amd as J
    g = torch.Generator(device=gpu)
    g.manual_seed(97)
    row = 1152 if k_type == O.TYPE_BF16 else 612
    n_pages = (5 << 30) // (128 * row) + 1
    lens = [131072, 70001, 5000]
    nblk = [(l + 127) // 128 for l in lens]
    used = torch.randperm(n_pages - 1, generator=g, device=gpu)[:sum(nblk) - 1]
    used = torch.cat([used, torch.tensor([n_pages - 1], device=gpu)])[torch.randperm(sum(nblk), generator=g, device=gpu)]
    pool = torch.empty((n_pages * 128, row), dtype=torch.uint8, device=gpu)     # pages no sequence owns stay uninitialised
    if k_type == O.TYPE_BF16:
        data = (torch.randn((sum(nblk) * 128, 576), generator=g, device=gpu) * 0.7).to(torch.bfloat16).view(torch.uint8)
    else:
        data = torch.empty((sum(nblk) * 128, 18, 34), dtype=torch.uint8, device=gpu)
        data[..., 0], data[..., 1] = 0x00, 0x28          # f16 1/32, little endian
        data[..., 2:] = torch.clamp(torch.round(torch.randn((sum(nblk) * 128, 18, 32), generator=g, device=gpu) * 16), -127, 127).to(torch.int8).view(torch.uint8)
        data = data.reshape(-1, 612)
    pool.view(n_pages, 128 * row)[used] = data.view(sum(nblk), 128 * row)
    bt = torch.full((3, max(nblk)), -7, dtype=torch.int32, device=gpu)
    bt_small = bt.clone()
    pos = 0
    for b in range(3):
        bt[b, :nblk[b]] = used[pos:pos + nblk[b]].to(torch.int32)
        bt_small[b, :nblk[b]] = torch.arange(pos, pos + nblk[b], dtype=torch.int32, device=gpu)
        pos += nblk[b]
    sl = torch.tensor(lens, dtype=torch.int32, device=gpu)
    q = torch.randn((3, 128, 1, 576), generator=g, device=gpu)
    kt = J.MLA_TYPE_BF16 if k_type == O.TYPE_BF16 else J.MLA_TYPE_Q8_0
    tk = pool.view(torch.int16) if k_type == O.TYPE_BF16 else pool
    td = data.view(torch.int16) if k_type == O.TYPE_BF16 else data
    kw = dict(dv=512, scale=U.SCALE, seq_lens=sl)
    info = J.plan(q, tk, kt, block_table=bt, **kw)
    assert info["variant"] == 2 and info["balanced"] == 1
    big = J.ggml_flash_attn_ext(q, tk, kt, block_table=bt, **kw)[..., :512].clone()
    small = J.ggml_flash_attn_ext(q, td, kt, block_table=bt_small, **kw)[..., :512]
    assert not torch.isnan(big).any() and torch.equal(big, small)
    uni = J.ggml_flash_attn_ext(q, tk, kt, block_table=bt, flags=J.MLA_FLAG_UNIFORM_SPLITS, **kw)[..., :512]
    ma, rl = O.errors(uni.cpu().numpy(), big.cpu().numpy())
    assert ma <= 5e-4 and rl <= 5e-4, (ma, rl)
    k2 = data.view(sum(nblk), 128, row)[nblk[0] + nblk[1]:].reshape(-1, row)[:lens[2]].cpu().numpy()
    if k_type == O.TYPE_BF16:
        k2 = k2.view(np.uint16)
    want = O.flash_attn_ext(q[2:3].cpu().numpy(), k2[None], k_type, dv=512, scale=U.SCALE)
    print(U.check(big[2:3].cpu().numpy(), want, "5000-token sequence in the 5 GiB pool"))


def test_full_size_config4_causal_independence(gpu):
    """BASELINE configs[3] at full size (B=4, H=16, 512 new tokens on 2048 cached, causal mask): query token t must not
    depend on keys after position 2048 + t.  Keys after 2048 + 255 are replaced by other values: the outputs of tokens
    0..255 stay bit-identical, later ones change; the last token's row equals the oracle."""
    import torch
    import jittorinfer_amd as J
    g = torch.Generator(device=gpu)
    g.manual_seed(6)
    B, H, n_new, n_old = 4, 16, 512, 2048
    L = n_new + n_old
    pages = B * L // 128
    pool = torch.randn((pages * 128, 576), generator=g, device=gpu).to(torch.bfloat16).view(torch.int16)
    bt = torch.randperm(pages, generator=g, device=gpu).to(torch.int32).reshape(B, L // 128).contiguous()
    sl = torch.full((B,), L, dtype=torch.int32, device=gpu)
    q = torch.randn((B, H, n_new, 576), generator=g, device=gpu)
    mask = torch.where(torch.arange(L, device=gpu)[None, :] > n_old + torch.arange(n_new, device=gpu)[:, None], float("-inf"), 0.0).to(torch.float16)
    kw = dict(dv=512, scale=U.SCALE, mask=mask, block_table=bt, seq_lens=sl)
    assert J.plan(q, pool, J.MLA_TYPE_BF16, **kw)["variant"] == 2
    base = J.ggml_flash_attn_ext(q, pool, J.MLA_TYPE_BF16, **kw)[..., :512].clone()
    pool2 = pool.clone()
    for b in range(B):
        pos = torch.arange(n_old + 256, L, device=gpu)
        rows = bt[b].long()[pos // 128] * 128 + pos % 128
        pool2[rows] = (torch.randn((len(pos), 576), generator=g, device=gpu) * 3).to(torch.bfloat16).view(torch.int16)
    other = J.ggml_flash_attn_ext(q, pool2, J.MLA_TYPE_BF16, **kw)[..., :512]
    assert torch.equal(base[:, :256], other[:, :256])
    assert not torch.equal(base[:, 256:], other[:, 256:])
    b = 2
    rows = (bt[b].long()[:, None] * 128 + torch.arange(128, device=gpu)[None, :]).reshape(-1)
    kb = pool[rows].cpu().numpy().view(np.uint16)[None]
    mh = mask[-1:].cpu().numpy().view(np.uint16)
    want = O.flash_attn_ext(q[b:b + 1, :, -1:].cpu().numpy(), kb, O.TYPE_BF16, dv=512, mask=mh, scale=U.SCALE)
    print(U.check(base[b:b + 1, -1:].cpu().numpy(), want, "config 4 full size, last token"))


def test_step_replayed_from_a_hip_graph(gpu):
    """mla_attn_launch (Q pre-pack, split-K kernel, combine) captured into a HIP graph: every replay, with eager work and
    synchronisations of the program's own in between and fresh inputs each time, equals the eager result bit for bit."""
    import ctypes as C
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(21)
    lens = [700, 513, 260]
    pool, bt, seqs = U.make_paged(rng, lens, O.TYPE_BF16)
    tq = torch.zeros((3, 128, 1, 576), dtype=torch.float32, device=gpu)
    tk = torch.from_numpy(pool.view(np.int16)).to(gpu)
    tb, tl = torch.from_numpy(bt).to(gpu), torch.tensor(lens, dtype=torch.int32, device=gpu)
    out = torch.zeros((3, 1, 128, 576), dtype=torch.float32, device=gpu)
    a, _, keep = J.capi.make_args(tq, tk, J.MLA_TYPE_BF16, dv=512, scale=U.SCALE, block_table=tb, seq_lens=tl, out=out)
    assert J.plan(tq, tk, J.MLA_TYPE_BF16, dv=512, scale=U.SCALE, block_table=tb, seq_lens=tl, out=out)["n_splits"] > 1
    lib = J.library()
    side = torch.cuda.Stream(gpu)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        graph.capture_begin()
        assert lib.mla_attn_launch(C.byref(a), C.c_void_p(side.cuda_stream)) == 0
        graph.capture_end()
    torch.cuda.synchronize()
    for it in range(4):
        q = rng.standard_normal((3, 128, 1, 576)).astype(np.float32)
        tq.copy_(torch.from_numpy(q).to(gpu))
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replayed = out.clone()
        out.fill_(float("nan"))
        J.ggml_flash_attn_ext(tq, tk, J.MLA_TYPE_BF16, dv=512, scale=U.SCALE, block_table=tb, seq_lens=tl, out=out)   # eager
        torch.cuda.synchronize()
        assert torch.equal(replayed[..., :512], out[..., :512]), "replay %d differs from the eager launch" % it
        if it == 0:
            print(U.check(out.cpu().numpy()[..., :512], U.oracle_per_seq(q, seqs, O.TYPE_BF16, 512), "graph replay"))


def test_graph_replay_with_sequence_lengths_changed_on_the_device(gpu):
    """The balanced page schedule is built on the device from seq_lens at every launch, so a captured launch follows
    lengths that change between replays (a serving loop appends a token per step and swaps sequences in and out): every
    replay equals the eager launch bit for bit and the oracle on the current prefixes, lengths of 0 included."""
    import ctypes as C
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(77)
    n_seq, cap = 24, 1536   # 24 x 12 pages: more than one page per workgroup, so the balanced schedule is planned
    pool, bt, seqs = U.make_paged(rng, [cap] * n_seq, O.TYPE_BF16)
    tq = torch.zeros((n_seq, 128, 1, 576), dtype=torch.float32, device=gpu)
    tk = torch.from_numpy(pool.view(np.int16)).to(gpu)
    tb = torch.from_numpy(bt).to(gpu)
    tl = torch.full((n_seq,), cap, dtype=torch.int32, device=gpu)
    out = torch.zeros((n_seq, 1, 128, 512), dtype=torch.float32, device=gpu)
    kw = dict(dv=512, scale=U.SCALE, block_table=tb, seq_lens=tl, out=out)
    a, _, keep = J.capi.make_args(tq, tk, J.MLA_TYPE_BF16, **kw)
    assert J.plan(tq, tk, J.MLA_TYPE_BF16, **kw)["balanced"] == 1
    lib = J.library()
    side = torch.cuda.Stream(gpu)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        graph.capture_begin()
        assert lib.mla_attn_launch(C.byref(a), C.c_void_p(side.cuda_stream)) == 0
        graph.capture_end()
    torch.cuda.synchronize()
    steps = [rng.integers(1, cap + 1, n_seq), np.full(n_seq, cap), rng.integers(0, 260, n_seq),
             np.where(np.arange(n_seq) % 3 == 0, 0, rng.integers(1, cap + 1, n_seq)), np.full(n_seq, 1)]
    for it, lens in enumerate(steps):
        q = rng.standard_normal((n_seq, 128, 1, 576)).astype(np.float32)
        tq.copy_(torch.from_numpy(q).to(gpu))
        tl.copy_(torch.from_numpy(lens.astype(np.int32)).to(gpu))
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replayed = out.clone()
        out.fill_(float("nan"))
        J.ggml_flash_attn_ext(tq, tk, J.MLA_TYPE_BF16, **kw)
        torch.cuda.synchronize()
        assert torch.equal(replayed.view(torch.int32), out.view(torch.int32)), "replay %d differs from the eager launch" % it
        got = replayed.cpu().numpy()
        some = list(range(6))
        want = U.oracle_per_seq(q[some], [seqs[b][:lens[b]] for b in some], O.TYPE_BF16, 512)
        print(it, U.check(got[some], want, "replay %d" % it))


@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_F16, O.TYPE_Q8_0])
@pytest.mark.parametrize("n_splits", [0, 1, 5])
def test_reference_style_batched_decode_through_the_mask(gpu, k_type, n_splits):
    """The reference's own decode batch (no block table): one shared cache, one query token per sequence, and the f16 mask
    (src/llama-context.cpp:364-404) selects every token's own cells.  The pipelined kernel visits only the key range a
    token's mask leaves open and divides that range into the KV splits."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(31 + n_splits)
    lens = [300, 512, 77, 1024, 5, 640, 128, 900]
    order = rng.permutation(len(lens))
    n_kv, start = 4352, {}
    pos = 17
    for s in order:                       # sequences sit in the cache in shuffled order with gaps between them
        start[s] = pos
        pos += lens[s] + int(rng.integers(0, 40))
    assert pos <= n_kv
    # (Q8_0 cells with one power-of-two block scale, as BASELINE's config 5 builds them: with arbitrary scales the f16 MFMA
    # operand alone costs a 5-key sequence up to 2^-11 |v| = 2.1e-3 in single elements)
    q8s = 1.0 / 32 if k_type == O.TYPE_Q8_0 else None
    k = U.encode_kv((rng.standard_normal((1, n_kv, 576)) * 30).astype(np.float32), k_type, q8_scale=q8s)   # other cells: wild values
    m = np.full((len(lens), n_kv), -np.inf, dtype=np.float32)
    for s, l in enumerate(lens):
        k[0, start[s]:start[s] + l] = U.encode_kv(rng.standard_normal((l, 576)).astype(np.float32), k_type, q8_scale=q8s)
        m[s, start[s]:start[s] + l] = 0.0
    m[3, start[3] + 100:start[3] + 400] = -np.inf       # a hole inside a sequence (cells of a removed span)
    mask = m.astype(np.float16).view(np.uint16)
    q = rng.standard_normal((1, 128, len(lens), 576)).astype(np.float32)
    tq = torch.from_numpy(q).to(gpu)
    tk = torch.from_numpy(k.view(np.int16) if k.dtype == np.uint16 else k).to(gpu)
    tm = torch.from_numpy(mask.view(np.float16)).to(gpu)
    info = J.plan(tq, tk, k_type, dv=512, scale=U.SCALE, mask=tm, n_splits=n_splits)
    assert info["variant"] == 2 and info["balanced"] == (2 if n_splits == 0 else 0)   # 0: the tiles of the 8 key ranges dealt out evenly
    got = _run(gpu, q, k, k_type, mask=mask, scale=U.SCALE, n_splits=n_splits)
    if n_splits == 0:
        uni = _run(gpu, q, k, k_type, mask=mask, scale=U.SCALE, flags=J.MLA_FLAG_UNIFORM_SPLITS)
        assert float(np.nanmax(np.abs(uni[..., :512] - got[..., :512]))) < 2e-3
    if k_type == O.TYPE_F16:
        want = O.flash_attn_ext_f64(q, k, k_type, dv=512, mask=mask, scale=U.SCALE)
    else:
        want = O.flash_attn_ext(q, k, k_type, dv=512, mask=mask, scale=U.SCALE)
    print(U.check(got[..., :512], want, "batched decode through the mask"))


@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_F16, O.TYPE_Q8_0])
@pytest.mark.parametrize("n_head,n_tok", [(16, 32), (32, 64), (24, 37), (16, 256), (8, 16), (16, 3), (16, 20), (1, 200), (64, 32), (48, 21), (40, 2)])
def test_few_heads_masked_launch_issued_in_two_forms(gpu, k_type, n_head, n_tok):
    """A masked launch over one cache with at most 32 heads and at most 256 query tokens is issued both as row blocks of 128
    rows and token by token (every token a sequence of n_head rows); the device runs the form with fewer tiles to visit.
    Three masks over the same cache and queries: a decode batch (every token its own cells, shuffled, with gaps, one token
    without any cell -> NaN rows, one with a hole) where the token form runs; a prompt chunk (causal over one sequence) where
    the row-block form runs; two sequences with half of the tokens each.  24 heads: tokens straddle the row blocks.  Up to 32 heads
    of 16-bit cells the token form is the k-split program; 33 to 64 heads, and Q8_0 cells (one power-of-two block scale, as in
    BASELINE's config 5), run the row-split program of the cache type on an operand image written token by token."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(1000 * n_head + n_tok)
    n_kv = 4096
    k = U.encode_kv(rng.standard_normal((1, n_kv, 576)).astype(np.float32), k_type, q8_scale=1.0 / 32 if k_type == O.TYPE_Q8_0 else None)
    q = rng.standard_normal((1, n_head, n_tok, 576)).astype(np.float32)
    masks = {}
    m = np.full((n_tok, n_kv), -np.inf, dtype=np.float32)       # decode batch
    pos, budget = 5, n_kv // n_tok
    for t in rng.permutation(n_tok):
        l = int(rng.integers(1, budget - 2))
        if t != 1:
            m[t, pos:pos + l] = 0.0
        pos += l + int(rng.integers(0, 3))
    t_hole = int(np.argmax((m == 0).sum(1)))
    cells = np.flatnonzero(m[t_hole] == 0)
    if len(cells) > 4:
        m[t_hole, cells[1]:cells[len(cells) // 2]] = -np.inf
    masks["decode batch"] = m
    m = np.full((n_tok, n_kv), -np.inf, dtype=np.float32)       # prompt chunk: token t sees cells 100 .. 100 + past + t
    past = 1500
    for t in range(n_tok):
        m[t, 100:100 + past + t + 1] = 0.0
    masks["prompt chunk"] = m
    m = np.full((n_tok, n_kv), -np.inf, dtype=np.float32)       # two sequences, each a chunk of half of the tokens
    for t in range(n_tok):
        first = t < n_tok // 2
        base, i = (64, t) if first else (2200, t - n_tok // 2)
        m[t, base:base + 700 + i + 1] = 0.0
    masks["two sequences"] = m
    tq, tk = torch.from_numpy(q).to(gpu), torch.from_numpy(k.view(np.int16) if k.dtype == np.uint16 else k).to(gpu)
    for what, m in masks.items():
        mask = m.astype(np.float16).view(np.uint16)
        tm = torch.from_numpy(mask.view(np.float16)).to(gpu)
        info = J.plan(tq, tk, k_type, dv=512, scale=U.SCALE, mask=tm)
        one_form = n_head == 64 and k_type != O.TYPE_Q8_0          # (a row block of 16-bit cells is two tokens exactly: nothing to gain)
        assert info["variant"] == 2 and info["balanced"] == (2 if one_form else 4)     # 4: both forms are launched
        got = _run(gpu, q, k, k_type, mask=mask, scale=U.SCALE)
        want = (O.flash_attn_ext_f64 if k_type == O.TYPE_F16 else O.flash_attn_ext)(q, k, k_type, dv=512, mask=mask, scale=U.SCALE)
        if what == "decode batch":
            assert np.isnan(want[0, 1]).all()
        # (Q8_0: Q as d * q rounded to the f16 MFMA operand moves a logit by up to 1e-3, which a token with a handful of cells and V
        # values several units apart turns into up to 2.5e-3 in single elements, rel-L2 near 3e-4: 3e-3 there, as in the random sweep)
        print(what, U.check(got[..., :512], want, what, max_abs=3e-3 if k_type == O.TYPE_Q8_0 else U.MAX_ABS_TOL))
        if k_type == O.TYPE_Q8_0:                                   # the same launch in the reference's own arithmetic
            exact = _run(gpu, q, k, k_type, mask=mask, scale=U.SCALE, flags=J.MLA_FLAG_Q8_EXACT)
            print(what, U.check(exact[..., :512], want, what + ", exact", max_abs=2e-5, rel_l2=1e-5))
    if n_tok == 32:                                                # the 576-wide V: both forms in each of the two passes
        mask = masks["decode batch"].astype(np.float16).view(np.uint16)
        got = _run(gpu, q, k, k_type, dv=576, mask=mask, scale=U.SCALE)
        want = (O.flash_attn_ext_f64 if k_type == O.TYPE_F16 else O.flash_attn_ext)(q, k, k_type, dv=576, mask=mask, scale=U.SCALE)
        print(U.check(got, want, "V := K", max_abs=3e-3 if k_type == O.TYPE_Q8_0 else U.MAX_ABS_TOL))


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_masked_launches_over_one_cache(gpu, seed):
    """Randomised masked launches over one contiguous cache (the reference's own graph form): 1 to 128 heads, 1 to 300 query
    tokens, every token a window of its own (some empty -> NaN rows, some with a hole), windows of neighbouring tokens disjoint,
    nested or overlapping at random -- which decides whether the launch runs as row blocks or token by token, with equal runs
    of the tile list or with workgroups of its own for every item -- bf16 and f16 cells, both V widths."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(4242 + seed)
    seen = set()
    for case in range(14):
        n_head = int(rng.choice([1, 3, 8, 16, 16, 24, 32, 32, 48, 64, 128]))
        n_tok = int(rng.choice([1, 2, 5, 8, 17, 32, 64, 100, 300])) if n_head <= 32 else int(rng.choice([1, 2, 5, 8, 17]))
        n_kv = 32 * int(rng.integers(4, 129))
        k_type = O.TYPE_BF16 if rng.integers(2) else O.TYPE_F16
        dv = 576 if rng.integers(5) == 0 else 512
        style = int(rng.integers(3))      # 0: decode batch (disjoint windows), 1: prompt chunk (nested windows), 2: anything
        m = np.full((n_tok, n_kv), -np.inf, dtype=np.float32)
        for t in range(n_tok):
            if rng.integers(12) == 0:
                continue
            if style == 0:
                w = max(1, n_kv // n_tok)
                lo, hi = t * w + int(rng.integers(0, max(1, w // 3))), (t + 1) * w
            elif style == 1:
                lo, hi = 7, min(n_kv, max(8, n_kv - n_tok + t))
            else:
                lo = int(rng.integers(0, n_kv)); hi = min(n_kv, lo + int(rng.integers(1, n_kv)))
            hi = min(max(hi, lo + 1), n_kv)
            m[t, lo:hi] = (rng.standard_normal(hi - lo) * 0.5).astype(np.float32) if rng.integers(3) == 0 else 0.0
            if hi - lo > 6 and rng.integers(4) == 0:
                m[t, lo + 2:lo + 2 + (hi - lo) // 2] = -np.inf
        mask = m.astype(np.float16).view(np.uint16)
        q = rng.standard_normal((1, n_head, n_tok, 576)).astype(np.float32)
        k = U.encode_kv(rng.standard_normal((1, n_kv, 576)).astype(np.float32), k_type)
        tq, tk = torch.from_numpy(q).to(gpu), torch.from_numpy(k.view(np.int16)).to(gpu)
        tm = torch.from_numpy(mask.view(np.float16)).to(gpu)
        info = J.plan(tq, tk, k_type, dv=dv, scale=U.SCALE, mask=tm)
        seen.add((info["variant"], info["balanced"]))
        got = _run(gpu, q, k, k_type, dv=dv, mask=mask, scale=U.SCALE)[..., :dv]
        want = (O.flash_attn_ext_f64 if k_type == O.TYPE_F16 else O.flash_attn_ext)(q, k, k_type, dv=dv, mask=mask, scale=U.SCALE)
        U.check(got, want, "case %d: H %d tok %d n_kv %d type %d dv %d style %d plan %s" % (case, n_head, n_tok, n_kv, k_type, dv, style, info))
    print(sorted(seen))


@pytest.mark.parametrize("k_type", [O.TYPE_F16, O.TYPE_BF16])
def test_repeated_launches_give_identical_results(gpu, k_type):
    """The same masked launch (ALiBi, then soft cap, then neither) 150 times each, other launches in between: every result equals
    the first bit for bit.  (A scalar load that the compiled code ahead of a wave program had left in flight once landed on the
    program's scale and flag words in about one launch of a hundred: one wave's rows wrong.  The programs now wait first.)"""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(5 + k_type)
    n_seq, n_head, n_tok, n_kv = 2, 128, 2, 640
    q = torch.from_numpy(rng.standard_normal((n_seq, n_head, n_tok, 576)).astype(np.float32)).to(gpu)
    k = torch.from_numpy(U.encode_kv(rng.standard_normal((n_seq, n_kv, 576)).astype(np.float32), k_type).view(np.int16)).to(gpu)
    m = (rng.standard_normal((n_tok, n_kv)) * 2).astype(np.float32)
    m[rng.random((n_tok, n_kv)) < 0.3] = -np.inf
    m[:, 600:] = -np.inf
    tm = torch.from_numpy(m.astype(np.float16)).to(gpu)
    pool, bt, _ = U.make_paged(rng, [1000] * 8, O.TYPE_BF16)
    qo = torch.from_numpy(rng.standard_normal((8, 16, 1, 576)).astype(np.float32)).to(gpu)
    po, bto = torch.from_numpy(pool.view(np.int16)).to(gpu), torch.from_numpy(bt).to(gpu)
    slo = torch.full((8,), 1000, dtype=torch.int32, device=gpu)
    oo = torch.empty((8, 1, 16, 576), dtype=torch.float32, device=gpu)
    settings = [(8.0, 0.0), (0.0, 30.0), (4.0, 5.0), (0.0, 0.0)]
    for i_set, (bias, cap) in enumerate(settings):
        out = torch.empty((n_seq, n_tok, n_head, 576), dtype=torch.float32, device=gpu)
        other = torch.empty_like(out)
        ob, oc = settings[(i_set + 2) % 4]
        ref, differ, where = None, 0, {}
        for i in range(150):
            if i % 3 == 0:
                J.ggml_flash_attn_ext(qo, po, O.TYPE_BF16, dv=512, scale=U.SCALE, block_table=bto, seq_lens=slo, out=oo)
            if i % 7 == 0:
                J.ggml_flash_attn_ext(q, k, k_type, dv=512, scale=U.SCALE, mask=tm, out=other, max_bias=ob, logit_softcap=oc)
            out.fill_(float("nan"))
            J.ggml_flash_attn_ext(q, k, k_type, dv=512, scale=U.SCALE, mask=tm, out=out, max_bias=bias, logit_softcap=cap)
            cur = out[..., :512].clone()
            if ref is None:
                ref = cur
            elif not torch.equal(cur, ref):
                differ += 1
                d = (cur - ref).abs().amax(-1)
                d = torch.where(torch.isnan(d), torch.full_like(d, 1e9), d)
                for idx in torch.nonzero(d > 0).tolist():
                    key = (i, idx[0], idx[1], idx[2] // 32, "%.1e" % float(d[idx[0], idx[1], idx[2] // 32 * 32:idx[2] // 32 * 32 + 32].max()))
                    where[key] = where.get(key, 0) + 1
        assert differ == 0, "bias %g cap %g: %d of 149 launches differ from the first; (launch, sequence, token, wave, max diff): rows %s" % (
            bias, cap, differ, sorted(where.items())[:24])
        assert bool(torch.isfinite(ref).all())


def test_repeated_launches_of_the_programs_with_idle_waves(gpu):
    """The same launches 100 times each, other launches in between, every result equal to the first bit for bit: a paged decode step
    of 64 heads (the two-row-block program: two waves without rows in a loop of their own) and a masked one of 48 heads with ALiBi and
    a soft cap over bf16 and over Q8_0 cells (the bias builds of the row-split programs)."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(77)
    lens = [1000, 333, 129, 2048, 77, 640]
    pool, bt, _ = U.make_paged(rng, lens, O.TYPE_BF16)
    q64 = torch.from_numpy(rng.standard_normal((len(lens), 64, 1, 576)).astype(np.float32)).to(gpu)
    tp, tb = torch.from_numpy(pool.view(np.int16)).to(gpu), torch.from_numpy(bt).to(gpu)
    tl = torch.tensor(lens, dtype=torch.int32, device=gpu)
    n_kv = 640
    q48 = torch.from_numpy(rng.standard_normal((2, 48, 1, 576)).astype(np.float32)).to(gpu)
    kb = torch.from_numpy(U.encode_kv(rng.standard_normal((2, n_kv, 576)).astype(np.float32), O.TYPE_BF16).view(np.int16)).to(gpu)
    kq = torch.from_numpy(U.encode_kv(rng.standard_normal((2, n_kv, 576)).astype(np.float32), O.TYPE_Q8_0)).to(gpu)
    m = (rng.standard_normal((1, n_kv)) * 2).astype(np.float32)
    m[rng.random((1, n_kv)) < 0.3] = -np.inf
    m[:, 0] = 0
    tm = torch.from_numpy(m.astype(np.float16)).to(gpu)
    launches = [
        ("64 heads, paged", lambda out: J.ggml_flash_attn_ext(q64, tp, O.TYPE_BF16, dv=512, scale=U.SCALE, block_table=tb, seq_lens=tl, out=out), (len(lens), 1, 64, 576)),
        ("48 heads, bf16 cells, ALiBi + soft cap", lambda out: J.ggml_flash_attn_ext(q48, kb, O.TYPE_BF16, dv=512, scale=U.SCALE, mask=tm, out=out, max_bias=8.0, logit_softcap=20.0), (2, 1, 48, 576)),
        ("48 heads, Q8_0 cells, ALiBi + soft cap", lambda out: J.ggml_flash_attn_ext(q48, kq, O.TYPE_Q8_0, dv=512, scale=U.SCALE, mask=tm, out=out, max_bias=8.0, logit_softcap=20.0), (2, 1, 48, 576)),
    ]
    for k, (what, f, shape) in enumerate(launches):
        out = torch.empty(shape, dtype=torch.float32, device=gpu)
        other = torch.empty(launches[(k + 1) % 3][2], dtype=torch.float32, device=gpu)
        ref, differ = None, 0
        for i in range(100):
            if i % 3 == 0:
                launches[(k + 1) % 3][1](other)
            out.fill_(float("nan"))
            f(out)
            cur = out[..., :512].clone()
            if ref is None:
                ref = cur
            elif not torch.equal(cur, ref):
                differ += 1
        assert differ == 0, "%s: %d of 99 launches differ from the first" % (what, differ)
        assert bool(torch.isfinite(ref).all()), what


@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_Q8_0])
@pytest.mark.parametrize("n_head,n_tok", [(128, 8), (16, 32), (16, 1), (48, 5)])
def test_mask_extents_left_by_the_launch_before(gpu, k_type, n_head, n_tok):
    """MLA_FLAG_MASK_EXTENTS_VALID: a launch with the same mask and shapes as the one before it on the same workspace, other
    queries and another cache, leaves out the scan of the mask and gives the result of a launch that scans (every kernel path that
    takes a mask: column-split, both forms of a few-head launch, k-split, row-split, Q8_0; contiguous and paged)."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(900 + n_head + n_tok)
    n_kv = 2048
    q8s = 1.0 / 32 if k_type == O.TYPE_Q8_0 else None
    m = np.full((n_tok, n_kv), -np.inf, dtype=np.float32)
    for t in range(n_tok):
        lo = int(rng.integers(0, n_kv - 64)); hi = min(n_kv, lo + int(rng.integers(33, 700)))
        m[t, lo:hi] = 0.0
    tm = torch.from_numpy(m.astype(np.float16)).to(gpu)
    for paged in (False, True):
        outs = []
        for layer in range(2):      # two "layers": other queries, another cache; the second is launched twice, with and without the flag
            q = torch.from_numpy(rng.standard_normal((1, n_head, n_tok, 576)).astype(np.float32)).to(gpu)
            kf = rng.standard_normal((1, n_kv, 576)).astype(np.float32)
            if paged:
                pool, bt, _ = U.make_paged(rng, [n_kv], k_type, q8_scale=q8s)
                kw = dict(block_table=torch.from_numpy(bt).to(gpu), seq_lens=torch.tensor([n_kv], dtype=torch.int32, device=gpu))
                k = torch.from_numpy(pool.view(np.int16) if pool.dtype == np.uint16 else pool).to(gpu)
            else:
                enc = U.encode_kv(kf, k_type, q8_scale=q8s)
                kw = {}
                k = torch.from_numpy(enc.view(np.int16) if enc.dtype == np.uint16 else enc).to(gpu)
            out = torch.full((1, n_tok, n_head, 576), float("nan"), dtype=torch.float32, device=gpu)
            J.ggml_flash_attn_ext(q, k, k_type, dv=512, scale=U.SCALE, mask=tm, out=out, **kw)
            if layer == 1:
                again = torch.full_like(out, float("nan"))
                J.ggml_flash_attn_ext(q, k, k_type, dv=512, scale=U.SCALE, mask=tm, out=again, flags=J.MLA_FLAG_MASK_EXTENTS_VALID, **kw)
                torch.cuda.synchronize()
                assert torch.equal(again[..., :512], out[..., :512]), "paged %d: the launch that reuses the extents differs" % paged
                assert bool(torch.isfinite(out[..., :512]).all())


@pytest.mark.parametrize("form", ["paged", "masked", "few heads", "contiguous"])
def test_one_long_sequence_in_256_splits(gpu, form):
    """One or two long sequences of 128 heads: the planner deals the keys out to 256 workgroups, every output row has up to 256 f16
    partials, and the combine pass for such rows lets four lanes share the walk over a row's splits.  Paged (33 000 and 20 000 keys:
    a balanced page schedule across both) and masked over one cache (two query tokens with windows of their own, one of them with a
    hole).  With f32 partials (16 heads over 33 000 paged keys: 256 pieces; 128 heads over 8192 contiguous keys: 64 one-page splits;
    V := K in its two passes) the four waves of a block share the walk."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(77)
    if form == "few heads":
        lens = [33000]
        pool, bt, seqs = U.make_paged(rng, lens, O.TYPE_F16)
        q = rng.standard_normal((1, 16, 1, 576)).astype(np.float32)
        got = _run(gpu, q, pool, O.TYPE_F16, bt=bt, lens=lens, scale=U.SCALE)
        want = np.stack([O.flash_attn_ext_f64(q[b:b + 1], k[None], O.TYPE_F16, dv=512, scale=U.SCALE)[0] for b, k in enumerate(seqs)])
    elif form == "contiguous":
        k = U.encode_kv(rng.standard_normal((1, 8192, 576)).astype(np.float32), O.TYPE_BF16)
        q = rng.standard_normal((1, 128, 1, 576)).astype(np.float32)
        tq, tk = torch.from_numpy(q).to(gpu), torch.from_numpy(k.view(np.int16)).to(gpu)
        assert J.plan(tq, tk, O.TYPE_BF16, dv=576, scale=U.SCALE)["n_splits"] == 64
        got = _run(gpu, q, k, O.TYPE_BF16, dv=576, scale=U.SCALE)
        want = O.flash_attn_ext(q, k, O.TYPE_BF16, dv=576, scale=U.SCALE)
        print(U.check(got, want, "many splits per row, V := K"))
        return
    elif form == "paged":
        lens = [33000, 20000]
        pool, bt, seqs = U.make_paged(rng, lens, O.TYPE_BF16)
        q = rng.standard_normal((2, 128, 1, 576)).astype(np.float32)
        tq, tk = torch.from_numpy(q).to(gpu), torch.from_numpy(pool.view(np.int16)).to(gpu)
        info = J.plan(tq, tk, O.TYPE_BF16, dv=512, scale=U.SCALE, block_table=torch.from_numpy(bt).to(gpu), seq_lens=torch.tensor(lens, dtype=torch.int32, device=gpu))
        assert info["variant"] == 2 and info["balanced"] == 1 and info["n_workgroups"] == 256
        got = _run(gpu, q, pool, O.TYPE_BF16, bt=bt, lens=lens, scale=U.SCALE)
        want = U.oracle_per_seq(q, seqs, O.TYPE_BF16, 512)
    else:
        n_kv = 40960
        k = U.encode_kv(rng.standard_normal((1, n_kv, 576)).astype(np.float32), O.TYPE_BF16)
        q = rng.standard_normal((1, 128, 2, 576)).astype(np.float32)
        m = np.full((2, n_kv), -np.inf, dtype=np.float32)
        m[0, 100:36000] = 0.0
        m[0, 5000:9000] = -np.inf
        m[1, 20000:40900] = 0.0
        mask = m.astype(np.float16).view(np.uint16)
        tq, tk = torch.from_numpy(q).to(gpu), torch.from_numpy(k.view(np.int16)).to(gpu)
        info = J.plan(tq, tk, O.TYPE_BF16, dv=512, scale=U.SCALE, mask=torch.from_numpy(mask.view(np.float16)).to(gpu))
        assert info["variant"] == 2 and info["balanced"] == 2 and info["n_row_blocks"] == 2
        got = _run(gpu, q, k, O.TYPE_BF16, mask=mask, scale=U.SCALE)
        want = O.flash_attn_ext(q, k, O.TYPE_BF16, dv=512, mask=mask, scale=U.SCALE)
    print(U.check(got[..., :512], want, "many splits per row, " + form))


def _run_flags(gpu, q, pool, k_type, bt, lens, flags):
    import torch
    import jittorinfer_amd as J
    tq = torch.from_numpy(q).to(gpu)
    tk = torch.from_numpy(pool.view(np.int16) if pool.dtype == np.uint16 else pool).to(gpu)
    tb, tl = torch.from_numpy(bt).to(gpu), torch.from_numpy(np.asarray(lens, dtype=np.int32)).to(gpu)
    out = torch.full((q.shape[0], q.shape[2], q.shape[1], 576), float("nan"), dtype=torch.float32, device=gpu)
    info = J.plan(tq, tk, k_type, dv=512, scale=U.SCALE, block_table=tb, seq_lens=tl, out=out, flags=flags)
    J.ggml_flash_attn_ext(tq, tk, k_type, dv=512, scale=U.SCALE, block_table=tb, seq_lens=tl, out=out, flags=flags)
    torch.cuda.synchronize()
    return out.cpu().numpy()[..., :512], info


@pytest.mark.parametrize("n_head", [32, 64])
@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_Q8_0])
@pytest.mark.parametrize("shape", ["many_short", "few_long_many_short", "one_sequence", "with_empties"])
def test_balanced_schedule_of_ragged_decode_batches(gpu, k_type, shape, n_head):
    """The pipelined kernel's balanced schedule (equal runs of the batch's page list per workgroup, pieces of several
    sequences inside one workgroup, whole-sequence pieces written without the combine pass) against the oracle and
    against the uniform-split plan of the same call."""
    import jittorinfer_amd as J
    rng = np.random.default_rng({"many_short": 1, "few_long_many_short": 2, "one_sequence": 3, "with_empties": 4}[shape])
    if shape == "many_short":
        lens = [int(x) for x in rng.integers(1, 3 * 128, size=150)]          # ~300 pages: runs of 2 pages cross sequence ends
    elif shape == "few_long_many_short":
        lens = [4000, 3777] + [int(x) for x in rng.integers(1, 200, size=40)]
    elif shape == "one_sequence":
        lens = [5000]
    else:
        lens = [0, 0, 700, 0, 129, 0, 0, 1, 128, 0]
    # Q8_0 pages as BASELINE's config 5 builds them (one power-of-two scale): with arbitrary block scales a lone key's
    # V value rounded to the f16 MFMA operand alone costs up to 2^-11 |v| = 2.2e-3 at |v| = 4.5, whatever the schedule
    pool, bt, seqs = U.make_paged(rng, np.maximum(lens, 1), k_type, q8_scale=1.0 / 32 if k_type == O.TYPE_Q8_0 else None)
    seqs = [s[:l] for s, l in zip(seqs, lens)]
    if len(lens) * bt.shape[1] <= 256:
        # the schedule is planned when the table allows more than one page per workgroup: columns no sequence reaches
        bt = np.concatenate([bt, np.full((len(lens), 300 - bt.shape[1]), -5, np.int32)], axis=1)
    q = rng.standard_normal((len(lens), n_head, 1, 576)).astype(np.float32)
    got, info = _run_flags(gpu, q, pool, k_type, bt, lens, 0)
    assert info["variant"] == 2 and info["balanced"] == 1 and info["n_workgroups"] == 256
    uni, info_u = _run_flags(gpu, q, pool, k_type, bt, lens, J.MLA_FLAG_UNIFORM_SPLITS)
    assert info_u["balanced"] == 0
    want = _want(q, seqs, k_type)
    print(U.check(got, want, "balanced schedule"), U.check(uni, want, "uniform splits"))


def test_balanced_schedule_limits(gpu):
    """A batch that already fills the GPU with one workgroup per sequence (nothing to split), one whose table holds no more
    pages than there are workgroups, or a block table so wide that a workgroup's run could exceed the 64 pages a wave
    indexes, keeps the uniform plan."""
    import torch
    import jittorinfer_amd as J
    q = torch.zeros((257, 16, 1, 576), device=gpu)
    pool = torch.zeros((128 * 4, 576), dtype=torch.int16, device=gpu)
    bt = torch.zeros((257, 4), dtype=torch.int32, device=gpu)
    sl = torch.ones(257, dtype=torch.int32, device=gpu)
    assert J.plan(q[:256], pool, J.MLA_TYPE_BF16, dv=512, scale=1.0, block_table=bt[:256], seq_lens=sl[:256])["balanced"] == 0   # one split: nothing to balance
    q8 = torch.zeros((8, 16, 1, 576), device=gpu)
    assert J.plan(q8, pool, J.MLA_TYPE_BF16, dv=512, scale=1.0, block_table=bt[:8], seq_lens=sl[:8])["balanced"] == 0   # 32 pages at most: one per workgroup anyway
    bt40 = torch.zeros((8, 40), dtype=torch.int32, device=gpu)
    assert J.plan(q8, pool, J.MLA_TYPE_BF16, dv=512, scale=1.0, block_table=bt40, seq_lens=sl[:8])["balanced"] == 1
    wide = torch.zeros((8, 4096), dtype=torch.int32, device=gpu)
    assert J.plan(q8, pool, J.MLA_TYPE_BF16, dv=512, scale=1.0, block_table=wide, seq_lens=sl[:8])["balanced"] == 0


def test_balanced_schedule_of_a_masked_launch_with_many_row_blocks(gpu):
    """320 query tokens x 16 heads = 40 row blocks over one cache of 2048 cells; every token sees its own window, some see
    nothing (NaN rows, like the reference), the windows of a row block's 8 tokens overlap only partly.  The workgroups'
    runs of the tile list cross row-block boundaries (40 key ranges of up to 64 tiles over 256 workgroups)."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(77)
    n_tok, n_kv = 320, 2048
    k = U.encode_kv(rng.standard_normal((1, n_kv, 576)).astype(np.float32), O.TYPE_BF16)
    m = np.full((n_tok, n_kv), -np.inf, dtype=np.float32)
    for t in range(n_tok):
        if t % 37 == 5:
            continue                                   # a token with no visible key at all
        centre = (t // 8) * 45 + int(rng.integers(0, 200))
        lo, hi = max(0, centre - int(rng.integers(1, 300))), min(n_kv, centre + int(rng.integers(1, 300)))
        m[t, lo:hi] = 0.0
    m[8:16] = -np.inf                                  # a whole row block without keys
    mask = m.astype(np.float16).view(np.uint16)
    q = rng.standard_normal((1, 16, n_tok, 576)).astype(np.float32)
    tq, tk = torch.from_numpy(q).to(gpu), torch.from_numpy(k.view(np.int16)).to(gpu)
    tm = torch.from_numpy(mask.view(np.float16)).to(gpu)
    info = J.plan(tq, tk, O.TYPE_BF16, dv=512, scale=U.SCALE, mask=tm)
    assert info["variant"] == 2 and info["balanced"] == 2 and info["n_row_blocks"] == 40
    got = _run(gpu, q, k, O.TYPE_BF16, mask=mask, scale=U.SCALE)
    want = O.flash_attn_ext(q, k, O.TYPE_BF16, dv=512, mask=mask, scale=U.SCALE)
    assert np.isnan(want[0, 5]).all() and np.isnan(want[0, 8:16]).all()
    print(U.check(got[..., :512], want, "masked launch, balanced schedule"))


def test_workspace_is_per_stream_and_survives_growth_and_capture(gpu):
    """The binding keeps one scratch area per (device, stream): launches on two streams must not share partials; a larger
    launch gets a new area while the old one stays allocated (a graph that recorded its address replays correctly
    afterwards); a first launch on a stream that is being captured allocates from the graph's pool and replays correctly."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(3)
    pool, bt, seqs = U.make_paged(rng, [900, 700], O.TYPE_BF16)
    q = rng.standard_normal((2, 128, 1, 576)).astype(np.float32)
    tq, tk = torch.from_numpy(q).to(gpu), torch.from_numpy(pool.view(np.int16)).to(gpu)
    tb, tl = torch.from_numpy(bt).to(gpu), torch.tensor([900, 700], dtype=torch.int32, device=gpu)
    kw = dict(dv=512, scale=U.SCALE, block_table=tb, seq_lens=tl)
    want = U.oracle_per_seq(q, seqs, O.TYPE_BF16, 512)
    s1, s2 = torch.cuda.Stream(gpu), torch.cuda.Stream(gpu)
    torch.cuda.synchronize()
    with torch.cuda.stream(s1):
        a1, o1, k1 = J.capi.make_args(tq, tk, J.MLA_TYPE_BF16, **kw)
    with torch.cuda.stream(s2):
        a2, o2, k2 = J.capi.make_args(tq, tk, J.MLA_TYPE_BF16, **kw)
    assert a1.workspace != a2.workspace
    with torch.cuda.stream(s1):
        r1 = J.ggml_flash_attn_ext(tq, tk, J.MLA_TYPE_BF16, **kw)
    with torch.cuda.stream(s2):
        r2 = J.ggml_flash_attn_ext(tq, tk, J.MLA_TYPE_BF16, **kw)
    torch.cuda.synchronize()
    assert torch.equal(r1[..., :512], r2[..., :512])
    print(U.check(r1.cpu().numpy()[..., :512], want, "two streams"))
    # a stream that has never launched, under capture (what `with torch.cuda.graph(g):` does): the area is made then and there
    out3 = torch.zeros((2, 1, 128, 576), dtype=torch.float32, device=gpu)
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        J.ggml_flash_attn_ext(tq, tk, J.MLA_TYPE_BF16, out=out3, **kw)
    torch.cuda.synchronize()
    # a much larger launch on the first stream replaces its area; the graph and the earlier argument block keep theirs
    big_pool, big_bt, _ = U.make_paged(rng, [128] * 64, O.TYPE_BF16)
    bq = torch.from_numpy(rng.standard_normal((64, 128, 1, 576)).astype(np.float32)).to(gpu)
    with torch.cuda.stream(s1):
        J.ggml_flash_attn_ext(bq, torch.from_numpy(big_pool.view(np.int16)).to(gpu), J.MLA_TYPE_BF16, dv=512, scale=U.SCALE,
                              block_table=torch.from_numpy(big_bt).to(gpu), seq_lens=torch.full((64,), 128, dtype=torch.int32, device=gpu), n_splits=1)
    torch.cuda.synchronize()
    for it in range(2):
        out3.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out3[..., :512], r1[..., :512]), "replay %d" % it


@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_F16, O.TYPE_Q8_0])
@pytest.mark.parametrize("masked", [False, True])
@pytest.mark.parametrize("n_head,n_tok", [(16, 1), (16, 8), (48, 3)])
def test_a_split_of_more_than_64_pages_of_a_cache_without_a_table(gpu, k_type, masked, n_head, n_tok):
    """A wave keeps the page ids of its split in the 64 lanes of one register.  A cache without a block table has no page ids
    to keep, so a split of it may be of any length: one workgroup walks 9248 keys here (a prompt chunk of many row blocks behind
    more than 8192 cached keys is planned that way), with the k-split program (16 rows), the column-split ones (128 and 144 rows)
    and the row-split one of a Q8_0 cache.  Every key carries a distinct weight, so a tile read from the wrong place shows."""
    rng = np.random.default_rng(n_head * 100 + n_tok * 10 + masked)
    n_kv = 8192 + 1024 + 32
    k = U.encode_kv(rng.standard_normal((1, n_kv, 576)).astype(np.float32), k_type, **({"q8_scale": 1.0 / 32} if k_type == O.TYPE_Q8_0 else {}))
    q = rng.standard_normal((1, n_head, n_tok, 576)).astype(np.float32)
    mask = None
    if masked:
        m = np.zeros((n_tok, n_kv), dtype=np.float32)
        for t in range(n_tok):
            m[t, n_kv - 40 * (n_tok - 1 - t):] = -np.inf   # causal tail of a chunk
            m[t, 3000 + 10 * t:3100] = -np.inf
        mask = m.astype(np.float16).view(np.uint16)
    got = _run(gpu, q, k, k_type, mask=mask, scale=U.SCALE, n_splits=1)
    # (an F16 cache against the oracle's float64 form: the reference sums V in f16 there, which over 9000 keys is its own noise)
    want = (O.flash_attn_ext_f64 if k_type == O.TYPE_F16 else O.flash_attn_ext)(q, k, k_type, dv=512, scale=U.SCALE, mask=mask)
    print(U.check(got[..., :512], want, "one split of 9248 keys"))


def test_prompt_chunk_behind_a_long_cache_without_a_table(gpu):
    """512 tokens x 128 heads behind 8192 cached keys, causal mask: 512 row blocks, one split each of up to 8704 keys (more than the 64
    pages a wave has lanes for), the row blocks taken in folded order; and 64 tokens x 128 heads over 40960 keys, whose 64 row
    blocks the tile schedule hands to 256 workgroups in runs of about 10 000 keys.  Checked on sampled rows against float64."""
    import torch
    import jittorinfer_amd as J
    g = torch.Generator(device="cpu").manual_seed(5)
    for n_tok, past in [(512, 8192), (64, 40960 - 64)]:
        n_kv = past + n_tok
        q = torch.randn(1, 128, n_tok, 576, generator=g).to(gpu)
        kv = (torch.randn(1, n_kv, 576, generator=g)).to(torch.bfloat16).to(gpu)
        mask = torch.full((n_tok, n_kv), float("-inf"), dtype=torch.float16)
        for t in range(n_tok):
            mask[t, : past + t + 1] = 0
        mask = mask.to(gpu)
        info = J.plan(q, kv.view(torch.int16), O.TYPE_BF16, mask=mask, scale=U.SCALE)
        assert info["variant"] == 2 and (info["n_splits"] == 1 if n_tok == 512 else info["balanced"] == 2), info
        out = J.ggml_flash_attn_ext(q, kv.view(torch.int16), O.TYPE_BF16, mask=mask, scale=U.SCALE)
        torch.cuda.synchronize()
        qc, kc = q[0].to(torch.bfloat16).double().cpu().numpy(), kv[0].double().cpu().numpy()
        worst = 0.0
        for (t, h) in [(0, 0), (n_tok - 1, 0), (n_tok - 1, 127), (n_tok // 2, 5), (7, 77), (n_tok - 2, 64)]:
            s = kc[: past + t + 1] @ qc[h, t] * U.SCALE
            p = np.exp(s - s.max())
            want = (p / p.sum()) @ kc[: past + t + 1, :512]
            worst = max(worst, float(np.abs(out[0, t, h, :512].cpu().numpy() - want).max()))
        print("tokens %d past %d: worst sampled difference %.2e" % (n_tok, past, worst))
        assert worst < U.MAX_ABS_TOL, (n_tok, past, worst)


@pytest.mark.parametrize("n_head", [128, 64])
def test_paged_decode_of_more_than_256_sequences_longest_first(gpu, n_head):
    """A paged decode batch of more than 256 sequences of 128 (64) heads is a workgroup per sequence, in rounds; the workgroups take the
    sequences by falling length (an order the pre-pass writes into the workspace).  300 ragged sequences, some empty, some equal:
    against the oracle, and bit for bit against the same launch in batch order (MLA_FLAG_UNIFORM_SPLITS)."""
    import torch
    import jittorinfer_amd as J
    rng = np.random.default_rng(300)
    lens = [int(x) for x in rng.integers(1, 140, size=300)]
    lens[7], lens[150], lens[299] = 0, 600, 333
    lens[20:24] = [77, 77, 77, 77]
    pool, bt, seqs = U.make_paged(rng, np.maximum(lens, 1), O.TYPE_BF16)
    seqs = [s[:l] for s, l in zip(seqs, lens)]
    q = rng.standard_normal((300, n_head, 1, 576)).astype(np.float32)
    tq, tk = torch.from_numpy(q).to(gpu), torch.from_numpy(pool.view(np.int16)).to(gpu)
    tb, tl = torch.from_numpy(bt).to(gpu), torch.from_numpy(np.asarray(lens, dtype=np.int32)).to(gpu)
    info = J.plan(tq, tk, O.TYPE_BF16, dv=512, scale=U.SCALE, block_table=tb, seq_lens=tl)
    assert info["variant"] == 2 and info["n_splits"] == 1 and info["balanced"] == 0 and info["n_workgroups"] == 300, info
    got, _ = _run_flags(gpu, q, pool, O.TYPE_BF16, bt, lens, 0)
    same, _ = _run_flags(gpu, q, pool, O.TYPE_BF16, bt, lens, J.MLA_FLAG_UNIFORM_SPLITS)
    assert np.array_equal(got, same, equal_nan=True), "longest first and batch order differ"
    want = U.oracle_per_seq(q, seqs, O.TYPE_BF16, 512)
    print(U.check(got, want, "300 sequences, longest first"))
