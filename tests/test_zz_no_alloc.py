"""mla_attn_launch_static (include/mla_attn.h): the entry point that brings its own scratch -- a file-scope device array -- and
allocates nothing.  Through the C ABI, against mla_attn_launch on the same inputs: the two run the same kernels with the same
plan, so the outputs are required to be bit-identical (well inside the 2e-3 / 1e-3 bar, which is checked against the oracle
too).  Two calls in a row, the second on a smaller input, so that what the first call left in the array is in the way."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O
from tests import util as U

pytestmark = pytest.mark.gpu


def _both(gpu, lens, n_head, k_type, seed):
    import torch
    import jittorinfer_amd as J
    lib = J.library()
    rng = np.random.default_rng(seed)
    pool, bt, seqs = U.make_paged(rng, lens, k_type)
    q = rng.standard_normal((len(lens), n_head, 1, 576)).astype(np.float32)
    tq, tk = torch.from_numpy(q).to(gpu), torch.from_numpy(pool.view(np.int16) if pool.dtype == np.uint16 else pool).to(gpu)
    tb, tl = torch.from_numpy(bt).to(gpu), torch.from_numpy(np.asarray(lens, dtype=np.int32)).to(gpu)
    outs = []
    st = C.c_void_p(torch.cuda.current_stream(gpu).cuda_stream)
    for fn in (lib.mla_attn_launch, lib.mla_attn_launch_static):
        out = torch.full((len(lens), 1, n_head, 576), float("nan"), dtype=torch.float32, device=gpu)
        a, _, keep = J.capi.make_args(tq, tk, k_type, dv=512, scale=U.SCALE, block_table=tb, seq_lens=tl, out=out)
        assert lib.mla_attn_workspace_size(C.byref(a)) > 0          # the case does use scratch (split-K partials, the Q image)
        if fn is lib.mla_attn_launch_static:
            a.workspace, a.workspace_size = None, 0                 # the entry point must not need the caller's workspace
        rc = fn(C.byref(a), st)
        assert rc == 0, rc
        torch.cuda.synchronize()
        outs.append(out.cpu().numpy())
    want = U.oracle_per_seq(q, seqs, k_type, 512)
    return outs[0], outs[1], want


@pytest.mark.parametrize("k_type", [O.TYPE_BF16, O.TYPE_Q8_0])
def test_static_scratch_entry_point_matches_the_workspace_one(gpu, k_type):
    for lens, n_head, seed in (([2048, 1500, 700], 128, 11), ([640], 16, 12)):      # the second call is the smaller one
        ref, got, want = _both(gpu, lens, n_head, k_type, seed)
        assert np.array_equal(ref[..., :512], got[..., :512]), "static-scratch result differs from the workspace result"
        assert np.isnan(got[..., 512:]).all()
        print(U.check(got[..., :512], want, "static scratch, %s" % lens))


def test_static_scratch_rejects_what_does_not_fit(gpu):
    """A call whose scratch exceeds the fixed array is refused with MLA_ERR_TOO_LARGE before anything is launched."""
    import torch
    import jittorinfer_amd as J
    lib = J.library()
    n_seq, n_head, pages = 128, 128, 4
    q = torch.zeros((n_seq, n_head, 1, 576), dtype=torch.float32, device=gpu)
    pool = torch.zeros((n_seq * pages * 128, 576), dtype=torch.int16, device=gpu)
    bt = torch.arange(n_seq * pages, dtype=torch.int32, device=gpu).reshape(n_seq, pages).contiguous()
    sl = torch.full((n_seq,), pages * 128, dtype=torch.int32, device=gpu)
    out = torch.zeros((n_seq, 1, n_head, 576), dtype=torch.float32, device=gpu)
    a, _, keep = J.capi.make_args(q, pool, J.MLA_TYPE_BF16, dv=512, scale=U.SCALE, block_table=bt, seq_lens=sl, out=out, n_splits=4)
    need = lib.mla_attn_workspace_size(C.byref(a))
    assert need > J.capi.MLA_ATTN_STATIC_WORKSPACE_MAX, need
    rc = lib.mla_attn_launch_static(C.byref(a), C.c_void_p(torch.cuda.current_stream(gpu).cuda_stream))
    assert rc == J.capi.MLA_ERR_TOO_LARGE, rc
