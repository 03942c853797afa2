"""Golden vectors produced by the reference's compiled ggml-cpu (tests/golden/gen_golden.py): the oracle (CPU) and
the HIP path (GPU) are both held to them."""
import os

import numpy as np
import pytest

from oracle import oracle as O
from tests import util as U
from tests.golden import cases

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "golden.npz"))


def _inputs(name):
    inp = cases.make_inputs(name)
    digest = bytes(GOLD[name + "/digest"]).decode()
    if digest != inp["digest"]:
        pytest.skip("seeded inputs differ from the ones the fixture was made with (different numpy?)")
    return inp


@pytest.mark.parametrize("name", list(cases.CASES))
def test_oracle_matches_golden(name):
    inp = _inputs(name)
    got = O.flash_attn_ext(inp["q"], inp["k"], inp["k_type"], dv=576, mask=inp["mask"], scale=inp["scale"], max_bias=inp["max_bias"], softcap=inp["softcap"])
    ma, rl = O.errors(got, GOLD[name])
    if inp["k_type"] == O.TYPE_F16:
        assert ma < 2e-3 and rl < 3e-4, (ma, rl)  # f16 accumulator: rounding flips from 1e-7 differences in the dots
    else:
        assert ma < 3e-6 and rl < 2e-6, (ma, rl)


@pytest.mark.gpu
@pytest.mark.parametrize("dv", [512, 576])
@pytest.mark.parametrize("name", list(cases.CASES))
def test_gpu_matches_golden(gpu, name, dv):
    import torch
    import jittorinfer_amd as J
    inp = _inputs(name)
    k = inp["k"]
    tk = torch.from_numpy(k.view(np.int16) if k.dtype == np.uint16 else k).to(gpu)
    tm = None if inp["mask"] is None else torch.from_numpy(inp["mask"].view(np.float16)).to(gpu)
    flags = J.MLA_FLAG_F16_ACC_STRICT if inp["k_type"] == O.TYPE_F16 else 0
    out = J.ggml_flash_attn_ext(torch.from_numpy(inp["q"]).to(gpu), tk, inp["k_type"], dv=dv, mask=tm, scale=inp["scale"], flags=flags,
                                max_bias=inp["max_bias"], logit_softcap=inp["softcap"])
    torch.cuda.synchronize()
    U.check(out.cpu().numpy()[..., :dv], GOLD[name][..., :dv], name)
