"""bench.py's command-line contract, as far as it can be checked without a GPU: more than one GPU is refused with a
message, the help text lists the measured configurations, and the product raises (no CPU path) when asked to compute
on a CPU tensor."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")] + list(args), capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _bench("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr) and "--gpus 2" in (r.stdout + r.stderr)


def test_help_names_the_configurations():
    r = _bench("--help")
    assert r.returncode == 0
    for word in ("--steps", "--warmup", "--gpus", "--config", "c3mask", "kvwrite", "layer", "--cpu-seqs"):
        assert word in r.stdout, word


def test_no_cpu_path():
    import torch
    import jittorinfer_amd as J
    q = torch.zeros((1, 16, 1, 576))
    k = torch.zeros((1, 32, 576), dtype=torch.int16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        J.ggml_flash_attn_ext(q, k, J.MLA_TYPE_BF16)


def test_workspace_areas_grow_by_at_least_half():
    """The Python layer's scratch areas: a run of requests that creep up retires a logarithmic number of areas, not one per
    request (checked on the CPU with a stand-in allocator: the policy is plain arithmetic)."""
    import types
    import jittorinfer_amd.capi as capi

    class FakeTensor:
        def __init__(self, n):
            self.n = n

        def numel(self):
            return self.n
    fake_torch = types.SimpleNamespace(empty=lambda n, dtype=None, device=None: FakeTensor(n), uint8=None,
                                       cuda=types.SimpleNamespace(current_stream=lambda d: types.SimpleNamespace(cuda_stream=7)))
    saved = dict(capi._workspaces), list(capi._retired)
    capi._workspaces.clear()
    capi._retired.clear()
    import sys
    real = sys.modules.get("torch")
    sys.modules["torch"] = fake_torch
    try:
        for step in range(8192):
            ws = capi._workspace("dev", (2 << 20) + 512 * 128 * step, stream=7)
            assert ws.numel() >= (2 << 20) + 512 * 128 * step
        assert len(capi._retired) <= 16, len(capi._retired)
        assert sum(w.numel() for w in capi._retired) <= 3 * ws.numel()
    finally:
        if real is not None:
            sys.modules["torch"] = real
        else:
            del sys.modules["torch"]
        capi._workspaces.clear()
        capi._workspaces.update(saved[0])
        capi._retired[:] = saved[1]
