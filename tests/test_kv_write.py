"""The oracle of the KV cache write (oracle/mla_oracle.c mla_oracle_kv_write), pinned without a GPU: against numpy
indexing plus the per-row converters (which tests/test_oracle.py pins exhaustively), and against the reference's own
compiled ggml_cpy when oracle/_ref is built.  Also: the ctypes mirror of mla_kv_write_args against the C header."""
import ctypes as C
import os
import subprocess
import tempfile

import numpy as np
import pytest

from oracle import oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TYPES = [O.TYPE_BF16, O.TYPE_F16, O.TYPE_Q8_0]


def _empty_cache(rng, n_rows, kv_type):
    if kv_type == O.TYPE_Q8_0:
        return rng.integers(0, 256, size=(n_rows, 612), dtype=np.uint8)
    return rng.integers(0, 65536, size=(n_rows, 576), dtype=np.uint16)


def _convert_rows(x, kv_type, q8_mode=1):
    if kv_type == O.TYPE_BF16:
        return O.f32_to_bf16(x)
    if kv_type == O.TYPE_F16:
        return O.f32_to_f16(x)
    return O.quantize_q8_0(x, q8_mode)


@pytest.mark.parametrize("kv_type", TYPES)
def test_rows_land_where_numpy_indexing_puts_them(kv_type):
    rng = np.random.default_rng(7)
    cache = _empty_cache(rng, 300, kv_type)
    before = cache.copy()
    x = (rng.standard_normal((37, 576)) * 3).astype(np.float32)
    dest = rng.permutation(300)[:37].astype(np.int64)
    dest[5] = -1      # skipped
    dest[9] = 300     # skipped
    O.kv_write(x, cache, kv_type, dest)
    want = before.copy()
    conv = _convert_rows(x, kv_type)
    for t, r in enumerate(dest):
        if 0 <= r < 300:
            want[r] = conv[t]
    assert np.array_equal(cache, want)
    untouched = np.setdiff1d(np.arange(300), dest)
    assert np.array_equal(cache[untouched], before[untouched])


def test_q8_0_write_uses_the_cpu_backend_quantizer_by_default():
    # a value whose scaled form is an exact .5: round-half-even (x86 CPU backend) and roundf (reference form) differ
    x = np.zeros((1, 576), dtype=np.float32)
    x[0, 0] = 127.0
    x[0, 1] = 2.5
    c1 = np.zeros((1, 612), dtype=np.uint8)
    c0 = np.zeros((1, 612), dtype=np.uint8)
    O.kv_write(x, c1, O.TYPE_Q8_0, [0], q8_mode=1)
    O.kv_write(x, c0, O.TYPE_Q8_0, [0], q8_mode=0)
    assert c1[0, 3].view(np.int8) == 2 and c0[0, 3].view(np.int8) == 3
    assert np.array_equal(c1, O.quantize_q8_0(x, 1)) and np.array_equal(c0, O.quantize_q8_0(x, 0))


@pytest.mark.parametrize("kv_type", TYPES)
def test_raw_rows_are_copied_unchanged(kv_type):
    rng = np.random.default_rng(8)
    cache = _empty_cache(rng, 64, kv_type)
    rows = _empty_cache(rng, 5, kv_type)
    dest = np.array([63, 0, 17, 18, 40])
    O.kv_write(rows, cache, kv_type, dest, src_type=kv_type)
    assert np.array_equal(cache[dest], rows)


@pytest.mark.skipif(not O.ref_available(), reason="oracle/_ref is not built")
@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("kv_head,n_tok", [(0, 1), (5, 40), (100, 28)])
def test_matches_the_reference_ggml_cpy(kv_type, kv_head, n_tok):
    rng = np.random.default_rng(9 + kv_head)
    cache = _empty_cache(rng, 128, kv_type)
    x = (rng.standard_normal((n_tok, 576)) * rng.choice([1e-3, 1.0, 40.0], size=(n_tok, 1))).astype(np.float32)
    x[0, :32] = 0.0   # an all-zero Q8_0 block
    want = O.ref_kv_cpy(x, cache.copy(), kv_type, kv_head)
    got = O.kv_write(x, cache.copy(), kv_type, np.arange(kv_head, kv_head + n_tok))
    assert np.array_equal(got, want)


def test_args_struct_matches_header():
    from jittorinfer_amd.capi import MlaKvWriteArgs
    src = ('#include <stdio.h>\n#include <stddef.h>\n#include "mla_kv_write.h"\nint main(){printf("%zu %zu %zu %zu\\n", '
           'sizeof(mla_kv_write_args), offsetof(mla_kv_write_args, kv), offsetof(mla_kv_write_args, rows), offsetof(mla_kv_write_args, positions));return 0;}\n')
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "t.c")
        exe = os.path.join(d, "t")
        open(c, "w").write(src)
        subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), c, "-o", exe], check=True)
        size, off_kv, off_rows, off_pos = map(int, subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split())
    assert C.sizeof(MlaKvWriteArgs) == size
    assert MlaKvWriteArgs.kv.offset == off_kv and MlaKvWriteArgs.rows.offset == off_rows and MlaKvWriteArgs.positions.offset == off_pos
