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


def test_rope_and_batch_structs_match_the_headers_and_the_checks_refuse_what_they_should():
    """mla_kv_write_rope_args / mla_front_op mirrors against the C compiler's view, and the argument checks of
    mla_kv_write_rope_check / mla_front_batch_check (host code: no GPU needed)."""
    import jittorinfer_amd as J
    from jittorinfer_amd.capi import MlaKvWriteRopeArgs, MlaFrontOp, MLA_FRONT_COPY, MLA_FRONT_KV_WRITE_ROPE
    src = ('#include <stdio.h>\n#include <stddef.h>\n#include "mla_kv_write.h"\nint main(){printf("%zu %zu %zu %zu %d %d\\n", '
           'sizeof(mla_kv_write_rope_args), offsetof(mla_kv_write_rope_args, rope), sizeof(mla_front_op), offsetof(mla_front_op, args), '
           'MLA_FRONT_COPY, MLA_FRONT_KV_WRITE_ROPE);return 0;}\n')
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "t.c")
        exe = os.path.join(d, "t")
        open(c, "w").write(src)
        subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), c, "-o", exe], check=True)
        vals = list(map(int, subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()))
    assert vals == [C.sizeof(MlaKvWriteRopeArgs), MlaKvWriteRopeArgs.rope.offset, C.sizeof(MlaFrontOp), MlaFrontOp.args.offset,
                    MLA_FRONT_COPY, MLA_FRONT_KV_WRITE_ROPE]

    lib = J.library()
    lib.mla_kv_write_rope_check.argtypes = [C.POINTER(MlaKvWriteRopeArgs)]
    lib.mla_front_batch_check.argtypes = [C.POINTER(MlaFrontOp), C.c_int32]

    def good():
        a = MlaKvWriteRopeArgs()
        a.w.n_tok, a.w.src_type, a.w.kv_type = 5, J.MLA_TYPE_F32, J.MLA_TYPE_BF16
        a.w.src, a.w.src_nb1, a.w.kv, a.w.kv_nb1, a.w.n_kv_rows = 0x1000, 2048, 0x100000, 1152, 64
        a.rope.src, a.rope.pos, a.rope.dst = 0x2000, 0x3000, 0x2000
        a.rope.ne[:], a.rope.src_nb[:], a.rope.dst_nb[:] = [64, 1, 5, 1], [4, 256, 256, 1280], [4, 256, 256, 1280]
        a.rope.n_dims, a.rope.mode, a.rope.n_ctx_orig, a.rope.freq_base, a.rope.freq_scale = 64, 0, 4096, 10000.0, 1.0
        a.rope.attn_factor, a.rope.beta_fast, a.rope.beta_slow = 1.0, 32.0, 1.0
        return a
    assert lib.mla_kv_write_rope_check(C.byref(good())) == 0
    for field, value, rc in (("rope.mode", 2, -6), ("rope.n_dims", 32, -1), ("rope.src", 0x2004, -3), ("rope.pos", None, -5),
                             ("w.src_type", J.MLA_TYPE_BF16, -2), ("w.src_nb1", 1024, -1), ("w.row0", 60, -1)):
        a = good()
        obj, name = (a.rope, field[5:]) if field.startswith("rope.") else (a.w, field[2:])
        setattr(obj, name, value)
        assert lib.mla_kv_write_rope_check(C.byref(a)) == rc, field
    a = good()
    a.rope.ne[2] = 4   # one k_pe row per new token
    assert lib.mla_kv_write_rope_check(C.byref(a)) == -1

    ops = (MlaFrontOp * 3)()
    a = good()
    ops[0].kind, ops[0].args = MLA_FRONT_KV_WRITE_ROPE, C.addressof(a)
    assert lib.mla_front_batch_check(ops, 1) == 0
    assert lib.mla_front_batch_check(ops, 0) == 0 and lib.mla_front_batch_check(None, 0) == 0
    assert lib.mla_front_batch_check(None, 1) == -5 and lib.mla_front_batch_check(ops, -1) == -1
    ops[1].kind, ops[1].args = 9, C.addressof(a)
    assert lib.mla_front_batch_check(ops, 2) == -2          # no such kind
    ops[1].kind, ops[1].args = MLA_FRONT_COPY, None
    assert lib.mla_front_batch_check(ops, 2) == -5
