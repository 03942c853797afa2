"""The drop-in boundary without a GPU: the library loads, exports every symbol include/*.h declares, and its mirror
of the reference's struct layouts / enum ordinals (jittorinfer_amd/csrc/ggml_abi.h) agrees with the real headers
-- live against oracle/_ref when that is built, and always against the committed copy of the reference's table."""
import ctypes as C
import json
import os
import re

import pytest

from oracle import oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden", "ggml_abi_table.json")


def _lib():
    import jittorinfer_amd as J
    return J.library()


def _mirror_table():
    lib = _lib()
    name, val = C.c_char_p(), C.c_int64()
    n = lib.mla_ggml_abi_table(-1, C.byref(name), C.byref(val))
    out = {}
    for i in range(n):
        lib.mla_ggml_abi_table(i, C.byref(name), C.byref(val))
        out[name.value.decode()] = val.value
    return out


def test_library_exports_every_declared_symbol():
    lib = _lib()
    declared = set()
    for hdr in ("mla_attn.h", "mla_kv_write.h", "mla_front.h", "mla_page_table.h", "ggml_mla_backend.h"):
        src = open(os.path.join(ROOT, "include", hdr)).read()
        src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
        declared |= set(re.findall(r"\b(mla_\w+|ggml_backend_\w+)\s*\(", src))
    declared -= {"mla_attn_args", "mla_attn_plan_info", "mla_page_table", "mla_kv_write_args"}
    assert {"mla_attn_launch", "mla_attn_workspace_size", "ggml_backend_init", "ggml_backend_score"} <= declared
    for sym in sorted(declared):
        assert hasattr(lib, sym), "library does not export %s" % sym


def test_mirror_matches_committed_reference_table():
    golden = json.load(open(GOLDEN))
    mirror = _mirror_table()
    assert set(mirror) == set(golden)
    bad = {k: (mirror[k], golden[k]) for k in golden if mirror[k] != golden[k]}
    assert not bad, bad


@pytest.mark.skipif(not O.ref_available(), reason="oracle/_ref is not built")
def test_mirror_matches_live_reference_headers():
    live = O.ref_abi_table()
    mirror = _mirror_table()
    assert live == mirror
    assert live == json.load(open(GOLDEN))


def test_args_struct_size_matches_header():
    """ctypes mirror of mla_attn_args vs the C compiler's view of include/mla_attn.h."""
    import subprocess
    import tempfile
    import jittorinfer_amd as J
    src = '#include <stdio.h>\n#include <stddef.h>\n#include "mla_attn.h"\nint main(){printf("%zu %zu %zu %zu\\n", sizeof(mla_attn_args), offsetof(mla_attn_args, kv), offsetof(mla_attn_args, workspace), sizeof(mla_attn_plan_info));return 0;}\n'
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "t.c")
        open(c, "w").write(src)
        exe = os.path.join(d, "t")
        subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), c, "-o", exe], check=True)
        out = subprocess.run([exe], check=True, stdout=subprocess.PIPE, text=True).stdout.split()
    assert int(out[0]) == C.sizeof(J.MlaAttnArgs)
    assert int(out[1]) == J.MlaAttnArgs.kv.offset
    assert int(out[2]) == J.MlaAttnArgs.workspace.offset
    assert int(out[3]) == C.sizeof(J.MlaPlanInfo)


def test_argument_validation_without_gpu():
    """Rejected arguments come back as negative codes before anything touches a device."""
    import jittorinfer_amd as J
    lib = _lib()
    a = J.MlaAttnArgs()
    assert lib.mla_attn_launch(C.byref(a), None) == -5          # null pointers
    a.q, a.kv, a.dst = 4096, 8192, 16384
    a.n_seq, a.n_head, a.n_tok, a.dk, a.dv = 1, 16, 1, 576, 512
    a.kv_type, a.q_type = J.MLA_TYPE_BF16, J.MLA_TYPE_F32
    a.q_nb1 = a.q_nb2 = a.q_nb3 = 2304
    a.kv_nb1, a.n_kv, a.dst_nb1, a.scale = 1152, 256, 2304, 0.1
    info = J.MlaPlanInfo()
    assert lib.mla_attn_plan(C.byref(a), C.byref(info)) == 0 and info.n_splits >= 1
    a.dk = 512
    assert lib.mla_attn_plan(C.byref(a), C.byref(info)) == -1    # head size other than 576
    a.dk, a.kv_type = 576, 2
    assert lib.mla_attn_plan(C.byref(a), C.byref(info)) == -2    # unsupported KV type
    a.kv_type, a.kv_nb1 = J.MLA_TYPE_BF16, 1150
    assert lib.mla_attn_plan(C.byref(a), C.byref(info)) == -3    # misaligned rows
    a.kv_nb1, a.max_bias = 1152, 1.0
    assert lib.mla_attn_plan(C.byref(a), C.byref(info)) == -6    # ALiBi without a mask
    a.max_bias = 0.0
    a.n_splits = 4
    assert lib.mla_attn_plan(C.byref(a), C.byref(info)) == 0
    assert lib.mla_attn_launch(C.byref(a), None) == -4           # split-K needs a workspace
    assert lib.ggml_backend_score() in (0, 100)


def _plan(**kw):
    """mla_attn_plan on made-up (never dereferenced) device addresses: the planner is host logic."""
    import jittorinfer_amd as J
    a = J.MlaAttnArgs()
    a.q, a.kv, a.dst = 4096, 8192, 16384
    a.n_seq, a.n_head, a.n_tok, a.dk, a.dv = 32, 128, 1, 576, 512
    a.kv_type, a.q_type = J.MLA_TYPE_BF16, J.MLA_TYPE_F32
    a.q_nb1 = a.q_nb2 = 2304
    a.q_nb3 = 2304 * 128
    a.kv_nb1, a.n_kv, a.dst_nb1, a.scale = 1152, 2048 * 128, 2304, 0.1
    a.block_table, a.bt_stride, a.seq_lens = 32768, 64, 65536
    for k, v in kw.items():
        setattr(a, k, v)
    info = J.MlaPlanInfo()
    rc = _lib().mla_attn_plan(C.byref(a), C.byref(info))
    return rc, info, _lib().mla_attn_workspace_size(C.byref(a))


def test_planner_schedules_without_gpu():
    """Which kernel and which split schedule the planner picks for the BASELINE shapes, and what the workspace holds."""
    import jittorinfer_amd as J
    rc, info, ws = _plan()                                       # config 3: 32 sequences x 64 pages
    assert rc == 0 and info.variant == 2 and info.balanced == 1 and info.n_workgroups == 256
    assert info.n_splits == 8 and info.split_tokens == 1024     # the uniform plan the balanced schedule replaces
    slots = 256 + 32                                            # f16 partials, (m, l), Q image, schedule
    assert ws >= slots * 128 * 512 * 2 + slots * 128 * 8 + 32 * 4 * 36 * 1024 + 33 * 4 + 256 * 32
    rc, info, _ = _plan(flags=J.MLA_FLAG_UNIFORM_SPLITS)
    assert rc == 0 and info.variant == 2 and info.balanced == 0 and info.n_workgroups == 256
    rc, info, _ = _plan(n_splits=4)                              # an explicit split count is honoured as it is
    assert rc == 0 and info.balanced == 0 and info.n_splits == 4
    rc, info, _ = _plan(n_seq=64, kv_type=J.MLA_TYPE_Q8_0, kv_nb1=612)   # config 5
    assert rc == 0 and info.variant == 2 and info.balanced == 1
    rc, info, _ = _plan(n_seq=256)                               # one workgroup per sequence fills the GPU: nothing to split
    assert rc == 0 and info.n_splits == 1 and info.balanced == 0
    rc, info, _ = _plan(n_seq=8, bt_stride=4096)                 # runs could exceed the 64 pages a wave indexes
    assert rc == 0 and info.balanced == 0 and info.n_splits * 64 * 128 >= 4096 * 128
    rc, info, _ = _plan(block_table=0, seq_lens=0, bt_stride=0, n_kv=8192, kv_nb3=8192 * 1152)   # contiguous KV: uniform splits
    assert rc == 0 and info.variant == 2 and info.balanced == 0 and info.n_splits == 8
    rc, info, _ = _plan(dv=576)                                  # V := K: two passes of the pipelined kernel (columns 0.., 64..)
    assert rc == 0 and info.variant == 2 and info.n_passes == 2 and info.balanced == 1
    rc, info, _ = _plan(dv=576, max_bias=8.0, mask=131072, mask_nb1=16384, mask_ne0=8192)   # ALiBi with a mask over 16-bit rows: the pipelined kernel has a build for it
    assert rc == 0 and info.variant == 2 and info.n_passes == 2
    rc, info, _ = _plan(dv=576, max_bias=8.0, mask=131072, mask_nb1=16384, mask_ne0=8192, kv_type=J.MLA_TYPE_Q8_0, kv_nb1=612)   # and over Q8_0 rows
    assert rc == 0 and info.variant == 2 and info.n_passes == 2
    rc, info, _ = _plan(dv=576, max_bias=8.0, mask=131072, mask_nb1=16384, mask_ne0=8192, flags=J.MLA_FLAG_BF16_DIRECT)   # not for the hi + lo bf16 program: the general kernel, 2 x 288 columns
    assert rc == 0 and info.variant == 0 and info.n_passes == 2
    rc, info, _ = _plan(logit_softcap=30.0)                      # softcap without a mask: general kernel, 64 rows per workgroup
    assert rc == 0 and info.variant == 0 and info.rows_per_wg == 64
    one = dict(n_seq=1, n_head=16, block_table=0, seq_lens=0, bt_stride=0, kv_nb3=0, kv_type=J.MLA_TYPE_F16)
    rc, info, _ = _plan(n_kv=1024, **one)                        # configs[0]: one short sequence, splits of one 32-key tile
    assert rc == 0 and info.variant == 2 and info.n_splits == 32 and info.split_tokens == 32
    rc, info, _ = _plan(n_kv=4096, **one)                        # 128 tiles: 4 MB of f32 partials, the most a few-head launch gets
    assert rc == 0 and info.n_splits == 128 and info.split_tokens == 32
    rc, info, _ = _plan(n_kv=16384, **one)                       # more tiles than that allows splits: whole pages again
    assert rc == 0 and info.n_splits == 128 and info.split_tokens == 128
    rc, info, _ = _plan(n_kv=1024, **{**one, "n_head": 128})
    assert rc == 0 and info.n_splits == 8 and info.split_tokens == 128
    # the reference's decode batch: one cache, one query token per sequence, the mask picks every token's cells
    batch = dict(n_seq=1, n_tok=32, block_table=0, seq_lens=0, bt_stride=0, n_kv=32 * 8192, kv_nb3=0, mask=131072, mask_nb1=2 * 32 * 8192, mask_ne0=32 * 8192)
    rc, info, _ = _plan(**batch)                                 # 128 heads: a query token fills a block of 128 rows
    assert rc == 0 and info.variant == 2 and info.balanced == 2 and info.n_row_blocks == 32
    rc, info, ws = _plan(n_head=16, **batch)                     # 16 heads: issued both as row blocks and token by token
    assert rc == 0 and info.variant == 2 and info.balanced == 4 and info.n_row_blocks == 4 and info.n_workgroups == 256
    assert ws >= (256 + 4) * 128 * 512 * 2 + 32 * 16 * 8         # the row-block form's partials hold the token form's; 16 key pairs per token
    for kw in (dict(n_head=48), dict(n_head=16, kv_type=J.MLA_TYPE_Q8_0, kv_nb1=612), dict(n_head=64, kv_type=J.MLA_TYPE_Q8_0, kv_nb1=612)):
        rc, info, ws2 = _plan(**{**batch, **kw})                # up to 64 heads, and Q8_0 cells: the token form is the row-split program
        assert rc == 0 and info.balanced == 4, kw
        assert ws2 >= 32 * 4 * 36 * 1024                        # ... which takes an operand image per token
    for kw in (dict(n_head=16, n_tok=2), dict(n_head=16, n_tok=257), dict(n_head=65), dict(n_head=64), dict(n_head=48, n_tok=1),
               dict(n_head=16, flags=J.MLA_FLAG_BF16_DIRECT), dict(n_head=16, max_bias=8.0)):
        rc, info, _ = _plan(**{**batch, **kw})                  # at most 32 rows, more than 256 tokens, more than 64 heads, two tokens to a row block exactly, ...: one form
        assert rc == 0 and info.balanced in (0, 2), kw


@pytest.mark.parametrize("gen,flags,name", [("gen_decode_asm.py", [], "mla_decode_asm.inc"), ("gen_decode_asm.py", ["--f16"], "mla_decode_asm_f16.inc"),
                                            ("gen_decode_asm.py", ["--mask"], "mla_decode_asm_mask.inc"),
                                            ("gen_decode_asm.py", ["--f16", "--mask"], "mla_decode_asm_f16_mask.inc"), ("gen_decode_asm.py", ["--q8"], "mla_decode_asm_q8.inc"),
                                            ("gen_decode_asm.py", ["--q8", "--mask"], "mla_decode_asm_q8_mask.inc"), ("gen_decode_asm.py", ["--cvt"], "mla_decode_asm_cvt.inc"),
                                            ("gen_decode_asm.py", ["--cvt", "--mask"], "mla_decode_asm_cvt_mask.inc"),
                                            ("gen_decode_cs_asm.py", [], "mla_decode_cs_bf16.inc"), ("gen_decode_cs_asm.py", ["--f16"], "mla_decode_cs_f16.inc"),
                                            ("gen_decode_cs_asm.py", ["--mask"], "mla_decode_cs_bf16_mask.inc"),
                                            ("gen_decode_cs_asm.py", ["--mask", "--bias"], "mla_decode_cs_bf16_bias.inc"),
                                            ("gen_decode_cs_asm.py", ["--f16", "--mask", "--bias"], "mla_decode_cs_f16_bias.inc"),
                                            ("gen_decode_cs_asm.py", ["--f16", "--mask"], "mla_decode_cs_f16_mask.inc"),
                                            ("gen_decode_cs_asm.py", ["--ks"], "mla_decode_ks_bf16.inc"), ("gen_decode_cs_asm.py", ["--ks", "--f16"], "mla_decode_ks_f16.inc"),
                                            ("gen_decode_cs_asm.py", ["--ks", "--mask"], "mla_decode_ks_bf16_mask.inc"),
                                            ("gen_decode_cs_asm.py", ["--ks", "--f16", "--mask"], "mla_decode_ks_f16_mask.inc"),
                                            ("gen_decode_cs_asm.py", ["--mask", "--stream"], "mla_decode_cs_bf16_mask_nt.inc"),
                                            ("gen_decode_cs_asm.py", ["--f16", "--mask", "--stream"], "mla_decode_cs_f16_mask_nt.inc"),
                                            ("gen_decode_cs_asm.py", ["--ks", "--mask", "--stream"], "mla_decode_ks_bf16_mask_nt.inc"),
                                            ("gen_decode_cs_asm.py", ["--ks", "--f16", "--mask", "--stream"], "mla_decode_ks_f16_mask_nt.inc"),
                                            ("gen_decode_cs_asm.py", ["--ks", "--mask", "--bias"], "mla_decode_ks_bf16_bias.inc"),
                                            ("gen_decode_cs_asm.py", ["--ks", "--f16", "--mask", "--bias"], "mla_decode_ks_f16_bias.inc"),
                                            ("gen_decode_asm.py", ["--cvt", "--mask", "--bias"], "mla_decode_asm_cvt_bias.inc"),
                                            ("gen_decode_asm.py", ["--f16", "--mask", "--bias"], "mla_decode_asm_f16_bias.inc"),
                                            ("gen_decode_asm.py", ["--q8", "--mask", "--bias"], "mla_decode_asm_q8_bias.inc"),
                                            ("gen_decode_cs_asm.py", ["--half"], "mla_decode_csh_bf16.inc"),
                                            ("gen_decode_cs_asm.py", ["--half", "--f16"], "mla_decode_csh_f16.inc")])
def test_committed_wave_programs_are_what_the_generator_emits(gen, flags, name):
    """The instruction streams the decode kernel includes are generated files: each equals the generator's output.  None of
    them touches v252..v255: the asm block's clobber list ends at v251, and the compiler keeps there what lives across the
    block (the lanes it spills scalar registers to among it).  The bias builds own v252 as well: their clobber list names it."""
    import re
    import subprocess
    import sys
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "jittorinfer_amd", "csrc")
    got = subprocess.run([sys.executable, os.path.join(csrc, gen)] + flags, capture_output=True, text=True, check=True).stdout
    with open(os.path.join(csrc, name)) as f:
        assert got == f.read(), "%s is stale: regenerate it with %s %s" % (name, gen, " ".join(flags))
    # a program takes and leaves the machine with nothing in flight: what the compiled code ahead of it left outstanding could land on
    # a register the program has written since, and the other way round
    lines = [ln for ln in got.splitlines() if ln.startswith('"')]
    assert lines[0] == '"s_waitcnt vmcnt(0) lgkmcnt(0)\\n\\t"' and lines[-1] == lines[0], (lines[0], lines[-1])
    for m in re.finditer(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]", got):
        hi = int(m.group(1)) if m.group(1) else int(m.group(3))
        assert hi <= (252 if "--bias" in flags else 251), "%s uses %s" % (name, m.group(0))
        if "--ks" in flags and "--mask" in flags:       # their clobber list leaves v192..v203 to the compiler as well
            lo = int(m.group(1)) if m.group(1) else int(m.group(2))
            assert hi < 192 or lo > 203, "%s uses %s" % (name, m.group(0))
    top = 99 if gen == "gen_decode_cs_asm.py" else 83
    for m in re.finditer(r"\bs(\d+)\b|\bs\[(\d+):(\d+)\]", got):      # scalar registers: inside the clobbered range s40..s83 (s99)
        lo, hi = (int(m.group(1)),) * 2 if m.group(1) else (int(m.group(2)), int(m.group(3)))
        assert 40 <= lo and hi <= top, "%s uses %s" % (name, m.group(0))


def test_python_constants_match_the_header():
    """The ctypes mirror restates the #defines of include/mla_attn.h (types, flags, errors): each one is compared with the header."""
    import re
    import jittorinfer_amd.capi as capi
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with open(os.path.join(root, "include", "mla_attn.h")) as f:
        text = f.read()
    defs = {m.group(1): m.group(2) for m in re.finditer(r"#define\s+(MLA_(?:TYPE|FLAG|ERR)_\w+)\s+\(?(-?\d+)u?\)?", text)}
    assert {"MLA_FLAG_F16_ACC_STRICT", "MLA_FLAG_UNIFORM_SPLITS", "MLA_FLAG_BF16_DIRECT", "MLA_TYPE_BF16", "MLA_TYPE_Q8_0"} <= set(defs)
    checked = 0
    for name, value in defs.items():
        if hasattr(capi, name):
            assert getattr(capi, name) == int(value), name
            checked += 1
    assert checked >= 6
