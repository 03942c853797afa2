"""supports_op against the launchers' own argument checks, on the CPU.

ggml_backend_sched asks every device `supports_op` per node and sends a node nobody takes to the CPU backend
(ggml/src/ggml-backend.cpp:820-846); a node this plugin takes and graph_compute then refuses fails the whole graph.
So for nodes generated around the shapes of the MLA layer -- dense and strided, aligned and misaligned views, every
cache type -- the test checks: supported => the launch check of the argument block graph_compute would build is 0;
and hand-made nodes that the launchers refuse (misaligned rows, short strides, foreign products) are not supported.
The tensors are ctypes mirrors of ggml_tensor, laid out by the offsets in tests/golden/ggml_abi_table.json (which
tests/test_abi.py keeps in step with the library and the reference's headers); nothing runs on a device.
"""
import ctypes as C
import json
import os

import numpy as np
import pytest

import jittorinfer_amd.capi as J

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ABI = json.load(open(os.path.join(ROOT, "tests", "golden", "ggml_abi_table.json")))


class Tensor(C.Structure):
    pass


Tensor._fields_ = [
    ("type", C.c_int32), ("_pad0", C.c_int32), ("buffer", C.c_void_p), ("ne", C.c_int64 * 4), ("nb", C.c_size_t * 4),
    ("op", C.c_int32), ("op_params", C.c_int32 * 16), ("flags", C.c_int32), ("src", C.POINTER(Tensor) * 10),
    ("view_src", C.POINTER(Tensor)), ("view_offs", C.c_size_t), ("data", C.c_void_p), ("name", C.c_char * 64),
    ("extra", C.c_void_p), ("padding", C.c_char * 8),
]

T = {k[len("GGML_TYPE_"):]: v for k, v in ABI.items() if k.startswith("GGML_TYPE_")}
OP = {k[len("GGML_OP_"):]: v for k, v in ABI.items() if k.startswith("GGML_OP_")}
BLOCK = {T["F32"]: (1, 4), T["F16"]: (1, 2), T["BF16"]: (1, 2), T["Q8_0"]: (32, 34), T["I32"]: (1, 4)}


def test_the_mirror_has_ggml_tensor_s_layout():
    for f in ("type", "buffer", "ne", "nb", "op", "op_params", "flags", "src", "view_src", "view_offs", "data", "name", "extra"):
        assert getattr(Tensor, f).offset == ABI["offsetof(ggml_tensor,%s)" % f], f
    assert C.sizeof(Tensor) == ABI["sizeof(ggml_tensor)"]


_keep = []


def tensor(typ, ne, nb=None, op="NONE", src=(), view_of=None, view_offs=0, params=(), data=None):
    """A ggml_tensor as ggml_new_tensor / ggml_view_* would fill it (ggml.c:1637-1720): contiguous strides unless given."""
    t = Tensor()
    t.type = T[typ]
    ne = list(ne) + [1] * (4 - len(ne))
    bs, ts = BLOCK[T[typ]]
    if nb is None:
        nb = [ts, ts * (ne[0] // bs), 0, 0]
        nb[2] = nb[1] * ne[1]
        nb[3] = nb[2] * ne[2]
    for i in range(4):
        t.ne[i], t.nb[i] = ne[i], nb[i]
    t.op = OP[op]
    for i, v in enumerate(params):
        t.op_params[i] = v
    for i, s in enumerate(src):
        if s is not None:
            t.src[i] = C.pointer(s)
    if view_of is not None:
        t.view_src = C.pointer(view_of)
        t.view_offs = view_offs
    if data is not None:
        t.data = data
    _keep.append(t)
    return t


def f32_bits(x):
    return int(np.float32(x).view(np.int32))


@pytest.fixture(scope="module")
def lib():
    lib = J.library()
    lib.mla_ggml_supports_node.argtypes = [C.c_void_p, C.POINTER(C.c_char_p)]
    lib.mla_ggml_node_launch_check.argtypes = [C.c_void_p]
    return lib


def verdict(lib, t):
    why = C.c_char_p()
    ok = lib.mla_ggml_supports_node(C.addressof(t), C.byref(why))
    return bool(ok), (why.value or b"").decode()


def attn_node(kv_type="BF16", n_head=16, n_tok=1, n_seq=2, n_kv=256, dv=512, q_nb=None, q_offs=0, k_nb1=None, k_offs=0,
              dst_ne0=None, dst_offs=0, mask=None, paged=None, max_bias=0.0, q_data=None):
    """The node as llm_attn_mla builds it: q [576, n_tok, n_head, n_seq] a permuted view, k the cache (or page pool), v a
    view of k's first dv columns, dst [dst_ne0, n_head, n_tok, n_seq]."""
    bs, ts = BLOCK[T[kv_type]]
    row = 576 // bs * ts
    if q_nb is None:
        q_nb = [4, 576 * 4 * n_head, 576 * 4, 576 * 4 * n_head * n_tok]     # [576, H, n_tok] storage seen as [576, n_tok, H]
    q_root = tensor("F32", [576, n_head, n_tok, n_seq])
    q = tensor("F32", [576, n_tok, n_head, n_seq], q_nb, op="PERMUTE", src=[q_root], view_of=q_root, view_offs=q_offs, data=q_data)
    k1 = k_nb1 or row
    k3 = 1 if paged else n_seq
    cache = tensor(kv_type, [576, n_kv, 1, k3], [ts, k1, k1 * n_kv, k1 * n_kv])
    k = cache if not k_offs else tensor(kv_type, [576, n_kv, 1, k3], [ts, k1, k1 * n_kv, k1 * n_kv], op="VIEW", src=[cache], view_of=cache, view_offs=k_offs)
    v = k if dv == 576 else tensor(kv_type, [dv, n_kv, 1, k3], [ts, k1, k1 * n_kv, k1 * n_kv], op="VIEW", src=[cache], view_of=cache, view_offs=k_offs)
    m = None
    if mask:
        m = tensor("F16", [mask[0], mask[1]])
    bt = lens = None
    if paged:
        bt, lens = tensor("I32", [paged, n_seq]), tensor("I32", [n_seq])
    d0 = dst_ne0 or dv
    droot = tensor("F32", [d0 + 8, n_head, n_tok, n_seq])
    dst = tensor("F32", [d0, n_head, n_tok, n_seq], [4, (d0 + 8) * 4, (d0 + 8) * 4 * n_head, (d0 + 8) * 4 * n_head * n_tok] if dst_offs else None,
                 op="FLASH_ATTN_EXT", src=[q, k, v, m, bt, lens], view_of=droot if dst_offs else None, view_offs=dst_offs,
                 params=[f32_bits(0.0417), f32_bits(max_bias), 0])
    return dst


def test_the_layer_s_nodes_are_taken(lib):
    for kv in ("BF16", "F16", "Q8_0"):
        assert verdict(lib, attn_node(kv))[0]
        assert verdict(lib, attn_node(kv, n_head=128, n_seq=32, n_kv=4096 * 128, paged=32))[0]
        assert verdict(lib, attn_node(kv, n_tok=64, n_seq=1, n_kv=1024, mask=(1024, 64)))[0]
        assert verdict(lib, attn_node(kv, dv=576, dst_ne0=576))[0]


@pytest.mark.parametrize("kw, clause", [
    (dict(q_offs=4), "16-byte"),                                   # q view starting one float in
    (dict(q_nb=[4, 2312, 2308 * 16, 2308 * 16 * 4]), "16-byte"),   # q rows 2308 bytes apart
    (dict(kv_type="F16", k_offs=2), "16-byte"),                    # cache view starting one element in
    (dict(kv_type="BF16", k_nb1=1160), "16-byte"),                 # cache rows 1160 bytes apart
    (dict(kv_type="Q8_0", k_offs=1), "2-byte"),
    (dict(kv_type="Q8_0", k_nb1=613), "2-byte"),
    (dict(dst_offs=8), "16-byte"),
    (dict(n_kv=200, paged=4), "128-token pages"),
    (dict(n_kv=256, paged=4, mask=(256, 1)), "mask narrower"),
    (dict(mask=(128, 1)), "mask narrower"),
    (dict(max_bias=8.0), "max_bias"),
    (dict(q_data=0x7f0000000004), "16-byte"),                      # allocated: the real address decides
])
def test_what_the_launch_refuses_is_not_taken(lib, kw, clause):
    node = attn_node(**kw)
    ok, why = verdict(lib, node)
    assert not ok and clause in why, why


def kv_write_nodes(kv_type, n_tok=5, n_rows=512, upd_type="F32", src_nb1=2304, src_offs=0, cache_offs=0, var_nb1=None, idx_type="I32"):
    bs, ts = BLOCK[T[kv_type]]
    row = 576 // bs * ts
    cache = tensor(kv_type, [576, n_rows])
    src_root = tensor("F32", [1024, n_tok])
    src = tensor("F32", [576, n_tok], [4, src_nb1, src_nb1 * n_tok, src_nb1 * n_tok], op="VIEW", src=[src_root], view_of=src_root, view_offs=src_offs)
    kview = tensor(kv_type, [576 * n_tok], op="VIEW", src=[cache], view_of=cache, view_offs=cache_offs)
    cpy = tensor(kv_type, [576 * n_tok], op="CPY", src=[src, kview], view_of=kview, view_offs=0)
    cpy.view_src = C.pointer(kview)
    v1 = var_nb1 or row
    var = cache if not var_nb1 else tensor(kv_type, [576, n_rows // 2], [ts, v1, v1 * (n_rows // 2), v1 * (n_rows // 2)], op="VIEW", src=[cache], view_of=cache)
    ubs, uts = BLOCK[T[upd_type]]
    upd = src if upd_type == "F32" else tensor(upd_type, [576, n_tok])
    idx = tensor(idx_type, [n_tok])
    sc = tensor(kv_type, list(var.ne), list(var.nb), op="SCATTER_UPDATE", src=[var, idx, upd], view_of=var)
    return cpy, sc


def test_cache_write_nodes(lib):
    for kv in ("BF16", "F16", "Q8_0"):
        cpy, sc = kv_write_nodes(kv)
        assert verdict(lib, cpy)[0] and verdict(lib, sc)[0]
        cpy, sc = kv_write_nodes(kv, upd_type=kv)
        assert verdict(lib, sc)[0]
        # update rows that are not 16-byte aligned / start one float in
        for kw in (dict(src_nb1=2308), dict(src_offs=4)):
            cpy, sc = kv_write_nodes(kv, **kw)
            assert not verdict(lib, cpy)[0] and not verdict(lib, sc)[0]
    # a cache view one element in: 16-bit caches refuse, and so does Q8_0 at an odd byte
    assert not verdict(lib, kv_write_nodes("BF16", cache_offs=2)[0])[0]
    assert not verdict(lib, kv_write_nodes("Q8_0", cache_offs=1)[0])[0]
    assert verdict(lib, kv_write_nodes("Q8_0", cache_offs=34)[0])[0]
    # scatter into cache rows spread two rows apart is fine; a stride that is not a multiple of 16 is not
    assert verdict(lib, kv_write_nodes("BF16", var_nb1=2304)[1])[0]
    assert not verdict(lib, kv_write_nodes("BF16", var_nb1=1156)[1])[0]
    assert verdict(lib, kv_write_nodes("F16", idx_type="I32")[1])[0]
    # a SCATTER_UPDATE whose result is not the cache
    cpy, sc = kv_write_nodes("BF16")
    other = tensor("BF16", [576, 512])
    sc.view_src = C.pointer(other)
    assert not verdict(lib, sc)[0]


def mul_mat_node(K, N, M, n_head, w_type="BF16", w_heads=None, x_nb1=None):
    w = tensor(w_type, [K, N, n_head if w_heads is None else w_heads])
    x = tensor("F32", [K, M, n_head], None if x_nb1 is None else [4, x_nb1, x_nb1 * M, x_nb1 * M * n_head])
    return tensor("F32", [N, M, n_head], op="MUL_MAT", src=[w, x])


def test_only_the_absorb_products_are_taken(lib):
    assert verdict(lib, mul_mat_node(128, 512, 4, 16))[0]            # q_nope . wk_b
    assert verdict(lib, mul_mat_node(512, 128, 4, 16, "F16"))[0]     # wv_b . kqv
    assert verdict(lib, mul_mat_node(192, 512, 1, 128))[0]
    for node in (mul_mat_node(2048, 2048, 4, 1),                     # a projection of the model
                 mul_mat_node(512, 10944, 4, 1),                     # an FFN product that happens to have K = 512
                 mul_mat_node(128, 512, 4, 16, w_heads=1),           # one matrix for all heads
                 mul_mat_node(128, 512, 4, 16, x_nb1=520),           # rows of src1 8 bytes apart from alignment
                 mul_mat_node(120, 512, 4, 16)):                     # K not a multiple of 16
        assert not verdict(lib, node)[0]


def test_supported_means_the_launch_check_passes(lib):
    """Generated nodes, valid and broken in every stride / offset / shape the launch checks look at."""
    rng = np.random.default_rng(11)
    pick = lambda *xs: xs[int(rng.integers(0, len(xs)))]
    taken = refused = 0
    for _ in range(4000):
        kind = pick("attn", "attn", "cpy", "scatter", "mul_mat", "cont", "rope", "concat")
        if kind == "attn":
            kv = pick("BF16", "F16", "Q8_0")
            n_head, n_tok, n_seq = pick(1, 16, 128), pick(1, 2, 64), pick(1, 3)
            paged = pick(None, None, 4, 1 << 24)
            n_kv = pick(128, 256, 200, 1024)
            row = 612 if kv == "Q8_0" else 1152
            node = attn_node(kv, n_head, n_tok, n_seq, n_kv, dv=pick(512, 512, 576), paged=paged,
                             q_offs=pick(0, 0, 0, 4, 16, 8), k_offs=pick(0, 0, 0, 1, 2, 16, 34), k_nb1=pick(None, None, row + 16, row + 2, row + 1, row - 2),
                             dst_offs=pick(0, 0, 16, 4), dst_ne0=pick(None, 576), mask=pick(None, None, (n_kv, n_tok), (n_kv, 64), (64, n_tok), (512 + n_kv, n_tok)),
                             max_bias=pick(0.0, 0.0, 8.0), q_data=pick(None, None, 0x7f0000000100, 0x7f0000000108))
        elif kind in ("cpy", "scatter"):
            kv = pick("BF16", "F16", "Q8_0")
            row = 612 if kv == "Q8_0" else 1152
            cpy, sc = kv_write_nodes(kv, n_tok=pick(0, 1, 5, 300), upd_type=pick("F32", "F32", kv), src_nb1=pick(2304, 2304, 2308, 4096, 2320, 1152),
                                     src_offs=pick(0, 0, 4, 16, 2), cache_offs=pick(0, 0, 1, 2, 34, 1152, 612), var_nb1=pick(None, None, 2 * row, row + 4, row + 2, row + 1),
                                     idx_type=pick("I32", "I32", "F32"))
            node = cpy if kind == "cpy" else sc
        elif kind == "mul_mat":
            node = mul_mat_node(pick(128, 512, 64, 120, 16, 8), pick(512, 128, 64, 100), pick(0, 1, 7, 4096), pick(1, 16, 128), pick("BF16", "F16"),
                                w_heads=pick(None, None, 1), x_nb1=pick(None, None, 520, 528, 2048))
        elif kind == "cont":
            ne = [pick(64, 128, 3), pick(1, 5), pick(1, 16), pick(1, 2)]
            src_root = tensor("F32", [256, 8, 16, 2])
            nb1 = pick(1024, 1028, 512)
            src = tensor("F32", ne, [4, nb1, nb1 * 8, nb1 * 8 * 16], op="VIEW", src=[src_root], view_of=src_root, view_offs=pick(0, 4, 2, 64))
            node = tensor("F32", [ne[0] * ne[1], ne[2], ne[3]], op="CONT", src=[src])
        elif kind == "rope":
            ne = [pick(64, 192, 1024), pick(1, 16), pick(1, 7, 70000), 1]
            x = tensor("F32", ne)
            pos = tensor("I32", [ne[2]])
            node = tensor("F32", ne, op="ROPE", src=[x, pos, None], params=[0, pick(64, 63, 2048, 192), pick(0, 2, 8), 0, 4096] + [f32_bits(v) for v in (1e4, 1.0, 0.0, 1.0, 32.0, 1.0)])
        else:
            a, b = tensor("F32", [512, 16, 3]), tensor("F32", [pick(64, 63), 16, 3])
            node = tensor("F32", [512 + b.ne[0], 16, 3], op="CONCAT", src=[a, b], params=[0])
        ok, why = verdict(lib, node)
        rc = lib.mla_ggml_node_launch_check(C.addressof(node))
        if ok:
            taken += 1
            assert rc == 0, (kind, why, rc)
        else:
            refused += 1
            assert why
    assert taken > 400 and refused > 400, (taken, refused)
