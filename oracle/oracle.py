"""ctypes front end of the CPU oracle (oracle/mla_oracle.c) and, when built, of the reference's own compiled
ggml (oracle/_ref/).  TEST INFRASTRUCTURE ONLY -- see oracle/__init__.py.

Array conventions (numpy, C order; ggml lists dimensions the other way round):
  q     float32 [n_seq, n_head, n_tok, 576]          ggml ne = {576, n_tok, n_head, n_seq}
  k     f16/bf16: uint16 [n_seq, n_kv, 576];  q8_0: uint8 [n_seq, n_kv, 612]
  mask  uint16 (f16 bits) [n_tok, n_kv] or None
  out   float32 [n_seq, n_tok, n_head, dv]
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

TYPE_F32, TYPE_F16, TYPE_Q8_0, TYPE_BF16 = 0, 1, 8, 30
Q8_ROW = 612


class _Tensor(C.Structure):
    _fields_ = [("type", C.c_int32), ("_pad", C.c_int32), ("ne", C.c_int64 * 4), ("nb", C.c_int64 * 4), ("data", C.c_void_p)]


def build(force=False):
    """Compile liboracle.so (and oracle/_ref when the reference tree is present) with the Makefile beside this file."""
    if force or not os.path.exists(os.path.join(HERE, "liboracle.so")) or (
            os.path.isdir("/root/reference/ggml") and not os.path.exists(os.path.join(HERE, "_ref", "libref_driver.so"))):
        subprocess.run(["make", "-C", HERE, "-j8"], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        _lib = C.CDLL(path)
        _lib.mla_oracle_flash_attn_ext.restype = C.c_int
        _lib.mla_oracle_flash_attn_ext.argtypes = [C.POINTER(_Tensor)] * 4 + [C.c_void_p, C.c_int64, C.c_float, C.c_float, C.c_float, C.c_int, C.c_int]
        _lib.mla_oracle_flash_attn_ext_f64.restype = C.c_int
        _lib.mla_oracle_flash_attn_ext_f64.argtypes = [C.POINTER(_Tensor)] * 4 + [C.c_void_p, C.c_int64, C.c_float, C.c_int, C.c_int]
        _lib.mla_oracle_kv_write.restype = C.c_int
        _lib.mla_oracle_kv_write.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_void_p, C.c_int, C.c_int64, C.c_int64, C.c_void_p, C.c_int]
        for name in ("mla_oracle_f32_to_bf16_row", "mla_oracle_f32_to_f16_row", "mla_oracle_bf16_to_f32_row", "mla_oracle_f16_to_f32_row"):
            getattr(_lib, name).argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
            getattr(_lib, name).restype = None
        _lib.mla_oracle_quantize_row_q8_0.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int]
        _lib.mla_oracle_quantize_row_q8_0.restype = None
        _lib.mla_oracle_dequantize_row_q8_0.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
        _lib.mla_oracle_dequantize_row_q8_0.restype = None
    return _lib


def ref_available():
    return os.path.exists(os.path.join(HERE, "_ref", "libref_driver.so"))


def ref():
    """The reference's compiled ggml behind oracle/ref_driver.c; None when oracle/_ref is not built."""
    global _ref
    if _ref is None and ref_available():
        C.CDLL(os.path.join(HERE, "_ref", "libggml_ref.so"), mode=C.RTLD_GLOBAL)
        _ref = C.CDLL(os.path.join(HERE, "_ref", "libref_driver.so"))
        _ref.ref_flash_attn_ext.restype = C.c_int
        _ref.ref_flash_attn_ext.argtypes = [C.c_int] + [C.c_int64] * 5 + [C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_float, C.c_float, C.c_void_p, C.c_int]
        _ref.ref_backend_flash_attn_ext.restype = C.c_int
        _ref.ref_backend_flash_attn_ext.argtypes = [C.c_char_p, C.c_int] + [C.c_int64] * 6 + [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                                    C.c_void_p, C.c_int64, C.c_void_p, C.c_float, C.c_float, C.c_float, C.c_int,
                                                    C.c_void_p, C.c_char_p, C.c_size_t, C.c_void_p, C.c_void_p]
        _ref.ref_kv_cpy.restype = C.c_int
        _ref.ref_kv_cpy.argtypes = [C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_int]
        _ref.ref_backend_kv_cpy.restype = C.c_int
        _ref.ref_backend_kv_cpy.argtypes = [C.c_char_p, C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_char_p, C.c_size_t]
        for name in ("ref_quantize_q8_0_ref", "ref_quantize_q8_0_cpu", "ref_dequantize_q8_0", "ref_f32_to_f16_row", "ref_f32_to_bf16_row", "ref_f16_to_f32_row"):
            getattr(_ref, name).argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
            getattr(_ref, name).restype = None
        _ref.ref_abi_table.restype = C.c_int
        _ref.ref_abi_table.argtypes = [C.c_int, C.POINTER(C.c_char_p), C.POINTER(C.c_int64)]
    return _ref


# ------------------------------------------------------------------ conversions

def _conv(name, x, in_dtype, out_dtype):
    x = np.ascontiguousarray(x, dtype=in_dtype)
    y = np.empty(x.shape, dtype=out_dtype)
    getattr(lib(), name)(x.ctypes.data, y.ctypes.data, x.size)
    return y


def f32_to_bf16(x): return _conv("mla_oracle_f32_to_bf16_row", x, np.float32, np.uint16)
def f32_to_f16(x): return _conv("mla_oracle_f32_to_f16_row", x, np.float32, np.uint16)
def bf16_to_f32(x): return _conv("mla_oracle_bf16_to_f32_row", x, np.uint16, np.float32)
def f16_to_f32(x): return _conv("mla_oracle_f16_to_f32_row", x, np.uint16, np.float32)


def quantize_q8_0(x, mode=0):
    """x float32 [..., n] (n % 32 == 0) -> uint8 [..., n/32*34].  mode 0: reference quantizer, 1: x86 CPU-backend one."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    n = x.shape[-1]
    assert n % 32 == 0
    y = np.empty(x.shape[:-1] + (n // 32 * 34,), dtype=np.uint8)
    lib().mla_oracle_quantize_row_q8_0(x.ctypes.data, y.ctypes.data, x.size, mode)
    return y


def dequantize_q8_0(y):
    y = np.ascontiguousarray(y, dtype=np.uint8)
    n = y.shape[-1] // 34 * 32
    x = np.empty(y.shape[:-1] + (n,), dtype=np.float32)
    lib().mla_oracle_dequantize_row_q8_0(y.ctypes.data, x.ctypes.data, x.size)
    return x


def make_q8_0(qs, d_f16_bits):
    """Assemble Q8_0 rows from int8 quants [..., n] and f16 scale bits [..., n/32] -> uint8 [..., n/32*34]."""
    qs = np.asarray(qs, dtype=np.int8)
    d = np.asarray(d_f16_bits, dtype=np.uint16)
    nb = qs.shape[-1] // 32
    out = np.empty(qs.shape[:-1] + (nb, 34), dtype=np.uint8)
    out[..., 0:2] = d.reshape(d.shape + (1,)).view(np.uint8).reshape(d.shape + (2,))
    out[..., 2:] = qs.reshape(qs.shape[:-1] + (nb, 32)).view(np.uint8)
    return out.reshape(qs.shape[:-1] + (nb * 34,))


def to_f32(k, k_type):
    if k_type == TYPE_BF16: return bf16_to_f32(k)
    if k_type == TYPE_F16: return f16_to_f32(k)
    if k_type == TYPE_Q8_0: return dequantize_q8_0(k)
    raise ValueError(k_type)


# ------------------------------------------------------------------ the op

def _desc(arr, type_id, ne, nb):
    t = _Tensor()
    t.type = type_id
    t.ne = (C.c_int64 * 4)(*ne)
    t.nb = (C.c_int64 * 4)(*nb)
    t.data = arr.ctypes.data
    return t


def _row_bytes(k_type, n=576):
    return n * 2 if k_type in (TYPE_F16, TYPE_BF16) else n // 32 * 34


def _prep(q, k, k_type, dv, mask):
    q = np.ascontiguousarray(q, dtype=np.float32)
    n3, H, N, DK = q.shape
    k = np.ascontiguousarray(k)
    n3k, n_kv = k.shape[0], k.shape[1]
    rb = _row_bytes(k_type, DK)
    assert k.dtype.itemsize * k.shape[2] == rb, (k.shape, k.dtype, rb)
    tq = _desc(q, TYPE_F32, (DK, N, H, n3), (4, DK * 4, DK * 4 * N, DK * 4 * N * H))
    tk = _desc(k, k_type, (DK, n_kv, 1, n3k), (2 if k_type != TYPE_Q8_0 else 34, rb, rb * n_kv, rb * n_kv))
    tv = _desc(k, k_type, (dv, n_kv, 1, n3k), (2 if k_type != TYPE_Q8_0 else 34, rb, rb * n_kv, rb * n_kv))
    tm = None
    if mask is not None:
        mask = np.ascontiguousarray(mask, dtype=np.uint16)
        assert mask.shape[0] >= N and mask.shape[1] >= n_kv
        tm = _desc(mask, TYPE_F16, (mask.shape[1], mask.shape[0], 1, 1), (2, mask.shape[1] * 2, 0, 0))
    return q, k, mask, tq, tk, tv, tm, (n3, H, N, DK)


def flash_attn_ext(q, k, k_type, dv=512, mask=None, scale=1.0, max_bias=0.0, softcap=0.0, q8_mode=1, n_threads=None):
    """The oracle: ggml-cpu's flash_attn_ext restated (oracle/mla_oracle.c).  Returns float32 [n_seq, n_tok, n_head, dv]."""
    q, k, mask, tq, tk, tv, tm, (n3, H, N, DK) = _prep(q, k, k_type, dv, mask)
    out = np.empty((n3, N, H, dv), dtype=np.float32)
    nt = n_threads or min(os.cpu_count() or 1, 16)
    rc = lib().mla_oracle_flash_attn_ext(C.byref(tq), C.byref(tk), C.byref(tv), C.byref(tm) if tm is not None else None,
                                         out.ctypes.data, dv, scale, max_bias, softcap, q8_mode, nt)
    if rc != 0:
        raise RuntimeError("mla_oracle_flash_attn_ext failed: %d" % rc)
    return out


def flash_attn_ext_f64(q, k, k_type, dv=512, mask=None, scale=1.0, q8_mode=1, n_threads=None):
    """softmax(scale q.k + mask).v evaluated in float64 on the same rounded inputs (no ALiBi / softcap)."""
    q, k, mask, tq, tk, tv, tm, (n3, H, N, DK) = _prep(q, k, k_type, dv, mask)
    out = np.empty((n3, N, H, dv), dtype=np.float32)
    nt = n_threads or min(os.cpu_count() or 1, 16)
    rc = lib().mla_oracle_flash_attn_ext_f64(C.byref(tq), C.byref(tk), C.byref(tv), C.byref(tm) if tm is not None else None,
                                             out.ctypes.data, dv, scale, q8_mode, nt)
    if rc != 0:
        raise RuntimeError("mla_oracle_flash_attn_ext_f64 failed: %d" % rc)
    return out


def ref_flash_attn_ext(q, k, k_type, mask=None, scale=1.0, max_bias=0.0, softcap=0.0, n_threads=None):
    """The reference's own compiled ggml-cpu (V := K, all 576 output columns).  float32 [n_seq, n_tok, n_head, 576]."""
    r = ref()
    if r is None:
        raise RuntimeError("oracle/_ref is not built")
    q = np.ascontiguousarray(q, dtype=np.float32)
    n3, H, N, DK = q.shape
    k = np.ascontiguousarray(k)
    assert k.shape[0] == n3
    n_kv = k.shape[1]
    if mask is not None:
        mask = np.ascontiguousarray(mask, dtype=np.uint16)
        assert mask.shape == (N, n_kv)
    out = np.empty((n3, N, H, DK), dtype=np.float32)
    nt = n_threads or min(os.cpu_count() or 1, 16)
    rc = r.ref_flash_attn_ext(k_type, DK, N, H, n3, n_kv, q.ctypes.data, k.ctypes.data, mask.ctypes.data if mask is not None else None,
                              scale, max_bias, softcap, out.ctypes.data, nt)
    if rc != 0:
        raise RuntimeError("ref_flash_attn_ext failed: %d" % rc)
    return out


def ref_backend_flash_attn_ext(so_path, q, k, k_type, dv=576, mask=None, block_table=None, seq_lens=None, scale=1.0,
                               max_bias=0.0, softcap=0.0, use_sched=False, q_second=None):
    """Run the node on a backend .so loaded by the reference's ggml_backend_load, through its ggml-backend API.
    k: [n_seq, n_kv, row] or, with a block table, the pool [n_rows, row].  Returns (float32 [n_seq, n_tok, n_head, 576], info).
    q_second: the graph gets a second attention node over the same cache and mask with these queries (as the layers of one llama
    graph share their mask); the result is then (out, out_second, info)."""
    r = ref()
    if r is None:
        raise RuntimeError("oracle/_ref is not built")
    q = np.ascontiguousarray(q, dtype=np.float32)
    n3, H, N, DK = q.shape
    k = np.ascontiguousarray(k)
    n_kv = k.shape[-2]
    mask_ne0 = 0
    if mask is not None:
        mask = np.ascontiguousarray(mask, dtype=np.uint16)
        mask_ne0 = mask.shape[1]
    max_blocks = 0
    if block_table is not None:
        block_table = np.ascontiguousarray(block_table, dtype=np.int32)
        seq_lens = np.ascontiguousarray(seq_lens, dtype=np.int32)
        max_blocks = block_table.shape[1]
    out = np.full((n3, N, H, DK), np.nan, dtype=np.float32)
    out_b = None
    if q_second is not None:
        q_second = np.ascontiguousarray(q_second, dtype=np.float32)
        assert q_second.shape == q.shape
        out_b = np.full((n3, N, H, DK), np.nan, dtype=np.float32)
    info = C.create_string_buffer(512)
    rc = r.ref_backend_flash_attn_ext(so_path.encode(), k_type, DK, dv, N, H, n3, n_kv, q.ctypes.data, k.ctypes.data,
                                      mask.ctypes.data if mask is not None else None, mask_ne0,
                                      block_table.ctypes.data if block_table is not None else None, max_blocks,
                                      seq_lens.ctypes.data if seq_lens is not None else None,
                                      scale, max_bias, softcap, int(use_sched), out.ctypes.data, info, 512,
                                      q_second.ctypes.data if q_second is not None else None, out_b.ctypes.data if out_b is not None else None)
    if rc != 0:
        raise RuntimeError("ref_backend_flash_attn_ext failed: %d (%s)" % (rc, info.value.decode()))
    if q_second is not None:
        return out, out_b, info.value.decode()
    return out, info.value.decode()


def ref_abi_table():
    r = ref()
    name, val = C.c_char_p(), C.c_int64()
    n = r.ref_abi_table(-1, C.byref(name), C.byref(val))
    out = {}
    for i in range(n):
        r.ref_abi_table(i, C.byref(name), C.byref(val))
        out[name.value.decode()] = val.value
    return out


# ------------------------------------------------------------------ error metrics used by every parity test

def errors(a, b):
    """(max-abs error, relative L2 error) of a against b."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.max(np.abs(a - b))), float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


def kv_write(src, cache, kv_type, dest_rows, src_type=TYPE_F32, q8_mode=1):
    """The cache write as ggml-cpu's ggml_cpy does it per row: cache (uint16 [rows, 576] or uint8 [rows, 612]) is updated
    in place and returned; src is float32 [n_tok, 576] (converted) or rows already in the cache type (copied)."""
    src = np.ascontiguousarray(src)
    assert cache.flags.c_contiguous
    dest = np.ascontiguousarray(dest_rows, dtype=np.int64)
    assert dest.shape == (src.shape[0],)
    rc = lib().mla_oracle_kv_write(src.ctypes.data, src_type, src.strides[0], src.shape[0], cache.ctypes.data, kv_type,
                                   cache.strides[0], cache.shape[0], dest.ctypes.data, q8_mode)
    if rc != 0:
        raise RuntimeError("mla_oracle_kv_write failed: %d" % rc)
    return cache


def ref_kv_cpy(kv_cur, cache, kv_type, kv_head, n_threads=4):
    """ggml_cpy(kv_cur, view of the cache at row kv_head) on the reference's compiled ggml-cpu; cache updated in place."""
    kv_cur = np.ascontiguousarray(kv_cur, dtype=np.float32)
    assert cache.flags.c_contiguous
    rc = ref().ref_kv_cpy(kv_type, cache.shape[0], kv_head, kv_cur.shape[0], kv_cur.ctypes.data, cache.ctypes.data, n_threads)
    if rc != 0:
        raise RuntimeError("ref_kv_cpy failed: %d" % rc)
    return cache


def ref_backend_kv_cpy(so_path, kv_cur, cache, kv_type, kv_head):
    """The same node computed by a backend plugin loaded through the reference's ggml_backend_load."""
    kv_cur = np.ascontiguousarray(kv_cur, dtype=np.float32)
    assert cache.flags.c_contiguous
    info = C.create_string_buffer(256)
    rc = ref().ref_backend_kv_cpy(so_path.encode(), kv_type, cache.shape[0], kv_head, kv_cur.shape[0], kv_cur.ctypes.data,
                                  cache.ctypes.data, info, 256)
    if rc != 0:
        raise RuntimeError("ref_backend_kv_cpy failed: %d (%s)" % (rc, info.value.decode()))
    return cache, info.value.decode()


# ------------------------------------------------------------------ the nodes either side of the attention node

class RopeParams(C.Structure):
    """ggml_rope_ext's scalar arguments (ggml/src/ggml.c:3413-3449); mode 0 = adjacent pairs, 2 = NeoX halves."""
    _fields_ = [("n_dims", C.c_int32), ("mode", C.c_int32), ("n_ctx_orig", C.c_int32), ("freq_base", C.c_float),
                ("freq_scale", C.c_float), ("ext_factor", C.c_float), ("attn_factor", C.c_float), ("beta_fast", C.c_float),
                ("beta_slow", C.c_float)]


def rope_params(n_dims=64, mode=0, n_ctx_orig=4096, freq_base=10000.0, freq_scale=1.0, ext_factor=0.0, attn_factor=1.0,
                beta_fast=32.0, beta_slow=1.0):
    return RopeParams(n_dims, mode, n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow)


def _front():
    l = lib()
    if not hasattr(l, "_front_ready"):
        l.mla_oracle_rope.restype = C.c_int
        l.mla_oracle_rope.argtypes = [C.c_void_p, C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.c_void_p, C.POINTER(C.c_int64),
                                      C.c_void_p, C.c_void_p, C.POINTER(RopeParams)]
        l.mla_oracle_mul_mat.restype = C.c_int
        l.mla_oracle_mul_mat.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.c_void_p,
                                         C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.c_void_p, C.c_void_p]
        l.mla_oracle_rope_corr_dims.restype = None
        l.mla_oracle_rope_corr_dims.argtypes = [C.c_int, C.c_int, C.c_float, C.c_float, C.c_float, C.POINTER(C.c_float)]
        l._front_ready = True
    return l


def _i64x4(v):
    return (C.c_int64 * 4)(*[int(x) for x in v])


def rope(x, pos, p, freq_factors=None):
    """GGML_OP_ROPE as ggml-cpu computes it.  x float32 [n_tok, n_head, ne0] (ggml ne = {ne0, n_head, n_tok}), any
    strides with a unit last one; pos int32 [n_tok]; returns a contiguous array of the same shape."""
    assert x.dtype == np.float32 and x.ndim == 3 and x.strides[2] == 4
    pos = np.ascontiguousarray(pos, dtype=np.int32)
    out = np.empty(x.shape, dtype=np.float32)
    ff = None if freq_factors is None else np.ascontiguousarray(freq_factors, dtype=np.float32)
    ne = _i64x4([x.shape[2], x.shape[1], x.shape[0], 1])
    nb = _i64x4([4, x.strides[1], x.strides[0], 0])
    dnb = _i64x4([4, out.strides[1], out.strides[0], 0])
    rc = _front().mla_oracle_rope(x.ctypes.data, ne, nb, out.ctypes.data, dnb, pos.ctypes.data,
                                  None if ff is None else ff.ctypes.data, C.byref(p))
    if rc != 0:
        raise RuntimeError("mla_oracle_rope failed: %d" % rc)
    return out


def rope_corr_dims(p):
    d = (C.c_float * 2)()
    _front().mla_oracle_rope_corr_dims(p.n_dims, p.n_ctx_orig, p.freq_base, p.beta_fast, p.beta_slow, d)
    return float(d[0]), float(d[1])


def mul_mat(a, a_type, b, with_abs=False):
    """GGML_OP_MUL_MAT: a = src0 [ne02, N, K] (uint16 bits for F16/BF16, float32 for F32), b = src1 float32 [ne12, M, K],
    any strides with a unit last one; out float32 [ne12, M, N] (ne12 % ne02 == 0, src0 broadcast over the quotient)."""
    assert a.ndim == 3 and b.ndim == 3 and b.dtype == np.float32 and a.strides[2] == a.itemsize and b.strides[2] == 4
    ne0 = _i64x4([a.shape[2], a.shape[1], a.shape[0], 1])
    nb0 = _i64x4([a.itemsize, a.strides[1], a.strides[0], 0])
    ne1 = _i64x4([b.shape[2], b.shape[1], b.shape[0], 1])
    nb1 = _i64x4([4, b.strides[1], b.strides[0], 0])
    out = np.empty((b.shape[0], b.shape[1], a.shape[1]), dtype=np.float32)
    ab = np.empty_like(out) if with_abs else None
    rc = _front().mla_oracle_mul_mat(a.ctypes.data, a_type, ne0, nb0, b.ctypes.data, ne1, nb1, out.ctypes.data,
                                     None if ab is None else ab.ctypes.data)
    if rc != 0:
        raise RuntimeError("mla_oracle_mul_mat failed: %d" % rc)
    return (out, ab) if with_abs else out


def mla_q_states(q, wkv_b, w_type, pos, p, n_head):
    """The query side of llm_attn_mla (src/llama-graph-attn.cpp:264-277 after the rope of
    src/llama-graph-deepseek2.cpp:216-222) from the oracle's own pieces: q float32 [n_tok, n_head*192], wkv_b
    [n_head*256, 512] in w_type; returns q_states float32 [n_head, n_tok, 576]."""
    n_tok = q.shape[0]
    q3 = q.reshape(n_tok, n_head, 192)
    q_pe = rope(np.ascontiguousarray(q3[:, :, 128:]), pos, p)                    # [n_tok, H, 64]
    wk_b = wkv_b.reshape(-1)[:n_head * 512 * 128].reshape(n_head, 512, 128)       # ggml ne = {128, 512, H}
    q_abs = mul_mat(wk_b, w_type, q3[:, :, :128].transpose(1, 0, 2))              # [H, n_tok, 512]
    return np.concatenate([q_abs, q_pe.transpose(1, 0, 2)], axis=2)


def mla_unabsorb(kqv, wkv_b, w_type, n_head):
    """The output side (src/llama-graph-attn.cpp:303-323): kqv float32 [n_head, n_tok, 512] -> float32 [n_tok, n_head*128]."""
    n_tok = kqv.shape[1]
    wv_b = wkv_b.reshape(-1)[n_head * 512 * 128:].reshape(n_head, 128, 512)       # ggml ne = {512, 128, H}
    o = mul_mat(wv_b, w_type, kqv)                                                # [H, n_tok, 128]
    return np.ascontiguousarray(o.transpose(1, 0, 2)).reshape(n_tok, n_head * 128)


def _ref_front():
    r = ref()
    if not hasattr(r, "_front_ready"):
        r.ref_rope.restype = C.c_int
        r.ref_rope.argtypes = [C.c_char_p, C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p,
                               C.POINTER(RopeParams), C.c_void_p, C.c_int]
        r.ref_mul_mat.restype = C.c_int
        r.ref_mul_mat.argtypes = [C.c_char_p, C.c_int] + [C.c_int64] * 5 + [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
        r.ref_mla_q_states.restype = C.c_int
        r.ref_mla_q_states.argtypes = [C.c_char_p, C.c_int, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p,
                                       C.POINTER(RopeParams), C.c_void_p, C.c_int]
        r.ref_mla_unabsorb.restype = C.c_int
        r.ref_mla_unabsorb.argtypes = [C.c_char_p, C.c_int, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
        r.ref_mla_layer.restype = C.c_int
        r.ref_mla_layer.argtypes = [C.c_char_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int64, C.c_int64, C.c_int, C.c_void_p, C.c_void_p,
                                    C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p,
                                    C.c_int]
        r.ref_random_front.restype = C.c_int
        r.ref_random_front.argtypes = [C.c_char_p, C.c_uint32, C.c_int64, C.c_int64, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                       C.c_void_p, C.c_void_p, C.POINTER(C.c_int32), C.c_int]
        r._front_ready = True
    return r


def _so(so_path):
    return None if so_path is None else so_path.encode()


def ref_rope(x, pos, p, freq_factors=None, so_path=None, n_threads=4):
    """One ROPE node on the reference's ggml-cpu (so_path None) or on the backend plugin loaded from so_path."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    pos = np.ascontiguousarray(pos, dtype=np.int32)
    ff = None if freq_factors is None else np.ascontiguousarray(freq_factors, dtype=np.float32)
    out = np.full(x.shape, np.nan, dtype=np.float32)
    rc = _ref_front().ref_rope(_so(so_path), x.shape[2], x.shape[1], x.shape[0], x.ctypes.data, pos.ctypes.data,
                               None if ff is None else ff.ctypes.data, C.byref(p), out.ctypes.data, n_threads)
    if rc != 0:
        raise RuntimeError("ref_rope failed: %d" % rc)
    return out


def ref_mul_mat(a, a_type, b, so_path=None, n_threads=4):
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b, dtype=np.float32)
    out = np.full((b.shape[0], b.shape[1], a.shape[1]), np.nan, dtype=np.float32)
    rc = _ref_front().ref_mul_mat(_so(so_path), a_type, a.shape[2], a.shape[1], a.shape[0], b.shape[1], b.shape[0],
                                  a.ctypes.data, b.ctypes.data, out.ctypes.data, n_threads)
    if rc != 0:
        raise RuntimeError("ref_mul_mat failed: %d" % rc)
    return out


def ref_mla_q_states(q, wkv_b, w_type, pos, p, n_head, so_path=None, n_threads=4):
    q = np.ascontiguousarray(q, dtype=np.float32)
    wkv_b = np.ascontiguousarray(wkv_b)
    pos = np.ascontiguousarray(pos, dtype=np.int32)
    n_tok = q.shape[0]
    out = np.full((n_head, n_tok, 576), np.nan, dtype=np.float32)
    rc = _ref_front().ref_mla_q_states(_so(so_path), w_type, n_head, n_tok, q.ctypes.data, wkv_b.ctypes.data, pos.ctypes.data,
                                       C.byref(p), out.ctypes.data, n_threads)
    if rc != 0:
        raise RuntimeError("ref_mla_q_states failed: %d" % rc)
    return out


def ref_mla_unabsorb(kqv, wkv_b, w_type, n_head, so_path=None, n_threads=4):
    kqv = np.ascontiguousarray(kqv, dtype=np.float32)
    wkv_b = np.ascontiguousarray(wkv_b)
    n_tok = kqv.shape[1]
    out = np.full((n_tok, n_head * 128), np.nan, dtype=np.float32)
    rc = _ref_front().ref_mla_unabsorb(_so(so_path), w_type, n_head, n_tok, kqv.ctypes.data, wkv_b.ctypes.data, out.ctypes.data,
                                       n_threads)
    if rc != 0:
        raise RuntimeError("ref_mla_unabsorb failed: %d" % rc)
    return out


def ref_random_front(seed, n_head, n_tok, n_ops, kv_type, a, b, pos, so_path=None, n_threads=4):
    """A graph of cont / rope_ext / concat nodes and the k side's rope -> concat -> cpy drawn from `seed` (oracle/ref_driver.c),
    allocated by ggml's graph allocator, on the reference's ggml-cpu (so_path None) or the backend plugin.  a: f32 [n_tok, n_head,
    192], b: f32 [n_tok, 576], pos: int32 [n_tok].  Returns (result f32 [n_tok, n_head, 192], cache rows as bytes, nodes)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    pos = np.ascontiguousarray(pos, dtype=np.int32)
    assert a.shape == (n_tok, n_head, 192) and b.shape == (n_tok, 576) and pos.shape == (n_tok,)
    out = np.full((n_tok, n_head, 192), np.nan, dtype=np.float32)
    cache = np.zeros((n_tok, 612 if kv_type == TYPE_Q8_0 else 1152), dtype=np.uint8)
    n_nodes = C.c_int32(0)
    rc = _ref_front().ref_random_front(_so(so_path), seed, n_head, n_tok, n_ops, kv_type, a.ctypes.data, b.ctypes.data, pos.ctypes.data,
                                       out.ctypes.data, cache.ctypes.data, C.byref(n_nodes), n_threads)
    if rc != 0:
        raise RuntimeError("ref_random_front(seed %d) failed: %d" % (seed, rc))
    return out, cache, n_nodes.value


def ref_mla_layer(mode, k_type, w_type, n_head, n_ctx, steps, wkv_b, kq_scale, so_path=None, v_type=TYPE_F16, block_table=None,
                  n_threads=4, rope_in_graph=False):
    """Steps of llm_attn_mla on one KV cache.  mode 0: the unfused graph the reference emits (src/llama-graph-attn.cpp:233-323)
    on its ggml-cpu, with a K cache of k_type and a transposed V cache of v_type; mode 1 / 2: the one-node form on the backend
    plugin at so_path under ggml_backend_sched, the cache written by CPY (1) or as a page pool by SCATTER_UPDATE with a block
    table (2).  steps = [(q f32 [n_tok, n_head, 192], kv_cur f32 [n_tok, 576]), ...], appended to the one sequence in order.
    rope_in_graph: q_pe and the last 64 values of the kv_cur rows arrive unrotated and the graph holds the model's own
    cont / rope_ext / view / concat nodes for them (src/llama-graph-deepseek2.cpp:216-236), positions = cache positions.
    Returns (outputs [f32 [n_tok, 128 * n_head] per step], on_backend flags per step, cache bytes after the last step)."""
    n_tok = np.array([q.shape[0] for q, _ in steps], dtype=np.int32)
    kv_head = np.concatenate([[0], np.cumsum(n_tok)[:-1]]).astype(np.int32)
    q = np.ascontiguousarray(np.concatenate([np.asarray(q, dtype=np.float32).reshape(-1) for q, _ in steps]))
    kv = np.ascontiguousarray(np.concatenate([np.asarray(k, dtype=np.float32).reshape(-1) for _, k in steps]))
    for qq, kk in steps:
        assert qq.shape[1:] == (n_head, 192) and kk.shape == (qq.shape[0], 576)
    wkv_b = np.ascontiguousarray(wkv_b)
    out = np.full((int(n_tok.sum()), n_head * 128), np.nan, dtype=np.float32)
    where = np.zeros(len(steps), dtype=np.int32)
    cache = np.zeros((n_ctx, 612 if k_type == TYPE_Q8_0 else 1152), dtype=np.uint8)
    bt = None if block_table is None else np.ascontiguousarray(block_table, dtype=np.int32)
    rc = _ref_front().ref_mla_layer(_so(so_path), mode | (8 if rope_in_graph else 0), k_type, v_type, w_type, n_head, n_ctx, len(steps), n_tok.ctypes.data,
                                    kv_head.ctypes.data, q.ctypes.data, kv.ctypes.data, wkv_b.ctypes.data, kq_scale,
                                    None if bt is None else bt.ctypes.data, 0 if bt is None else bt.shape[-1], out.ctypes.data,
                                    where.ctypes.data, cache.ctypes.data, n_threads)
    if rc != 0:
        raise RuntimeError("ref_mla_layer(mode %d%s) failed: %d" % (mode, ", rope in the graph" if rope_in_graph else "", rc))
    ends = np.cumsum(n_tok)
    return [out[e - n:e] for e, n in zip(ends, n_tok)], where, cache
