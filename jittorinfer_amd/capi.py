"""ctypes binding of include/mla_attn.h.  PyTorch is used for device memory and streams only."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))

MLA_TYPE_F32, MLA_TYPE_F16, MLA_TYPE_Q8_0, MLA_TYPE_BF16 = 0, 1, 8, 30
MLA_FLAG_F16_ACC_STRICT = 1
MLA_FLAG_UNIFORM_SPLITS = 2
MLA_FLAG_BF16_DIRECT = 4
MLA_FLAG_MASK_EXTENTS_VALID = 8
MLA_FLAG_Q8_EXACT = 16
MLA_ERR_TOO_LARGE = -7
MLA_ATTN_STATIC_WORKSPACE_MAX = 48 << 20
PAGE_TOKENS = 128
ROW_BYTES = {MLA_TYPE_F16: 1152, MLA_TYPE_BF16: 1152, MLA_TYPE_Q8_0: 612}


class MlaAttnArgs(C.Structure):
    _fields_ = [
        ("n_seq", C.c_int32), ("n_head", C.c_int32), ("n_tok", C.c_int32), ("dk", C.c_int32), ("dv", C.c_int32),
        ("q_type", C.c_int32), ("kv_type", C.c_int32), ("flags", C.c_uint32),
        ("scale", C.c_float), ("max_bias", C.c_float), ("logit_softcap", C.c_float),
        ("q", C.c_void_p), ("q_nb1", C.c_int64), ("q_nb2", C.c_int64), ("q_nb3", C.c_int64),
        ("kv", C.c_void_p), ("kv_nb1", C.c_int64), ("kv_nb3", C.c_int64), ("n_kv", C.c_int64),
        ("mask", C.c_void_p), ("mask_nb1", C.c_int64), ("mask_ne0", C.c_int64),
        ("block_table", C.c_void_p), ("bt_stride", C.c_int64), ("seq_lens", C.c_void_p),
        ("dst", C.c_void_p), ("dst_nb1", C.c_int64),
        ("workspace", C.c_void_p), ("workspace_size", C.c_size_t),
        ("n_splits", C.c_int32), ("rows_per_wg", C.c_int32),
    ]


class MlaPlanInfo(C.Structure):
    _fields_ = [("variant", C.c_int32), ("rows_per_wg", C.c_int32), ("n_row_blocks", C.c_int32), ("n_splits", C.c_int32),
                ("split_tokens", C.c_int32), ("n_passes", C.c_int32), ("lds_bytes", C.c_int64), ("balanced", C.c_int32),
                ("n_workgroups", C.c_int32)]


def library_path():
    # JITTORINFER_AMD_LIB: development override (an experimental build of the same library)
    return os.environ.get("JITTORINFER_AMD_LIB") or os.path.join(HERE, "libggml-hip-mla.so")


_lib = None


def library():
    """The HIP library; raises if it has not been built (python -m jittorinfer_amd.build)."""
    global _lib
    if _lib is None:
        path = library_path()
        if not os.path.exists(path):
            raise RuntimeError("%s is missing: build it with `python jittorinfer_amd/build.py` (there is no CPU fallback)" % path)
        lib = C.CDLL(path)
        lib.mla_attn_workspace_size.restype = C.c_size_t
        lib.mla_attn_workspace_size.argtypes = [C.POINTER(MlaAttnArgs)]
        lib.mla_attn_plan.restype = C.c_int
        lib.mla_attn_plan.argtypes = [C.POINTER(MlaAttnArgs), C.POINTER(MlaPlanInfo)]
        lib.mla_attn_launch.restype = C.c_int
        lib.mla_attn_launch.argtypes = [C.POINTER(MlaAttnArgs), C.c_void_p]
        for name in ("mla_attn_launch_partials", "mla_attn_launch_combine", "mla_attn_launch_kernel", "mla_attn_launch_static"):
            getattr(lib, name).restype = C.c_int
            getattr(lib, name).argtypes = [C.POINTER(MlaAttnArgs), C.c_void_p]
        lib.mla_hbm_copy_launch.restype = C.c_int
        lib.mla_hbm_copy_launch.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
        lib.mla_kv_write_launch.restype = C.c_int
        lib.mla_kv_write_launch.argtypes = [C.POINTER(MlaKvWriteArgs), C.c_void_p]
        for name, cls in (("mla_rope_launch", MlaRopeArgs), ("mla_mul_mat_launch", MlaMulMatArgs), ("mla_copy_f32_launch", MlaCopyArgs),
                          ("mla_kv_write_rope_launch", MlaKvWriteRopeArgs)):
            getattr(lib, name).restype = C.c_int
            getattr(lib, name).argtypes = [C.POINTER(cls), C.c_void_p]
        lib.mla_front_batch_launch.restype = C.c_int
        lib.mla_front_batch_launch.argtypes = [C.POINTER(MlaFrontOp), C.c_int32, C.c_void_p]
        lib.mla_page_table_create.restype = C.c_void_p
        lib.mla_page_table_create.argtypes = [C.c_int32] * 3
        lib.mla_page_table_free.argtypes = [C.c_void_p]
        lib.mla_page_table_clear.argtypes = [C.c_void_p]
        lib.mla_page_table_find_slot.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]
        lib.mla_page_table_seq_rm.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_int32]
        lib.mla_page_table_seq_cp.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32] + [C.POINTER(C.c_int32)] * 3
        lib.mla_page_table_seq_unshare.argtypes = [C.c_void_p, C.c_int32] + [C.POINTER(C.c_int32)] * 3
        lib.mla_page_table_seq_keep.argtypes = [C.c_void_p, C.c_int32]
        lib.mla_page_table_seq_add.argtypes = [C.c_void_p] + [C.c_int32] * 4
        lib.mla_page_table_defrag.argtypes = [C.c_void_p, C.POINTER(C.c_int32)]
        for name in ("mla_page_table_seq_len", "mla_page_table_free_pages", "mla_page_table_used_cells"):
            getattr(lib, name).restype = C.c_int32
        lib.mla_page_table_seq_len.argtypes = [C.c_void_p, C.c_int32]
        lib.mla_page_table_free_pages.argtypes = [C.c_void_p]
        lib.mla_page_table_used_cells.argtypes = [C.c_void_p]
        lib.mla_page_table_fill_inputs.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]
        lib.mla_attn_target_arch.restype = C.c_char_p
        lib.ggml_backend_init.restype = C.c_void_p
        lib.ggml_backend_score.restype = C.c_int
        lib.mla_ggml_abi_table.restype = C.c_int
        lib.mla_ggml_abi_table.argtypes = [C.c_int, C.POINTER(C.c_char_p), C.POINTER(C.c_int64)]
        _lib = lib
    return _lib


class MlaKvWriteArgs(C.Structure):
    """mla_kv_write_args of include/mla_kv_write.h."""
    _fields_ = [("n_tok", C.c_int32), ("src_type", C.c_int32), ("kv_type", C.c_int32), ("rows_type", C.c_int32),
                ("src", C.c_void_p), ("src_nb1", C.c_int64), ("kv", C.c_void_p), ("kv_nb1", C.c_int64), ("n_kv_rows", C.c_int64),
                ("row0", C.c_int64), ("rows", C.c_void_p), ("block_table", C.c_void_p), ("bt_stride", C.c_int64),
                ("seq_ids", C.c_void_p), ("positions", C.c_void_p)]


_workspaces = {}
_retired = []


def _workspace(device, nbytes, stream=None):
    """The scratch area of a launch: one per (device, stream) -- launches on different streams run side by side and each
    needs its own partials, Q image and schedule.  An area that has been handed out is not freed while work may use it: a launch
    queued earlier or recorded into a HIP graph keeps its address, so a larger request gets a new area and the old one is retired.
    Areas grow by at least half (requests that creep up -- a decode loop adding one key per step -- retire O(log size) areas, not
    one per step); release_workspaces() drops what has been retired.  Under graph capture the new area comes from the graph's own
    memory pool, like any tensor made during capture."""
    import torch
    if stream is None:
        stream = torch.cuda.current_stream(device).cuda_stream
    key = (device, int(stream))
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        have = 0
        if ws is not None:
            _retired.append(ws)
            have = ws.numel()
        ws = torch.empty(max(nbytes, have + have // 2, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def release_workspaces(stream=None, device=None):
    """Drops the retired scratch areas and, for a stream that is given (a raw handle; with its device), that stream's current one --
    to be called when the stream is destroyed, or at any point where no launch that used them is still queued or held in a HIP
    graph that will be replayed: the call synchronizes the device first and refuses to run under graph capture."""
    import torch
    if torch.cuda.is_current_stream_capturing():
        raise RuntimeError("release_workspaces: not under graph capture")
    torch.cuda.synchronize(device)
    _retired.clear()
    if stream is not None:
        dev = torch.device("cuda", torch.cuda.current_device()) if device is None else device
        _workspaces.pop((dev, int(stream)), None)


def make_args(q, k, kv_type, dv=512, mask=None, scale=1.0, max_bias=0.0, logit_softcap=0.0, block_table=None,
              seq_lens=None, out=None, n_splits=0, flags=0, rows_per_wg=0, stream=None):
    """Builds (args, out, keepalive) from torch tensors on one gfx950 device, for a launch on `stream` (a raw handle; None: the
    current torch stream) -- the workspace is that stream's.

    q     float32 [n_seq, n_head, n_tok, 576] (any strides with a contiguous last dim)
    k     the latent KV rows: [n_seq, n_kv, row] (uint8/int16/bfloat16/float16 with `row` 1152/612 bytes) or,
          with a block table, the page pool [n_rows, row] (n_rows a multiple of 128)
    mask  float16 [>= n_tok, mask_ne0] or None;  block_table int32 [n_seq, max_blocks];  seq_lens int32 [n_seq]
    out   float32 [n_seq, n_tok, n_head, 576] (ggml's dst layout); created if None.  dv columns of each row are written.
    """
    import torch
    assert q.dtype == torch.float32 and q.dim() == 4 and q.shape[-1] == 576 and q.stride(-1) == 1
    n_seq, n_head, n_tok, _ = q.shape
    row = ROW_BYTES[kv_type]
    a = MlaAttnArgs()
    a.n_seq, a.n_head, a.n_tok, a.dk, a.dv = n_seq, n_head, n_tok, 576, dv
    a.q_type, a.kv_type, a.flags = MLA_TYPE_F32, kv_type, flags
    a.scale, a.max_bias, a.logit_softcap = scale, max_bias, logit_softcap
    a.q = q.data_ptr()
    a.q_nb1, a.q_nb2, a.q_nb3 = q.stride(2) * 4, q.stride(1) * 4, q.stride(0) * 4
    es = k.element_size()
    assert k.stride(-1) == 1 and k.shape[-1] * es == row, (k.shape, k.dtype)
    a.kv = k.data_ptr()
    if block_table is not None:
        assert k.dim() == 2 and k.shape[0] % PAGE_TOKENS == 0
        a.kv_nb1, a.kv_nb3, a.n_kv = k.stride(0) * es, 0, k.shape[0]
        assert block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.shape[0] == n_seq and block_table.is_contiguous()
        assert seq_lens.dtype == torch.int32 and seq_lens.numel() == n_seq and seq_lens.is_contiguous()
        a.block_table, a.bt_stride, a.seq_lens = block_table.data_ptr(), block_table.shape[1], seq_lens.data_ptr()
    else:
        assert k.dim() == 3 and k.shape[0] in (1, n_seq)
        a.kv_nb1, a.kv_nb3, a.n_kv = k.stride(1) * es, (k.stride(0) * es if k.shape[0] > 1 else 0), k.shape[1]
    if mask is not None:
        assert mask.dtype == torch.float16 and mask.dim() == 2 and mask.stride(1) == 1 and mask.shape[0] >= n_tok
        a.mask, a.mask_nb1, a.mask_ne0 = mask.data_ptr(), mask.stride(0) * 2, mask.shape[1]
    if out is None:
        out = torch.empty((n_seq, n_tok, n_head, 576), dtype=torch.float32, device=q.device)
    assert out.dtype == torch.float32 and out.is_contiguous() and out.shape[:3] == (n_seq, n_tok, n_head) and out.shape[3] >= dv
    a.dst, a.dst_nb1 = out.data_ptr(), out.shape[3] * 4
    a.n_splits = n_splits
    a.rows_per_wg = rows_per_wg
    need = library().mla_attn_workspace_size(C.byref(a))
    ws = _workspace(q.device, need, stream)
    a.workspace, a.workspace_size = ws.data_ptr(), ws.numel()
    return a, out, (q, k, mask, block_table, seq_lens, ws)


def ggml_flash_attn_ext(q, k, kv_type, dv=512, mask=None, scale=1.0, max_bias=0.0, logit_softcap=0.0, *,
                        block_table=None, seq_lens=None, out=None, n_splits=0, flags=0, rows_per_wg=0, stream=None):
    """GGML_OP_FLASH_ATTN_EXT of the reference (ggml_flash_attn_ext(ctx, q, k, v, mask, scale, max_bias,
    logit_softcap), ggml/src/ggml.c:3988) for the MLA shape, on the current torch stream.  v is the first `dv`
    columns of k's rows.  Returns dst in ggml's layout: float32 [n_seq, n_tok, n_head, 576] with dv columns valid."""
    import torch
    if not q.is_cuda:
        raise RuntimeError("jittorinfer_amd runs on a gfx950 GPU only (there is no CPU path)")
    a, out, keep = make_args(q, k, kv_type, dv, mask, scale, max_bias, logit_softcap, block_table, seq_lens, out, n_splits, flags, rows_per_wg, stream)
    st = stream if stream is not None else torch.cuda.current_stream(q.device).cuda_stream
    rc = library().mla_attn_launch(C.byref(a), C.c_void_p(st))
    if rc != 0:
        raise RuntimeError("mla_attn_launch failed with code %d" % rc)
    return out


def plan(q, k, kv_type, **kw):
    a, _, keep = make_args(q, k, kv_type, **kw)
    info = MlaPlanInfo()
    rc = library().mla_attn_plan(C.byref(a), C.byref(info))
    if rc != 0:
        raise RuntimeError("mla_attn_plan failed with code %d" % rc)
    return {f: getattr(info, f) for f, _ in MlaPlanInfo._fields_}


def hbm_copy(src, dst, stream=None):
    import torch
    st = stream if stream is not None else torch.cuda.current_stream(src.device).cuda_stream
    rc = library().mla_hbm_copy_launch(src.data_ptr(), dst.data_ptr(), src.numel() * src.element_size(), C.c_void_p(st))
    if rc != 0:
        raise RuntimeError("mla_hbm_copy_launch failed with code %d" % rc)


def kv_write(src, cache, kv_type, *, row0=None, rows=None, block_table=None, seq_ids=None, positions=None, stream=None,
             k_pe=None, rope=None, batch=None):
    """The KV cache write (ggml_cpy of src/llama-graph-attn.cpp:236-241 / ggml_scatter_update of :380-383) on the current
    torch stream.  src: float32 [n_tok, 576] (converted to the cache type on write) or rows already in the cache type;
    cache: [n_rows, row] in the storage type (row = 1152 or 612 bytes).  Exactly one addressing mode: row0 (consecutive
    rows), rows (int32/int64 [n_tok] row indices), or block_table + seq_ids + positions (128-token pages).
    k_pe + rope: values 512 .. 575 of every row are k_pe (float32 [n_tok, 64], not yet rotated) rotated on the way
    (mla_kv_write_rope_launch); rope = dict(pos=..., and the keywords of ggml_rope_ext).  batch: a FrontBatch that takes
    the launch instead of the stream."""
    import torch
    if not src.is_cuda:
        raise RuntimeError("jittorinfer_amd runs on a gfx950 GPU only (there is no CPU path)")
    ra = None
    if k_pe is not None:
        ra = MlaKvWriteRopeArgs()
        a = ra.w
        kw = dict(rope)
        rpos = kw.pop("pos")
        assert k_pe.dtype == torch.float32 and k_pe.dim() == 2 and k_pe.shape == (src.shape[0], 64) and k_pe.stride(1) == 1
        _fill_rope_args(ra.rope, k_pe.unsqueeze(1), rpos, k_pe.unsqueeze(1), **kw)
    else:
        a = MlaKvWriteArgs()
    a.n_tok = src.shape[0]
    a.kv_type = kv_type
    a.src_type = MLA_TYPE_F32 if src.dtype == torch.float32 else kv_type
    assert src.dim() == 2 and src.stride(1) == 1 and cache.dim() == 2 and cache.stride(1) == 1
    assert cache.shape[1] * cache.element_size() == ROW_BYTES[kv_type]
    if a.src_type == MLA_TYPE_F32:
        assert src.shape[1] == 576 or (ra is not None and src.shape[1] >= 512)
    else:
        assert src.shape[1] * src.element_size() == ROW_BYTES[kv_type]
    a.src, a.src_nb1 = src.data_ptr(), src.stride(0) * src.element_size()
    a.kv, a.kv_nb1, a.n_kv_rows = cache.data_ptr(), cache.stride(0) * cache.element_size(), cache.shape[0]
    assert (row0 is not None) + (rows is not None) + (block_table is not None) == 1
    if row0 is not None:
        a.row0 = row0
    elif rows is not None:
        assert rows.dtype in (torch.int32, torch.int64) and rows.is_contiguous() and rows.numel() == a.n_tok
        a.rows, a.rows_type = rows.data_ptr(), 1 if rows.dtype == torch.int64 else 0
    else:
        for t in (block_table, seq_ids, positions):
            assert t.dtype == torch.int32 and t.is_contiguous()
        assert block_table.dim() == 2 and seq_ids.numel() == a.n_tok and positions.numel() == a.n_tok
        a.block_table, a.bt_stride = block_table.data_ptr(), block_table.shape[1]
        a.seq_ids, a.positions = seq_ids.data_ptr(), positions.data_ptr()
    if batch is not None:
        batch.add(MLA_FRONT_KV_WRITE_ROPE if ra is not None else MLA_FRONT_KV_WRITE, ra if ra is not None else a)
        return cache
    st = stream if stream is not None else torch.cuda.current_stream(src.device).cuda_stream
    rc = library().mla_kv_write_rope_launch(C.byref(ra), C.c_void_p(st)) if ra is not None else library().mla_kv_write_launch(C.byref(a), C.c_void_p(st))
    if rc != 0:
        raise RuntimeError("mla_kv_write%s_launch failed with code %d" % ("_rope" if ra is not None else "", rc))
    return cache


class MlaRopeArgs(C.Structure):
    """mla_rope_args of include/mla_front.h."""
    _fields_ = [("src", C.c_void_p), ("ne", C.c_int64 * 4), ("src_nb", C.c_int64 * 4), ("dst", C.c_void_p), ("dst_nb", C.c_int64 * 4),
                ("pos", C.c_void_p), ("freq_factors", C.c_void_p), ("n_dims", C.c_int32), ("mode", C.c_int32),
                ("n_ctx_orig", C.c_int32), ("freq_base", C.c_float), ("freq_scale", C.c_float), ("ext_factor", C.c_float),
                ("attn_factor", C.c_float), ("beta_fast", C.c_float), ("beta_slow", C.c_float)]


class MlaMulMatArgs(C.Structure):
    """mla_mul_mat_args of include/mla_front.h."""
    _fields_ = [("w_type", C.c_int32), ("_pad", C.c_int32), ("w", C.c_void_p), ("K", C.c_int64), ("N", C.c_int64),
                ("w_ne2", C.c_int64), ("w_ne3", C.c_int64), ("w_nb1", C.c_int64), ("w_nb2", C.c_int64), ("w_nb3", C.c_int64),
                ("x", C.c_void_p), ("M", C.c_int64), ("ne2", C.c_int64), ("ne3", C.c_int64), ("x_nb1", C.c_int64),
                ("x_nb2", C.c_int64), ("x_nb3", C.c_int64), ("dst", C.c_void_p), ("d_nb1", C.c_int64), ("d_nb2", C.c_int64),
                ("d_nb3", C.c_int64)]


class MlaCopyArgs(C.Structure):
    """mla_copy_args of include/mla_front.h."""
    _fields_ = [("src", C.c_void_p), ("dst", C.c_void_p), ("ne", C.c_int64 * 4), ("src_nb", C.c_int64 * 4), ("dst_nb", C.c_int64 * 4)]


class MlaKvWriteRopeArgs(C.Structure):
    """mla_kv_write_rope_args of include/mla_kv_write.h."""
    _fields_ = [("w", MlaKvWriteArgs), ("rope", MlaRopeArgs)]


class MlaFrontOp(C.Structure):
    """mla_front_op of include/mla_front.h."""
    _fields_ = [("kind", C.c_int32), ("_pad", C.c_int32), ("args", C.c_void_p)]


MLA_FRONT_ROPE, MLA_FRONT_MUL_MAT, MLA_FRONT_COPY, MLA_FRONT_KV_WRITE, MLA_FRONT_KV_WRITE_ROPE = range(5)


class FrontBatch:
    """Independent launches of ggml_rope_ext / ggml_mul_mat / copy_f32 / kv_write collected (pass batch=...) and issued as one
    dispatch by launch() (mla_front_batch_launch).  None of them may read or write what another one writes."""

    def __init__(self):
        self.ops = []

    def add(self, kind, args):
        self.ops.append((kind, args))

    def launch(self, stream=None, device=None):
        import torch
        n = len(self.ops)
        arr = (MlaFrontOp * max(n, 1))()
        for i, (kind, args) in enumerate(self.ops):
            arr[i].kind, arr[i].args = kind, C.addressof(args)
        st = stream if stream is not None else torch.cuda.current_stream(device).cuda_stream
        rc = library().mla_front_batch_launch(arr, n, C.c_void_p(st))
        if rc != 0:
            raise RuntimeError("mla_front_batch_launch failed with code %d" % rc)
        self.ops = []


def _gpu_only(t):
    if not t.is_cuda:
        raise RuntimeError("jittorinfer_amd runs on a gfx950 GPU only (there is no CPU path)")


def _stream(t, stream):
    import torch
    return stream if stream is not None else torch.cuda.current_stream(t.device).cuda_stream


def _nb4(t):
    """ggml-order byte strides / sizes of a torch tensor of up to 4 dims (last torch dim = ggml dim 0)."""
    es = t.element_size()
    ne = list(reversed(t.shape)) + [1] * (4 - t.dim())
    nb = [s * es for s in reversed(t.stride())]
    while len(nb) < 4:
        nb.append(nb[-1] * ne[len(nb) - 1])
    return ne, nb


def _fill_rope_args(a, x, pos, out, *, n_dims, mode=0, n_ctx_orig=0, freq_base=10000.0, freq_scale=1.0, ext_factor=0.0, attn_factor=1.0,
                    beta_fast=32.0, beta_slow=1.0, freq_factors=None):
    import torch
    assert pos.dtype == torch.int32 and pos.is_contiguous() and pos.numel() == x.shape[0]
    ne, nb = _nb4(x)
    _, dnb = _nb4(out)
    a.src, a.dst, a.pos = x.data_ptr(), out.data_ptr(), pos.data_ptr()
    a.ne[:], a.src_nb[:], a.dst_nb[:] = ne, nb, dnb
    if freq_factors is not None:
        assert freq_factors.dtype == torch.float32 and freq_factors.is_contiguous() and freq_factors.numel() >= n_dims // 2
        a.freq_factors = freq_factors.data_ptr()
    a.n_dims, a.mode, a.n_ctx_orig = n_dims, mode, n_ctx_orig
    a.freq_base, a.freq_scale, a.ext_factor, a.attn_factor = freq_base, freq_scale, ext_factor, attn_factor
    a.beta_fast, a.beta_slow = beta_fast, beta_slow


def ggml_rope_ext(x, pos, *, n_dims, mode=0, n_ctx_orig=0, freq_base=10000.0, freq_scale=1.0, ext_factor=0.0, attn_factor=1.0,
                  beta_fast=32.0, beta_slow=1.0, freq_factors=None, out=None, stream=None, batch=None):
    """ggml_rope_ext (ggml/src/ggml.c:3495-3501) on the current torch stream.  x: float32 [n_tok, n_head, ne0] (ggml ne =
    {ne0, n_head, n_tok}), unit stride in the last dimension; pos: int32 [n_tok]; out: same shape (default: a new
    contiguous tensor; pass out=x to rotate in place)."""
    import torch
    _gpu_only(x)
    assert x.dtype == torch.float32 and x.dim() == 3 and x.stride(2) == 1
    assert pos.dtype == torch.int32 and pos.is_contiguous() and pos.numel() == x.shape[0]
    if out is None:
        out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    assert out.shape == x.shape and out.dtype == torch.float32 and out.stride(2) == 1
    a = MlaRopeArgs()
    _fill_rope_args(a, x, pos, out, n_dims=n_dims, mode=mode, n_ctx_orig=n_ctx_orig, freq_base=freq_base, freq_scale=freq_scale,
                    ext_factor=ext_factor, attn_factor=attn_factor, beta_fast=beta_fast, beta_slow=beta_slow, freq_factors=freq_factors)
    if batch is not None:
        batch.add(MLA_FRONT_ROPE, a)
        return out
    rc = library().mla_rope_launch(C.byref(a), C.c_void_p(_stream(x, stream)))
    if rc != 0:
        raise RuntimeError("mla_rope_launch failed with code %d" % rc)
    return out


def ggml_mul_mat(w, w_type, x, *, out=None, stream=None, batch=None):
    """ggml_mul_mat(src0 = w, src1 = x) for the absorb products (src/llama-graph-attn.cpp:264-275, :303-317).
    w: [w_ne2, N, K] 16-bit storage (bf16 / f16 bits, any 2-byte dtype), x: float32 [ne2, M, K], unit stride in the
    last dimension of both, ne2 % w_ne2 == 0; returns float32 [ne2, M, N]."""
    import torch
    _gpu_only(x)
    assert w.dim() == 3 and x.dim() == 3 and w.element_size() == 2 and x.dtype == torch.float32
    assert w.stride(2) == 1 and x.stride(2) == 1 and w.shape[2] == x.shape[2]
    if out is None:
        out = torch.empty((x.shape[0], x.shape[1], w.shape[1]), dtype=torch.float32, device=x.device)
    assert out.shape == (x.shape[0], x.shape[1], w.shape[1]) and out.dtype == torch.float32 and out.stride(2) == 1
    a = MlaMulMatArgs()
    a.w_type, a.w, a.x, a.dst = w_type, w.data_ptr(), x.data_ptr(), out.data_ptr()
    a.K, a.N, a.w_ne2, a.w_ne3 = w.shape[2], w.shape[1], w.shape[0], 1
    a.M, a.ne2, a.ne3 = x.shape[1], x.shape[0], 1
    a.w_nb1, a.w_nb2 = w.stride(1) * 2, w.stride(0) * 2
    a.x_nb1, a.x_nb2 = x.stride(1) * 4, x.stride(0) * 4
    a.d_nb1, a.d_nb2 = out.stride(1) * 4, out.stride(0) * 4
    a.w_nb3, a.x_nb3, a.d_nb3 = a.w_nb2 * a.w_ne2, a.x_nb2 * a.ne2, a.d_nb2 * a.ne2
    if batch is not None:
        batch.add(MLA_FRONT_MUL_MAT, a)
        return out
    rc = library().mla_mul_mat_launch(C.byref(a), C.c_void_p(_stream(x, stream)))
    if rc != 0:
        raise RuntimeError("mla_mul_mat_launch failed with code %d" % rc)
    return out


def copy_f32(src, dst, stream=None, batch=None):
    """Strided float32 copy (ggml_cont; each half of ggml_concat): dst[...] = src[...], same shape, any strides with a
    unit last one."""
    import torch
    _gpu_only(src)
    assert src.dtype == torch.float32 and dst.dtype == torch.float32 and src.shape == dst.shape and src.dim() <= 4
    assert src.stride(-1) == 1 and dst.stride(-1) == 1
    a = MlaCopyArgs()
    ne, nb = _nb4(src)
    _, dnb = _nb4(dst)
    a.src, a.dst = src.data_ptr(), dst.data_ptr()
    a.ne[:], a.src_nb[:], a.dst_nb[:] = ne, nb, dnb
    if batch is not None:
        batch.add(MLA_FRONT_COPY, a)
        return dst
    rc = library().mla_copy_f32_launch(C.byref(a), C.c_void_p(_stream(src, stream)))
    if rc != 0:
        raise RuntimeError("mla_copy_f32_launch failed with code %d" % rc)
    return dst


class PageTable:
    """Host-side page allocator / block-table builder (include/mla_page_table.h): the paged counterpart of the reference's
    llama_kv_cache bookkeeping (src/llama-kv-cache.cpp) and of the mask builder of llama_set_inputs.  numpy in, numpy out."""

    def __init__(self, n_pages, n_seq_max, max_blocks):
        self._lib = library()
        self.n_pages, self.n_seq_max, self.max_blocks = n_pages, n_seq_max, max_blocks
        self._h = self._lib.mla_page_table_create(n_pages, n_seq_max, max_blocks)
        if not self._h:
            raise ValueError("mla_page_table_create rejected the sizes")

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.mla_page_table_free(self._h)
            self._h = None

    def clear(self):
        self._lib.mla_page_table_clear(self._h)

    def find_slot(self, seq_id, pos):
        """Cache rows (int32 [n_tokens]) of the batch's tokens, or None when the batch does not fit (nothing is changed);
        other errors raise."""
        import numpy as np
        seq_id = np.ascontiguousarray(seq_id, dtype=np.int32)
        pos = np.ascontiguousarray(pos, dtype=np.int32)
        rows = np.empty(len(seq_id), dtype=np.int32)
        rc = self._lib.mla_page_table_find_slot(self._h, len(seq_id), seq_id.ctypes.data, pos.ctypes.data, rows.ctypes.data)
        if rc == -1:
            return None
        if rc != 0:
            raise ValueError("mla_page_table_find_slot: %d" % rc)
        return rows

    def seq_rm(self, seq_id, p0=-1, p1=-1):
        return self._lib.mla_page_table_seq_rm(self._h, seq_id, p0, p1) == 0

    def seq_cp(self, src, dst, p0=-1, p1=-1):
        """Returns (src_row, dst_row, n_rows): the row run the caller copies on the device (n_rows may be 0)."""
        a, b, n = C.c_int32(0), C.c_int32(0), C.c_int32(0)
        rc = self._lib.mla_page_table_seq_cp(self._h, src, dst, p0, p1, C.byref(a), C.byref(b), C.byref(n))
        if rc != 0:
            raise ValueError("mla_page_table_seq_cp: %d" % rc)
        return a.value, b.value, n.value

    def seq_unshare(self, seq_id):
        """Gives the sequence a private copy of a partly used last page that other sequences map too (after seq_cp + a roll-back
        into the shared prefix); returns (src_row, dst_row, n_rows) to copy on the device (n_rows may be 0), None when no page is free."""
        a, b, n = C.c_int32(0), C.c_int32(0), C.c_int32(0)
        rc = self._lib.mla_page_table_seq_unshare(self._h, seq_id, C.byref(a), C.byref(b), C.byref(n))
        if rc == -1:
            return None
        if rc != 0:
            raise ValueError("mla_page_table_seq_unshare: %d" % rc)
        return a.value, b.value, n.value

    def seq_keep(self, seq_id):
        return self._lib.mla_page_table_seq_keep(self._h, seq_id) == 0

    def seq_add(self, seq_id, p0, p1, delta):
        """True when nothing had to move (no cell in the range, or delta 0); False: refused, cached positions cannot be shifted."""
        return self._lib.mla_page_table_seq_add(self._h, seq_id, p0, p1, delta) == 0

    def defrag(self):
        """Number of row runs to copy on the device: always 0, freed pages need no compaction."""
        n = C.c_int32(-1)
        rc = self._lib.mla_page_table_defrag(self._h, C.byref(n))
        if rc != 0:
            raise ValueError("mla_page_table_defrag: %d" % rc)
        return n.value

    def seq_len(self, seq_id):
        return self._lib.mla_page_table_seq_len(self._h, seq_id)

    @property
    def free_pages(self):
        return self._lib.mla_page_table_free_pages(self._h)

    @property
    def used_cells(self):
        return self._lib.mla_page_table_used_cells(self._h)

    def fill_inputs(self, seq_ids):
        """(block_table int32 [n_seqs, max_blocks], seq_lens int32 [n_seqs]): src[4] / src[5] of the attention node."""
        import numpy as np
        seq_ids = np.ascontiguousarray(seq_ids, dtype=np.int32)
        bt = np.empty((len(seq_ids), self.max_blocks), dtype=np.int32)
        sl = np.empty(len(seq_ids), dtype=np.int32)
        rc = self._lib.mla_page_table_fill_inputs(self._h, len(seq_ids), seq_ids.ctypes.data, bt.ctypes.data, sl.ctypes.data)
        if rc != 0:
            raise ValueError("mla_page_table_fill_inputs: %d" % rc)
        return bt, sl
