// ggml backend plugin "HIP-MLA": a drop-in for the reference's backend plugin interface that executes
// GGML_OP_FLASH_ATTN_EXT nodes of the absorbed-MLA shape on an MI355X through the kernels of mla_kernels.hip.
//
// It answers the four vtables of ggml/src/ggml-backend-impl.h (buffer type :17-35, buffer :41-69, backend
// :89-130, device :143-192, reg :198-214) and exports ggml_backend_init / ggml_backend_score, the symbols
// load_backend looks up with dlsym (ggml/src/ggml-backend-reg.cpp:234-250).  The in-tree template for the wiring
// is the CANN backend (ggml/src/ggml-cann/ggml-cann.cpp:2228-2432, :2487-2550); nothing of it is reused.
//
// The host's ggml is not linked: struct layouts come from ggml_abi.h.  ggml_backend_buffer_init is taken from the
// host process with dlsym when it is there (so the host's ggml_backend_buffer_free pairs with its own allocation).
//
// Node contract (see include/ggml_mla_backend.h): src[0]=q F32 [576,n_tok,H,B]; src[1]=k F16|BF16|Q8_0
// [576,n_kv,1,B|1]; src[2]=v: k itself or a 512/576-wide view of k at offset 0; src[3]=mask F16 or NULL;
// optional src[4]=I32 block table [max_blocks,B] and src[5]=I32 [B] sequence lengths; dst F32 [576,H,n_tok,B].

#include <hip/hip_runtime.h>
#include <dlfcn.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/ggml_mla_backend.h"
#include "../../include/mla_front.h"
#include "../../include/mla_kv_write.h"
#include "../../include/mla_attn.h"
#include "ggml_abi.h"

using namespace ggml_abi;

namespace {

void log_error(const char * fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    fprintf(stderr, "ggml-hip-mla: ");
    vfprintf(stderr, fmt, ap);
    fprintf(stderr, "\n");
    va_end(ap);
}

#define HIP_OK(expr) ((expr) == hipSuccess)

// ---------------------------------------------------------------- per-device state

struct device_ctx {
    int         index;
    std::string name;         // "HIPMLA0"
    std::string description;  // hipDeviceProp_t::name
    backend_buffer_type buft;
    backend_buffer_type host_buft;   // pinned host memory (the reference's "CANN_Host", ggml/src/ggml-cann/ggml-cann.cpp:1252-1365)
    std::string         host_name;   // "HIPMLA0_Host"
};

struct buffer_ctx {
    int    device;
    void * base;
};

struct backend_ctx {
    int         device;
    std::string name;
    hipStream_t stream;
    void *      workspace      = nullptr;
    size_t      workspace_size = 0;
    bool        f16_strict     = false;   // F16 KV: replay ggml-cpu's f16 accumulator instead of accumulating in f32
    bool        q8_exact       = false;   // Q8_0 KV: the reference's integer block dots and f32 V instead of f16 matrix-core operands (MLA_FLAG_Q8_EXACT)
    bool        bf16_direct    = false;   // BF16 KV: the hi + lo bf16 program instead of the one that converts the tiles to f16 (MLA_FLAG_BF16_DIRECT)
    // The attention nodes of the layers of one graph share their mask (one KQ_mask tensor per graph, src/llama-graph-deepseek2.cpp:99-103):
    // the key extents the first of them leaves in the workspace serve the others (MLA_FLAG_MASK_EXTENTS_VALID).  ext_key: the
    // arguments of the launch whose extents the workspace holds, q / kv / dst blanked; valid inside one graph_compute call, while no
    // node writes the mask and nothing else uses the workspace.
    bool          reuse_mask_extents = true;
    bool          log_schedule       = false;   // GGML_HIP_MLA_DEBUG=schedule: the levels front_flush issues, on stderr
    bool          batch_front        = true;    // the nodes around the attention node as dispatches of several nodes each (front_collect / front_flush)
    bool          ext_key_valid      = false;
    mla_attn_args ext_key;
};

std::vector<device_ctx *>     g_device_ctx;
std::vector<backend_device *> g_devices;
backend_reg                   g_reg;
std::once_flag                g_once;
std::atomic<int64_t>          g_mask_extent_reuses{ 0 };
uint8_t                       g_guid[16] = { 0x6d, 0x6c, 0x61, 0x2d, 0x68, 0x69, 0x70, 0x2d, 0x67, 0x66, 0x78, 0x39, 0x35, 0x30, 0x00, 0x01 };

int64_t nelements(const tensor * t) { return t->ne[0] * t->ne[1] * t->ne[2] * t->ne[3]; }
bool    is_empty(const tensor * t) { return nelements(t) == 0; }

// bytes spanned by a tensor with ggml strides (ggml_nbytes, ggml/src/ggml.c) for the types this backend sees
size_t type_size(int type) {
    switch (type) {
        case TYPE_F32: case TYPE_I32: return 4;
        case TYPE_F16: case TYPE_BF16: case TYPE_I16: return 2;
        case TYPE_I8: return 1;
        case TYPE_I64: case TYPE_F64: return 8;
        case TYPE_Q8_0: return sizeof(block_q8_0);
        default: return 0;
    }
}
int64_t blck_size(int type) { return type == TYPE_Q8_0 ? 32 : 1; }
size_t  tensor_nbytes(const tensor * t) {
    if (is_empty(t)) return 0;
    const int64_t blck = blck_size(t->type);
    size_t nbytes;
    if (blck == 1) {
        nbytes = type_size(t->type);
        for (int i = 0; i < MAX_DIMS; i++) nbytes += (t->ne[i] - 1) * t->nb[i];
    } else {
        nbytes = t->ne[0] * t->nb[0] / blck;
        for (int i = 1; i < MAX_DIMS; i++) nbytes += (t->ne[i] - 1) * t->nb[i];
    }
    return nbytes;
}
bool is_contiguous(const tensor * t) {
    size_t next = type_size(t->type);
    if (t->ne[0] != blck_size(t->type) && t->nb[0] != next) return false;
    next *= t->ne[0] / blck_size(t->type);
    for (int i = 1; i < MAX_DIMS; i++) {
        if (t->ne[i] != 1 && t->nb[i] != next) return false;
        next *= t->ne[i];
    }
    return true;
}

// ---------------------------------------------------------------- buffer

void buffer_free(backend_buffer * buffer) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    (void) hipSetDevice(ctx->device);
    (void) hipFree(ctx->base);
    delete ctx;
}
void * buffer_get_base(backend_buffer * buffer) { return ((buffer_ctx *) buffer->context)->base; }

void buffer_memset_tensor(backend_buffer * buffer, tensor * t, uint8_t value, size_t offset, size_t size) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    (void) hipSetDevice(ctx->device);
    if (!HIP_OK(hipMemset((char *) t->data + offset, value, size)) || !HIP_OK(hipDeviceSynchronize())) log_error("memset_tensor failed");
}
void buffer_set_tensor(backend_buffer * buffer, tensor * t, const void * data, size_t offset, size_t size) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    (void) hipSetDevice(ctx->device);
    if (!HIP_OK(hipMemcpy((char *) t->data + offset, data, size, hipMemcpyHostToDevice))) log_error("set_tensor failed");
}
void buffer_get_tensor(backend_buffer * buffer, const tensor * t, void * data, size_t offset, size_t size) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    (void) hipSetDevice(ctx->device);
    if (!HIP_OK(hipMemcpy(data, (const char *) t->data + offset, size, hipMemcpyDeviceToHost))) log_error("get_tensor failed");
}
const char * buft_get_name(backend_buffer_type * buft);
bool buffer_cpy_tensor(backend_buffer * buffer, const tensor * src, tensor * dst) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    if (!src->buffer || !src->buffer->buft) return false;
    const size_t n = tensor_nbytes(src);
    (void) hipSetDevice(ctx->device);
    backend_buffer_type * sb = src->buffer->buft;
    if (sb->iface.is_host && sb->iface.is_host(sb)) {
        return HIP_OK(hipMemcpy(dst->data, src->data, n, hipMemcpyHostToDevice));
    }
    if (sb->iface.get_name == buft_get_name) {  // one of ours (any device)
        return HIP_OK(hipMemcpy(dst->data, src->data, n, hipMemcpyDeviceToDevice));
    }
    return false;
}
void buffer_clear(backend_buffer * buffer, uint8_t value) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    (void) hipSetDevice(ctx->device);
    if (!HIP_OK(hipMemset(ctx->base, value, buffer->size)) || !HIP_OK(hipDeviceSynchronize())) log_error("clear failed");
}

const backend_buffer_i k_buffer_iface = {
    /* free_buffer   */ buffer_free,
    /* get_base      */ buffer_get_base,
    /* init_tensor   */ nullptr,
    /* memset_tensor */ buffer_memset_tensor,
    /* set_tensor    */ buffer_set_tensor,
    /* get_tensor    */ buffer_get_tensor,
    /* cpy_tensor    */ buffer_cpy_tensor,
    /* clear         */ buffer_clear,
    /* reset         */ nullptr,
};

typedef backend_buffer * (*buffer_init_fn)(backend_buffer_type *, backend_buffer_i, void *, size_t);

backend_buffer * make_buffer(backend_buffer_type * buft, const backend_buffer_i & iface, void * context, size_t size) {
    static buffer_init_fn host_init = (buffer_init_fn) dlsym(RTLD_DEFAULT, "ggml_backend_buffer_init");
    if (host_init) return host_init(buft, iface, context, size);
    // stand-alone use (no ggml in the process): same object the host would have built (ggml-backend.cpp buffer_init)
    return new backend_buffer{ iface, buft, context, size, BUFFER_USAGE_ANY };
}

// ---------------------------------------------------------------- buffer type

const char * buft_get_name(backend_buffer_type * buft) { return ((device_ctx *) buft->context)->name.c_str(); }

backend_buffer * buft_alloc_buffer(backend_buffer_type * buft, size_t size) {
    device_ctx * dc = (device_ctx *) buft->context;
    if (!HIP_OK(hipSetDevice(dc->index))) return nullptr;
    void * p = nullptr;
    if (size == 0) size = 1;
    const hipError_t e = hipMalloc(&p, size);
    if (e != hipSuccess) {
        log_error("allocating %.2f MiB on device %d failed: %s", size / 1048576.0, dc->index, hipGetErrorString(e));
        return nullptr;
    }
    return make_buffer(buft, k_buffer_iface, new buffer_ctx{ dc->index, p }, size);
}
size_t buft_get_alignment(backend_buffer_type *) { return 256; }
bool   buft_is_host(backend_buffer_type *) { return false; }

// ---------------------------------------------------------------- pinned host buffer type
// What the reference asks a GPU device for to hold the CPU backend's compute buffer and the logits, "for faster transfer
// of the intermediate state" (src/llama-context-load-utils.cpp:116-123, src/llama-context.cpp:181): host memory that
// the CPU backend computes in (is_host) and that copies to and from the device need no staging for.  Counterpart of
// ggml_backend_cann_host_buffer_type (ggml/src/ggml-cann/ggml-cann.cpp:1323-1365); the buffer functions are the plain
// memory operations of the CPU buffer (ggml/src/ggml-backend.cpp:2022-2085), which this library cannot borrow without
// linking ggml.

struct host_buffer_ctx {
    void * base;
    bool   pinned;   // false: the pinned allocation failed and the buffer is ordinary aligned memory
};

void host_buffer_free(backend_buffer * buffer) {
    host_buffer_ctx * ctx = (host_buffer_ctx *) buffer->context;
    if (ctx->pinned) (void) hipHostFree(ctx->base); else free(ctx->base);
    delete ctx;
}
void * host_buffer_get_base(backend_buffer * buffer) { return ((host_buffer_ctx *) buffer->context)->base; }
void host_buffer_memset_tensor(backend_buffer *, tensor * t, uint8_t value, size_t offset, size_t size) { memset((char *) t->data + offset, value, size); }
void host_buffer_set_tensor(backend_buffer *, tensor * t, const void * data, size_t offset, size_t size) { memcpy((char *) t->data + offset, data, size); }
void host_buffer_get_tensor(backend_buffer *, const tensor * t, void * data, size_t offset, size_t size) { memcpy(data, (const char *) t->data + offset, size); }
bool host_buffer_cpy_tensor(backend_buffer *, const tensor * src, tensor * dst) {
    if (!src->buffer || !src->buffer->buft) return false;
    backend_buffer_type * sb = src->buffer->buft;
    if (!(sb->iface.is_host && sb->iface.is_host(sb))) return false;
    memcpy(dst->data, src->data, tensor_nbytes(src));
    return true;
}
void host_buffer_clear(backend_buffer * buffer, uint8_t value) { memset(((host_buffer_ctx *) buffer->context)->base, value, buffer->size); }

const backend_buffer_i k_host_buffer_iface = {
    /* free_buffer   */ host_buffer_free,
    /* get_base      */ host_buffer_get_base,
    /* init_tensor   */ nullptr,
    /* memset_tensor */ host_buffer_memset_tensor,
    /* set_tensor    */ host_buffer_set_tensor,
    /* get_tensor    */ host_buffer_get_tensor,
    /* cpy_tensor    */ host_buffer_cpy_tensor,
    /* clear         */ host_buffer_clear,
    /* reset         */ nullptr,
};

const char * host_buft_get_name(backend_buffer_type * buft) { return ((device_ctx *) buft->context)->host_name.c_str(); }
backend_buffer * host_buft_alloc_buffer(backend_buffer_type * buft, size_t size) {
    device_ctx * dc = (device_ctx *) buft->context;
    if (size == 0) size = 1;
    void * p = nullptr;
    bool pinned = HIP_OK(hipSetDevice(dc->index)) && hipHostMalloc(&p, size, hipHostMallocDefault) == hipSuccess && p;
    if (!pinned) {
        // like the reference's host buffer (ggml-cann.cpp:1327-1331): fall back to ordinary memory rather than fail
        (void) hipGetLastError();
        log_error("pinning %.2f MiB of host memory failed: using pageable memory", size / 1048576.0);
        if (posix_memalign(&p, 64, size) != 0) return nullptr;
    }
    return make_buffer(buft, k_host_buffer_iface, new host_buffer_ctx{ p, pinned }, size);
}
size_t host_buft_get_alignment(backend_buffer_type *) { return 64; }
bool   host_buft_is_host(backend_buffer_type *) { return true; }

// ---------------------------------------------------------------- op support

bool is_noop(int op) { return op == OP_NONE || op == OP_RESHAPE || op == OP_VIEW || op == OP_PERMUTE || op == OP_TRANSPOSE; }

const tensor * view_root(const tensor * t, size_t * offs) {
    *offs = 0;
    while (t->view_src) { *offs += t->view_offs; t = t->view_src; }
    return t;
}

// The address the launchers' alignment checks see: the tensor's own once it is allocated, before that a stand-in with the
// same low bits (every ggml buffer aligns its tensors to at least 32 bytes, TENSOR_ALIGNMENT in ggml-impl.h, so the offset
// of a view inside its root decides).
const void * addr_of(const tensor * t) {
    if (!t) return nullptr;
    if (t->data) return t->data;
    size_t offs;
    (void) view_root(t, &offs);
    return (const void *) ((uintptr_t) 1 << 20 | offs);
}

// Every *_ok function below does two things: the clauses only the graph can show (which tensor is a view of which, how
// dst relates to the sources), and then the argument block graph_compute would pass, handed to the launcher's own check
// -- so a node the device reports as supported is one the launch accepts (ggml_backend_sched sends a refused node to
// the CPU backend instead, ggml-backend.cpp:820-846).

void fill_attn_args(const tensor * dst, mla_attn_args * a) {
    const tensor * q = dst->src[0], * k = dst->src[1], * v = dst->src[2], * mask = dst->src[3];
    const tensor * bt = dst->src[4], * lens = dst->src[5];
    memset(a, 0, sizeof(*a));
    a->n_seq = (int32_t) q->ne[3]; a->n_head = (int32_t) q->ne[2]; a->n_tok = (int32_t) q->ne[1];
    a->dk = 576; a->dv = (int32_t) v->ne[0];
    a->q_type = MLA_TYPE_F32; a->kv_type = k->type;
    memcpy(&a->scale, (const char *) dst->op_params + 0, 4);
    memcpy(&a->max_bias, (const char *) dst->op_params + 4, 4);
    memcpy(&a->logit_softcap, (const char *) dst->op_params + 8, 4);
    a->q = addr_of(q); a->q_nb1 = (int64_t) q->nb[1]; a->q_nb2 = (int64_t) q->nb[2]; a->q_nb3 = (int64_t) q->nb[3];
    a->kv = addr_of(k); a->kv_nb1 = (int64_t) k->nb[1]; a->kv_nb3 = k->ne[3] == 1 ? 0 : (int64_t) k->nb[3]; a->n_kv = k->ne[1];
    if (mask) { a->mask = addr_of(mask); a->mask_nb1 = (int64_t) mask->nb[1]; a->mask_ne0 = mask->ne[0]; }
    if (bt) { a->block_table = (const int32_t *) addr_of(bt); a->bt_stride = bt->ne[0]; a->seq_lens = (const int32_t *) addr_of(lens); }
    a->dst = (float *) addr_of(dst); a->dst_nb1 = (int64_t) dst->nb[1];
}

// Fills `why` (if given) with the first violated clause of the node contract.
bool mla_node_ok(const tensor * dst, const char ** why) {
    const char * dummy;
    if (!why) why = &dummy;
    const tensor * q = dst->src[0], * k = dst->src[1], * v = dst->src[2], * mask = dst->src[3];
    const tensor * bt = dst->src[4], * lens = dst->src[5];
    if (!q || !k || !v) { *why = "missing q/k/v"; return false; }
    if (q->type != TYPE_F32 || q->nb[0] != 4) { *why = "q must be F32 with contiguous rows"; return false; }
    if (q->ne[0] != 576 || k->ne[0] != 576) { *why = "head size must be 576 (512 latent + 64 rope)"; return false; }
    if (q->ne[1] < 1 || q->ne[2] < 1 || q->ne[3] < 1 || q->ne[1] > 0x7fffffff || q->ne[2] > 0x7fffffff || q->ne[3] > 0x7fffffff) { *why = "q must have 1 .. 2^31-1 tokens, heads and sequences"; return false; }
    if (k->type != TYPE_F16 && k->type != TYPE_BF16 && k->type != TYPE_Q8_0) { *why = "k must be F16, BF16 or Q8_0"; return false; }
    if (k->ne[2] != 1) { *why = "MLA has a single latent KV head"; return false; }
    if (k->nb[0] != type_size(k->type)) { *why = "k rows must be contiguous"; return false; }
    if (v->type != k->type) { *why = "v must have k's type"; return false; }
    if (v->ne[0] != 512 && v->ne[0] != 576) { *why = "v must be 512 or 576 wide"; return false; }
    if (v->ne[1] != k->ne[1] || v->ne[2] != 1 || v->ne[3] != k->ne[3]) { *why = "v must cover the same rows as k"; return false; }
    if (v != k) {  // must alias k: the same latent row supplies both
        size_t ko, vo;
        const tensor * kr = view_root(k, &ko), * vr = view_root(v, &vo);
        if (kr != vr || ko != vo || v->nb[1] != k->nb[1] || v->nb[3] != k->nb[3]) { *why = "v must be a view of k's rows at offset 0"; return false; }
    }
    if (dst->type != TYPE_F32 || dst->nb[0] != 4 || dst->ne[0] < v->ne[0]) { *why = "dst must be F32 rows of >= dv floats"; return false; }
    if (dst->ne[1] != q->ne[2] || dst->ne[2] != q->ne[1] || dst->ne[3] != q->ne[3]) { *why = "dst must be [*, H, n_tok, B]"; return false; }
    if (dst->nb[2] != dst->nb[1] * (size_t) dst->ne[1] || dst->nb[3] != dst->nb[2] * (size_t) dst->ne[2]) { *why = "dst rows must be evenly strided"; return false; }
    if (mask) {
        if (mask->type != TYPE_F16 || !is_contiguous(mask) || mask->ne[2] != 1 || mask->ne[3] != 1) { *why = "mask must be contiguous F16 2-D"; return false; }
        if (mask->ne[1] < q->ne[1]) { *why = "mask has fewer rows than query tokens"; return false; }
    }
    if ((bt != nullptr) != (lens != nullptr)) { *why = "block table and sequence lengths come together"; return false; }
    if (bt) {
        if (bt->type != TYPE_I32 || lens->type != TYPE_I32 || !is_contiguous(bt) || !is_contiguous(lens)) { *why = "block table / lengths must be contiguous I32"; return false; }
        if (bt->ne[1] != q->ne[3] || nelements(lens) != q->ne[3]) { *why = "block table / lengths must have one row per sequence"; return false; }
        if (k->ne[3] != 1) { *why = "with a block table k is the page pool [576, rows, 1, 1]"; return false; }
        // every position a sequence can reach has a mask column
        if (mask && mask->ne[0] < bt->ne[0] * MLA_PAGE_TOKENS) { *why = "mask narrower than the block table's reach"; return false; }
    } else {
        if (k->ne[3] != q->ne[3] && k->ne[3] != 1) { *why = "k batch must equal q batch or be 1"; return false; }
        if (mask && mask->ne[0] < k->ne[1]) { *why = "mask narrower than n_kv"; return false; }
    }
    mla_attn_args a;
    fill_attn_args(dst, &a);
    mla_attn_plan_info info;
    switch (mla_attn_plan(&a, &info)) {
        case 0: return true;
        case MLA_ERR_BAD_ALIGNMENT: *why = "q, dst rows must be 16-byte aligned, k rows 16-byte (Q8_0: 2-byte) aligned and hold 576 values"; return false;
        case MLA_ERR_UNSUPPORTED: *why = "max_bias needs a mask"; return false;
        default: *why = "shape outside the launch limits (rows <= 2^31-1, page pool of whole 128-token pages, <= 2^23 pages per sequence)"; return false;
    }
}

// The KV cache write of llm_attn_mla (src/llama-graph-attn.cpp:236-241): CPY of f32 rows [576, n_tok] into a contiguous
// view of a BF16 / F16 / Q8_0 cache with the same number of elements; and SCATTER_UPDATE (ggml.c:3203-3223): rows of
// `updates` (cache type or F32) into rows indices[i] of a [576, n_rows] cache.
void fill_kv_cpy_args(const tensor * op, mla_kv_write_args * a) {
    const tensor * src = op->src[0];
    memset(a, 0, sizeof(*a));
    a->n_tok = (int32_t) src->ne[1]; a->src_type = MLA_TYPE_F32; a->kv_type = op->type;
    a->src = addr_of(src); a->src_nb1 = (int64_t) src->nb[1];
    a->kv = const_cast<void *>(addr_of(op)); a->kv_nb1 = op->type == TYPE_Q8_0 ? 612 : 1152; a->n_kv_rows = src->ne[1]; a->row0 = 0;
}

void fill_kv_scatter_args(const tensor * op, mla_kv_write_args * a) {
    const tensor * var = op->src[0], * idx = op->src[1], * upd = op->src[2];
    memset(a, 0, sizeof(*a));
    a->n_tok = (int32_t) upd->ne[1]; a->src_type = upd->type == TYPE_F32 ? MLA_TYPE_F32 : var->type; a->kv_type = var->type;
    a->src = addr_of(upd); a->src_nb1 = (int64_t) upd->nb[1];
    a->kv = const_cast<void *>(addr_of(var)); a->kv_nb1 = (int64_t) var->nb[1]; a->n_kv_rows = var->ne[1];
    a->rows = addr_of(idx); a->rows_type = idx->type == TYPE_I64 ? 1 : 0;
}

const char * kv_write_why(int rc) {
    return rc == MLA_ERR_BAD_ALIGNMENT ? "rows must be 16-byte aligned (Q8_0 cache: 2-byte, Q8_0 row copies: 4-byte)"
         : rc == MLA_ERR_BAD_SHAPE     ? "rows shorter than 576 values"
                                       : "refused by the launch check";
}

bool kv_cpy_ok(const tensor * op, const char ** why) {
    const char * dummy; if (!why) why = &dummy;
    const tensor * src = op->src[0];
    if (!src || src->type != TYPE_F32 || src->ne[0] != 576 || src->ne[2] != 1 || src->ne[3] != 1) { *why = "source must be F32 [576, n_tok]"; return false; }
    if (src->nb[0] != 4 || src->ne[1] > 0x7fffffff) { *why = "source rows must be dense, at most 2^31-1 of them"; return false; }
    if (op->type != TYPE_BF16 && op->type != TYPE_F16 && op->type != TYPE_Q8_0) { *why = "destination must be BF16, F16 or Q8_0"; return false; }
    if (!is_contiguous(op) || nelements(op) != nelements(src)) { *why = "destination must be a contiguous view with as many elements"; return false; }
    mla_kv_write_args a;
    fill_kv_cpy_args(op, &a);
    const int rc = mla_kv_write_check(&a);
    if (rc) { *why = kv_write_why(rc); return false; }
    return true;
}

bool kv_scatter_ok(const tensor * op, const char ** why) {
    const char * dummy; if (!why) why = &dummy;
    const tensor * var = op->src[0], * idx = op->src[1], * upd = op->src[2];
    if (!var || !idx || !upd) { *why = "missing operand"; return false; }
    if (var->ne[0] != 576 || upd->ne[0] != 576 || var->ne[2] != 1 || var->ne[3] != 1 || upd->ne[2] != 1 || upd->ne[3] != 1) { *why = "cache and updates must be [576, rows]"; return false; }
    if (var->type != TYPE_BF16 && var->type != TYPE_F16 && var->type != TYPE_Q8_0) { *why = "cache must be BF16, F16 or Q8_0"; return false; }
    if (upd->type != var->type && upd->type != TYPE_F32) { *why = "updates must have the cache type or be F32"; return false; }
    if ((idx->type != TYPE_I32 && idx->type != TYPE_I64) || !is_contiguous(idx) || idx->ne[0] != upd->ne[1]) { *why = "indices must be contiguous I32/I64, one per update row"; return false; }
    if (var->nb[0] != type_size(var->type) || upd->nb[0] != type_size(upd->type)) { *why = "cache and update rows must be dense"; return false; }
    if (var->ne[1] > 0x7fffffff || upd->ne[1] > 0x7fffffff) { *why = "too many rows"; return false; }
    {   // the node's result is the cache itself, updated in place (ggml.c:3203-3223 makes it a view of src[0])
        size_t oo, vo;
        if (view_root(op, &oo) != view_root(var, &vo) || oo != vo) { *why = "the node must be a view of the cache"; return false; }
    }
    mla_kv_write_args a;
    fill_kv_scatter_args(op, &a);
    const int rc = mla_kv_write_check(&a);
    if (rc) { *why = kv_write_why(rc); return false; }
    return true;
}

// The nodes llm_attn_mla and the DeepSeek-V2 graph put either side of the attention node
// (src/llama-graph-deepseek2.cpp:216-233, src/llama-graph-attn.cpp:264-277, :303-323): CONT and CONCAT of f32 tensors with
// dense rows, ROPE (normal / NeoX pairing, f32), and the two per-head products with the halves of kv_b: the absorb
// product q_nope . wk_b ([n_tok x 128] . [128 x 512] per head) and the un-absorb product wv_b . kqv ([n_tok x 512] . [512 x 128]).
bool f32_rows(const tensor * t) { return t && t->type == TYPE_F32 && t->nb[0] == 4 && !(t->nb[1] & 3) && !(t->nb[2] & 3) && !(t->nb[3] & 3); }

void fill_copy_args(const void * src, const size_t * src_nb, const int64_t * ne, const void * dst, const size_t * dst_nb, mla_copy_args * a) {
    a->src = src; a->dst = const_cast<void *>(dst);
    for (int i = 0; i < 4; i++) { a->ne[i] = ne[i]; a->src_nb[i] = (int64_t) src_nb[i]; a->dst_nb[i] = (int64_t) dst_nb[i]; }
}

// CONT: the destination is walked in the source's shape -- same element order (ggml_cont_2d)
void fill_cont_args(const tensor * op, mla_copy_args * a) {
    const tensor * src = op->src[0];
    const size_t dnb[4] = { 4, (size_t) src->ne[0] * 4, (size_t) (src->ne[0] * src->ne[1]) * 4, (size_t) (src->ne[0] * src->ne[1] * src->ne[2]) * 4 };
    fill_copy_args(addr_of(src), src->nb, src->ne, addr_of(op), dnb, a);
}

bool cont_ok(const tensor * op, const char ** why) {
    const char * dummy; if (!why) why = &dummy;
    const tensor * src = op->src[0];
    if (!f32_rows(src)) { *why = "source must be F32 with dense rows"; return false; }
    if (op->type != TYPE_F32 || !is_contiguous(op) || nelements(op) != nelements(src)) { *why = "destination must be contiguous F32 with as many elements"; return false; }
    mla_copy_args a;
    fill_cont_args(op, &a);
    if (mla_copy_f32_check(&a)) { *why = "refused by the launch check"; return false; }
    return true;
}

bool concat_ok(const tensor * op, const char ** why) {
    const char * dummy; if (!why) why = &dummy;
    const tensor * a = op->src[0], * b = op->src[1];
    int32_t dim; memcpy(&dim, op->op_params, 4);
    if (!f32_rows(a) || !f32_rows(b) || !f32_rows(op)) { *why = "operands must be F32 with dense rows"; return false; }
    if (dim < 0 || dim > 3) { *why = "bad dimension"; return false; }
    for (int i = 0; i < 4; i++)
        if (i == dim ? op->ne[i] != a->ne[i] + b->ne[i] : (op->ne[i] != a->ne[i] || op->ne[i] != b->ne[i])) { *why = "shapes do not concatenate"; return false; }
    mla_copy_args c;
    fill_copy_args(addr_of(a), a->nb, a->ne, addr_of(op), op->nb, &c);
    if (mla_copy_f32_check(&c)) { *why = "refused by the launch check"; return false; }
    fill_copy_args(addr_of(b), b->nb, b->ne, (const char *) addr_of(op) + (size_t) a->ne[dim] * op->nb[dim], op->nb, &c);
    if (mla_copy_f32_check(&c)) { *why = "refused by the launch check"; return false; }
    return true;
}

void fill_rope_args(const tensor * op, mla_rope_args * a) {
    const tensor * x = op->src[0];
    memset(a, 0, sizeof(*a));
    a->src = addr_of(x); a->dst = const_cast<void *>(addr_of(op)); a->pos = (const int32_t *) addr_of(op->src[1]);
    a->freq_factors = op->src[2] ? (const float *) addr_of(op->src[2]) : nullptr;
    for (int i = 0; i < 4; i++) { a->ne[i] = x->ne[i]; a->src_nb[i] = (int64_t) x->nb[i]; a->dst_nb[i] = (int64_t) op->nb[i]; }
    int32_t prm[11]; memcpy(prm, op->op_params, sizeof(prm));   // ggml.c:3431-3441
    a->n_dims = prm[1]; a->mode = prm[2]; a->n_ctx_orig = prm[4];
    memcpy(&a->freq_base, prm + 5, 4); memcpy(&a->freq_scale, prm + 6, 4); memcpy(&a->ext_factor, prm + 7, 4);
    memcpy(&a->attn_factor, prm + 8, 4); memcpy(&a->beta_fast, prm + 9, 4); memcpy(&a->beta_slow, prm + 10, 4);
}

bool rope_ok(const tensor * op, const char ** why) {
    const char * dummy; if (!why) why = &dummy;
    const tensor * x = op->src[0], * pos = op->src[1], * ff = op->src[2];
    if (!f32_rows(x) || !f32_rows(op)) { *why = "source and destination must be F32 with dense rows"; return false; }
    for (int i = 0; i < 4; i++) if (op->ne[i] != x->ne[i]) { *why = "shape mismatch"; return false; }
    if (!pos || pos->type != TYPE_I32 || !is_contiguous(pos) || nelements(pos) != x->ne[2]) { *why = "positions must be contiguous I32, one per token"; return false; }
    mla_rope_args a;
    fill_rope_args(op, &a);
    if (ff && (ff->type != TYPE_F32 || !is_contiguous(ff) || ff->ne[0] < a.n_dims / 2)) { *why = "frequency factors must be contiguous F32 [n_dims/2]"; return false; }
    switch (mla_rope_check(&a)) {
        case 0: return true;
        case MLA_ERR_UNSUPPORTED: *why = "only the normal and the NeoX pairing"; return false;
        default: *why = "n_dims must be even, <= ne0 and <= 512; at most 65535 tokens per launch"; return false;
    }
}

void fill_mul_mat_args(const tensor * op, mla_mul_mat_args * a) {
    const tensor * w = op->src[0], * x = op->src[1];
    memset(a, 0, sizeof(*a));
    a->w_type = w->type; a->w = addr_of(w); a->x = addr_of(x); a->dst = const_cast<void *>(addr_of(op));
    a->K = w->ne[0]; a->N = w->ne[1]; a->w_ne2 = w->ne[2]; a->w_ne3 = w->ne[3];
    a->M = x->ne[1]; a->ne2 = x->ne[2]; a->ne3 = x->ne[3];
    a->w_nb1 = (int64_t) w->nb[1]; a->w_nb2 = (int64_t) w->nb[2]; a->w_nb3 = (int64_t) w->nb[3];
    a->x_nb1 = (int64_t) x->nb[1]; a->x_nb2 = (int64_t) x->nb[2]; a->x_nb3 = (int64_t) x->nb[3];
    a->d_nb1 = (int64_t) op->nb[1]; a->d_nb2 = (int64_t) op->nb[2]; a->d_nb3 = (int64_t) op->nb[3];
}

bool mul_mat_ok(const tensor * op, const char ** why) {
    const char * dummy; if (!why) why = &dummy;
    const tensor * w = op->src[0], * x = op->src[1];
    if (!w || !x) { *why = "missing operand"; return false; }
    if ((w->type != TYPE_F16 && w->type != TYPE_BF16) || w->nb[0] != 2) { *why = "src0 must be F16 or BF16 with dense rows"; return false; }
    if (x->type != TYPE_F32 || x->nb[0] != 4 || op->type != TYPE_F32 || op->nb[0] != 4) { *why = "src1 and dst must be F32 with dense rows"; return false; }
    if (w->ne[0] != x->ne[0]) { *why = "src0 and src1 rows differ in length"; return false; }
    if (op->ne[0] != w->ne[1] || op->ne[1] != x->ne[1] || op->ne[2] != x->ne[2] || op->ne[3] != x->ne[3]) { *why = "dst must be [N, M, ne12, ne13]"; return false; }
    // only the two products the kernels were built and measured for: one small matrix per head, one side of it the
    // latent width.  A model's other F16 / BF16 products (wq, wo, the FFN) stay with the backend that owns their weights.
    const int64_t K = w->ne[0], N = w->ne[1];
    if (!((K == 512 && N <= 512) || (N == 512 && K <= 512)) || w->ne[2] != x->ne[2] || w->ne[3] != 1) { *why = "only the per-head absorb ([K<=512] x 512) and un-absorb (512 x [N<=512]) products"; return false; }
    mla_mul_mat_args a;
    fill_mul_mat_args(op, &a);
    switch (mla_mul_mat_check(&a)) {
        case 0: return true;
        case MLA_ERR_BAD_ALIGNMENT: *why = "rows must be 16-byte aligned"; return false;
        case MLA_ERR_UNSUPPORTED: *why = "K must be a multiple of 16"; return false;
        default: *why = "too many batches or rows for one launch"; return false;
    }
}

bool device_supports_op(backend_device *, const tensor * op) {
    if (is_noop(op->op)) return true;
    if (op->op == OP_FLASH_ATTN_EXT) return mla_node_ok(op, nullptr);
    if (op->op == OP_CPY) return kv_cpy_ok(op, nullptr);
    if (op->op == OP_SCATTER_UPDATE) return kv_scatter_ok(op, nullptr);
    if (op->op == OP_CONT) return cont_ok(op, nullptr);
    if (op->op == OP_CONCAT) return concat_ok(op, nullptr);
    if (op->op == OP_ROPE) return rope_ok(op, nullptr);
    if (op->op == OP_MUL_MAT) return mul_mat_ok(op, nullptr);
    return false;
}

// ---------------------------------------------------------------- backend (stream)

const char * backend_get_name(backend * be) { return ((backend_ctx *) be->context)->name.c_str(); }

void backend_free(backend * be) {
    backend_ctx * ctx = (backend_ctx *) be->context;
    (void) hipSetDevice(ctx->device);
    (void) hipStreamSynchronize(ctx->stream);
    if (ctx->workspace) (void) hipFree(ctx->workspace);
    (void) hipStreamDestroy(ctx->stream);
    delete ctx;
    delete be;
}

void backend_set_tensor_async(backend * be, tensor * t, const void * data, size_t offset, size_t size) {
    backend_ctx * ctx = (backend_ctx *) be->context;
    (void) hipSetDevice(ctx->device);
    if (!HIP_OK(hipMemcpyAsync((char *) t->data + offset, data, size, hipMemcpyHostToDevice, ctx->stream))) log_error("set_tensor_async failed");
}
void backend_get_tensor_async(backend * be, const tensor * t, void * data, size_t offset, size_t size) {
    backend_ctx * ctx = (backend_ctx *) be->context;
    (void) hipSetDevice(ctx->device);
    if (!HIP_OK(hipMemcpyAsync(data, (const char *) t->data + offset, size, hipMemcpyDeviceToHost, ctx->stream))) log_error("get_tensor_async failed");
}
void backend_synchronize(backend * be) {
    backend_ctx * ctx = (backend_ctx *) be->context;
    (void) hipSetDevice(ctx->device);
    if (!HIP_OK(hipStreamSynchronize(ctx->stream))) log_error("synchronize failed");
}

int compute_flash_attn(backend_ctx * ctx, const tensor * dst) {
    const char * why = nullptr;
    if (!mla_node_ok(dst, &why)) {
        const tensor * q = dst->src[0], * k = dst->src[1];
        log_error("FLASH_ATTN_EXT node '%s' rejected: %s (q '%s' [%lld,%lld,%lld,%lld], k '%s' [%lld,%lld,%lld,%lld])", dst->name, why,
                  q ? q->name : "-", q ? (long long) q->ne[0] : 0, q ? (long long) q->ne[1] : 0, q ? (long long) q->ne[2] : 0, q ? (long long) q->ne[3] : 0,
                  k ? k->name : "-", k ? (long long) k->ne[0] : 0, k ? (long long) k->ne[1] : 0, k ? (long long) k->ne[2] : 0, k ? (long long) k->ne[3] : 0);
        return STATUS_FAILED;
    }
    const tensor * q = dst->src[0], * k = dst->src[1], * v = dst->src[2], * bt = dst->src[4];
    if (!q->data || !k->data || !dst->data || v->data != k->data) { log_error("node '%s': operands not allocated, or v does not alias k", dst->name); return STATUS_FAILED; }
    for (int i = 3; i < 6; i++) if (dst->src[i] && !dst->src[i]->data) { log_error("node '%s': operands not allocated", dst->name); return STATUS_FAILED; }

    mla_attn_args a;
    fill_attn_args(dst, &a);
    if (ctx->f16_strict && k->type == TYPE_F16) a.flags |= MLA_FLAG_F16_ACC_STRICT;
    if (ctx->q8_exact && k->type == TYPE_Q8_0) a.flags |= MLA_FLAG_Q8_EXACT;
    if (ctx->bf16_direct) a.flags |= MLA_FLAG_BF16_DIRECT;

    const size_t need = mla_attn_workspace_size(&a);
    if (need > ctx->workspace_size) {
        // grow the scratch area; work already queued on the stream may still be using the old one
        if (!HIP_OK(hipStreamSynchronize(ctx->stream))) return STATUS_FAILED;
        if (ctx->workspace) (void) hipFree(ctx->workspace);
        ctx->workspace = nullptr; ctx->workspace_size = 0; ctx->ext_key_valid = false;
        if (!HIP_OK(hipMalloc(&ctx->workspace, need))) { log_error("workspace of %zu bytes: out of memory", need); return STATUS_ALLOC_FAILED; }
        ctx->workspace_size = need;
    }
    a.workspace = ctx->workspace; a.workspace_size = ctx->workspace_size;
    // what the extents, their layout and their place in the workspace depend on: everything but the operands that change from layer
    // to layer -- and of those the alignment, which the planner looks at (a Q8_0 cache that is not 16-byte aligned runs on an f16 copy,
    // with extents per row block where the aligned form has them per token)
    mla_attn_args key;
    memcpy(&key, &a, sizeof(key));
    key.q   = (const void *) ((uintptr_t) a.q & 15);
    key.kv  = (const void *) ((uintptr_t) a.kv & 15);
    key.dst = (float *) ((uintptr_t) a.dst & 15);
    const bool same_mask = a.mask && ctx->reuse_mask_extents && ctx->ext_key_valid && memcmp(&key, &ctx->ext_key, sizeof(key)) == 0;
    if (same_mask) { a.flags |= MLA_FLAG_MASK_EXTENTS_VALID; g_mask_extent_reuses++; }
    const int rc = mla_attn_launch(&a, ctx->stream);
    ctx->ext_key_valid = false;
    if (rc != 0) { log_error("mla_attn_launch failed for node '%s': %d", dst->name, rc); return STATUS_FAILED; }
    if (a.mask) { memcpy(&ctx->ext_key, &key, sizeof(key)); ctx->ext_key_valid = true; }
    return STATUS_SUCCESS;
}

int compute_kv_write(backend_ctx * ctx, const tensor * dst) {
    const char * why = nullptr;
    mla_kv_write_args a;
    if (dst->op == OP_CPY) {
        if (!kv_cpy_ok(dst, &why)) { log_error("CPY node '%s' rejected: %s", dst->name, why); return STATUS_FAILED; }
        if (!dst->src[0]->data || !dst->data) { log_error("node '%s': operands not allocated", dst->name); return STATUS_FAILED; }
        fill_kv_cpy_args(dst, &a);
    } else {
        if (!kv_scatter_ok(dst, &why)) { log_error("SCATTER_UPDATE node '%s' rejected: %s", dst->name, why); return STATUS_FAILED; }
        for (int i = 0; i < 3; i++) if (!dst->src[i]->data) { log_error("node '%s': operands not allocated", dst->name); return STATUS_FAILED; }
        fill_kv_scatter_args(dst, &a);
    }
    const int rc = mla_kv_write_launch(&a, ctx->stream);
    if (rc != 0) { log_error("mla_kv_write_launch failed for node '%s': %d", dst->name, rc); return STATUS_FAILED; }
    return STATUS_SUCCESS;
}

int launch_copy(backend_ctx * ctx, const tensor * node, const mla_copy_args * a) {
    const int rc = mla_copy_f32_launch(a, ctx->stream);
    if (rc != 0) { log_error("mla_copy_f32_launch failed for node '%s': %d", node->name, rc); return STATUS_FAILED; }
    return STATUS_SUCCESS;
}

int compute_front(backend_ctx * ctx, const tensor * dst) {
    const char * why = nullptr;
    for (int i = 0; i < 3; i++) if (dst->src[i] && !dst->src[i]->data) { log_error("node '%s': operands not allocated", dst->name); return STATUS_FAILED; }
    if (!dst->data) { log_error("node '%s': destination not allocated", dst->name); return STATUS_FAILED; }
    if (dst->op == OP_CONT) {
        if (!cont_ok(dst, &why)) { log_error("CONT node '%s' rejected: %s", dst->name, why); return STATUS_FAILED; }
        mla_copy_args a;
        fill_cont_args(dst, &a);
        return launch_copy(ctx, dst, &a);
    }
    if (dst->op == OP_CONCAT) {
        if (!concat_ok(dst, &why)) { log_error("CONCAT node '%s' rejected: %s", dst->name, why); return STATUS_FAILED; }
        const tensor * a = dst->src[0], * b = dst->src[1];
        int32_t dim; memcpy(&dim, dst->op_params, 4);
        mla_copy_args c;
        fill_copy_args(a->data, a->nb, a->ne, dst->data, dst->nb, &c);
        const int st = launch_copy(ctx, dst, &c);
        if (st != STATUS_SUCCESS) return st;
        fill_copy_args(b->data, b->nb, b->ne, (char *) dst->data + (size_t) a->ne[dim] * dst->nb[dim], dst->nb, &c);
        return launch_copy(ctx, dst, &c);
    }
    if (dst->op == OP_ROPE) {
        if (!rope_ok(dst, &why)) { log_error("ROPE node '%s' rejected: %s", dst->name, why); return STATUS_FAILED; }
        mla_rope_args a;
        fill_rope_args(dst, &a);
        const int rc = mla_rope_launch(&a, ctx->stream);
        if (rc != 0) { log_error("mla_rope_launch failed for node '%s': %d", dst->name, rc); return STATUS_FAILED; }
        return STATUS_SUCCESS;
    }
    if (!mul_mat_ok(dst, &why)) { log_error("MUL_MAT node '%s' rejected: %s", dst->name, why); return STATUS_FAILED; }
    mla_mul_mat_args a;
    fill_mul_mat_args(dst, &a);
    const int rc = mla_mul_mat_launch(&a, ctx->stream);
    if (rc != 0) { log_error("mla_mul_mat_launch failed for node '%s': %d", dst->name, rc); return STATUS_FAILED; }
    return STATUS_SUCCESS;
}

// ---- the nodes around the attention node, scheduled as dispatches of several nodes each (mla_front_batch_launch)
//
// graph_compute collects the run of nodes between two attention nodes, works out which of them depend on which from the
// memory they read and write, and issues them level by level: all nodes of a level in one dispatch.  The reference's
// executors run a graph node by node (ggml-cpu: one pass of the thread pool per node, ggml-cpu.c:15230-15268; CANN: one
// or more aclnn calls per node, ggml-cann.cpp:1761-1800); here a node of a decode step moves a few MB and a launch of its
// own costs it 4 - 5 us.  Two rewrites shorten the dependency chains; both leave every node's own result where the graph
// says it is, so that a consumer this backend does not see (another split of ggml_backend_sched) still finds it:
//  * a ROPE whose source is a CONT of this run reads the CONT's source instead (the kernel takes strided rows; the CONT
//    still runs, in the same dispatch -- unless the ROPE rotates in place in the CONT's memory, which is where the graph
//    allocator puts it: then the CONT's result would be overwritten unread and the CONT is left out);
//  * a cache write (CPY / SCATTER_UPDATE) whose new rows are CONCAT(latent, view of ROPE(k_pe)) reads the latent rows and
//    the unrotated k_pe and rotates on the way (mla_kv_write_rope_launch: bit-identical to the chain); the ROPE and the
//    CONCAT still run.
// Neither is applied when a node between the producer and the consumer writes what the consumer would now read later.
// The dependencies are those of the memory, not of the graph's edges: the graph allocator (ggml-alloc.c) hands a tensor's
// memory to a later node once its last consumer in node order has run, so two nodes without an edge between them may
// still have to keep their order.
struct mem_range { const char * lo, * hi; };
inline bool overlaps(const mem_range & a, const mem_range & b) { return a.lo < b.hi && b.lo < a.hi; }
inline mem_range range_of(const tensor * t) { return mem_range{ (const char *) t->data, (const char *) t->data + tensor_nbytes(t) }; }

struct front_item {
    const tensor * node;
    int            n_ops;
    mla_front_op   ops[2];
    union { mla_rope_args rope; mla_mul_mat_args mm; mla_copy_args copy; mla_kv_write_args kvw; mla_kv_write_rope_args kvr; } args[2];
    int            n_reads;
    mem_range      reads[6];
    mem_range      write;
    const tensor * rope_src;   // ROPE items: the tensor the launch reads its rows from (the node's source, or that CONT's source)
    int            level;
};

constexpr int FRONT_WINDOW = 64;

std::atomic<int64_t> g_front_dispatches{ 0 }, g_front_nodes{ 0 };

int find_item(const std::vector<front_item> & w, const tensor * node) {
    for (int i = (int) w.size() - 1; i >= 0; i--) if (w[i].node == node) return i;
    return -1;
}
bool written_after(const std::vector<front_item> & w, int i, const mem_range & r) {
    for (size_t k = (size_t) i + 1; k < w.size(); k++) if (overlaps(w[k].write, r)) return true;
    return false;
}
// ... by an item strictly between items i and j
bool written_between(const std::vector<front_item> & w, int i, int j, const mem_range & r) {
    for (int k = i + 1; k < j; k++) if (overlaps(w[k].write, r)) return true;
    return false;
}

// Appends `node` to the run; validation as in compute_front / compute_kv_write.
int front_collect(std::vector<front_item> & w, const tensor * node) {
    const char * why = nullptr;
    for (int i = 0; i < 3; i++) if (node->src[i] && !node->src[i]->data) { log_error("node '%s': operands not allocated", node->name); return STATUS_FAILED; }
    if (!node->data) { log_error("node '%s': destination not allocated", node->name); return STATUS_FAILED; }
    w.emplace_back();
    front_item & it = w.back();
    const int self = (int) w.size() - 1;
    memset(&it, 0, sizeof(it));
    it.node = node; it.n_ops = 1; it.write = range_of(node);
    auto reads = [&](const tensor * t) { if (t && it.n_reads < 6) it.reads[it.n_reads++] = range_of(t); };
    switch (node->op) {
        case OP_CONT: {
            if (!cont_ok(node, &why)) { log_error("CONT node '%s' rejected: %s", node->name, why); return STATUS_FAILED; }
            fill_cont_args(node, &it.args[0].copy);
            it.ops[0] = mla_front_op{ MLA_FRONT_COPY, 0, &it.args[0].copy };
            reads(node->src[0]);
            break;
        }
        case OP_CONCAT: {
            if (!concat_ok(node, &why)) { log_error("CONCAT node '%s' rejected: %s", node->name, why); return STATUS_FAILED; }
            const tensor * a = node->src[0], * b = node->src[1];
            int32_t dim; memcpy(&dim, node->op_params, 4);
            fill_copy_args(a->data, a->nb, a->ne, node->data, node->nb, &it.args[0].copy);
            fill_copy_args(b->data, b->nb, b->ne, (char *) node->data + (size_t) a->ne[dim] * node->nb[dim], node->nb, &it.args[1].copy);
            it.n_ops = 2;
            it.ops[0] = mla_front_op{ MLA_FRONT_COPY, 0, &it.args[0].copy };
            it.ops[1] = mla_front_op{ MLA_FRONT_COPY, 0, &it.args[1].copy };
            reads(a); reads(b);
            break;
        }
        case OP_ROPE: {
            if (!rope_ok(node, &why)) { log_error("ROPE node '%s' rejected: %s", node->name, why); return STATUS_FAILED; }
            mla_rope_args & a = it.args[0].rope;
            fill_rope_args(node, &a);
            it.rope_src = node->src[0];
            const tensor * x = node->src[0];
            const int ci = x->op == OP_CONT ? find_item(w, x) : -1;
            if (ci >= 0 && ci != self && f32_rows(x->src[0]) && x->src[0]->data) {
                const tensor * xs = x->src[0];
                bool same = true;
                for (int i = 0; i < 4; i++) same = same && xs->ne[i] == x->ne[i];
                mla_rope_args f = a;
                f.src = xs->data;
                for (int i = 0; i < 4; i++) f.src_nb[i] = (int64_t) xs->nb[i];
                // (the CONT's source as it was when the CONT ran, and the CONT's result as the CONT left it: nothing in between wrote either)
                if (same && mla_rope_check(&f) == 0 && !written_after(w, ci, range_of(xs)) && !written_between(w, ci, self, range_of(x))) {
                    a = f; it.rope_src = xs;
                    // the graph allocator lets a ROPE rotate in place (ggml-alloc.c: ggml_op_can_inplace): the CONT's result is
                    // then overwritten whole by this node, and when nothing in between reads it the CONT has no work left
                    bool read_between = false;
                    for (int k = ci + 1; k < self && !read_between; k++)
                        for (int r = 0; r < w[k].n_reads && !read_between; r++) read_between = overlaps(w[k].reads[r], w[ci].write);
                    if (node->data == x->data && tensor_nbytes(node) == tensor_nbytes(x) && !read_between) {
                        w[ci].n_ops = 0; w[ci].n_reads = 0; w[ci].write = mem_range{ nullptr, nullptr };
                    }
                }
            }
            it.ops[0] = mla_front_op{ MLA_FRONT_ROPE, 0, &a };
            reads(it.rope_src); reads(node->src[1]); reads(node->src[2]);
            break;
        }
        case OP_MUL_MAT: {
            if (!mul_mat_ok(node, &why)) { log_error("MUL_MAT node '%s' rejected: %s", node->name, why); return STATUS_FAILED; }
            fill_mul_mat_args(node, &it.args[0].mm);
            it.ops[0] = mla_front_op{ MLA_FRONT_MUL_MAT, 0, &it.args[0].mm };
            reads(node->src[0]); reads(node->src[1]);
            break;
        }
        default: {   // OP_CPY, OP_SCATTER_UPDATE
            mla_kv_write_args & a = it.args[0].kvw;
            const tensor * rows;
            if (node->op == OP_CPY) {
                if (!kv_cpy_ok(node, &why)) { log_error("CPY node '%s' rejected: %s", node->name, why); return STATUS_FAILED; }
                fill_kv_cpy_args(node, &a);
                rows = node->src[0];
            } else {
                if (!kv_scatter_ok(node, &why)) { log_error("SCATTER_UPDATE node '%s' rejected: %s", node->name, why); return STATUS_FAILED; }
                fill_kv_scatter_args(node, &a);
                rows = node->src[2];
                it.write = range_of(node->src[0]);
                reads(node->src[1]);
            }
            it.ops[0] = mla_front_op{ MLA_FRONT_KV_WRITE, 0, &a };
            // new rows = CONCAT(latent [512, n_tok], view of ROPE(k_pe [64, 1, n_tok])): the rope on the way into the cache
            const int ki = rows->op == OP_CONCAT ? find_item(w, rows) : -1;
            bool folded = false;
            if (ki >= 0 && ki != self && rows->type == TYPE_F32) {
                const tensor * lat = rows->src[0], * pe = rows->src[1];
                int32_t dim; memcpy(&dim, rows->op_params, 4);
                size_t off = 0;
                const tensor * r = pe ? view_root(pe, &off) : nullptr;
                const int ri = r && r->op == OP_ROPE ? find_item(w, r) : -1;
                if (dim == 0 && lat && lat->ne[0] == 512 && pe->ne[0] == 64 && ri >= 0 && off == 0 && is_contiguous(r) && r->ne[0] == 64 && r->ne[1] == 1 &&
                    r->ne[3] == 1 && pe->ne[1] == r->ne[2] && pe->ne[2] == 1 && pe->ne[3] == 1 && pe->nb[1] == 256 && lat->ne[1] == rows->ne[1] && lat->ne[2] == 1 && lat->ne[3] == 1) {
                    mla_kv_write_rope_args f;
                    f.w = a;
                    f.w.src = lat->data; f.w.src_nb1 = (int64_t) lat->nb[1];
                    f.rope = w[ri].args[0].rope;
                    const mem_range pe_src = range_of(w[ri].rope_src);
                    // (what the chain read is still what it was, and its intermediate results are what it left: the rotated k_pe up to the
                    // CONCAT, the CONCAT's rows up to this node)
                    if (mla_kv_write_rope_check(&f) == 0 && !written_between(w, ri, ki, range_of(r)) && !written_between(w, ki, self, range_of(rows)) &&
                        !written_after(w, ki, range_of(lat)) && !written_after(w, ri, pe_src) &&
                        !written_after(w, ri, range_of(r->src[1])) && !(r->src[2] && written_after(w, ri, range_of(r->src[2])))) {
                        it.args[0].kvr = f;
                        it.ops[0] = mla_front_op{ MLA_FRONT_KV_WRITE_ROPE, 0, &it.args[0].kvr };
                        reads(lat); it.reads[it.n_reads++] = pe_src; reads(r->src[1]); reads(r->src[2]);
                        folded = true;
                    }
                }
            }
            if (!folded) reads(rows);
            break;
        }
    }
    it.level = 0;
    for (int i = 0; i < self; i++) {
        const front_item & e = w[i];
        bool dep = overlaps(e.write, it.write);
        for (int k = 0; k < it.n_reads && !dep; k++) dep = overlaps(e.write, it.reads[k]);
        for (int k = 0; k < e.n_reads && !dep; k++) dep = overlaps(e.reads[k], it.write);
        if (dep && e.level + 1 > it.level) it.level = e.level + 1;
    }
    return STATUS_SUCCESS;
}

int front_flush(backend_ctx * ctx, std::vector<front_item> & w) {
    int max_level = -1;
    for (const front_item & it : w) if (it.level > max_level) max_level = it.level;
    if (ctx->log_schedule)
        for (const front_item & it : w)
            fprintf(stderr, "ggml-hip-mla: schedule: level %d  op %2d x%d  %-24s writes %p+%zu  reads %p %p %p\n", it.level, it.node->op, it.n_ops, it.node->name,
                    (const void *) it.write.lo, (size_t) (it.write.hi - it.write.lo), it.n_reads > 0 ? (const void *) it.reads[0].lo : nullptr,
                    it.n_reads > 1 ? (const void *) it.reads[1].lo : nullptr, it.n_reads > 2 ? (const void *) it.reads[2].lo : nullptr);
    std::vector<mla_front_op> ops;
    for (int level = 0; level <= max_level; level++) {
        ops.clear();
        for (const front_item & it : w)
            if (it.level == level)
                for (int k = 0; k < it.n_ops; k++) ops.push_back(it.ops[k]);
        if (ops.empty()) continue;
        const int rc = mla_front_batch_launch(ops.data(), (int32_t) ops.size(), ctx->stream);
        if (rc != 0) {
            for (const front_item & it : w) if (it.level == level) log_error("level %d holds node '%s'", level, it.node->name);
            log_error("mla_front_batch_launch failed: %d", rc);
            return STATUS_FAILED;
        }
        g_front_dispatches++;
    }
    g_front_nodes += (int64_t) w.size();
    w.clear();
    return STATUS_SUCCESS;
}

int backend_graph_compute(backend * be, cgraph * g) {
    backend_ctx * ctx = (backend_ctx *) be->context;
    if (!HIP_OK(hipSetDevice(ctx->device))) return STATUS_FAILED;
    ctx->ext_key_valid = false;   // (the mask is an input of the graph: it may have been set anew since the last call)
    std::vector<front_item> window;
    window.reserve(FRONT_WINDOW);   // the items hold pointers into themselves: the vector never grows past this
    for (int i = 0; i < g->n_nodes; i++) {
        const tensor * node = g->nodes[i];
        if (is_empty(node) || is_noop(node->op)) continue;
        // a node that writes into the mask whose extents the workspace holds (none of the reference's graphs has one) ends their validity
        if (ctx->ext_key_valid && node->data && ctx->ext_key.mask && node->op != OP_FLASH_ATTN_EXT) {
            const char * m0 = (const char *) ctx->ext_key.mask, * m1 = m0 + (size_t) ctx->ext_key.mask_nb1 * (size_t) ctx->ext_key.n_tok;
            const char * d0 = (const char *) node->data, * d1 = d0 + tensor_nbytes(node);
            if (d0 < m1 && m0 < d1) ctx->ext_key_valid = false;
        }
        int st;
        switch (node->op) {
            case OP_FLASH_ATTN_EXT:
                st = front_flush(ctx, window);
                if (st == STATUS_SUCCESS) st = compute_flash_attn(ctx, node);
                break;
            case OP_CPY: case OP_SCATTER_UPDATE: case OP_CONT: case OP_CONCAT: case OP_ROPE: case OP_MUL_MAT:
                if (!ctx->batch_front) { st = node->op == OP_CPY || node->op == OP_SCATTER_UPDATE ? compute_kv_write(ctx, node) : compute_front(ctx, node); break; }
                st = front_collect(window, node);
                if (st == STATUS_SUCCESS && (int) window.size() == FRONT_WINDOW) st = front_flush(ctx, window);
                break;
            default: log_error("op %d of node '%s' is not supported", node->op, node->name); return STATUS_FAILED;
        }
        if (st != STATUS_SUCCESS) return st;
    }
    return front_flush(ctx, window);
}

// Events (ggml-backend-impl.h:120-122, :132-135, :183-185; the reference's own: ggml-cann.cpp:2192-2219, :2365-2410): what
// ggml_backend_sched uses instead of full synchronisations when
// it keeps several copies of a graph's inputs in flight (ggml-backend.cpp:1508-1530, :1576-1580).
bool event_is_ours(const backend_event * ev);
void backend_event_record(backend * be, backend_event * ev) {
    backend_ctx * ctx = (backend_ctx *) be->context;
    (void) hipSetDevice(ctx->device);
    if (!HIP_OK(hipEventRecord((hipEvent_t) ev->context, ctx->stream))) log_error("event_record failed");
}
void backend_event_wait(backend * be, backend_event * ev) {
    backend_ctx * ctx = (backend_ctx *) be->context;
    (void) hipSetDevice(ctx->device);
    if (event_is_ours(ev)) {
        if (!HIP_OK(hipStreamWaitEvent(ctx->stream, (hipEvent_t) ev->context, 0))) log_error("event_wait failed");
    } else if (ev->device && ev->device->iface.event_synchronize) {
        ev->device->iface.event_synchronize(ev->device, ev);   // another backend's event: wait for it on the host
    }
}

const backend_i k_backend_iface = {
    /* get_name           */ backend_get_name,
    /* free               */ backend_free,
    /* set_tensor_async   */ backend_set_tensor_async,
    /* get_tensor_async   */ backend_get_tensor_async,
    /* cpy_tensor_async   */ nullptr,
    /* synchronize        */ backend_synchronize,
    /* graph_plan_create  */ nullptr,
    /* graph_plan_free    */ nullptr,
    /* graph_plan_update  */ nullptr,
    /* graph_plan_compute */ nullptr,
    /* graph_compute      */ backend_graph_compute,
    /* event_record       */ backend_event_record,
    /* event_wait         */ backend_event_wait,
};

// ---------------------------------------------------------------- device

const char * device_get_name(backend_device * dev) { return ((device_ctx *) dev->context)->name.c_str(); }
const char * device_get_description(backend_device * dev) { return ((device_ctx *) dev->context)->description.c_str(); }
void device_get_memory(backend_device * dev, size_t * free, size_t * total) {
    device_ctx * dc = (device_ctx *) dev->context;
    *free = *total = 0;
    if (HIP_OK(hipSetDevice(dc->index))) (void) hipMemGetInfo(free, total);
}
int  device_get_type(backend_device *) { return DEVICE_TYPE_GPU; }
void device_get_props(backend_device * dev, dev_props * props) {
    props->name        = device_get_name(dev);
    props->description = device_get_description(dev);
    props->type        = DEVICE_TYPE_GPU;
    device_get_memory(dev, &props->memory_free, &props->memory_total);
    props->caps = dev_caps{ /* async */ true, /* host_buffer */ true, /* buffer_from_host_ptr */ false, /* events */ true };
}
// params (the string ggml_backend_dev_init hands through, ggml-backend.cpp:505-508) or the environment may ask for
// "f16_acc=strict": attention over an F16 cache then reproduces ggml-cpu's f16 accumulator (ggml-cpu.c:12066-12080)
// instead of the f32 accumulation that is closer to the exact value.
backend * device_init_backend(backend_device * dev, const char * params) {
    device_ctx * dc = (device_ctx *) dev->context;
    if (!HIP_OK(hipSetDevice(dc->index))) return nullptr;
    backend_ctx * ctx = new backend_ctx;
    ctx->device = dc->index;
    ctx->name   = dc->name;
    const char * env = getenv("GGML_HIP_MLA_F16_ACC");
    ctx->f16_strict = (params && strstr(params, "f16_acc=strict")) || (env && strcmp(env, "strict") == 0);
    const char * env_q8 = getenv("GGML_HIP_MLA_Q8");
    ctx->q8_exact = (params && strstr(params, "q8=exact")) || (env_q8 && strcmp(env_q8, "exact") == 0);
    const char * env_bf = getenv("GGML_HIP_MLA_BF16");
    ctx->bf16_direct = (params && strstr(params, "bf16=direct")) || (env_bf && strcmp(env_bf, "direct") == 0);
    const char * env_ext = getenv("GGML_HIP_MLA_MASK_EXTENTS");   // "rescan": every attention node scans its mask itself
    ctx->reuse_mask_extents = !((params && strstr(params, "mask_extents=rescan")) || (env_ext && strcmp(env_ext, "rescan") == 0));
    const char * env_dbg = getenv("GGML_HIP_MLA_DEBUG");
    ctx->log_schedule = env_dbg && strstr(env_dbg, "schedule");
    const char * env_batch = getenv("GGML_HIP_MLA_BATCH");   // "off": every node a launch of its own
    ctx->batch_front = !((params && strstr(params, "batch=off")) || (env_batch && strcmp(env_batch, "off") == 0));
    if (!HIP_OK(hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking))) { delete ctx; return nullptr; }
    return new backend{ &g_guid, k_backend_iface, dev, ctx };
}
backend_buffer_type * device_get_buffer_type(backend_device * dev) { return &((device_ctx *) dev->context)->buft; }
bool device_supports_buft(backend_device * dev, backend_buffer_type * buft) { return buft == device_get_buffer_type(dev); }
backend_buffer_type * device_get_host_buffer_type(backend_device * dev) { return &((device_ctx *) dev->context)->host_buft; }

backend_event * device_event_new(backend_device * dev) {
    device_ctx * dc = (device_ctx *) dev->context;
    hipEvent_t ev = nullptr;
    if (!HIP_OK(hipSetDevice(dc->index)) || !HIP_OK(hipEventCreateWithFlags(&ev, hipEventDisableTiming))) return nullptr;
    return new backend_event{ dev, ev };
}
void device_event_free(backend_device *, backend_event * ev) {
    if (!ev) return;
    (void) hipEventDestroy((hipEvent_t) ev->context);
    delete ev;
}
void device_event_synchronize(backend_device *, backend_event * ev) {
    if (!HIP_OK(hipEventSynchronize((hipEvent_t) ev->context))) log_error("event_synchronize failed");
}
bool event_is_ours(const backend_event * ev) { return ev && ev->device && ev->device->iface.event_new == device_event_new; }

const backend_device_i k_device_iface = {
    /* get_name             */ device_get_name,
    /* get_description      */ device_get_description,
    /* get_memory           */ device_get_memory,
    /* get_type             */ device_get_type,
    /* get_props            */ device_get_props,
    /* init_backend         */ device_init_backend,
    /* get_buffer_type      */ device_get_buffer_type,
    /* get_host_buffer_type */ device_get_host_buffer_type,
    /* buffer_from_host_ptr */ nullptr,
    /* supports_op          */ device_supports_op,
    /* supports_buft        */ device_supports_buft,
    /* offload_op           */ nullptr,
    /* event_new            */ device_event_new,
    /* event_free           */ device_event_free,
    /* event_synchronize    */ device_event_synchronize,
};

// ---------------------------------------------------------------- registry

const char * reg_get_name(backend_reg *) { return "HIP-MLA"; }
size_t       reg_get_device_count(backend_reg *) { return g_devices.size(); }
backend_device * reg_get_device(backend_reg *, size_t index) { return index < g_devices.size() ? g_devices[index] : nullptr; }
// The reference probes for "ggml_backend_set_n_threads", "ggml_backend_set_abort_callback" and
// "ggml_backend_comm_init*" (src/llama-context-load-utils.cpp:72-76, :360-385); none applies here.
void * reg_get_proc_address(backend_reg *, const char *) { return nullptr; }

int gfx950_device_count() {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) { (void) hipGetLastError(); return 0; }
    int ok = 0;
    for (int i = 0; i < n; i++) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, i) != hipSuccess) continue;
        if (strncmp(prop.gcnArchName, "gfx950", 6) == 0) ok++;
    }
    return ok;
}

void init_registry() {
    g_reg.api_version = BACKEND_API_VERSION;
    g_reg.iface       = backend_reg_i{ reg_get_name, reg_get_device_count, reg_get_device, reg_get_proc_address };
    g_reg.context     = nullptr;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) { (void) hipGetLastError(); n = 0; }
    for (int i = 0; i < n; i++) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, i) != hipSuccess) continue;
        if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) continue;  // the kernels exist for gfx950 only
        device_ctx * dc = new device_ctx;
        dc->index       = i;
        dc->name        = "HIPMLA" + std::to_string(i);
        dc->description = prop.name;
        backend_device * dev = new backend_device{ k_device_iface, &g_reg, dc };
        dc->buft.iface   = backend_buffer_type_i{ buft_get_name, buft_alloc_buffer, buft_get_alignment, nullptr, nullptr, buft_is_host };
        dc->buft.device  = dev;
        dc->buft.context = dc;
        dc->host_name         = dc->name + "_Host";
        dc->host_buft.iface   = backend_buffer_type_i{ host_buft_get_name, host_buft_alloc_buffer, host_buft_get_alignment, nullptr, nullptr, host_buft_is_host };
        dc->host_buft.device  = dev;
        dc->host_buft.context = dc;
        g_device_ctx.push_back(dc);
        g_devices.push_back(dev);
    }
}

struct abi_entry { const char * name; int64_t value; };
#define E(n, v) { n, (int64_t) (v) }
const abi_entry k_abi_table[] = {
    E("sizeof(ggml_tensor)", sizeof(tensor)),
    E("offsetof(ggml_tensor,type)", offsetof(tensor, type)), E("offsetof(ggml_tensor,buffer)", offsetof(tensor, buffer)),
    E("offsetof(ggml_tensor,ne)", offsetof(tensor, ne)), E("offsetof(ggml_tensor,nb)", offsetof(tensor, nb)),
    E("offsetof(ggml_tensor,op)", offsetof(tensor, op)), E("offsetof(ggml_tensor,op_params)", offsetof(tensor, op_params)),
    E("offsetof(ggml_tensor,flags)", offsetof(tensor, flags)), E("offsetof(ggml_tensor,src)", offsetof(tensor, src)),
    E("offsetof(ggml_tensor,view_src)", offsetof(tensor, view_src)), E("offsetof(ggml_tensor,view_offs)", offsetof(tensor, view_offs)),
    E("offsetof(ggml_tensor,data)", offsetof(tensor, data)), E("offsetof(ggml_tensor,name)", offsetof(tensor, name)),
    E("offsetof(ggml_tensor,extra)", offsetof(tensor, extra)),
    E("GGML_MAX_DIMS", MAX_DIMS), E("GGML_MAX_SRC", MAX_SRC), E("GGML_MAX_OP_PARAMS", MAX_OP_PARAMS), E("GGML_MAX_NAME", MAX_NAME),
    E("GGML_KQ_MASK_PAD", KQ_MASK_PAD),
    E("sizeof(ggml_cgraph)", sizeof(cgraph)), E("offsetof(ggml_cgraph,n_nodes)", offsetof(cgraph, n_nodes)), E("offsetof(ggml_cgraph,nodes)", offsetof(cgraph, nodes)),
    E("sizeof(ggml_backend_buffer_type_i)", sizeof(backend_buffer_type_i)), E("sizeof(ggml_backend_buffer_type)", sizeof(backend_buffer_type)),
    E("offsetof(ggml_backend_buffer_type,device)", offsetof(backend_buffer_type, device)), E("offsetof(ggml_backend_buffer_type,context)", offsetof(backend_buffer_type, context)),
    E("sizeof(ggml_backend_buffer_i)", sizeof(backend_buffer_i)), E("sizeof(ggml_backend_buffer)", sizeof(backend_buffer)),
    E("offsetof(ggml_backend_buffer,buft)", offsetof(backend_buffer, buft)), E("offsetof(ggml_backend_buffer,context)", offsetof(backend_buffer, context)),
    E("offsetof(ggml_backend_buffer,size)", offsetof(backend_buffer, size)), E("offsetof(ggml_backend_buffer,usage)", offsetof(backend_buffer, usage)),
    E("sizeof(ggml_backend_i)", sizeof(backend_i)), E("offsetof(ggml_backend_i,graph_compute)", offsetof(backend_i, graph_compute)),
    E("offsetof(ggml_backend_i,synchronize)", offsetof(backend_i, synchronize)),
    E("sizeof(ggml_backend)", sizeof(backend)), E("offsetof(ggml_backend,iface)", offsetof(backend, iface)),
    E("offsetof(ggml_backend,device)", offsetof(backend, device)), E("offsetof(ggml_backend,context)", offsetof(backend, context)),
    E("sizeof(ggml_backend_device_i)", sizeof(backend_device_i)), E("offsetof(ggml_backend_device_i,supports_op)", offsetof(backend_device_i, supports_op)),
    E("sizeof(ggml_backend_device)", sizeof(backend_device)), E("offsetof(ggml_backend_device,reg)", offsetof(backend_device, reg)),
    E("offsetof(ggml_backend_device,context)", offsetof(backend_device, context)),
    E("sizeof(ggml_backend_reg_i)", sizeof(backend_reg_i)), E("sizeof(ggml_backend_reg)", sizeof(backend_reg)),
    E("offsetof(ggml_backend_reg,iface)", offsetof(backend_reg, iface)), E("offsetof(ggml_backend_reg,context)", offsetof(backend_reg, context)),
    E("sizeof(ggml_backend_dev_props)", sizeof(dev_props)), E("offsetof(ggml_backend_dev_props,type)", offsetof(dev_props, type)),
    E("offsetof(ggml_backend_dev_props,caps)", offsetof(dev_props, caps)),
    E("sizeof(ggml_backend_event)", sizeof(backend_event)),
    E("GGML_BACKEND_API_VERSION", BACKEND_API_VERSION),
    E("GGML_TYPE_F32", TYPE_F32), E("GGML_TYPE_F16", TYPE_F16), E("GGML_TYPE_Q8_0", TYPE_Q8_0), E("GGML_TYPE_I8", TYPE_I8),
    E("GGML_TYPE_I32", TYPE_I32), E("GGML_TYPE_BF16", TYPE_BF16), E("GGML_TYPE_COUNT", TYPE_COUNT),
    E("GGML_OP_NONE", OP_NONE), E("GGML_OP_CPY", OP_CPY), E("GGML_OP_CONT", OP_CONT), E("GGML_OP_RESHAPE", OP_RESHAPE),
    E("GGML_OP_VIEW", OP_VIEW), E("GGML_OP_PERMUTE", OP_PERMUTE), E("GGML_OP_TRANSPOSE", OP_TRANSPOSE),
    E("GGML_OP_FLASH_ATTN_EXT", OP_FLASH_ATTN_EXT), E("GGML_OP_SCATTER_UPDATE", OP_SCATTER_UPDATE), E("GGML_OP_COUNT", OP_COUNT),
    E("GGML_OP_ROPE", OP_ROPE), E("GGML_OP_MUL_MAT", OP_MUL_MAT), E("GGML_OP_CONCAT", OP_CONCAT),
    E("GGML_STATUS_ALLOC_FAILED", STATUS_ALLOC_FAILED), E("GGML_STATUS_FAILED", STATUS_FAILED), E("GGML_STATUS_SUCCESS", STATUS_SUCCESS),
    E("GGML_STATUS_ABORTED", STATUS_ABORTED),
    E("GGML_BACKEND_DEVICE_TYPE_CPU", DEVICE_TYPE_CPU), E("GGML_BACKEND_DEVICE_TYPE_GPU", DEVICE_TYPE_GPU),
    E("GGML_BACKEND_BUFFER_USAGE_ANY", BUFFER_USAGE_ANY), E("GGML_BACKEND_BUFFER_USAGE_COMPUTE", BUFFER_USAGE_COMPUTE),
    E("GGML_PREC_DEFAULT", PREC_DEFAULT), E("GGML_PREC_F32", PREC_F32),
    E("GGML_TENSOR_FLAG_INPUT", TENSOR_FLAG_INPUT), E("GGML_TENSOR_FLAG_OUTPUT", TENSOR_FLAG_OUTPUT),
    E("sizeof(block_q8_0)", sizeof(block_q8_0)),
};

}  // namespace

extern "C" {

void * ggml_backend_init(void) {
    std::call_once(g_once, init_registry);
    return &g_reg;
}

int ggml_backend_score(void) { return gfx950_device_count() > 0 ? 100 : 0; }

int64_t mla_ggml_mask_extent_reuses(void) { return g_mask_extent_reuses.load(); }
int64_t mla_ggml_front_dispatches(void) { return g_front_dispatches.load(); }
int64_t mla_ggml_front_nodes(void) { return g_front_nodes.load(); }

void * ggml_backend_hip_mla_reg(void) { return ggml_backend_init(); }

int mla_ggml_abi_table(int i, const char ** name, int64_t * value) {
    const int n = (int) (sizeof(k_abi_table) / sizeof(k_abi_table[0]));
    if (i < 0 || i >= n) return n;
    *name  = k_abi_table[i].name;
    *value = k_abi_table[i].value;
    return n;
}

void mla_ggml_buffer_free(void * buffer) {
    backend_buffer * b = (backend_buffer *) buffer;
    if (!b) return;
    if (b->iface.free_buffer) b->iface.free_buffer(b);
    delete b;
}

int mla_ggml_supports_node(const void * node, const char ** why) {
    const tensor * t = (const tensor *) node;
    const char * dummy; if (!why) why = &dummy;
    *why = "";
    if (is_noop(t->op)) return 1;
    switch (t->op) {
        case OP_FLASH_ATTN_EXT: return mla_node_ok(t, why) ? 1 : 0;
        case OP_CPY: return kv_cpy_ok(t, why) ? 1 : 0;
        case OP_SCATTER_UPDATE: return kv_scatter_ok(t, why) ? 1 : 0;
        case OP_CONT: return cont_ok(t, why) ? 1 : 0;
        case OP_CONCAT: return concat_ok(t, why) ? 1 : 0;
        case OP_ROPE: return rope_ok(t, why) ? 1 : 0;
        case OP_MUL_MAT: return mul_mat_ok(t, why) ? 1 : 0;
        default: *why = "op not taken by this backend"; return 0;
    }
}

int mla_ggml_node_launch_check(const void * node) {
    const tensor * t = (const tensor *) node;
    switch (t->op) {
        case OP_FLASH_ATTN_EXT: { mla_attn_args a; fill_attn_args(t, &a); mla_attn_plan_info info; return mla_attn_plan(&a, &info); }
        case OP_CPY: { mla_kv_write_args a; fill_kv_cpy_args(t, &a); return mla_kv_write_check(&a); }
        case OP_SCATTER_UPDATE: { mla_kv_write_args a; fill_kv_scatter_args(t, &a); return mla_kv_write_check(&a); }
        case OP_CONT: { mla_copy_args a; fill_cont_args(t, &a); return mla_copy_f32_check(&a); }
        case OP_CONCAT: {
            const tensor * x = t->src[0], * y = t->src[1];
            int32_t dim; memcpy(&dim, t->op_params, 4);
            mla_copy_args c;
            fill_copy_args(addr_of(x), x->nb, x->ne, addr_of(t), t->nb, &c);
            const int rc = mla_copy_f32_check(&c);
            if (rc) return rc;
            fill_copy_args(addr_of(y), y->nb, y->ne, (const char *) addr_of(t) + (size_t) x->ne[dim] * t->nb[dim], t->nb, &c);
            return mla_copy_f32_check(&c);
        }
        case OP_ROPE: { mla_rope_args a; fill_rope_args(t, &a); return mla_rope_check(&a); }
        case OP_MUL_MAT: { mla_mul_mat_args a; fill_mul_mat_args(t, &a); return mla_mul_mat_check(&a); }
        default: return is_noop(t->op) ? 0 : MLA_ERR_UNSUPPORTED;
    }
}

}  // extern "C"
