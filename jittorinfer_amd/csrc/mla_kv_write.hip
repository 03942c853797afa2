// Latent-KV cache write for gfx950: new rows of 576 values -> cache rows (bf16 / f16 / Q8_0), consecutive, scattered by
// row index, or through the block table.  HBM-bound: every source byte is read once, every cache byte written once.
//
// One thread = 8 consecutive values of a row (72 threads per row): two 16-byte loads, one 16-byte store for the 16-bit
// types.  Q8_0: the 4 threads of a 32-value block (an aligned lane quad) agree on amax with two DPP-free shuffles, then
// every thread writes its 8 int8 values and the quarter-0 thread the block scale, the way ggml-cpu's x86 quantizer does it
// (ggml-cpu-quants.c:855-900: d = amax/127 stored as f16, id = 127/amax, round half to even).

#include "mla_front_bodies.hpp"

using namespace mla;
using namespace mla::front;

namespace {

template <int KVT, bool CONVERT, bool ROPE>
__global__ void __launch_bounds__(256) mla_kv_write_kernel(const WParams p) {
    kv_write_body<KVT, CONVERT, ROPE>(p, Blk{ blockIdx.x, 0, 0, gridDim.x });
}

template <int KVT> hipError_t launch_kvt(const WParams & p, dim3 grid, bool convert, bool rope, hipStream_t st) {
    if (rope)         hipLaunchKernelGGL((mla_kv_write_kernel<KVT, true, true>), grid, dim3(256), 0, st, p);
    else if (convert) hipLaunchKernelGGL((mla_kv_write_kernel<KVT, true, false>), grid, dim3(256), 0, st, p);
    else              hipLaunchKernelGGL((mla_kv_write_kernel<KVT, false, false>), grid, dim3(256), 0, st, p);
    return hipGetLastError();
}

hipError_t launch_typed(int kv_type, const WParams & p, dim3 grid, bool convert, bool rope, hipStream_t st) {
    switch (kv_type) {
        case MLA_TYPE_BF16: return launch_kvt<SRC_BF16>(p, grid, convert, rope, st);
        case MLA_TYPE_F16:  return launch_kvt<SRC_F16>(p, grid, convert, rope, st);
        default:            return launch_kvt<SRC_Q8>(p, grid, convert, rope, st);
    }
}

}  // namespace

extern "C" int mla_kv_write_check(const mla_kv_write_args * a) {
    if (!a) return MLA_ERR_NULL;
    if (a->n_tok < 0 || a->n_kv_rows < 0) return MLA_ERR_BAD_SHAPE;
    if (a->kv_type != MLA_TYPE_BF16 && a->kv_type != MLA_TYPE_F16 && a->kv_type != MLA_TYPE_Q8_0) return MLA_ERR_BAD_TYPE;
    if (a->src_type != MLA_TYPE_F32 && a->src_type != a->kv_type) return MLA_ERR_BAD_TYPE;
    if (a->rows_type != 0 && a->rows_type != 1) return MLA_ERR_BAD_TYPE;
    if (a->n_tok == 0) return 0;
    if (!a->src || !a->kv) return MLA_ERR_NULL;
    const bool convert = a->src_type == MLA_TYPE_F32;
    const bool q8 = a->kv_type == MLA_TYPE_Q8_0;
    const int64_t row_bytes = q8 ? Q8_ROW : ROW_BYTES;
    if (a->kv_nb1 < row_bytes || a->src_nb1 < (convert ? DK * 4 : row_bytes)) return MLA_ERR_BAD_SHAPE;
    if (q8) {
        if (((uintptr_t) a->kv & 1) || (a->kv_nb1 & 1)) return MLA_ERR_BAD_ALIGNMENT;
        if (!convert && (((uintptr_t) a->kv & 3) || (a->kv_nb1 & 3) || ((uintptr_t) a->src & 3) || (a->src_nb1 & 3))) return MLA_ERR_BAD_ALIGNMENT;
    } else if (((uintptr_t) a->kv & 15) || (a->kv_nb1 & 15)) return MLA_ERR_BAD_ALIGNMENT;
    if (convert ? (((uintptr_t) a->src & 15) || (a->src_nb1 & 15)) : (!q8 && (((uintptr_t) a->src & 15) || (a->src_nb1 & 15)))) return MLA_ERR_BAD_ALIGNMENT;
    if (a->block_table) {
        if (!a->seq_ids || !a->positions || a->bt_stride < 1) return MLA_ERR_NULL;
    } else if (!a->rows && (a->row0 < 0 || a->row0 + a->n_tok > a->n_kv_rows)) return MLA_ERR_BAD_SHAPE;
    return 0;
}

extern "C" int mla_kv_write_launch(const mla_kv_write_args * a, void * stream) {
    const int rc = mla_kv_write_check(a);
    if (rc) return rc;
    if (a->n_tok == 0) return 0;
    WParams p;
    const dim3 grid = make_kv_write_params(a, &p);
    return (int) launch_typed(a->kv_type, p, grid, a->src_type == MLA_TYPE_F32, false, (hipStream_t) stream);
}

extern "C" int mla_kv_write_rope_check(const mla_kv_write_rope_args * a) {
    if (!a) return MLA_ERR_NULL;
    if (a->w.src_type != MLA_TYPE_F32) return MLA_ERR_BAD_TYPE;
    const mla_rope_args & r = a->rope;
    // the latent rows need only their first 512 values: checked as rows of 576 minus what k_pe supplies
    mla_kv_write_args w = a->w;
    if (w.n_tok > 0 && w.src_nb1 >= 512 * 4 && w.src_nb1 < DK * 4) w.src_nb1 = DK * 4;
    int rc = mla_kv_write_check(&w);
    if (rc) return rc;
    if (r.n_dims != 64 || r.ne[0] != 64 || r.ne[1] != 1 || r.ne[2] != a->w.n_tok || r.ne[3] != 1) return MLA_ERR_BAD_SHAPE;
    if (r.mode != MLA_ROPE_MODE_NORM) return MLA_ERR_UNSUPPORTED;
    if (r.src_nb[0] != 4) return MLA_ERR_BAD_SHAPE;
    if (a->w.n_tok == 0) return 0;
    if (!r.src || !r.pos) return MLA_ERR_NULL;
    if (((uintptr_t) r.src & 15) || (r.src_nb[2] & 15)) return MLA_ERR_BAD_ALIGNMENT;
    return 0;
}

extern "C" int mla_kv_write_rope_launch(const mla_kv_write_rope_args * a, void * stream) {
    const int rc = mla_kv_write_rope_check(a);
    if (rc) return rc;
    if (a->w.n_tok == 0) return 0;
    WParams p;
    const dim3 grid = make_kv_write_rope_params(a, &p);
    return (int) launch_typed(a->w.kv_type, p, grid, true, true, (hipStream_t) stream);
}
