// Latent-KV cache write for gfx950: new rows of 576 values -> cache rows (bf16 / f16 / Q8_0), consecutive, scattered by
// row index, or through the block table.  HBM-bound: every source byte is read once, every cache byte written once.
//
// One thread = 8 consecutive values of a row (72 threads per row): two 16-byte loads, one 16-byte store for the 16-bit
// types.  Q8_0: the 4 threads of a 32-value block (an aligned lane quad) agree on amax with two DPP-free shuffles, then
// every thread writes its 8 int8 values and the quarter-0 thread the block scale, the way ggml-cpu's x86 quantizer does it
// (ggml-cpu-quants.c:855-900: d = amax/127 stored as f16, id = 127/amax, round half to even).

#include "mla_common.hpp"
#include "../../include/mla_kv_write.h"

using namespace mla;

namespace {

struct WParams {
    const char * src; int64_t src_nb1;
    char * kv; int64_t kv_nb1, n_kv_rows, row0;
    const void * rows; int rows_i64;
    const int32_t * block_table; int64_t bt_stride;
    const int32_t * seq_ids; const int32_t * positions;
    int n_tok;
};

__device__ __forceinline__ int64_t dest_row(const WParams & p, int t) {
    if (p.block_table) {
        const int pos = p.positions[t];
        if (pos < 0 || pos / MLA_PAGE_TOKENS >= p.bt_stride) return -1;
        const int64_t page = p.block_table[(int64_t) p.seq_ids[t] * p.bt_stride + pos / MLA_PAGE_TOKENS];
        return page < 0 ? -1 : page * MLA_PAGE_TOKENS + pos % MLA_PAGE_TOKENS;
    }
    if (p.rows) return p.rows_i64 ? ((const int64_t *) p.rows)[t] : (int64_t) ((const int32_t *) p.rows)[t];
    return p.row0 + t;
}

// KVT: SRC_BF16 / SRC_F16 / SRC_Q8.  CONVERT: source rows are f32; otherwise they already have the cache type.
template <int KVT, bool CONVERT>
__global__ void __launch_bounds__(256) mla_kv_write_kernel(const WParams p) {
    constexpr int GROUPS = CONVERT || KVT != SRC_Q8 ? 72 : 0;   // 8-value groups per row
    if constexpr (!CONVERT) {
        // raw row copy: 16-bit rows are 72 chunks of 16 bytes; Q8_0 rows are 153 words of 4 bytes
        constexpr int UNITS = KVT == SRC_Q8 ? Q8_ROW / 4 : 72;
        const int64_t gid = (int64_t) blockIdx.x * 256 + threadIdx.x;
        const int t = (int) (gid / UNITS), u = (int) (gid - (int64_t) t * UNITS);
        if (t >= p.n_tok) return;
        const int64_t r = dest_row(p, t);
        if (r < 0 || r >= p.n_kv_rows) return;
        if constexpr (KVT == SRC_Q8) *(unsigned *) (p.kv + r * p.kv_nb1 + 4 * u) = *(const unsigned *) (p.src + (int64_t) t * p.src_nb1 + 4 * u);
        else *(u32x4 *) (p.kv + r * p.kv_nb1 + 16 * u) = *(const u32x4 *) (p.src + (int64_t) t * p.src_nb1 + 16 * u);
        return;
    } else {
        const int64_t gid = (int64_t) blockIdx.x * 256 + threadIdx.x;
        const int t = (int) (gid / GROUPS), u = (int) (gid - (int64_t) t * GROUPS);
        const bool live = t < p.n_tok;
        const int tc = live ? t : p.n_tok - 1;
        const float * s = (const float *) (p.src + (int64_t) tc * p.src_nb1) + 8 * u;
        const f32x4 x0 = *(const f32x4 *) s, x1 = *(const f32x4 *) (s + 4);
        const float x[8] = { x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w };
        const int64_t r = live ? dest_row(p, t) : -1;
        const bool ok = r >= 0 && r < p.n_kv_rows;
        if constexpr (KVT != SRC_Q8) {
            if (!ok) return;
            constexpr bool F16 = KVT == SRC_F16;
            *(u32x4 *) (p.kv + r * p.kv_nb1 + 16 * u) =
                u32x4{ pack2<F16>(x[0], x[1]), pack2<F16>(x[2], x[3]), pack2<F16>(x[4], x[5]), pack2<F16>(x[6], x[7]) };
        } else {
            // 72 groups per row and 256 threads per block: 72 and 256 are multiples of 4, so the 4 groups of a block of 32
            // values sit in one aligned lane quad of one wave
            float amax = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(x[e]));
            amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
            amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
            if (!ok) return;
            const float d  = amax / 127.0f;
            const float id = amax != 0.f ? 127.0f / amax : 0.f;
            const int b = u >> 2, qt = u & 3;
            char * blk = p.kv + r * p.kv_nb1 + 34 * b;
            if (qt == 0) *(unsigned short *) blk = (unsigned short) f32_to_f16_bits(d);
            unsigned short * qs = (unsigned short *) (blk + 2 + 8 * qt);   // 2-byte aligned
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int a = (int) rintf(x[2 * e] * id), c = (int) rintf(x[2 * e + 1] * id);
                qs[e] = (unsigned short) ((a & 0xff) | ((c & 0xff) << 8));
            }
        }
    }
}

template <int KVT> hipError_t launch_kvt(const WParams & p, bool convert, hipStream_t st) {
    const int units = convert || KVT != SRC_Q8 ? 72 : Q8_ROW / 4;
    const int64_t threads = (int64_t) p.n_tok * units;
    const dim3 grid((unsigned) ((threads + 255) / 256));
    if (convert) hipLaunchKernelGGL((mla_kv_write_kernel<KVT, true>), grid, dim3(256), 0, st, p);
    else         hipLaunchKernelGGL((mla_kv_write_kernel<KVT, false>), grid, dim3(256), 0, st, p);
    return hipGetLastError();
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
    const bool convert = a->src_type == MLA_TYPE_F32;

    WParams p;
    p.src = (const char *) a->src; p.src_nb1 = a->src_nb1;
    p.kv = (char *) a->kv; p.kv_nb1 = a->kv_nb1; p.n_kv_rows = a->n_kv_rows; p.row0 = a->row0;
    p.rows = a->rows; p.rows_i64 = a->rows_type;
    p.block_table = a->block_table; p.bt_stride = a->bt_stride; p.seq_ids = a->seq_ids; p.positions = a->positions;
    p.n_tok = a->n_tok;
    hipError_t e;
    switch (a->kv_type) {
        case MLA_TYPE_BF16: e = launch_kvt<SRC_BF16>(p, convert, (hipStream_t) stream); break;
        case MLA_TYPE_F16:  e = launch_kvt<SRC_F16>(p, convert, (hipStream_t) stream); break;
        default:            e = launch_kvt<SRC_Q8>(p, convert, (hipStream_t) stream); break;
    }
    return (int) e;
}
