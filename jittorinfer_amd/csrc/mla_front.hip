// The nodes either side of the MLA attention node, for gfx950: rotary embedding (YaRN), the batched absorb products on
// the matrix cores, and strided f32 copies (ggml_cont, the halves of ggml_concat).
//
// Rotary embedding: one workgroup per (token, group of heads).  Its first threads build the (cos, sin) table of the
// token with the arithmetic of ggml-cpu (ggml/src/ggml-cpu/ggml-cpu.c:10272-10307): theta starts at the position and is
// multiplied by theta_scale once per pair, in f32, in order; the YaRN blend is fma(interp, 1 - mix, extrap * mix), the
// form the reference's x86 build evaluates; theta_scale, the correction dims and the magnitude scale come from the
// host's libm exactly as the reference computes them (powf / logf).  Then every thread rotates pairs:
// fma(x0, cos, -(x1 * sin)), fma(x0, sin, x1 * cos).  HBM-bound: each value is read once and written once.
//
// Absorb products: dst[n, m, b] = sum_k w[k, n, b / r] * bf16|f16(x[k, m, b]), f32 accumulation in
// v_mfma_f32_32x32x16_{bf16,f16}.  A workgroup owns 128 outputs n (one block of 32 per wave) and 32 / 64 / 128 rows m.
// Weights go from HBM straight into the MFMA operand registers of the one wave that needs them (no other wave of the
// workgroup uses the same weight rows, so LDS would add nothing), one K chunk of 128 ahead of the MFMAs; the f32
// activation rows are rounded to the weight type on their way into LDS (what ggml-cpu's from_float does into its work
// buffer, ggml-cpu.c:8571-8606) and shared by the four waves.  Decode shapes (m <= 32) are bound by the weight stream
// from HBM, prefill shapes by the matrix cores.

#include <math.h>

#include "mla_front_bodies.hpp"

using namespace mla;
using namespace mla::front;

namespace {

__global__ void __launch_bounds__(256) mla_rope_kernel(const RopeP p) {
    __shared__ __attribute__((aligned(16))) char lds[ROPE_LDS];
    rope_body(p, Blk{ blockIdx.x, blockIdx.y, blockIdx.z, gridDim.x }, lds);
}

template <bool F16, int MB>
__global__ void __launch_bounds__(256) mla_mul_mat_kernel(const MmP p) {
    __shared__ __attribute__((aligned(16))) char lds[MM_LDS<MB>];
    mm_body<F16, MB>(p, xcd_grouped(Blk{ blockIdx.x, blockIdx.y, blockIdx.z, gridDim.x }, gridDim.y, gridDim.z), lds);
}

template <bool F16>
__global__ void __launch_bounds__(256) mla_mul_mat_small_kernel(const MmP p) {
    __shared__ __attribute__((aligned(16))) char lds[MS_LDS];
    mm_small_body<F16>(p, xcd_grouped(Blk{ blockIdx.x, blockIdx.y, blockIdx.z, gridDim.x }, gridDim.y, gridDim.z), lds);
}

// Many rows m with K = 128, 256 or 512 (a prefill chunk through the absorb products): bound by the f32 activations
// and results moving through HBM, not by the matrix cores, so the kernel is a software pipeline around the loads.  A
// workgroup keeps its 128 weight rows (all of K) in MFMA operand registers and walks over tiles of 64 rows m; while the
// MFMAs of one 64 x 128 activation chunk run out of LDS, the next chunk's global loads are in flight, and it is rounded
// into the other LDS buffer at the end of the step: one barrier per chunk.
template <bool F16, int KCH>
__global__ void __launch_bounds__(256) mla_mul_mat_stream_kernel(const MmP p, const int tiles_per_wg) {
    constexpr int TM = 64, OB_PITCH = 128 + 4;
    __shared__ __attribute__((aligned(16))) char lds[2][TM * MM_PITCH];
    __shared__ __attribute__((aligned(16))) float obuf[TM * OB_PITCH];
    // whole 128-wide n tiles and 16-byte aligned result rows: results are written row-wise through LDS
    const bool vec_store = p.N % 128 == 0 && !(p.d_nb1 & 15) && !(p.d_nb2 & 15) && !(p.d_nb3 & 15) && !((uintptr_t) p.dst & 15);
    const int     lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // dispatch index i runs on XCD i % 8: remapped so that the workgroups that read the same activation rows (the n tiles
    // of one run of m tiles) sit on one XCD and share its L2
    unsigned bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
    {
        const unsigned G = gridDim.x * gridDim.y * gridDim.z;
        if ((G & 7) == 0 && gridDim.x > 1) {   // (with one n tile nothing is shared, and the plain order measured 12 % faster)
            const unsigned id = (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
            const unsigned v  = (id & 7) * (G >> 3) + (id >> 3);
            bx = v % gridDim.x; by = (v / gridDim.x) % gridDim.y; bz = v / (gridDim.x * gridDim.y);
        }
    }
    const int64_t i2 = bz % p.ne2, i3 = bz / p.ne2;
    const char *  X  = p.x + i2 * p.x_nb2 + i3 * p.x_nb3;
    char *        D  = p.dst + i2 * p.d_nb2 + i3 * p.d_nb3;
    const int64_t n0 = (int64_t) bx * 128 + wave * 32;
    const int64_t n  = n0 + (lane & 31);
    const char *  wrow = p.w + (i2 / p.r2) * p.w_nb2 + (i3 / p.r3) * p.w_nb3 + min(n, p.N - 1) * p.w_nb1 + (lane >> 5) * 16;
    const int64_t n_tiles = (p.M + TM - 1) / TM;
    const int64_t t0 = (int64_t) by * tiles_per_wg, t1 = min(t0 + tiles_per_wg, n_tiles);
    if (t0 >= t1) return;

    u32x4 wf[KCH * 8];
#pragma unroll
    for (int i = 0; i < KCH * 8; i++) wf[i] = *(const u32x4 *) (wrow + i * 32);

    // a chunk = 64 rows x 128 k of f32: thread t takes float4 number (t & 31) of rows (t >> 5) + 8 i
    const int srow = threadIdx.x >> 5, sc4 = threadIdx.x & 31;
    float4    st[8];
    auto load_chunk = [&](int64_t tile, int kc) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int64_t m = tile * TM + srow + 8 * i;
            st[i] = m < p.M ? *(const float4 *) (X + m * p.x_nb1 + (int64_t) (kc * MM_KC + sc4 * 4) * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    auto stage_chunk = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            u32x2 v;
            v[0] = pack2<F16>(st[i].x, st[i].y); v[1] = pack2<F16>(st[i].z, st[i].w);
            *(u32x2 *) (lds[buf] + (srow + 8 * i) * MM_PITCH + sc4 * 8) = v;
        }
    };

    f32x16 acc[2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 16; j++) acc[i][j] = 0.f;

    load_chunk(t0, 0);
    stage_chunk(0);
    __syncthreads();
    int buf = 0;
    for (int64_t tile = t0; tile < t1; tile++) {
#pragma unroll
        for (int kc = 0; kc < KCH; kc++) {
            const bool last_kc = kc == KCH - 1;
            const bool more = !last_kc || tile + 1 < t1;
            if (more) load_chunk(last_kc ? tile + 1 : tile, last_kc ? 0 : kc + 1);
#pragma unroll
            for (int ks = 0; ks < 8; ks++)
#pragma unroll
                for (int mb = 0; mb < 2; mb++) {
                    const u32x4 af = *(const u32x4 *) (lds[buf] + (mb * 32 + (lane & 31)) * MM_PITCH + ks * 32 + (lane >> 5) * 16);
                    acc[mb] = mfma32<F16>(af, wf[kc * 8 + ks], acc[mb]);
                }
            if (last_kc) {
                if (vec_store) {
                    // through LDS, so that a row's 128 results leave as one 512-byte run (32 lanes x 16 bytes) instead of
                    // four 128-byte pieces written by four waves at different times
#pragma unroll
                    for (int mb = 0; mb < 2; mb++)
#pragma unroll
                        for (int j = 0; j < 16; j++)
                            obuf[(mb * 32 + (j >> 2) * 8 + (lane >> 5) * 4 + (j & 3)) * OB_PITCH + wave * 32 + (lane & 31)] = acc[mb][j];
                    __syncthreads();
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        const int     r = srow + 8 * i;
                        const int64_t m = tile * TM + r;
                        if (m < p.M) *(float4 *) (D + m * p.d_nb1 + ((int64_t) bx * 128 + sc4 * 4) * 4) = *(const float4 *) (obuf + r * OB_PITCH + sc4 * 4);
                    }
                } else if (n < p.N) {
#pragma unroll
                    for (int mb = 0; mb < 2; mb++)
#pragma unroll
                        for (int j = 0; j < 16; j++) {
                            const int64_t m = tile * TM + mb * 32 + (j >> 2) * 8 + (lane >> 5) * 4 + (j & 3);
                            if (m < p.M) ((float *) (D + m * p.d_nb1))[n] = acc[mb][j];
                        }
                }
#pragma unroll
                for (int mb = 0; mb < 2; mb++)
#pragma unroll
                    for (int j = 0; j < 16; j++) acc[mb][j] = 0.f;
            }
            if (more) stage_chunk(buf ^ 1);
            __syncthreads();
            buf ^= 1;
        }
    }
}

template <bool F16>
hipError_t launch_mm_stream(const MmP & p, int64_t batches, hipStream_t st) {
    const int64_t n_tiles = (p.M + 63) / 64, gx = (p.N + 127) / 128;
    int64_t groups = (1024 + gx * batches - 1) / (gx * batches);   // about four workgroups per CU in total
    if (groups > n_tiles) groups = n_tiles;
    const int  tiles_per_wg = (int) ((n_tiles + groups - 1) / groups);
    const dim3 grid((unsigned) gx, (unsigned) ((n_tiles + tiles_per_wg - 1) / tiles_per_wg), (unsigned) batches);
    switch (p.K / MM_KC) {
        case 1:  hipLaunchKernelGGL((mla_mul_mat_stream_kernel<F16, 1>), grid, dim3(256), 0, st, p, tiles_per_wg); break;
        case 2:  hipLaunchKernelGGL((mla_mul_mat_stream_kernel<F16, 2>), grid, dim3(256), 0, st, p, tiles_per_wg); break;
        default: hipLaunchKernelGGL((mla_mul_mat_stream_kernel<F16, 4>), grid, dim3(256), 0, st, p, tiles_per_wg); break;
    }
    return hipGetLastError();
}

template <typename T>
__global__ void __launch_bounds__(256) mla_copy_kernel(const CopyP p) {
    copy_body<T>(p, Blk{ blockIdx.x, blockIdx.y, blockIdx.z, gridDim.x });
}

// Several independent launches in one dispatch: op i owns the workgroups first[i] .. first[i + 1] - 1 and runs its body
// with the block index it would have had in a grid of its own.  What this buys is the dispatches not made: the nodes
// ahead of the attention node of a decode step are 2 - 20 MB of traffic each, a launch of its own costs such a node 4 - 5
// us from its first wave to the next kernel's, and the chip has room for all of them at once.
enum { B_ROPE = 0, B_MM_SMALL, B_MM_SMALL_F16, B_MM_TILE1, B_MM_TILE1_F16, B_COPY1, B_COPY4,
       B_KVW_BF16, B_KVW_F16, B_KVW_Q8, B_KVW_BF16_ROPE, B_KVW_F16_ROPE, B_KVW_Q8_ROPE, B_KVW_BF16_RAW, B_KVW_Q8_RAW };

struct BatchOp {
    int kind; unsigned gx, gy, gz;
    union { RopeP rope; MmP mm; CopyP copy; WParams kvw; } u;
};
struct BatchP {
    int n;
    unsigned first[MLA_FRONT_BATCH_MAX + 1];   // multiples of 8: every op's first workgroup runs on XCD 0 (xcd_grouped)
    BatchOp op[MLA_FRONT_BATCH_MAX];
};

// LDS: as much as the largest body of the batch needs (given with the launch), so that a batch without the K-split
// product keeps the occupancy of its members
__host__ __device__ constexpr int batch_lds_of(int kind) {
    return kind == B_ROPE ? ROPE_LDS : kind == B_MM_SMALL || kind == B_MM_SMALL_F16 ? MS_LDS : kind == B_MM_TILE1 || kind == B_MM_TILE1_F16 ? MM_LDS<1> : 0;
}

__global__ void __launch_bounds__(256) mla_front_batch_kernel(const BatchP p) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    int i = 0;
    while (i + 1 < p.n && blockIdx.x >= p.first[i + 1]) i++;
    const BatchOp & op = p.op[i];
    const unsigned l = blockIdx.x - p.first[i];
    if (l >= op.gx * op.gy * op.gz) return;   // the padding up to the next op's start
    const Blk b{ l % op.gx, (l / op.gx) % op.gy, l / (op.gx * op.gy), op.gx };
    switch (op.kind) {
        case B_ROPE:          rope_body(op.u.rope, b, lds); break;
        case B_MM_SMALL:      mm_small_body<false>(op.u.mm, xcd_grouped(b, op.gy, op.gz), lds); break;
        case B_MM_SMALL_F16:  mm_small_body<true>(op.u.mm, xcd_grouped(b, op.gy, op.gz), lds); break;
        case B_MM_TILE1:      mm_body<false, 1>(op.u.mm, xcd_grouped(b, op.gy, op.gz), lds); break;
        case B_MM_TILE1_F16:  mm_body<true, 1>(op.u.mm, xcd_grouped(b, op.gy, op.gz), lds); break;
        case B_COPY1:         copy_body<float>(op.u.copy, b); break;
        case B_COPY4:         copy_body<float4>(op.u.copy, b); break;
        case B_KVW_BF16:      kv_write_body<SRC_BF16, true, false>(op.u.kvw, b); break;
        case B_KVW_F16:       kv_write_body<SRC_F16, true, false>(op.u.kvw, b); break;
        case B_KVW_Q8:        kv_write_body<SRC_Q8, true, false>(op.u.kvw, b); break;
        case B_KVW_BF16_ROPE: kv_write_body<SRC_BF16, true, true>(op.u.kvw, b); break;
        case B_KVW_F16_ROPE:  kv_write_body<SRC_F16, true, true>(op.u.kvw, b); break;
        case B_KVW_Q8_ROPE:   kv_write_body<SRC_Q8, true, true>(op.u.kvw, b); break;
        case B_KVW_BF16_RAW:  kv_write_body<SRC_BF16, false, false>(op.u.kvw, b); break;   // (f16 rows are copied the same way)
        default:              kv_write_body<SRC_Q8, false, false>(op.u.kvw, b); break;
    }
}

template <bool F16>
hipError_t launch_mm(const mla_mul_mat_args * a, hipStream_t st) {
    MmP  p;
    dim3 grid;
    switch (make_mm_params(a, &p, &grid)) {
        case MM_STREAM: return launch_mm_stream<F16>(p, a->ne2 * a->ne3, st);
        case MM_SMALL:  hipLaunchKernelGGL((mla_mul_mat_small_kernel<F16>), grid, dim3(256), 0, st, p); break;
        case MM_TILE1:  hipLaunchKernelGGL((mla_mul_mat_kernel<F16, 1>), grid, dim3(256), 0, st, p); break;
        case MM_TILE2:  hipLaunchKernelGGL((mla_mul_mat_kernel<F16, 2>), grid, dim3(256), 0, st, p); break;
        default:        hipLaunchKernelGGL((mla_mul_mat_kernel<F16, 4>), grid, dim3(256), 0, st, p); break;
    }
    return hipGetLastError();
}

int check_op(const mla_front_op & op) {
    if (!op.args) return MLA_ERR_NULL;
    switch (op.kind) {
        case MLA_FRONT_ROPE:          return mla_rope_check((const mla_rope_args *) op.args);
        case MLA_FRONT_MUL_MAT:       return mla_mul_mat_check((const mla_mul_mat_args *) op.args);
        case MLA_FRONT_COPY:          return mla_copy_f32_check((const mla_copy_args *) op.args);
        case MLA_FRONT_KV_WRITE:      return mla_kv_write_check((const mla_kv_write_args *) op.args);
        case MLA_FRONT_KV_WRITE_ROPE: return mla_kv_write_rope_check((const mla_kv_write_rope_args *) op.args);
        default:                      return MLA_ERR_BAD_TYPE;
    }
}

int launch_alone(const mla_front_op & op, void * stream) {
    switch (op.kind) {
        case MLA_FRONT_ROPE:          return mla_rope_launch((const mla_rope_args *) op.args, stream);
        case MLA_FRONT_MUL_MAT:       return mla_mul_mat_launch((const mla_mul_mat_args *) op.args, stream);
        case MLA_FRONT_COPY:          return mla_copy_f32_launch((const mla_copy_args *) op.args, stream);
        case MLA_FRONT_KV_WRITE:      return mla_kv_write_launch((const mla_kv_write_args *) op.args, stream);
        default:                      return mla_kv_write_rope_launch((const mla_kv_write_rope_args *) op.args, stream);
    }
}

// Fills `b` when the op has a body in the batch kernel; 0: it has none (a launch of its own); -1: nothing to do.
int make_batch_op(const mla_front_op & op, BatchOp * b) {
    dim3 grid(0, 1, 1);
    switch (op.kind) {
        case MLA_FRONT_ROPE: {
            const mla_rope_args * a = (const mla_rope_args *) op.args;
            if (a->ne[0] * a->ne[1] * a->ne[2] * a->ne[3] == 0) return -1;
            grid = make_rope_params(a, &b->u.rope);
            b->kind = B_ROPE;
            break;
        }
        case MLA_FRONT_MUL_MAT: {
            const mla_mul_mat_args * a = (const mla_mul_mat_args *) op.args;
            if (a->N * a->M * a->ne2 * a->ne3 == 0) return -1;
            const bool f16 = a->w_type == MLA_TYPE_F16;
            switch (make_mm_params(a, &b->u.mm, &grid)) {
                case MM_SMALL: b->kind = f16 ? B_MM_SMALL_F16 : B_MM_SMALL; break;
                case MM_TILE1: b->kind = f16 ? B_MM_TILE1_F16 : B_MM_TILE1; break;
                default: return 0;
            }
            break;
        }
        case MLA_FRONT_COPY: {
            const mla_copy_args * a = (const mla_copy_args *) op.args;
            if (a->ne[0] * a->ne[1] * a->ne[2] * a->ne[3] == 0) return -1;
            b->kind = make_copy_params(a, &b->u.copy, &grid) ? B_COPY4 : B_COPY1;
            break;
        }
        case MLA_FRONT_KV_WRITE: {
            const mla_kv_write_args * a = (const mla_kv_write_args *) op.args;
            if (a->n_tok == 0) return -1;
            grid = make_kv_write_params(a, &b->u.kvw);
            if (a->src_type == MLA_TYPE_F32) b->kind = a->kv_type == MLA_TYPE_BF16 ? B_KVW_BF16 : a->kv_type == MLA_TYPE_F16 ? B_KVW_F16 : B_KVW_Q8;
            else                             b->kind = a->kv_type == MLA_TYPE_Q8_0 ? B_KVW_Q8_RAW : B_KVW_BF16_RAW;
            break;
        }
        default: {
            const mla_kv_write_rope_args * a = (const mla_kv_write_rope_args *) op.args;
            if (a->w.n_tok == 0) return -1;
            grid = make_kv_write_rope_params(a, &b->u.kvw);
            b->kind = a->w.kv_type == MLA_TYPE_BF16 ? B_KVW_BF16_ROPE : a->w.kv_type == MLA_TYPE_F16 ? B_KVW_F16_ROPE : B_KVW_Q8_ROPE;
            break;
        }
    }
    b->gx = grid.x; b->gy = grid.y; b->gz = grid.z;
    return 1;
}

}  // namespace

extern "C" int mla_rope_check(const mla_rope_args * a) {
    if (!a) return MLA_ERR_NULL;
    for (int i = 0; i < 4; i++) if (a->ne[i] < 0) return MLA_ERR_BAD_SHAPE;
    if (a->n_dims <= 0 || (a->n_dims & 1) || a->n_dims > a->ne[0] || a->n_dims > 2 * ROPE_MAX_PAIRS) return MLA_ERR_BAD_SHAPE;
    if (a->mode != MLA_ROPE_MODE_NORM && a->mode != MLA_ROPE_MODE_NEOX) return MLA_ERR_UNSUPPORTED;
    if (a->src_nb[0] != 4 || a->dst_nb[0] != 4) return MLA_ERR_BAD_SHAPE;
    if (a->ne[0] * a->ne[1] * a->ne[2] * a->ne[3] == 0) return 0;
    if (!a->src || !a->dst || !a->pos) return MLA_ERR_NULL;
    if (a->ne[2] > 65535 || a->ne[3] > 65535) return MLA_ERR_BAD_SHAPE;
    for (int i = 1; i < 4; i++) if ((a->src_nb[i] & 3) || (a->dst_nb[i] & 3)) return MLA_ERR_BAD_ALIGNMENT;
    if (((uintptr_t) a->src & 3) || ((uintptr_t) a->dst & 3)) return MLA_ERR_BAD_ALIGNMENT;
    return 0;
}

extern "C" int mla_rope_launch(const mla_rope_args * a, void * stream) {
    const int rc = mla_rope_check(a);
    if (rc) return rc;
    if (a->ne[0] * a->ne[1] * a->ne[2] * a->ne[3] == 0) return 0;
    RopeP p;
    const dim3 grid = make_rope_params(a, &p);
    hipLaunchKernelGGL(mla_rope_kernel, grid, dim3(256), 0, (hipStream_t) stream, p);
    return (int) hipGetLastError();
}

extern "C" int mla_mul_mat_check(const mla_mul_mat_args * a) {
    if (!a) return MLA_ERR_NULL;
    if (a->w_type != MLA_TYPE_F16 && a->w_type != MLA_TYPE_BF16) return MLA_ERR_BAD_TYPE;
    if (a->K < 0 || a->N < 0 || a->M < 0 || a->w_ne2 < 1 || a->w_ne3 < 1 || a->ne2 < 0 || a->ne3 < 0) return MLA_ERR_BAD_SHAPE;
    if (a->ne2 % a->w_ne2 || a->ne3 % a->w_ne3) return MLA_ERR_BAD_SHAPE;
    if (a->N * a->M * a->ne2 * a->ne3 == 0) return 0;
    if (a->K < 16 || a->K % 16) return MLA_ERR_UNSUPPORTED;
    if (!a->w || !a->x || !a->dst) return MLA_ERR_NULL;
    if (a->ne2 * a->ne3 > 65535 || (a->M + 31) / 32 > 65535) return MLA_ERR_BAD_SHAPE;
    if (!al16(a->w) || !al16(a->x) || (a->w_nb1 & 15) || (a->w_nb2 & 15) || (a->w_nb3 & 15) || (a->x_nb1 & 15) || (a->x_nb2 & 15) ||
        (a->x_nb3 & 15) || ((uintptr_t) a->dst & 3) || (a->d_nb1 & 3) || (a->d_nb2 & 3) || (a->d_nb3 & 3))
        return MLA_ERR_BAD_ALIGNMENT;
    if (a->w_nb1 < a->K * 2 || a->x_nb1 < a->K * 4 || a->d_nb1 < a->N * 4) return MLA_ERR_BAD_SHAPE;
    return 0;
}

extern "C" int mla_mul_mat_launch(const mla_mul_mat_args * a, void * stream) {
    const int rc = mla_mul_mat_check(a);
    if (rc) return rc;
    if (a->N * a->M * a->ne2 * a->ne3 == 0) return 0;
    const hipError_t e = a->w_type == MLA_TYPE_F16 ? launch_mm<true>(a, (hipStream_t) stream) : launch_mm<false>(a, (hipStream_t) stream);
    return (int) e;
}

extern "C" int mla_copy_f32_check(const mla_copy_args * a) {
    if (!a) return MLA_ERR_NULL;
    for (int i = 0; i < 4; i++) if (a->ne[i] < 0) return MLA_ERR_BAD_SHAPE;
    if (a->src_nb[0] != 4 || a->dst_nb[0] != 4) return MLA_ERR_BAD_SHAPE;
    if (a->ne[0] * a->ne[1] * a->ne[2] * a->ne[3] == 0) return 0;
    if (!a->src || !a->dst) return MLA_ERR_NULL;
    for (int i = 1; i < 4; i++) if ((a->src_nb[i] & 3) || (a->dst_nb[i] & 3)) return MLA_ERR_BAD_ALIGNMENT;
    if (((uintptr_t) a->src & 3) || ((uintptr_t) a->dst & 3)) return MLA_ERR_BAD_ALIGNMENT;
    return 0;
}

extern "C" int mla_copy_f32_launch(const mla_copy_args * a, void * stream) {
    const int rc = mla_copy_f32_check(a);
    if (rc) return rc;
    if (a->ne[0] * a->ne[1] * a->ne[2] * a->ne[3] == 0) return 0;
    CopyP p;
    dim3  grid;
    if (make_copy_params(a, &p, &grid)) hipLaunchKernelGGL(mla_copy_kernel<float4>, grid, dim3(256), 0, (hipStream_t) stream, p);
    else                                hipLaunchKernelGGL(mla_copy_kernel<float>, grid, dim3(256), 0, (hipStream_t) stream, p);
    return (int) hipGetLastError();
}

extern "C" int mla_front_batch_check(const mla_front_op * ops, int32_t n_ops) {
    if (n_ops < 0) return MLA_ERR_BAD_SHAPE;
    if (n_ops && !ops) return MLA_ERR_NULL;
    for (int i = 0; i < n_ops; i++) {
        const int rc = check_op(ops[i]);
        if (rc) return rc;
    }
    return 0;
}

extern "C" int mla_front_batch_launch(const mla_front_op * ops, int32_t n_ops, void * stream) {
    const int rc = mla_front_batch_check(ops, n_ops);   // all of them, before anything is launched
    if (rc) return rc;
    BatchP p;
    p.n = 0; p.first[0] = 0;
    auto flush = [&]() -> int {
        if (p.n == 0) return 0;
        int lds = 0;
        for (int i = 0; i < p.n; i++) lds = batch_lds_of(p.op[i].kind) > lds ? batch_lds_of(p.op[i].kind) : lds;
        hipLaunchKernelGGL(mla_front_batch_kernel, dim3(p.first[p.n]), dim3(256), lds, (hipStream_t) stream, p);
        p.n = 0;
        return (int) hipGetLastError();
    };
    // the products last: the short ops are chains of latencies (a table of angles, a barrier, one pass over a few rows) that
    // the product's workgroups, dispatched behind them, cover (a layer's decode step: 1.6 us less than products first)
    for (int pass = 0; pass < 2; pass++)
        for (int i = 0; i < n_ops; i++) {
            if ((ops[i].kind == MLA_FRONT_MUL_MAT) != (pass == 1)) continue;
            const int has = make_batch_op(ops[i], &p.op[p.n]);
            if (has < 0) continue;
            if (has == 0) {
                const int e = launch_alone(ops[i], stream);
                if (e) return e;
                continue;
            }
            const BatchOp & b = p.op[p.n];
            p.first[p.n + 1] = p.first[p.n] + ((b.gx * b.gy * b.gz + 7u) & ~7u);
            if (++p.n == MLA_FRONT_BATCH_MAX) {
                const int e = flush();
                if (e) return e;
            }
        }
    return flush();
}
