// Pipelined split-K flash-decode kernel for the common MLA decode shape on gfx950:
// bf16 or f16 latent KV rows of 576 (V = first 512 columns), no mask / ALiBi / softcap, any number of rows
// (query token x head pairs) in blocks of 128 per workgroup.
//
// One workgroup = 4 waves = 128 rows x one KV split.  Per 32-token tile:
//   KV tile:  HBM -> LDS directly (global_load_lds_dwordx4, no registers), three tiles in flight/resident
//   S^T = K.Q^T   36 x v_mfma_f32_32x32x16 (K fragment ds_read_b128, Q resident in 144 VGPRs)
//   softmax       on the accumulator layout, running max kept lazily (rescale only when it grows by > 2^TAU)
//   O^T += V^T.P^T  16 d-blocks x 2 k-steps, V^T fragments by ds_read_b64_tr_b16 from the same row-major tile;
//                 for bf16, P is fed as hi + lo bf16 halves (two MFMAs per fragment) so that the product keeps
//                 ~16 mantissa bits of P -- a single bf16 P would leave a 1.7e-3 relative L2 error.
// The QK^T of tile i+1 is issued interleaved with the softmax of tile i so the VALU work hides under MFMA time.
// Rows past the end of a sequence inside the last tile are loaded as copies of the last valid row (finite data)
// and get probability exactly 0.

#include "mla_common.hpp"

namespace mla {
namespace {

constexpr int   NBUF           = 3;
constexpr int   CHUNKS_PER_ROW = PITCH / 16;                // 73: 72 data chunks + 1 pad chunk
constexpr int   TILE_CHUNKS    = TILE_TOK * CHUNKS_PER_ROW; // 2336
constexpr int   N_DMA          = (TILE_CHUNKS + NTHREADS - 1) / NTHREADS;  // 10 issue slots per thread, the last partial
constexpr float TAU            = 8.0f;  // lazy-rescale threshold in log2 units: probabilities stay below 2^8

typedef __attribute__((ext_vector_type(2))) float    f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16   bf16x2;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;

template <bool F16> __device__ __forceinline__ unsigned int cvt_pk(float a, float b) {
    if constexpr (F16) return bitcast<unsigned int>(__builtin_convertvector(f32x2{ a, b }, f16x2));
    else               return bitcast<unsigned int>(__builtin_convertvector(f32x2{ a, b }, bf16x2));
}

// max over the two lanes that share an attention row (lanes l and l^32)
__device__ __forceinline__ float pair_max(float v) {
    typedef __attribute__((ext_vector_type(2))) unsigned int u2;
    const unsigned int x = __float_as_uint(v);
    const u2 r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    return fmaxf(__uint_as_float(r.x), __uint_as_float(r.y));
}
__device__ __forceinline__ float pair_sum(float v) {
    typedef __attribute__((ext_vector_type(2))) unsigned int u2;
    const unsigned int x = __float_as_uint(v);
    const u2 r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    return __uint_as_float(r.x) + __uint_as_float(r.y);
}

template <bool F16>
__global__ void __launch_bounds__(NTHREADS) mla_decode_kernel(const KParams p) {
    constexpr bool SPLIT = !F16;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];  // [NBUF][TILE_BYTES]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 5, rl = lane & 31;
    const int b = blockIdx.z, split = blockIdx.x;

    const int seq_len  = p.block_table ? min(p.seq_lens[b], (int) p.bt_stride * MLA_PAGE_TOKENS) : (int) p.n_kv;
    const int kv_begin = split * p.split_tokens;
    const int kv_end   = min(seq_len, kv_begin + p.split_tokens);
    if (kv_begin >= kv_end && !(seq_len <= 0 && split == 0)) return;
    const int n_tiles = (kv_end - kv_begin + TILE_TOK - 1) / TILE_TOK;

    const int  row       = blockIdx.y * 128 + wave * 32 + rl;
    const bool row_valid = row < p.n_rows;
    const int  rowc      = row_valid ? row : p.n_rows - 1;
    const int  tq        = rowc / p.n_head;
    const int  head      = rowc - tq * p.n_head;

    // ---- KV tile: HBM -> LDS with the LDS-DMA form of the global load (no VGPR data path).
    // Chunk c of the padded tile image lives at LDS byte 16*c; it is row c/73, 16-byte column c%73 (column 72 = pad,
    // filled with a harmless copy of column 71).  Issue slot j of this thread moves chunk j*256 + tid; within a
    // wave the 64 chunks of a slot are contiguous in LDS (base in M0, lane i at +16*i), as that load form requires.
    // The loads are issued from inline asm on purpose: the compiler then does not serialise later LDS reads behind
    // them; completion is awaited explicitly (vmcnt(0) + workgroup barrier) before a tile is first read.
    const int c0_row = tid / CHUNKS_PER_ROW, c0_col = tid - c0_row * CHUNKS_PER_ROW;
    auto dma_tile = [&](int it, int buf_off) {
        const int t0     = kv_begin + it * TILE_TOK;
        const int nvalid = min(TILE_TOK, kv_end - t0);
        const char * base;
        if (p.block_table) {
            int page = p.block_table[(int64_t) b * p.bt_stride + (t0 >> 7)];
            page     = max(0, min(page, p.n_pool_pages - 1));
            base     = p.kv + ((int64_t) page * MLA_PAGE_TOKENS + (t0 & 127)) * p.kv_nb1;
        } else {
            base = p.kv + (int64_t) t0 * p.kv_nb1 + (int64_t) b * p.kv_nb3;
        }
        int r = c0_row, col = c0_col;
        const unsigned lds0 = (unsigned) (uintptr_t) (LDS_PTR(unsigned char)) (smem + buf_off) + wave * 1024;
#pragma unroll
        for (int j = 0; j < N_DMA; j++) {
            if (j * NTHREADS + tid < TILE_CHUNKS) {
                const char * gp = base + (int64_t) min(r, nvalid - 1) * p.kv_nb1 + min(col, CHUNKS_PER_ROW - 2) * 16;
                const unsigned m0v = __builtin_amdgcn_readfirstlane(lds0 + j * NTHREADS * 16);
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gp), "s"(m0v) : "memory");
            }
            // chunk index advances by 256 = 3 rows + 37 chunks
            col += NTHREADS - 3 * CHUNKS_PER_ROW;
            r += 3;
            if (col >= CHUNKS_PER_ROW) { col -= CHUNKS_PER_ROW; r += 1; }
        }
    };

    // ---- Q -> registers (MFMA B layout), rounded to the KV type as ggml-cpu rounds it (ggml-cpu.c:12034-12035)
    u32x4 qreg[KSTEPS];
    {
        const float * qrow = (const float *) (p.q + (int64_t) tq * p.q_nb1 + (int64_t) head * p.q_nb2 + (int64_t) b * p.q_nb3);
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ks++) {
            const f32x4 x0 = *(const f32x4 *) (qrow + 16 * ks + 8 * g);
            const f32x4 x1 = *(const f32x4 *) (qrow + 16 * ks + 8 * g + 4);
            qreg[ks] = u32x4{ cvt_pk<F16>(x0.x, x0.y), cvt_pk<F16>(x0.z, x0.w), cvt_pk<F16>(x1.x, x1.y), cvt_pk<F16>(x1.z, x1.w) };
        }
    }

    f32x16 acc[16];
#pragma unroll
    for (int i = 0; i < 16; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[i][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    const float c_log2 = p.scale * LOG2E;  // > 0 (checked on the host)

    const int k_off = rl * PITCH + g * 16;
    const int v_off = (4 * g + ((lane & 15) >> 2)) * PITCH + (((lane >> 4) & 1) * 16 + (lane & 3) * 4) * 2;

    auto qk = [&](int buf_off) -> f32x16 {
        f32x16 s;
#pragma unroll
        for (int e = 0; e < 16; e++) s[e] = 0.f;
        const unsigned char * tile = smem + buf_off;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ks++) {
            const u32x4 a = *(LDS_PTR(const u32x4)) (tile + k_off + ks * 32);
            s = mfma32<F16>(a, qreg[ks], s);
        }
        return s;
    };

    // softmax of one tile's scores; leaves P^T (hi, lo) in MFMA B layout.  n_valid < 32 only for the last tile.
    u32x4 p_hi[2], p_lo[2];
    auto softmax = [&](f32x16 & s, int n_valid) {
        if (n_valid < TILE_TOK) {
#pragma unroll
            for (int e = 0; e < 16; e++)
                if (8 * (e >> 2) + 4 * g + (e & 3) >= n_valid) s[e] = -INFINITY;
        }
        float tmax = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
        tmax = fmaxf(tmax, fmaxf(fmaxf(fmaxf(s[8], s[9]), fmaxf(s[10], s[11])), fmaxf(fmaxf(s[12], s[13]), fmaxf(s[14], s[15]))));
        tmax = pair_max(tmax) * c_log2;
        if (__any(tmax > m_run + TAU)) {
            const float m_new = fmaxf(m_run, tmax);
            const float alpha = (m_run == -INFINITY) ? 0.f : fast_exp2(m_run - m_new);
#pragma unroll
            for (int i = 0; i < 16; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[i][e] *= alpha;
            l_run *= alpha;
            m_run = m_new;
        }
        const float neg_m = (m_run == -INFINITY) ? 0.f : -m_run;
        float lsum = 0.f;
#pragma unroll
        for (int e = 0; e < 16; e++) {
            s[e] = fast_exp2(fmaf(s[e], c_log2, neg_m));
            lsum += s[e];
        }
        l_run += lsum;
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            unsigned int h[4];
#pragma unroll
            for (int j = 0; j < 4; j++) h[j] = cvt_pk<F16>(s[8 * kk + 2 * j], s[8 * kk + 2 * j + 1]);
            p_hi[kk] = u32x4{ h[0], h[1], h[2], h[3] };
            if constexpr (SPLIT) {
                unsigned int l[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float r0 = s[8 * kk + 2 * j] - __uint_as_float(h[j] << 16);
                    const float r1 = s[8 * kk + 2 * j + 1] - __uint_as_float(h[j] & 0xffff0000u);
                    l[j] = cvt_pk<F16>(r0, r1);
                }
                p_lo[kk] = u32x4{ l[0], l[1], l[2], l[3] };
            }
        }
    };

    auto pv = [&](int buf_off) {
        const unsigned char * tile = smem + buf_off + v_off;
#pragma unroll
        for (int i = 0; i < 16; i++) {
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
                const unsigned char * vp = tile + (16 * kk) * PITCH + i * 64;
                const u32x2 a0 = bitcast<u32x2>(__builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4)) (vp)));
                const u32x2 a1 = bitcast<u32x2>(__builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4)) (vp + 8 * PITCH)));
                const u32x4 a  = { a0.x, a0.y, a1.x, a1.y };
                acc[i] = mfma32<F16>(a, p_hi[kk], acc[i]);
                if constexpr (SPLIT) acc[i] = mfma32<F16>(a, p_lo[kk], acc[i]);
            }
        }
    };

    auto wait_tiles = [&]() {
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's LDS-DMA writes have landed
        __syncthreads();
    };

    // ---- pipeline
    int off0 = 0, off1 = TILE_BYTES, off2 = 2 * TILE_BYTES;  // LDS offsets of tiles it, it+1, it+2
    f32x16 s_cur;
    if (n_tiles > 0) {
        dma_tile(0, off0);
        if (n_tiles > 1) dma_tile(1, off1);
        wait_tiles();
        s_cur = qk(off0);
    }
    for (int it = 0; it < n_tiles; it++) {
        const int n_valid = min(TILE_TOK, kv_end - (kv_begin + it * TILE_TOK));
        if (it + 2 < n_tiles) dma_tile(it + 2, off2);
        // QK^T of the next tile (for the last tile this reads a stale buffer and the result is dropped)
        f32x16 s_next = qk(off1);
        softmax(s_cur, n_valid);
        pv(off0);
        s_cur = s_next;
        const int t = off0; off0 = off1; off1 = off2; off2 = t;
        wait_tiles();
    }

    // ---- epilogue
    const float l_tot = pair_sum(l_run);
    if (!row_valid) return;
    if (p.n_splits == 1) {
        const float inv = 1.0f / l_tot;
        float * o = p.dst + ((int64_t) b * p.n_rows + row) * p.dst_stride;
#pragma unroll
        for (int i = 0; i < 16; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                *(f32x4 *) (o + i * 32 + 8 * j + 4 * g) = f32x4{ acc[i][4 * j] * inv, acc[i][4 * j + 1] * inv, acc[i][4 * j + 2] * inv, acc[i][4 * j + 3] * inv };
    } else {
        const int64_t prow = ((int64_t) b * p.n_splits + split) * p.n_rows + row;
        float * o = p.part_o + prow * p.dv_total;
#pragma unroll
        for (int i = 0; i < 16; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                *(f32x4 *) (o + i * 32 + 8 * j + 4 * g) = f32x4{ acc[i][4 * j], acc[i][4 * j + 1], acc[i][4 * j + 2], acc[i][4 * j + 3] };
        if (g == 0) {
            p.part_ml[prow * 2]     = m_run;
            p.part_ml[prow * 2 + 1] = l_tot;
        }
    }
}

}  // namespace

size_t decode_fast_lds_bytes() { return (size_t) NBUF * TILE_BYTES; }

bool decode_fast_applicable(const mla_attn_args * a) {
    if (a->kv_type != MLA_TYPE_BF16 && a->kv_type != MLA_TYPE_F16) return false;
    if (a->dv != 512 || (a->flags & MLA_FLAG_F16_ACC_STRICT)) return false;
    if (a->mask || a->logit_softcap != 0.0f || a->max_bias > 0.0f) return false;
    if (!(a->scale > 0.0f) || !(a->scale < INFINITY)) return false;
    if ((int64_t) a->n_tok * a->n_head <= 64) return false;  // few rows: the general kernel's d-split wave layout wastes less
    return true;
}

hipError_t launch_decode_fast(const KParams & kp, int kv_type, dim3 grid, hipStream_t st) {
    const size_t lds = decode_fast_lds_bytes();
    static bool  attr_done[2] = { false, false };
    const int    v = kv_type == MLA_TYPE_F16 ? 1 : 0;
    const void * fn = v ? (const void *) mla_decode_kernel<true> : (const void *) mla_decode_kernel<false>;
    if (!attr_done[v]) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        attr_done[v] = true;
    }
    if (v) hipLaunchKernelGGL(mla_decode_kernel<true>, grid, dim3(NTHREADS), lds, st, kp);
    else   hipLaunchKernelGGL(mla_decode_kernel<false>, grid, dim3(NTHREADS), lds, st, kp);
    return hipGetLastError();
}

}  // namespace mla
