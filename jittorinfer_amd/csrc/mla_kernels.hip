// Absorbed-MLA attention for gfx950 (MI355X): hand-written HIP kernels behind the C ABI of include/mla_attn.h.
//
// The op is GGML_OP_FLASH_ATTN_EXT as ggml-cpu computes it (ggml/src/ggml-cpu/ggml-cpu.c:11914-12124 of the
// reference) specialised to what llm_attn_mla feeds it (src/llama-graph-attn.cpp:259-315): Q rows of 576,
// one latent K row of 576 per cached token shared by every head, V = the first 512 (or all 576) columns of
// the same row.  A "row" below is one (query token, head) pair; all rows of a sequence read the same KV rows.
//
// Data flow of the tiled kernel (mla_attn_tile_kernel):
//   HBM --16-byte coalesced loads (through the block table)--> registers --(dequant)--> LDS tile [32 tokens][576]
//   S^T[token, row]  = K_tile . Q^T      v_mfma_f32_32x32x16_{bf16,f16}, K from LDS (ds_read_b128), Q in VGPRs
//   online softmax on S^T in its accumulator layout (one row per lane pair, exchange across lanes 32 apart)
//   O^T[d, row]     += V_tile^T . P^T    same MFMA; V^T fragments come from the SAME row-major LDS tile through
//                                        ds_read_b64_tr_b16, P^T is the S^T accumulator re-packed in registers
// so a KV tile is read from HBM once per workgroup and serves every head the workgroup owns.
// Split-K partials (unnormalised O, running max, running sum) go to the workspace and are merged by
// mla_attn_combine_kernel with the usual log-sum-exp rule.
//
// gfx950 only: v_mfma_f32_32x32x16_*, ds_read_b64_tr_b16, 160 KB LDS, 64-wide waves.

#include <atomic>
#include "mla_common.hpp"
#include <string.h>
#include <algorithm>
#include <stdlib.h>

using namespace mla;

namespace {

// ---------------------------------------------------------------------------------------------------------------
// Tiled MFMA kernel.
//   SRC  : storage type of the KV rows
//   NDB  : number of 32-wide d blocks of the output this launch produces (16 -> 512 columns, 9 -> 288 columns)
//   WM   : waves along rows (each wave owns 32 rows); WD: waves along d (each owns NDB/WD blocks); WM*WD == 4
// grid = (n_splits, n_row_blocks, n_seq), block = 256.
// ---------------------------------------------------------------------------------------------------------------
template <int SRC, int NDB, int WM, int WD>
__global__ void __launch_bounds__(NTHREADS) mla_attn_tile_kernel(const KParams p) {
    constexpr bool F16   = (SRC != SRC_BF16);  // LDS element type: f16 for f16 and Q8_0 sources, bf16 for bf16
    constexpr bool SPLIT = !F16;               // bf16 P is split into hi + lo so that P.V keeps ~16 mantissa bits
    constexpr int  NDBW  = NDB / WD;
    constexpr int  RBLK  = 32 * WM;
    static_assert(WM * WD == 4 && NDB % WD == 0, "wave layout");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // smem: [2][TILE_BYTES] tile double buffer, then (Q8 only) [Q8_TILE_RAW] raw staging

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm   = wave / WD;
    const int wd   = wave % WD;
    const int g    = lane >> 5;  // which half of the k-slots this lane feeds
    const int rl   = lane & 31;  // MFMA column: the attention row this lane owns
    const int b    = blockIdx.z;
    const int split = blockIdx.x;

    const int seq_len  = p.block_table ? min(p.seq_lens[b], (int) p.bt_stride * MLA_PAGE_TOKENS) : (int) p.n_kv;
    int kv_begin = split * p.split_tokens;
    int kv_end   = min(seq_len, kv_begin + p.split_tokens);
    if (p.mask_ext) {
        // only the keys that the mask leaves open for some row of this block (16 (first, one past the last) pairs per 128
        // rows from mla_mask_extent_kernel, rounded outwards to tiles), and the KV splits divide that range, not the
        // cache.  A split left without keys runs no tile and its (m, l) = (-inf, 0) tells the combine pass so; with one
        // split the rows then come out NaN like the reference's.
        int mlo = 0x7fffffff, mhi = 0;
        const int eb = blockIdx.y * RBLK / 128;
        for (int c = 0; c < 16; c++) {
            mlo = min(mlo, p.mask_ext[(eb * 16 + c) * 2]);
            mhi = max(mhi, p.mask_ext[(eb * 16 + c) * 2 + 1]);
        }
        const int hi = min(seq_len, (mhi + TILE_TOK - 1) / TILE_TOK * TILE_TOK), lo = min(mlo / TILE_TOK * TILE_TOK, hi);
        const int chunk = ((hi - lo + p.n_splits - 1) / p.n_splits + TILE_TOK - 1) / TILE_TOK * TILE_TOK;
        kv_begin = min(hi, lo + split * chunk);
        kv_end   = min(hi, kv_begin + chunk);
    } else if (kv_begin >= kv_end && !(seq_len <= 0 && split == 0)) return;  // nothing to do; the combine pass knows

    const int  row       = blockIdx.y * RBLK + wm * 32 + rl;
    const bool row_valid = row < p.n_rows;
    const int  rowc      = row_valid ? row : p.n_rows - 1;
    const int  tq        = rowc / p.n_head;  // query token of this row
    const int  head      = rowc - tq * p.n_head;

    // ---- Q -> registers in MFMA B layout: k-step ks holds d = 16*ks + 8*g .. +7 of row `rl`
    u32x4 qreg[KSTEPS];
    {
        const float * qrow = (const float *) (p.q + (int64_t) tq * p.q_nb1 + (int64_t) head * p.q_nb2 + (int64_t) b * p.q_nb3);
        if constexpr (SRC == SRC_Q8) {
            // ggml-cpu quantizes Q to Q8_0 when K is Q8_0 (ggml-cpu.c:313-322, :12034-12035): per 32-block
            // d = amax/127 (stored as f16), id = 127/amax, q = round-half-even(x*id) (ggml-cpu-quants.c:855-900).
            // The MFMA operand is the dequantized value q * f16(d), rounded to f16.
#pragma unroll
            for (int j = 0; j < KSTEPS / 2; j++) {
                f32x4 x[4];
                x[0] = *(const f32x4 *) (qrow + 32 * j + 8 * g);
                x[1] = *(const f32x4 *) (qrow + 32 * j + 8 * g + 4);
                x[2] = *(const f32x4 *) (qrow + 32 * j + 16 + 8 * g);
                x[3] = *(const f32x4 *) (qrow + 32 * j + 16 + 8 * g + 4);
                float amax = 0.f;
#pragma unroll
                for (int e = 0; e < 4; e++)
#pragma unroll
                    for (int c = 0; c < 4; c++) amax = fmaxf(amax, fabsf(x[e][c]));
                amax           = fmaxf(amax, xor32(amax));
                const float d  = f16_bits_to_f32(f32_to_f16_bits(amax / 127.0f));
                const float id = amax != 0.f ? 127.0f / amax : 0.f;
                float y[16];
#pragma unroll
                for (int e = 0; e < 4; e++)
#pragma unroll
                    for (int c = 0; c < 4; c++) y[e * 4 + c] = rintf(x[e][c] * id) * d;
                u32x4 lo, hi;
                lo.x = pack2<true>(y[0], y[1]);   lo.y = pack2<true>(y[2], y[3]);
                lo.z = pack2<true>(y[4], y[5]);   lo.w = pack2<true>(y[6], y[7]);
                hi.x = pack2<true>(y[8], y[9]);   hi.y = pack2<true>(y[10], y[11]);
                hi.z = pack2<true>(y[12], y[13]); hi.w = pack2<true>(y[14], y[15]);
                qreg[2 * j]     = lo;
                qreg[2 * j + 1] = hi;
            }
        } else {
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ks++) {
                const f32x4 x0 = *(const f32x4 *) (qrow + 16 * ks + 8 * g);
                const f32x4 x1 = *(const f32x4 *) (qrow + 16 * ks + 8 * g + 4);
                u32x4 v;
                v.x = pack2<F16>(x0.x, x0.y); v.y = pack2<F16>(x0.z, x0.w);
                v.z = pack2<F16>(x1.x, x1.y); v.w = pack2<F16>(x1.z, x1.w);
                qreg[ks] = v;
            }
        }
    }

    // ALiBi slope of this row's head (ggml-cpu.c:11985-11989, :12006-12008); 1 when max_bias == 0
    float slope = 1.0f;
    if (p.max_bias > 0.0f) {
        slope = head < p.n_head_log2 ? powf(p.m0, (float) (head + 1)) : powf(p.m1, (float) (2 * (head - p.n_head_log2) + 1));
    }
    const float scale_eff = p.softcap != 0.0f ? p.scale / p.softcap : p.scale;
    const char * mask_row = p.mask ? p.mask + (int64_t) tq * p.mask_nb1 : nullptr;

    f32x16 acc[NDBW];
#pragma unroll
    for (int i = 0; i < NDBW; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[i][e] = 0.f;
    float m_run = -INFINITY;  // running max, log2 units
    float l_run = 0.f;        // running sum (this lane's 16 of the 32 tokens of each tile)

    const int n_tiles = (kv_end - kv_begin + TILE_TOK - 1) / TILE_TOK;

    // ---- staging: global -> registers -> LDS
    constexpr int N_PRE = (SRC == SRC_Q8) ? (Q8_TILE_RAW / 16 + NTHREADS - 1) / NTHREADS : (TILE_TOK * (ROW_BYTES / 16)) / NTHREADS;  // 5 or 9
    u32x4 pre[N_PRE];

    auto tile_row_ptr = [&](int ic) -> const char * {  // address of logical KV row ic of this sequence
        if (p.block_table) {
            int page = p.block_table[(int64_t) b * p.bt_stride + (ic >> 7)];
            page = max(0, min(page, p.n_pool_pages - 1));  // a corrupt table must not turn into a wild address
            return p.kv + ((int64_t) page * MLA_PAGE_TOKENS + (ic & 127)) * p.kv_nb1;
        }
        return p.kv + (int64_t) ic * p.kv_nb1 + (int64_t) b * p.kv_nb3;
    };

    auto prefetch = [&](int it) {
        const int t0   = kv_begin + it * TILE_TOK;
        const int nrow = min(TILE_TOK, kv_end - t0);
        if constexpr (SRC == SRC_Q8) {
            if (p.rows_contig && nrow == TILE_TOK) {
                const char * base = tile_row_ptr(t0);
#pragma unroll
                for (int j = 0; j < N_PRE; j++) {
                    const int c = tid + j * NTHREADS;
                    if (c < Q8_TILE_RAW / 16) pre[j] = *(const u32x4 *) (base + (int64_t) c * 16);
                }
            } else {
                // generic: 2-byte granules, row by row (rows are only 2-byte aligned); zero past the end
#pragma unroll
                for (int j = 0; j < N_PRE; j++) {
                    const int c = tid + j * NTHREADS;
                    unsigned short h[8];
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        const int off = c * 16 + e * 2;
                        const int r   = off / Q8_ROW;
                        unsigned short v = 0;
                        if (c < Q8_TILE_RAW / 16 && r < nrow) v = *(const unsigned short *) (tile_row_ptr(t0 + r) + (off - r * Q8_ROW));
                        h[e] = v;
                    }
                    u32x4 v;
                    v.x = h[0] | ((unsigned) h[1] << 16); v.y = h[2] | ((unsigned) h[3] << 16);
                    v.z = h[4] | ((unsigned) h[5] << 16); v.w = h[6] | ((unsigned) h[7] << 16);
                    pre[j] = v;
                }
            }
        } else {
            if (p.rows_contig && nrow == TILE_TOK) {
                const char * base = tile_row_ptr(t0);
#pragma unroll
                for (int j = 0; j < N_PRE; j++) pre[j] = *(const u32x4 *) (base + (int64_t) (tid + j * NTHREADS) * 16);
            } else {
#pragma unroll
                for (int j = 0; j < N_PRE; j++) {
                    const int c   = tid + j * NTHREADS;
                    const int r   = c / (ROW_BYTES / 16);
                    const int col = c - r * (ROW_BYTES / 16);
                    u32x4 v = { 0u, 0u, 0u, 0u };
                    if (r < nrow) v = *(const u32x4 *) (tile_row_ptr(t0 + r) + col * 16);
                    pre[j] = v;
                }
            }
        }
    };

    auto commit = [&](int buf) {  // registers -> LDS (for Q8: raw bytes into the staging area)
        if constexpr (SRC == SRC_Q8) {
            unsigned char * raw = smem + 2 * TILE_BYTES;
#pragma unroll
            for (int j = 0; j < N_PRE; j++) {
                const int c = tid + j * NTHREADS;
                if (c < Q8_TILE_RAW / 16) *(LDS_PTR(u32x4)) (raw + c * 16) = pre[j];
            }
        } else {
            unsigned char * tile = smem + buf * TILE_BYTES;
#pragma unroll
            for (int j = 0; j < N_PRE; j++) {
                const int c   = tid + j * NTHREADS;
                const int r   = c / (ROW_BYTES / 16);
                const int col = c - r * (ROW_BYTES / 16);
                *(LDS_PTR(u32x4)) (tile + r * PITCH + col * 16) = pre[j];
            }
        }
    };

    // Q8_0 only: raw staging area -> f16 tile.  One (row, block) pair per work item: value = q * f32(d), rounded to
    // f16 (the reference dequantizes to f32, ggml-quants.c:357-373; q*d has <= 19 significant bits, f16 keeps 11).
    auto dequant = [&](int buf) {
        if constexpr (SRC == SRC_Q8) {
            const unsigned char * raw  = smem + 2 * TILE_BYTES;
            unsigned char *       tile = smem + buf * TILE_BYTES;
            for (int w = tid; w < TILE_TOK * 18; w += NTHREADS) {
                const int r  = w / 18;
                const int bk = w - r * 18;
                LDS_PTR(const unsigned short) src = (LDS_PTR(const unsigned short)) (raw + r * Q8_ROW + bk * 34);
                const float d = f16_bits_to_f32(src[0]);
                unsigned int o[16];
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const unsigned int pr = src[1 + e];
                    const float a = (float) (int) (signed char) (pr & 0xff) * d;
                    const float c = (float) (int) (signed char) (pr >> 8) * d;
                    o[e] = pack2<true>(a, c);
                }
                LDS_PTR(u32x4) dstp = (LDS_PTR(u32x4)) (tile + r * PITCH + bk * 64);
                dstp[0] = u32x4{ o[0], o[1], o[2], o[3] };
                dstp[1] = u32x4{ o[4], o[5], o[6], o[7] };
                dstp[2] = u32x4{ o[8], o[9], o[10], o[11] };
                dstp[3] = u32x4{ o[12], o[13], o[14], o[15] };
            }
        }
    };

    // per-lane LDS offsets
    const int k_off = rl * PITCH + g * 16;  // K fragment of S^T = K.Q^T: token rl, d = 16*ks + 8*g..+7
    // V^T fragment via ds_read_b64_tr_b16: within each 16-lane group, lane s supplies the address of token (s/4),
    // columns 4*(s%4)..+3 of the group's 16 columns, and receives 4 tokens of column s.
    const int v_off = (4 * g + ((lane & 15) >> 2)) * PITCH + (((lane >> 4) & 1) * 16 + (lane & 3) * 4) * 2;

    if (n_tiles > 0) {
        prefetch(0);
        commit(0);
        if constexpr (SRC == SRC_Q8) { __syncthreads(); dequant(0); }
    }
    __syncthreads();

    for (int it = 0; it < n_tiles; it++) {
        const int  buf      = it & 1;
        const bool has_next = it + 1 < n_tiles;
        if (has_next) prefetch(it + 1);

        const unsigned char * tile = smem + buf * TILE_BYTES;
        const int             t0   = kv_begin + it * TILE_TOK;

        // ---- S^T = K . Q^T
        f32x16 s;
#pragma unroll
        for (int e = 0; e < 16; e++) s[e] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ks++) {
            const u32x4 a = *(LDS_PTR(const u32x4)) (tile + k_off + ks * 32);
            s = mfma32<F16>(a, qreg[ks], s);
        }

        // ---- scores in log2 units; accumulator element e is token 8*(e/4) + 4*g + e%4 of the tile
        float tmax = -INFINITY;
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int ic = t0 + 8 * (e >> 2) + 4 * g + (e & 3);
            float v = s[e] * scale_eff;
            if (p.softcap != 0.0f) v = p.softcap * tanhf(v);
            if (mask_row) {
                float mv = -INFINITY;
                if (ic < p.mask_ne0) mv = f16_bits_to_f32(*(const unsigned short *) (mask_row + (int64_t) ic * 2));
                v += slope * mv;
            }
            v *= LOG2E;
            if (ic >= kv_end) v = -INFINITY;
            s[e] = v;
            tmax = fmaxf(tmax, v);
        }
        tmax = fmaxf(tmax, xor32(tmax));
        const float m_new = fmaxf(m_run, tmax);
        if (__any(m_new > m_run)) {
            const float alpha = (m_run == -INFINITY) ? 0.f : fast_exp2(m_run - m_new);  // 1 where the max did not move
#pragma unroll
            for (int i = 0; i < NDBW; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[i][e] *= alpha;
            l_run *= alpha;
            m_run = m_new;
        }
        const float m_use = (m_run == -INFINITY) ? 0.f : m_run;
        float lsum = 0.f;
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const float pe = fast_exp2(s[e] - m_use);
            s[e] = pe;
            lsum += pe;
        }
        l_run += lsum;

        // ---- P^T as MFMA B operand: k-step kk uses accumulator elements 8*kk .. 8*kk+7
        u32x4 p_hi[2], p_lo[2];
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            u32x4 h;
            h.x = pack2<F16>(s[8 * kk + 0], s[8 * kk + 1]); h.y = pack2<F16>(s[8 * kk + 2], s[8 * kk + 3]);
            h.z = pack2<F16>(s[8 * kk + 4], s[8 * kk + 5]); h.w = pack2<F16>(s[8 * kk + 6], s[8 * kk + 7]);
            p_hi[kk] = h;
            if constexpr (SPLIT) {
                float r[8];
#pragma unroll
                for (int e = 0; e < 8; e++) r[e] = s[8 * kk + e] - round_trip<F16>(s[8 * kk + e]);
                u32x4 l;
                l.x = pack2<F16>(r[0], r[1]); l.y = pack2<F16>(r[2], r[3]);
                l.z = pack2<F16>(r[4], r[5]); l.w = pack2<F16>(r[6], r[7]);
                p_lo[kk] = l;
            }
        }

        // ---- O^T += V^T . P^T ; V^T fragments straight from the row-major tile via the transposing LDS read
#pragma unroll
        for (int i = 0; i < NDBW; i++) {
            const int dcol = p.d_off + (wd * NDBW + i) * 32;  // first column of this 32-wide block
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
                const unsigned char * vp = tile + v_off + (16 * kk) * PITCH + dcol * 2;
                const s16x4 t0v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4)) (vp));
                const s16x4 t1v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4)) (vp + 8 * PITCH));
                const u32x2 a0 = bitcast<u32x2>(t0v), a1 = bitcast<u32x2>(t1v);
                const u32x4 a  = { a0.x, a0.y, a1.x, a1.y };
                acc[i] = mfma32<F16>(a, p_hi[kk], acc[i]);
                if constexpr (SPLIT) acc[i] = mfma32<F16>(a, p_lo[kk], acc[i]);
            }
        }

        if (has_next) {
            commit(buf ^ 1);
            if constexpr (SRC == SRC_Q8) { __syncthreads(); dequant(buf ^ 1); }
        }
        __syncthreads();
    }

    // ---- epilogue
    const float l_tot = l_run + xor32(l_run);
    if (!row_valid) return;
    const int64_t orow = (int64_t) b * p.n_rows + row;
    if (p.n_splits == 1) {
        const float inv = 1.0f / l_tot;  // l == 0 (every key masked, or an empty sequence) gives NaN like the reference
        float * o = p.dst + orow * p.dst_stride + p.d_off;
#pragma unroll
        for (int i = 0; i < NDBW; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                f32x4 v = { acc[i][4 * j] * inv, acc[i][4 * j + 1] * inv, acc[i][4 * j + 2] * inv, acc[i][4 * j + 3] * inv };
                *(f32x4 *) (o + (wd * NDBW + i) * 32 + 8 * j + 4 * g) = v;
            }
    } else {
        const int64_t prow   = ((int64_t) b * p.n_splits + split) * p.n_rows + row;
        const int64_t pblock = ((int64_t) b * p.n_splits + split) * p.n_rows * p.dv_total;
        // partial = O / l of this split, stored as f16 in layout [column/8][row][8]: coalesced for the writers here and
        // for the combine pass, and half the bytes of f32 (the 2^-11 rounding is averaged over the splits)
        const float pinv = 1.0f / l_tot;
        if (p.part_f32) {
            float * o = (float *) p.part_o + prow * p.dv_total + p.d_off;
#pragma unroll
            for (int i = 0; i < NDBW; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    f32x4 v = { acc[i][4 * j] * pinv, acc[i][4 * j + 1] * pinv, acc[i][4 * j + 2] * pinv, acc[i][4 * j + 3] * pinv };
                    *(f32x4 *) (o + (wd * NDBW + i) * 32 + 8 * j + 4 * g) = v;
                }
        } else
#pragma unroll
        for (int i = 0; i < NDBW; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int d0 = p.d_off + (wd * NDBW + i) * 32 + 8 * j + 4 * g;
                u32x2 v = { pack2<true>(acc[i][4 * j] * pinv, acc[i][4 * j + 1] * pinv), pack2<true>(acc[i][4 * j + 2] * pinv, acc[i][4 * j + 3] * pinv) };
                *(u32x2 *) (p.part_o + pblock + ((int64_t) (d0 >> 3) * p.n_rows + row) * 8 + (d0 & 7)) = v;
            }
        if (wd == 0 && g == 0 && p.d_off == 0) {
            p.part_ml[prow * 2]     = m_run;
            p.part_ml[prow * 2 + 1] = l_tot;
        }
    }
}

// Where the partials of a row sit.  Uniform splits: slots b*n_splits .. +nvalid, each holding all n_rows rows.  Balanced
// schedule: the workgroups whose runs of the unit list touch the item (the sequence b, or with a mask the row block of
// the row), slot = workgroup + item (see mla_decode_kernel), each holding p.slot_rows rows; lrow = the row inside a slot.
// nvalid < 0: one workgroup had the whole item and wrote the final rows itself.
// A launch issued in two forms (p.dual; the combine pass gets the row-block form's parameters): p.form tells which one ran; in the
// token form an item is a query token and a slot holds its n_head rows.
__device__ __forceinline__ void partial_slots(const KParams & p, int b, int row, int seq_len, int & slot0, int & nvalid, int & lrow, int & slot_rows) {
    lrow = row;
    slot_rows = p.slot_rows;
    if (!p.balanced) {
        nvalid = (seq_len + p.split_tokens - 1) / p.split_tokens;
        nvalid = p.rel_splits ? p.n_splits : min(nvalid, p.n_splits);
        slot0  = b * p.n_splits;
        return;
    }
    int item = p.balanced == 2 ? row / 128 : b, n_units = p.n_units;
    if (p.balanced == 2) lrow = row - item * 128;
    if (p.dual && *p.form == 3) { item = row / p.n_head; lrow = row - item * p.n_head; slot_rows = p.n_head; n_units = p.n_tok; }
    if (p.balanced >= 2 && p.wg_first[1]) {   // aligned schedule of a masked launch: every item has workgroups of its own
        const int * W = p.wg_first + 8;
        nvalid = W[item + 1] - W[item];
        slot0  = nvalid ? W[item] + item : 0;
        if (nvalid == 1) nvalid = -1;
        return;
    }
    const int before = p.sched[item], mine = p.sched[item + 1] - before, total = p.sched[n_units];
    const int quota = (total + p.n_wg - 1) / p.n_wg;
    if (mine == 0) { slot0 = 0; nvalid = 0; return; }
    const int w0 = before / quota, w1 = (before + mine - 1) / quota;
    slot0  = w0 + item;
    nvalid = w1 - w0 + 1;
    if (nvalid == 1) nvalid = -1;
}

// Log-sum-exp merge of the split-K partials: out = sum_c (O_c/l_c) l_c 2^(m_c - M) / sum_c l_c 2^(m_c - M).
// Partials hold O_c/l_c as f16, laid out [seq][split][column/8][row][8].  One thread = one row and two groups of 8 columns 128
// columns apart: 16-byte loads, splits in groups of 8 so that all the loads of a group (8 (m, l) pairs, 16 partial chunks) are in
// flight together, and the weights of a group of splits are worked out once for both column groups.  A wave covers 16 rows x 4
// column groups (twice): it reads runs of 256 bytes (16 rows of one column group are contiguous in the partial layout) and writes
// 128 contiguous bytes per row.  grid = (ceil(rows/16), ceil(dv/256), n_seq), block = 256 = 16 rows x 16 column groups (x 2).
__global__ void __launch_bounds__(256) mla_attn_combine_kernel(const KParams p) {
    const int b = blockIdx.z;
    const int row = blockIdx.x * 16 + (threadIdx.x & 15);
    const int cg  = blockIdx.y * 32 + (threadIdx.x >> 4);
    const int seq_len = p.block_table ? min(p.seq_lens[b], (int) p.bt_stride * MLA_PAGE_TOKENS) : (int) p.n_kv;
    if (row >= p.n_rows || cg * 8 >= p.dv_total) return;
    const bool two = (cg + 16) * 8 < p.dv_total;   // the second column group exists
    int slot0, nvalid, lrow, slot_rows;
    partial_slots(p, b, row, seq_len, slot0, nvalid, lrow, slot_rows);
    if (nvalid < 0) return;

    const float2 *   ml = (const float2 *) p.part_ml + (int64_t) slot0 * slot_rows + lrow;
    const _Float16 * po = p.part_o + (int64_t) slot0 * slot_rows * p.dv_total + ((int64_t) cg * slot_rows + lrow) * 8;
    const int64_t ml_step = slot_rows, po_step = (int64_t) slot_rows * p.dv_total, second = two ? (int64_t) 16 * slot_rows * 8 : 0;

    float M = -INFINITY, L = 0.f;
    float o[16] = { 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f };
    for (int c0 = 0; c0 < nvalid; c0 += 8) {
        float2 mlv[8];
        u32x4  hv[8], hw[8];
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int c = min(c0 + k, nvalid - 1);  // past the end: a duplicate of the last split, given weight 0 below
            mlv[k] = ml[c * ml_step];
            hv[k]  = *(const u32x4 *) (po + c * po_step);
            hw[k]  = *(const u32x4 *) (po + c * po_step + second);
        }
        float Mg = M;
#pragma unroll
        for (int k = 0; k < 8; k++) if (c0 + k < nvalid) Mg = fmaxf(Mg, mlv[k].x);
        if (Mg == -INFINITY) continue;  // every split so far saw only masked keys
        const float r = fast_exp2(M - Mg);  // 0 when M was -inf
        M = Mg;
        L *= r;
#pragma unroll
        for (int k = 0; k < 16; k++) o[k] *= r;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            // l_c 2^(m_c - M); a split that saw only masked keys (m_c = -inf) and the padding of the group get 0
            const float w = (c0 + k < nvalid && mlv[k].x != -INFINITY) ? mlv[k].y * fast_exp2(mlv[k].x - M) : 0.f;
            L += w;
            if (w == 0.f) continue;  // its partial may hold anything (0/0 of a split without a key), never multiply it in
            const unsigned h[8] = { hv[k].x, hv[k].y, hv[k].z, hv[k].w, hw[k].x, hw[k].y, hw[k].z, hw[k].w };
#pragma unroll
            for (int e = 0; e < 8; e++) {
                o[2 * e]     += f16_bits_to_f32(h[e] & 0xffff) * w;
                o[2 * e + 1] += f16_bits_to_f32(h[e] >> 16) * w;
            }
        }
    }
    const float inv = 1.0f / L;  // no valid key at all: 0 * inf = NaN, like the reference
    float * out = p.dst + ((int64_t) b * p.n_rows + row) * p.dst_stride + p.v_col0 + cg * 8;
    *(f32x4 *) out       = f32x4{ o[0] * inv, o[1] * inv, o[2] * inv, o[3] * inv };
    *(f32x4 *) (out + 4) = f32x4{ o[4] * inv, o[5] * inv, o[6] * inv, o[7] * inv };
    if (two) {
        *(f32x4 *) (out + 128) = f32x4{ o[8] * inv, o[9] * inv, o[10] * inv, o[11] * inv };
        *(f32x4 *) (out + 132) = f32x4{ o[12] * inv, o[13] * inv, o[14] * inv, o[15] * inv };
    }
}

// The same merge for rows with many splits (one or two long sequences: 256 pieces of one row's output): the walk over the splits of
// a row is a chain of load latencies when one thread makes it, so SL = 4 or 16 lanes share it -- lane `sl` of such a group takes
// splits sl, sl + SL, ... (up to 16 of them in flight), and the group merges its (M, L, O) triples with lane shuffles at the end.
// A wave covers 64 / SL rows x one group of 8 columns x SL split lanes.  grid = (ceil(rows * SL / 64), dv/32, n_seq), block = 256 =
// 4 waves = 4 column groups.  One sequence of 128 heads x 131 072 keys in 256 splits: step 96.3 us with one thread per (row, column
// group), 72.1 us with four lanes, 67.7 us with sixteen (the decode kernel alone: 47 us).
template <int G, int SL>
__device__ __forceinline__ void combine_wide_walk(const float2 * ml, const _Float16 * po, int64_t ml_step, int64_t po_step, int nvalid, int sl, float & M, float & L, float (&o)[8]) {
    for (int c0 = sl; c0 < nvalid; c0 += SL * G) {
        float2 mlv[G];
        u32x4  hv[G];
#pragma unroll
        for (int k = 0; k < G; k++) {
            const int c = min(c0 + SL * k, nvalid - 1);  // past the end: a duplicate of the last split, given weight 0 below
            mlv[k] = ml[c * ml_step];
            hv[k]  = *(const u32x4 *) (po + c * po_step);
        }
        float Mg = M;
#pragma unroll
        for (int k = 0; k < G; k++) if (c0 + SL * k < nvalid) Mg = fmaxf(Mg, mlv[k].x);
        if (Mg == -INFINITY) continue;  // every split so far saw only masked keys
        const float r = fast_exp2(M - Mg);  // 0 when M was -inf
        M = Mg;
        L *= r;
#pragma unroll
        for (int k = 0; k < 8; k++) o[k] *= r;
#pragma unroll
        for (int k = 0; k < G; k++) {
            const float w = (c0 + SL * k < nvalid && mlv[k].x != -INFINITY) ? mlv[k].y * fast_exp2(mlv[k].x - M) : 0.f;
            L += w;
            if (w == 0.f) continue;  // its partial may hold anything (0/0 of a split without a key), never multiply it in
            const unsigned h[4] = { hv[k].x, hv[k].y, hv[k].z, hv[k].w };
#pragma unroll
            for (int e = 0; e < 4; e++) {
                o[2 * e]     += f16_bits_to_f32(h[e] & 0xffff) * w;
                o[2 * e + 1] += f16_bits_to_f32(h[e] >> 16) * w;
            }
        }
    }
}
template <int SL>
__global__ void __launch_bounds__(256) mla_attn_combine_wide_kernel(const KParams p) {
    const int b = blockIdx.z, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sl = lane % SL;
    const int row = blockIdx.x * (64 / SL) + lane / SL;
    const int cg  = blockIdx.y * 4 + wave;
    const int seq_len = p.block_table ? min(p.seq_lens[b], (int) p.bt_stride * MLA_PAGE_TOKENS) : (int) p.n_kv;
    // (rows past the end keep their lanes: the shuffles below want whole groups; they work on the last row and store nothing)
    const int rrow = min(row, p.n_rows - 1);
    if (cg * 8 >= p.dv_total) return;
    int slot0, nvalid, lrow, slot_rows;
    partial_slots(p, b, rrow, seq_len, slot0, nvalid, lrow, slot_rows);
    if (nvalid < 0) return;   // (the same for the lanes of a group)

    const float2 *   ml = (const float2 *) p.part_ml + (int64_t) slot0 * slot_rows + lrow;
    const _Float16 * po = p.part_o + (int64_t) slot0 * slot_rows * p.dv_total + ((int64_t) cg * slot_rows + lrow) * 8;
    const int64_t ml_step = slot_rows, po_step = (int64_t) slot_rows * p.dv_total;

    float M = -INFINITY, L = 0.f;
    float o[8] = { 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f };
    // 16 splits per lane in flight, or 4 when the row has few (the host picks this kernel by the longest rows of the launch)
    if (nvalid > 4 * SL) combine_wide_walk<16, SL>(ml, po, ml_step, po_step, nvalid, sl, M, L, o);
    else                 combine_wide_walk<4, SL>(ml, po, ml_step, po_step, nvalid, sl, M, L, o);
    // the group's triples -> one: common maximum, rescale, add
    float Mq = M;
#pragma unroll
    for (int d = 1; d < SL; d <<= 1) Mq = fmaxf(Mq, __shfl_xor(Mq, d, 64));
    const float rs = (M == -INFINITY) ? 0.f : fast_exp2(M - Mq);   // (a lane without a valid split: nothing to add; Mq = -inf too: L stays 0)
    L *= rs;
#pragma unroll
    for (int k = 0; k < 8; k++) o[k] *= rs;
#pragma unroll
    for (int d = 1; d < SL; d <<= 1) {
        L += __shfl_xor(L, d, 64);
#pragma unroll
        for (int k = 0; k < 8; k++) o[k] += __shfl_xor(o[k], d, 64);
    }
    if (row >= p.n_rows || sl >= 4) return;
    const float inv = 1.0f / L;  // no valid key at all: 0 * inf = NaN, like the reference
    float * out = p.dst + ((int64_t) b * p.n_rows + row) * p.dst_stride + p.v_col0 + cg * 8 + 2 * sl;   // lane sl stores columns 2 sl, 2 sl + 1
    float2 v;
    v.x = (sl == 0 ? o[0] : sl == 1 ? o[2] : sl == 2 ? o[4] : o[6]) * inv;
    v.y = (sl == 0 ? o[1] : sl == 1 ? o[3] : sl == 2 ? o[5] : o[7]) * inv;
    *(float2 *) out = v;
}

// The same merge over f32 partials (rows of dv_total floats; small problems).  One thread = one (row, group of 4 columns),
// lanes along the columns of a row.  grid = (ceil(rows/2), 1, n_seq), block = 256 = 2 rows x 128 column groups (dv <= 512)
// or (rows, 1, n_seq) with 144 active threads for dv = 576: blockDim covers one or two rows, see the launch.
// G splits are loaded together (a split past the end is a duplicate of the last one with weight 0): small problems are
// latency-bound, so the group should cover every split of a row in one round -- a ragged batch of short sequences has up to 32
// one-page pieces per sequence -- without issuing many times the loads a row with two or three splits needs.
template <int G>
__device__ __forceinline__ void combine_f32_row(const float2 * ml, const float * po, int64_t ml_step, int64_t po_step, int nvalid, float * dst) {
    float M = -INFINITY, L = 0.f;
    f32x4 o = { 0.f, 0.f, 0.f, 0.f };
    for (int c0 = 0; c0 < nvalid; c0 += G) {
        float2 mlv[G];
        f32x4  xv[G];
#pragma unroll
        for (int k = 0; k < G; k++) {
            const int c = min(c0 + k, nvalid - 1);
            mlv[k] = ml[c * ml_step];
            xv[k]  = *(const f32x4 *) (po + c * po_step);
        }
        float Mg = M;
#pragma unroll
        for (int k = 0; k < G; k++) if (c0 + k < nvalid) Mg = fmaxf(Mg, mlv[k].x);
        if (Mg == -INFINITY) continue;  // every split so far saw only masked keys
        const float r = fast_exp2(M - Mg);  // 0 when M was -inf
        M = Mg;
        L *= r;
        o.x *= r; o.y *= r; o.z *= r; o.w *= r;
#pragma unroll
        for (int k = 0; k < G; k++) {
            const float w = (c0 + k < nvalid && mlv[k].x != -INFINITY) ? mlv[k].y * fast_exp2(mlv[k].x - M) : 0.f;
            L += w;
            if (w == 0.f) continue;  // that split saw only masked keys (or is padding): its partial may hold anything
            o.x += xv[k].x * w; o.y += xv[k].y * w; o.z += xv[k].z * w; o.w += xv[k].w * w;
        }
    }
    const float inv = 1.0f / L;  // no valid key at all: 0 * inf = NaN, like the reference
    *(f32x4 *) dst = f32x4{ o.x * inv, o.y * inv, o.z * inv, o.w * inv };
}

__global__ void __launch_bounds__(256) mla_attn_combine_f32_kernel(const KParams p, int groups_per_row) {
    const int b = blockIdx.z;
    const int rows_per_block = 256 / groups_per_row;
    const int row = blockIdx.x * rows_per_block + threadIdx.x / groups_per_row;
    const int cg  = threadIdx.x % groups_per_row;
    const int seq_len = p.block_table ? min(p.seq_lens[b], (int) p.bt_stride * MLA_PAGE_TOKENS) : (int) p.n_kv;
    if (row >= p.n_rows || (int) threadIdx.x >= rows_per_block * groups_per_row || cg * 4 >= p.dv_total) return;
    int slot0, nvalid, lrow, slot_rows;
    partial_slots(p, b, row, seq_len, slot0, nvalid, lrow, slot_rows);
    if (nvalid < 0) return;
    const float2 * ml = (const float2 *) p.part_ml + (int64_t) slot0 * slot_rows + lrow;
    const float *  po = (const float *) p.part_o + ((int64_t) slot0 * slot_rows + lrow) * p.dv_total + cg * 4;
    const int64_t ml_step = slot_rows, po_step = (int64_t) slot_rows * p.dv_total;
    float * dst = p.dst + ((int64_t) b * p.n_rows + row) * p.dst_stride + p.v_col0 + cg * 4;
    if (nvalid <= 4)       combine_f32_row<4>(ml, po, ml_step, po_step, nvalid, dst);
    else if (nvalid <= 16) combine_f32_row<16>(ml, po, ml_step, po_step, nvalid, dst);
    else                   combine_f32_row<32>(ml, po, ml_step, po_step, nvalid, dst);
}

// f32 partials, rows with more than 32 splits (a single sequence of a decode step: 64 one-page splits at 8192 keys, 256 pieces at
// 131 072): the four waves of a block share the walk over the splits of one row -- wave w takes splits w, w + 4, ..., 16 in flight,
// for 64 groups of 4 columns -- and meet in LDS.  grid = (rows, ceil(dv / 256), n_seq), block = 256.
__global__ void __launch_bounds__(256) mla_attn_combine_f32_wide_kernel(const KParams p) {
    __shared__ float red[4][6][64];
    constexpr int G = 16;
    const int b = blockIdx.z, row = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int cg = min((int) blockIdx.y * 64 + lane, p.dv_total / 4 - 1);   // (lanes past the row's end repeat its last group and store nothing)
    const int seq_len = p.block_table ? min(p.seq_lens[b], (int) p.bt_stride * MLA_PAGE_TOKENS) : (int) p.n_kv;
    int slot0, nvalid, lrow, slot_rows;
    partial_slots(p, b, row, seq_len, slot0, nvalid, lrow, slot_rows);
    if (nvalid < 0) return;   // (uniform over the block: one row)
    const float2 * ml = (const float2 *) p.part_ml + (int64_t) slot0 * slot_rows + lrow;
    const float *  po = (const float *) p.part_o + ((int64_t) slot0 * slot_rows + lrow) * p.dv_total + cg * 4;
    const int64_t ml_step = slot_rows, po_step = (int64_t) slot_rows * p.dv_total;
    float M = -INFINITY, L = 0.f;
    f32x4 o = { 0.f, 0.f, 0.f, 0.f };
    for (int c0 = wave; c0 < nvalid; c0 += 4 * G) {
        float2 mlv[G];
        f32x4  xv[G];
#pragma unroll
        for (int k = 0; k < G; k++) {
            const int c = min(c0 + 4 * k, nvalid - 1);
            mlv[k] = ml[c * ml_step];
            xv[k]  = *(const f32x4 *) (po + c * po_step);
        }
        float Mg = M;
#pragma unroll
        for (int k = 0; k < G; k++) if (c0 + 4 * k < nvalid) Mg = fmaxf(Mg, mlv[k].x);
        if (Mg == -INFINITY) continue;  // every split so far saw only masked keys
        const float r = fast_exp2(M - Mg);  // 0 when M was -inf
        M = Mg;
        L *= r;
        o.x *= r; o.y *= r; o.z *= r; o.w *= r;
#pragma unroll
        for (int k = 0; k < G; k++) {
            const float w = (c0 + 4 * k < nvalid && mlv[k].x != -INFINITY) ? mlv[k].y * fast_exp2(mlv[k].x - M) : 0.f;
            L += w;
            if (w == 0.f) continue;  // that split saw only masked keys (or is padding): its partial may hold anything
            o.x += xv[k].x * w; o.y += xv[k].y * w; o.z += xv[k].z * w; o.w += xv[k].w * w;
        }
    }
    red[wave][0][lane] = M; red[wave][1][lane] = L;
    red[wave][2][lane] = o.x; red[wave][3][lane] = o.y; red[wave][4][lane] = o.z; red[wave][5][lane] = o.w;
    __syncthreads();
    if (wave != 0 || (int) blockIdx.y * 64 + lane >= p.dv_total / 4) return;
    float Mq = fmaxf(fmaxf(red[0][0][lane], red[1][0][lane]), fmaxf(red[2][0][lane], red[3][0][lane]));
    float Lq = 0.f;
    f32x4 oq = { 0.f, 0.f, 0.f, 0.f };
#pragma unroll
    for (int w = 0; w < 4; w++) {
        const float mw = red[w][0][lane];
        const float rs = mw == -INFINITY ? 0.f : fast_exp2(mw - Mq);   // (a wave without a valid split adds nothing)
        Lq += red[w][1][lane] * rs;
        oq.x += red[w][2][lane] * rs; oq.y += red[w][3][lane] * rs; oq.z += red[w][4][lane] * rs; oq.w += red[w][5][lane] * rs;
    }
    const float inv = 1.0f / Lq;  // no valid key at all: 0 * inf = NaN, like the reference
    float * dst = p.dst + ((int64_t) b * p.n_rows + row) * p.dst_stride + p.v_col0 + cg * 4;
    *(f32x4 *) dst = f32x4{ oq.x * inv, oq.y * inv, oq.z * inv, oq.w * inv };
}

// ---------------------------------------------------------------------------------------------------------------
// Replay of ggml-cpu's own arithmetic, key by key (ggml-cpu.c:12028-12124), for comparisons with the reference's node and for
// problems too small for operand rounding to average out.  Two kernels: the logits' dots, then one block per row walking the keys.
//   F16 KV, MLA_FLAG_F16_ACC_STRICT: f32 dot of f16-rounded Q with f16 K; the f16 accumulator of ggml-cpu.c:12066-12080 with the
//     x86 F16 vector forms :621-659, :718-765 (f32 FMA, result rounded to f16 after every scale and every multiply-add).
//   Q8_0 KV, MLA_FLAG_Q8_EXACT (and by itself for caches of at most one page per sequence): Q quantized to Q8_0 the way the x86 CPU
//     backend does it (ggml-cpu-quants.c:855-900), the integer block dots times d_q * d_k of ggml-cpu-quants.c:3814-4241, V = q * d
//     in f32 (ggml-quants.c:357-373) and the f32 accumulator of ggml-cpu.c:12081-12095 -- no operand is rounded to 16 bits.
// Both over a contiguous cache or through the block table.
// ---------------------------------------------------------------------------------------------------------------
__device__ __forceinline__ const char * ref_kv_row(const KParams & p, int b, int64_t ic) {
    if (p.block_table) {
        const int page = min(max(p.block_table[(int64_t) b * p.bt_stride + (ic >> 7)], 0), p.n_pool_pages - 1);
        return p.kv + ((int64_t) page * MLA_PAGE_TOKENS + (ic & (MLA_PAGE_TOKENS - 1))) * p.kv_nb1;
    }
    return p.kv + ic * p.kv_nb1 + (int64_t) b * p.kv_nb3;
}
__device__ __forceinline__ int ref_seq_len(const KParams & p, int b) {
    return p.block_table ? max(min(p.seq_lens[b], (int) p.bt_stride * MLA_PAGE_TOKENS), 0) : (int) p.n_kv;
}

// grid (ceil(max_len / 64), n_rows, n_seq), block 256: a wave takes 16 keys; scores[(b * n_rows + row) * max_len + ic]
template <int KVT>
__global__ void __launch_bounds__(256) mla_ref_scores_kernel(const KParams p, float * scores, const int64_t max_len) {
    __shared__ signed char qq[DK];
    __shared__ float dq[DK / 32];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = blockIdx.y, b = blockIdx.z;
    const int seq_len = ref_seq_len(p, b);
    const int ic0 = blockIdx.x * 64 + wave * 16;
    if (blockIdx.x * 64 >= seq_len) return;   // (uniform over the block)
    const int tq = row / p.n_head, head = row - tq * p.n_head;
    const float * qrow = (const float *) (p.q + (int64_t) tq * p.q_nb1 + (int64_t) head * p.q_nb2 + (int64_t) b * p.q_nb3);
    float * out = scores + ((int64_t) b * p.n_rows + row) * max_len;
    if constexpr (KVT == MLA_TYPE_Q8_0) {
        // Q -> Q8_0: per block of 32 d = amax / 127 (kept as f16), id = 127 / amax, q = round-half-even(x * id)
        for (int e = threadIdx.x; e < DK; e += 256) {   // (the 32 lanes of a half wave hold one block)
            const float x = qrow[e];
            float amax = fabsf(x);
#pragma unroll
            for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
            const float id = amax != 0.f ? 127.0f / amax : 0.f;
            qq[e] = (signed char) (int) rintf(x * id);
            if ((e & 31) == 0) dq[e >> 5] = f16_bits_to_f32(f32_to_f16_bits(amax / 127.0f));
        }
        __syncthreads();
        const int h = lane >> 5, i = lane & 31;
        for (int k = 0; k < 16; k++) {
            const int ic = ic0 + k;
            if (ic >= seq_len) break;
            const unsigned char * krow = (const unsigned char *) ref_kv_row(p, b, ic);
            float acc = 0.f;
#pragma unroll
            for (int j = 0; j < 9; j++) {
                const int blk = 2 * j + h;
                int sumi = (int) qq[blk * 32 + i] * (int) (signed char) krow[blk * 34 + 2 + i];
#pragma unroll
                for (int o = 16; o > 0; o >>= 1) sumi += __shfl_xor(sumi, o, 64);
                const float dk = f16_bits_to_f32(*(const unsigned short *) (krow + blk * 34));
                acc += (float) sumi * (dq[blk] * dk);
            }
            acc += __shfl_xor(acc, 32, 64);
            if (lane == 0) out[ic] = acc;
        }
    } else {
        for (int k = 0; k < 16; k++) {
            const int ic = ic0 + k;
            if (ic >= seq_len) break;
            const unsigned short * krow = (const unsigned short *) ref_kv_row(p, b, ic);
            float sum = 0.f;
            for (int d = lane; d < DK; d += 64) sum += (float) (_Float16) qrow[d] * f16_bits_to_f32(krow[d]);
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
            if (lane == 0) out[ic] = sum;
        }
    }
}

// One block per output row, one thread per output column; the keys are walked in chunks of STRICT_CHUNK:
//   (a) the logits of the chunk (scale, softcap, ALiBi slope x mask), one key per thread,
//   (b) their running maximum by a prefix scan -- the maximum before key k decides which branch ggml-cpu takes at k
//       and what it feeds expf -- which gives every key its (ms, vs) pair without walking the keys,
//   (c) the walk itself, per column: acc = acc * ms where the maximum moved, acc = fma(v, vs, acc), S = S * ms + vs, exactly the
//       operations of the reference, in its order (F16 KV: both results rounded to f16, as its f16 accumulator does); the V values
//       of eight keys are in flight at a time.
constexpr int STRICT_CHUNK = 1024;
template <int KVT>
__global__ void __launch_bounds__(576) mla_ref_walk_kernel(const KParams p, const float * scores, const int64_t max_len) {  // grid (n_rows, n_seq), block 512 | 576
    __shared__ __attribute__((aligned(16))) float lg[STRICT_CHUNK], pa[STRICT_CHUNK], pb[STRICT_CHUNK];   // logits (-inf: skipped key); scan buffers, then ms / vs
    const int tid = threadIdx.x, nth = blockDim.x, row = blockIdx.x, b = blockIdx.y;
    const int tq = row / p.n_head, head = row - tq * p.n_head;
    const int n_kv = ref_seq_len(p, b);
    float slope = 1.0f;
    if (p.max_bias > 0.0f) slope = head < p.n_head_log2 ? powf(p.m0, (float) (head + 1)) : powf(p.m1, (float) (2 * (head - p.n_head_log2) + 1));
    const float scale_eff = p.softcap != 0.0f ? p.scale / p.softcap : p.scale;
    const char * mask_row = p.mask ? p.mask + (int64_t) tq * p.mask_nb1 + (int64_t) b * p.mask_nb3 : nullptr;
    const float * srow = scores + ((int64_t) b * p.n_rows + row) * max_len;
    const bool col = tid < p.dv_total;
    const int  c   = col ? tid : 0;
    // where column c sits inside a row, and (Q8_0) where its block's scale does
    const int voff = KVT == MLA_TYPE_Q8_0 ? (c >> 5) * 34 + 2 + (c & 31) : 2 * c, doff = (c >> 5) * 34;
    auto value = [&](const char * r) -> float {
        if constexpr (KVT == MLA_TYPE_Q8_0) return (float) (int) *(const signed char *) (r + voff) * f16_bits_to_f32(*(const unsigned short *) (r + doff));
        else return f16_bits_to_f32(*(const unsigned short *) (r + voff));
    };
    float acc = 0.f, S = 0.f, M = -INFINITY;   // M: the maximum over the chunks before this one (the same in every thread)
    for (int c0 = 0; c0 < n_kv; c0 += STRICT_CHUNK) {
        const int n = min(STRICT_CHUNK, n_kv - c0);
        for (int k = tid; k < n; k += nth) {
            const int ic = c0 + k;
            // (a key past the mask's width counts as masked, as in the other kernels)
            const float mv = !mask_row ? 0.0f : ic < p.mask_ne0 ? slope * f16_bits_to_f32(*(const unsigned short *) (mask_row + (int64_t) ic * 2)) : -INFINITY;
            float sv = -INFINITY;   // ggml-cpu skips a key whose mask value is -inf (ggml-cpu.c:12041-12044)
            if (mv != -INFINITY) {
                sv = srow[ic] * scale_eff;
                if (p.softcap != 0.0f) sv = p.softcap * tanhf(sv);
                sv += mv;
            }
            lg[k] = sv; pa[k] = sv;
        }
        __syncthreads();
        float * src = pa, * dst = pb;   // inclusive prefix maximum (Hillis-Steele, ping-pong)
        for (int off = 1; off < n; off <<= 1) {
            for (int k = tid; k < n; k += nth) dst[k] = k >= off ? fmaxf(src[k], src[k - off]) : src[k];
            __syncthreads();
            float * t = src; src = dst; dst = t;
        }
        float ms2[2], vs2[2];   // n <= 1024 and nth >= 512: at most two keys per thread
        int nk = 0;
        for (int k = tid; k < n; k += nth, nk++) {
            const float mprev = k > 0 ? fmaxf(M, src[k - 1]) : M;
            const float sv = lg[k];
            float ms = 1.0f, vs = -1.0f;   // vs < 0 marks a skipped key
            if (sv != -INFINITY || mask_row == nullptr) {
                if (sv > mprev) { ms = expf(mprev - sv); vs = 1.0f; }
                else            { vs = expf(sv - mprev); }
            }
            ms2[nk] = ms; vs2[nk] = vs;
        }
        const float m_chunk = src[n - 1];
        __syncthreads();
        nk = 0;
        for (int k = tid; k < n; k += nth, nk++) { pa[k] = ms2[nk]; pb[k] = vs2[nk]; }
        if (tid < 8 && n + tid < ((n + 7) & ~7)) { pa[n + tid] = 1.0f; pb[n + tid] = -1.0f; }   // pad the last group of eight with skipped keys
        __syncthreads();
        M = fmaxf(M, m_chunk);
        if (col) {
            float vn[8];
#pragma unroll
            for (int j = 0; j < 8; j++) vn[j] = value(ref_kv_row(p, b, c0 + min(j, n - 1)));
            for (int k0 = 0; k0 < n; k0 += 8) {
                float v8[8];
#pragma unroll
                for (int j = 0; j < 8; j++) v8[j] = vn[j];
#pragma unroll
                for (int j = 0; j < 8; j++) vn[j] = value(ref_kv_row(p, b, c0 + min(k0 + 8 + j, n - 1)));   // the next eight, in flight during this group
                const f32x4 m0 = *(const f32x4 *) (pa + k0), m1 = *(const f32x4 *) (pa + k0 + 4);
                const f32x4 w0 = *(const f32x4 *) (pb + k0), w1 = *(const f32x4 *) (pb + k0 + 4);
                const float ms8[8] = { m0.x, m0.y, m0.z, m0.w, m1.x, m1.y, m1.z, m1.w };
                const float vs8[8] = { w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w };
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    // acc * ms is the identity where the maximum did not move (ms = 1), so no branch on it
                    float scaled, next;
                    if constexpr (KVT == MLA_TYPE_F16) {
                        scaled = (float) (_Float16) (acc * ms8[j]);
                        next   = (float) (_Float16) fmaf(v8[j], vs8[j], scaled);
                    } else {
                        scaled = acc * ms8[j];
                        next   = fmaf(v8[j], vs8[j], scaled);
                    }
                    const bool skip = vs8[j] < 0.0f;
                    acc = skip ? acc : next;
                    S   = skip ? S : S * ms8[j] + vs8[j];
                }
            }
        }
        __syncthreads();
    }
    if (col) p.dst[((int64_t) b * p.n_rows + row) * p.dst_stride + tid] = acc * (1.0f / S);
}


__global__ void __launch_bounds__(256) mla_hbm_copy_kernel(const u32x4 * __restrict__ src, u32x4 * __restrict__ dst, size_t n16) {
    size_t       i      = (size_t) blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t) gridDim.x * 256;
    for (; i < n16; i += stride) dst[i] = src[i];
}

// ---------------------------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------------------------

// Scratch of mla_attn_launch_static: one copy per device, at the address hipGetSymbolAddress reports there (g_scratch_ptr).
// In host code the array's name is only a handle for that lookup, never an address.
static __device__ __align__(256) unsigned char scratch[MLA_ATTN_STATIC_WORKSPACE_MAX];
static std::atomic<void *> g_scratch_ptr[MLA_MAX_DEVICES];   // (per device; threads that look it up together store the same value)

struct Plan {
    int    variant;  // 0 tiled, 1 strict f16
    int    wm, wd, rblk, n_row_blocks;
    int    n_splits, split_tokens;
    int    n_passes, ndb;
    size_t lds_bytes;
    size_t ws_part_o, ws_part_ml, ws_scores, ws_qpack, ws_maskext, ws_sched, ws_kvcopy;
    int64_t kvcopy_rows;
    int    part_f32;
    int    balanced, n_wg, n_units;   // balanced schedule of the pipelined kernel (1: ragged paged decode, 2: masked launch)
    int    dual;                      // the masked launch is issued in two forms, see token_form_candidate
    int    seq_sorted;                // paged decode of more than 256 sequences: workgroups take the sequences longest first
};

int validate(const mla_attn_args * a) {
    if (!a) return MLA_ERR_NULL;
    if (!a->q || !a->kv || !a->dst) return MLA_ERR_NULL;
    if (a->n_seq < 1 || a->n_head < 1 || a->n_tok < 1) return MLA_ERR_BAD_SHAPE;
    if (a->dk != DK || (a->dv != 512 && a->dv != 576)) return MLA_ERR_BAD_SHAPE;
    if (a->q_type != MLA_TYPE_F32) return MLA_ERR_BAD_TYPE;
    if (a->kv_type != MLA_TYPE_BF16 && a->kv_type != MLA_TYPE_F16 && a->kv_type != MLA_TYPE_Q8_0) return MLA_ERR_BAD_TYPE;
    if ((a->flags & MLA_FLAG_F16_ACC_STRICT) && a->kv_type != MLA_TYPE_F16) return MLA_ERR_UNSUPPORTED;
    if ((a->flags & MLA_FLAG_Q8_EXACT) && a->kv_type != MLA_TYPE_Q8_0) return MLA_ERR_UNSUPPORTED;
    if (a->n_kv < 0 || a->n_kv > 0x7fffffff) return MLA_ERR_BAD_SHAPE;
    if ((int64_t) a->n_tok * a->n_head > 0x7fffffff) return MLA_ERR_BAD_SHAPE;
    if (((uintptr_t) a->q & 15) || (a->q_nb1 & 15) || (a->q_nb2 & 15) || (a->q_nb3 & 15)) return MLA_ERR_BAD_ALIGNMENT;
    if (((uintptr_t) a->dst & 15) || (a->dst_nb1 & 15) || a->dst_nb1 < (int64_t) a->dv * 4) return MLA_ERR_BAD_ALIGNMENT;
    if (a->kv_type == MLA_TYPE_Q8_0) {
        if (((uintptr_t) a->kv & 1) || (a->kv_nb1 & 1) || (a->kv_nb3 & 1) || a->kv_nb1 < Q8_ROW) return MLA_ERR_BAD_ALIGNMENT;
    } else {
        if (((uintptr_t) a->kv & 15) || (a->kv_nb1 & 15) || (a->kv_nb3 & 15) || a->kv_nb1 < ROW_BYTES) return MLA_ERR_BAD_ALIGNMENT;
    }
    if (a->mask) {
        if ((a->mask_nb1 & 1) || ((uintptr_t) a->mask & 1) || a->mask_ne0 < 0) return MLA_ERR_BAD_ALIGNMENT;
    }
    if (a->max_bias > 0.0f && !a->mask) return MLA_ERR_UNSUPPORTED;  // ggml.c:4005-4007
    if (a->block_table) {
        if (!a->seq_lens || a->bt_stride < 1) return MLA_ERR_NULL;
        if (a->n_kv < MLA_PAGE_TOKENS || a->n_kv % MLA_PAGE_TOKENS) return MLA_ERR_BAD_SHAPE;  // pool of whole pages
        if (a->bt_stride > (1 << 23)) return MLA_ERR_BAD_SHAPE;
    }
    if (a->n_splits < 0) return MLA_ERR_BAD_SHAPE;
    if (a->rows_per_wg != 0 && a->rows_per_wg != 32 && a->rows_per_wg != 64 && a->rows_per_wg != 128) return MLA_ERR_BAD_SHAPE;
    return 0;
}

// The reference's batched decode with few heads per device (one cache shared by the sequences, one query token each, the f16 mask
// selects each token's cells; 16 heads at tensor-parallel degree 8): a block of 128 rows holds the rows of 8 tokens and visits the
// cells of all 8, seven eighths of them masked for any one row.  Taken token by token -- every query token a sequence of its own
// with one token of n_head rows (at most 32: the k-split program), all on the same cache, its mask row that sequence's mask -- a
// workgroup only visits the cells its token may attend to.  For a prompt chunk of one sequence it is the other way round: the
// tokens of a block share their cells, and the token form would read them once per token.  The arguments do not tell the two
// apart, the mask on the device does: such a launch is issued in both forms at once, to a kernel that holds the programs of both;
// every workgroup adds up the tiles either form would visit (from the mask extents) and runs the cheaper one.
// Up to 32 heads of 16-bit cells the token form is the k-split program; from 33 to 64 heads, and for Q8_0 cells the wave program copies
// as raw tiles, it is the row-split program of the cache type (one or two of its four waves with rows), which takes an operand
// image of its own (token_image_bytes; written by more layers of the pack launch).  Not 64 heads of 16-bit cells: a row block is
// two tokens exactly, the token form never visits fewer tiles and its tile costs the same (32 tokens x 8192 cells: 99.5 us
// per step against 98.3 us).  48 heads: 113 -> 98 us; Q8_0 cells, 16 / 32 / 64 heads: 105 -> 85, 94 -> 86, 95 -> 89 us.
static bool token_form_candidate(const mla_attn_args * a, const Plan & pl) {
    if (a->n_head > 32 && a->kv_type != MLA_TYPE_Q8_0 && 128 % a->n_head == 0) return false;
    return pl.variant == 2 && pl.balanced == 2 && a->n_tok <= 256 && a->n_head <= 64 && (int64_t) a->n_tok * a->n_head > 32 && a->n_tok > 1 &&
           pl.kvcopy_rows == 0 && !(a->flags & MLA_FLAG_BF16_DIRECT) && a->logit_softcap == 0.0f && !(a->max_bias > 0.0f);
}
static size_t token_image_bytes(const mla_attn_args * a) {
    return a->kv_type == MLA_TYPE_Q8_0 || a->n_head > 32 ? decode_fast_qpack_bytes(a->n_tok, 1) : 0;
}

int make_plan(const mla_attn_args * a, Plan * pl) {
    const int rc = validate(a);
    if (rc) return rc;
    const int64_t n_rows  = (int64_t) a->n_tok * a->n_head;
    const int64_t max_len = a->block_table ? a->bt_stride * MLA_PAGE_TOKENS : a->n_kv;
    *pl = Plan{};
    // The replay of the reference's own arithmetic (mla_ref_scores_kernel, mla_ref_walk_kernel): asked for by flag, and taken by
    // itself for a Q8_0 cache of at most one page per sequence -- with so few keys one of them can carry a row, and then the
    // 16-bit operands the matrix cores are fed (q * d has 19 significant bits) show in single output elements -- while the walk
    // stays short: rows x keys up to what 16 384 rows over a full page are
    const bool q8_small = a->kv_type == MLA_TYPE_Q8_0 && max_len <= MLA_PAGE_TOKENS && a->rows_per_wg == 0 &&
                          (int64_t) a->n_seq * n_rows * (max_len > 0 ? max_len : 1) <= (int64_t) 16384 * MLA_PAGE_TOKENS;
    if ((a->flags & (MLA_FLAG_F16_ACC_STRICT | MLA_FLAG_Q8_EXACT)) || q8_small) {
        pl->variant   = 1;
        pl->n_splits  = 1;
        pl->n_passes  = 1;
        pl->ws_scores = (size_t) a->n_seq * n_rows * (size_t) (max_len > 0 ? max_len : 1) * sizeof(float);
        pl->split_tokens = (int) max_len;
        return 0;
    }
    if (decode_fast_applicable(a) && a->rows_per_wg == 0) { pl->variant = 2; pl->n_passes = a->dv == 576 ? 2 : 1; pl->ndb = 16; pl->wm = 4; pl->wd = 1; }
    else if (a->dv == 576) { pl->n_passes = 2; pl->ndb = 9; pl->wm = 4; pl->wd = 1; }
    else {
        pl->n_passes = 1; pl->ndb = 16;
        int rpw = a->rows_per_wg;
        if (rpw == 0) rpw = n_rows > 32 ? 64 : 32;   // 128 rows per workgroup (4 x 1 waves) spills: 2.3 times slower than 64 (2 x 2) at 128 heads
        if (rpw == 128)     { pl->wm = 4; pl->wd = 1; }
        else if (rpw == 64) { pl->wm = 2; pl->wd = 2; }
        else                { pl->wm = 1; pl->wd = 4; }
    }
    pl->rblk         = 32 * pl->wm;
    pl->n_row_blocks = (int) ((n_rows + pl->rblk - 1) / pl->rblk);
    // split the KV range so that about two workgroups per CU exist (256 CUs), in units of whole pages
    int64_t n_pages = (max_len + MLA_PAGE_TOKENS - 1) / MLA_PAGE_TOKENS;
    if (n_pages < 1) n_pages = 1;
    int64_t splits = a->n_splits;
    if (splits == 0) {
        const int64_t wgs = (int64_t) a->n_seq * pl->n_row_blocks;
        splits = (256 + wgs - 1) / wgs;
        if (pl->wd > 1) splits *= 2;  // small-row shapes leave room for two workgroups per CU
    }
    // with a block table that kernel indexes at most 64 pages per split (63 with a mask, whose splits need not start on a page boundary)
    const int64_t max_pages = pl->variant == 2 && a->mask ? 63 : 64;
    if (pl->variant == 2 && a->block_table && splits * max_pages < n_pages) splits = (n_pages + max_pages - 1) / max_pages;
    if (splits > n_pages) splits = n_pages;
    if (splits < 1) splits = 1;
    const int64_t pages_per_split = (n_pages + splits - 1) / splits;
    pl->split_tokens = (int) (pages_per_split * MLA_PAGE_TOKENS);
    pl->n_splits     = (int) ((n_pages + pages_per_split - 1) / pages_per_split);
    // A launch that leaves most CUs without a workgroup even with one page per split and whose partials stay small (one or two short
    // sequences of a few heads: BASELINE's configs[0]) is split by 32-key tiles instead: the wave programs start a split at any tile
    // (a page holds four), and what a workgroup of such a launch spends per tile it saves in full (configs[0] 14.4 -> 13.0 us; one
    // sequence of 16 heads x 4096 keys 17.2 -> 14.9 us, two 19.1 -> 16.2 us).  Up to 4 MB of f32 partials for at most 32 rows, 1 MB
    // beyond (128 rows: a partial is 64 KB of f32, twice a tile of KV; every finer split measured slower there): past that the
    // combine pass loses more than the kernel gains (16 heads x 8192 keys in 256 splits: 17.5 -> 21.3 us).
    if (pl->variant == 2 && a->n_splits == 0 && pages_per_split == 1 && !a->mask && a->kv_type != MLA_TYPE_Q8_0) {
        const int64_t n_tiles = (max_len + TILE_TOK - 1) / TILE_TOK, wgs = (int64_t) a->n_seq * pl->n_row_blocks;
        const int64_t lim = (int64_t) (n_rows <= 32 ? 4 : 1) << 20;
        const int64_t want = std::min<int64_t>({ n_tiles, 256 / wgs, lim / ((int64_t) a->n_seq * n_rows * 512 * 4) });
        if (want > pl->n_splits) {
            const int64_t tiles_per_split = (n_tiles + want - 1) / want;
            pl->split_tokens = (int) (tiles_per_split * TILE_TOK);
            pl->n_splits     = (int) ((n_tiles + tiles_per_split - 1) / tiles_per_split);
        }
    }
    pl->lds_bytes    = pl->variant == 2 ? decode_fast_lds_bytes(decode_fast_q8_copy_rows(a) > 0 ? MLA_TYPE_F16 : a->kv_type) : 2 * TILE_BYTES + (a->kv_type == MLA_TYPE_Q8_0 ? Q8_TILE_RAW : 0);
    if (pl->variant == 2) pl->ws_qpack = decode_fast_qpack_bytes(a->n_seq, pl->n_row_blocks);
    if (pl->variant == 2) { pl->kvcopy_rows = decode_fast_q8_copy_rows(a); pl->ws_kvcopy = (size_t) pl->kvcopy_rows * ROW_BYTES; }
    if (pl->variant == 2 && a->mask) pl->ws_maskext = (size_t) pl->n_row_blocks * 16 * 2 * sizeof(int);  // 16 (first, last) pairs per row block
    if (pl->variant == 0 && a->mask) {
        // the general kernel visits only the key range the mask leaves open, when the extent pass can read the mask rows
        // (8-byte loads over whole groups of 8 keys)
        const int64_t nk = a->block_table ? a->bt_stride * MLA_PAGE_TOKENS : a->n_kv;
        if (nk % 8 == 0 && a->mask_ne0 >= nk && !(a->mask_nb1 & 7) && !((uintptr_t) a->mask & 7))
            pl->ws_maskext = (size_t) ((n_rows + 127) / 128) * 16 * 2 * sizeof(int);
    }
    // A paged decode batch (one row block per sequence, no mask) that needs KV splits anyway: the pipelined kernel's
    // workgroups take equal runs of the page list of all sequences instead of equal shares of the longest possible
    // sequence, so a ragged batch keeps every CU busy.  One workgroup per CU; a run must fit the 64 page ids a wave holds.
    // The same for a masked launch over one contiguous cache (the reference's batched decode): equal runs of the tiles of
    // the key ranges the row blocks may attend to.
    if (pl->variant == 2 && a->n_splits == 0 && pl->n_splits > 1 && !(a->flags & MLA_FLAG_UNIFORM_SPLITS)) {
        // (with at most one page per workgroup even when every sequence is full there is nothing to balance: the uniform
        // plan already hands out single pages, and the schedule itself costs a small batch 1.6 us)
        if (a->block_table && !a->mask && pl->n_row_blocks == 1 && a->n_seq <= 256 && (int64_t) a->n_seq * n_pages > 256 &&
            ((int64_t) a->n_seq * n_pages + 255) / 256 <= 64) {
            pl->balanced = 1; pl->n_units = a->n_seq;
        } else if (a->mask && !a->block_table && a->n_seq == 1 && pl->n_row_blocks <= 256) {
            pl->balanced = 2; pl->n_units = pl->n_row_blocks;
        }
        if (pl->balanced) {
            pl->n_wg = 256;
            pl->ws_sched = (size_t) ((pl->n_units + 1 + 63) / 64 * 64 + pl->n_wg * 8) * sizeof(int);
        }
    }
    // A paged decode batch of more than 256 sequences with a workgroup each runs in rounds: its sequences are taken longest first
    // (an order the pre-pass writes; ws_sched holds it)
    if (pl->variant == 2 && !pl->balanced && pl->n_splits == 1 && pl->n_row_blocks == 1 && a->block_table && !a->mask &&
        a->n_seq > 256 && a->n_seq <= 4096 && !(a->flags & MLA_FLAG_UNIFORM_SPLITS)) {
        pl->seq_sorted = 1;
        pl->ws_sched = (size_t) a->n_seq * sizeof(int);
    }
    if (token_form_candidate(a, *pl)) {
        pl->dual = 1;
        pl->ws_maskext = (size_t) a->n_tok * 16 * 2 * sizeof(int);   // 16 pairs per query token
        pl->ws_qpack  += token_image_bytes(a);
        pl->ws_sched   = (size_t) ((std::max(pl->n_units, a->n_tok) + 1 + 63) / 64 * 64 + pl->n_wg * 8) * sizeof(int);
    }
    if (pl->n_splits > 1) {
        // f32 partials while they are small (no second rounding of O on top of the MFMA operands' one), f16 beyond: there the
        // partial traffic counts, and the rounding (2^-12 relative per split) is averaged over long contexts
        // (the two forms of a launch issued in both share the area: the token form's n_wg + n_tok slots of n_head <= 32 rows fit
        // into the row-block form's n_wg + n_units slots of 128 rows)
        const size_t n_slots = pl->balanced ? (size_t) pl->n_wg + pl->n_units : (size_t) a->n_seq * pl->n_splits;
        const size_t slot_rows = pl->balanced == 2 ? 128 : (size_t) n_rows;
        const size_t n_part = n_slots * slot_rows * (pl->variant == 2 ? 512 : a->dv);
        pl->part_f32   = n_part * sizeof(float) <= ((size_t) 32 << 20);
        pl->ws_part_o  = n_part * (pl->part_f32 ? sizeof(float) : sizeof(_Float16));
        pl->ws_part_ml = n_slots * slot_rows * 2 * sizeof(float);
    }
    return 0;
}

size_t align256(size_t x) { return (x + 255) & ~(size_t) 255; }
size_t plan_ws(const Plan & pl) {
    return align256(pl.ws_part_o) + align256(pl.ws_part_ml) + align256(pl.ws_scores) + align256(pl.ws_qpack) + align256(pl.ws_maskext) + align256(pl.ws_sched) + align256(pl.ws_kvcopy);
}

template <int SRC, int NDB, int WM, int WD>
hipError_t launch_tile(const KParams & kp, dim3 grid, size_t lds, hipStream_t st) {
    auto kern = mla_attn_tile_kernel<SRC, NDB, WM, WD>;
    static bool attr_done[MLA_MAX_DEVICES];
    const hipError_t e = raise_lds_limit((const void *) kern, attr_done);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, grid, dim3(NTHREADS), lds, st, kp);
    return hipGetLastError();
}

template <int SRC>
hipError_t launch_tile_src(const Plan & pl, const KParams & kp, dim3 grid, hipStream_t st) {
    if (pl.ndb == 9) return launch_tile<SRC, 9, 4, 1>(kp, grid, pl.lds_bytes, st);
    if (pl.wm == 4) return launch_tile<SRC, 16, 4, 1>(kp, grid, pl.lds_bytes, st);
    if (pl.wm == 2) return launch_tile<SRC, 16, 2, 2>(kp, grid, pl.lds_bytes, st);
    return launch_tile<SRC, 16, 1, 4>(kp, grid, pl.lds_bytes, st);
}

}  // namespace

extern "C" {

const char * mla_attn_target_arch(void) { return "gfx950 (mla_attn tiled MFMA kernels, " __DATE__ ")"; }

size_t mla_attn_workspace_size(const mla_attn_args * args) {
    Plan pl;
    if (make_plan(args, &pl)) return 0;
    return plan_ws(pl);
}

int mla_attn_plan(const mla_attn_args * args, mla_attn_plan_info * out) {
    Plan pl;
    const int rc = make_plan(args, &pl);
    if (rc) return rc;
    if (!out) return MLA_ERR_NULL;
    const int a_n_seq = args->n_seq;
    out->variant      = pl.variant;
    out->rows_per_wg  = pl.rblk;
    out->n_row_blocks = pl.n_row_blocks;
    out->n_splits     = pl.n_splits;
    out->split_tokens = pl.split_tokens;
    out->n_passes     = pl.n_passes;
    out->lds_bytes    = (int64_t) pl.lds_bytes;
    out->balanced     = pl.dual ? 4 : pl.balanced;
    out->n_workgroups = pl.balanced ? pl.n_wg : pl.n_splits * pl.n_row_blocks * a_n_seq;
    return 0;
}

// phases: bit 0 = the attention kernels (partials or final output), bit 1 = the combine pass,
// bit 2 = the small passes ahead of the pipelined kernel (Q operand image, key extent of the mask)
static int launch_phases(const mla_attn_args * a, void * stream, int phases) {
    Plan pl;
    const int rc = make_plan(a, &pl);
    if (rc) return rc;
    const size_t need = plan_ws(pl);
    if (need > 0 && (!a->workspace || a->workspace_size < need || ((uintptr_t) a->workspace & 255))) return MLA_ERR_WORKSPACE;
    hipStream_t st = (hipStream_t) stream;

    KParams kp{};
    kp.q = (const char *) a->q; kp.q_nb1 = a->q_nb1; kp.q_nb2 = a->q_nb2; kp.q_nb3 = a->q_nb3;
    kp.kv = (const char *) a->kv; kp.kv_nb1 = a->kv_nb1; kp.kv_nb3 = a->kv_nb3; kp.n_kv = a->n_kv;
    kp.mask = (const char *) a->mask; kp.mask_nb1 = a->mask_nb1; kp.mask_ne0 = a->mask_ne0; kp.mask_nb3 = 0;   // (shared by the sequences, ggml-cpu.c:12024)
    kp.block_table = a->block_table; kp.bt_stride = a->bt_stride; kp.seq_lens = a->seq_lens;
    kp.dst = a->dst; kp.dst_stride = a->dst_nb1 / 4;
    kp.n_head = a->n_head; kp.n_tok = a->n_tok; kp.n_rows = a->n_tok * a->n_head;
    kp.n_splits = pl.n_splits; kp.split_tokens = pl.split_tokens;
    kp.dv_total = a->dv;
    kp.scale = a->scale; kp.softcap = a->logit_softcap; kp.max_bias = a->max_bias;
    kp.n_head_log2 = 1 << (int) floor(log2((double) a->n_head));
    kp.m0 = powf(2.0f, -(a->max_bias) / kp.n_head_log2);
    kp.m1 = powf(2.0f, -(a->max_bias / 2.0f) / kp.n_head_log2);
    { const float c = a->scale * LOG2E; memcpy(&kp.c_log2_bits, &c, 4); }
    kp.n_pool_pages = (int) (a->n_kv / MLA_PAGE_TOKENS);
    kp.rows_contig = a->kv_nb1 == (a->kv_type == MLA_TYPE_Q8_0 ? Q8_ROW : ROW_BYTES) && (((uintptr_t) a->kv & 15) == 0) &&
                     (a->block_table || (a->kv_nb3 & 15) == 0);
    char * ws = (char *) a->workspace;
    kp.part_o  = (_Float16 *) ws;
    kp.part_f32 = pl.part_f32;
    kp.rel_splits = a->mask != nullptr && (pl.variant == 2 || pl.ws_maskext > 0);
    kp.balanced = pl.balanced; kp.n_wg = pl.n_wg; kp.n_seq_sched = a->n_seq; kp.n_units = pl.n_units;
    kp.bf16_direct = (a->flags & MLA_FLAG_BF16_DIRECT) ? 1 : 0;
    kp.slot_rows = pl.balanced == 2 ? 128 : kp.n_rows;
    kp.part_ml = (float *) (ws + align256(pl.ws_part_o));
    float * scores = (float *) (ws + align256(pl.ws_part_o) + align256(pl.ws_part_ml));
    kp.q_pack = ws + align256(pl.ws_part_o) + align256(pl.ws_part_ml) + align256(pl.ws_scores);
    kp.mask_ext = pl.ws_maskext ? (int *) (ws + align256(pl.ws_part_o) + align256(pl.ws_part_ml) + align256(pl.ws_scores) + align256(pl.ws_qpack)) : nullptr;
    kp.sched = (int *) (ws + align256(pl.ws_part_o) + align256(pl.ws_part_ml) + align256(pl.ws_scores) + align256(pl.ws_qpack) + align256(pl.ws_maskext));
    kp.wg_first = kp.sched + (std::max(pl.n_units, pl.dual ? a->n_tok : 0) + 1 + 63) / 64 * 64;
    kp.seq_order = pl.seq_sorted ? kp.sched : nullptr;
    // the token form of a launch issued in two forms (see token_form_candidate): every query token a sequence of one token
    KParams kt = kp;
    if (pl.dual) {
        kp.dual = 1; kt.dual = 2;
        kp.form = kt.form = kp.wg_first;   // (a masked launch has no use for that table)
        kt.q_nb3 = a->q_nb1; kt.kv_nb3 = 0; kt.mask_nb3 = a->mask_nb1;
        kt.q_pack = (char *) kp.q_pack + decode_fast_qpack_bytes(a->n_seq, pl.n_row_blocks);   // (behind the row-block form's image)
        kt.n_tok = 1; kt.n_rows = a->n_head; kt.slot_rows = a->n_head;
        kt.balanced = 3; kt.n_units = a->n_tok; kt.n_seq_sched = a->n_tok;
    }

    if (pl.variant == 1) {
        if (!(phases & 1)) return 0;
        const int64_t max_len = a->block_table ? a->bt_stride * MLA_PAGE_TOKENS : a->n_kv;
        const bool q8 = a->kv_type == MLA_TYPE_Q8_0;
        if (max_len > 0) {
            dim3 g1((unsigned) ((max_len + 63) / 64), (unsigned) kp.n_rows, (unsigned) a->n_seq);
            if (q8) hipLaunchKernelGGL(mla_ref_scores_kernel<MLA_TYPE_Q8_0>, g1, dim3(256), 0, st, kp, scores, max_len);
            else    hipLaunchKernelGGL(mla_ref_scores_kernel<MLA_TYPE_F16>, g1, dim3(256), 0, st, kp, scores, max_len);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return (int) e;
        }
        dim3 g2((unsigned) kp.n_rows, (unsigned) a->n_seq);
        if (q8) hipLaunchKernelGGL(mla_ref_walk_kernel<MLA_TYPE_Q8_0>, g2, dim3(a->dv == 576 ? 576 : 512), 0, st, kp, (const float *) scores, max_len);
        else    hipLaunchKernelGGL(mla_ref_walk_kernel<MLA_TYPE_F16>, g2, dim3(a->dv == 576 ? 576 : 512), 0, st, kp, (const float *) scores, max_len);
        return (int) hipGetLastError();
    }

    dim3 grid((unsigned) pl.n_splits, (unsigned) pl.n_row_blocks, (unsigned) a->n_seq);
    if (pl.balanced) grid = dim3((unsigned) pl.n_wg, 1, 1);
    int kv_type = a->kv_type;
    if (pl.kvcopy_rows > 0) {
        // Q8_0 cache + mask that the Q8_0 wave program cannot copy as raw tiles: expand the cache to f16 rows (a pre-pass like
        // the Q image) and run the masked f16 build on them
        char * copy = ws + align256(pl.ws_part_o) + align256(pl.ws_part_ml) + align256(pl.ws_scores) + align256(pl.ws_qpack) + align256(pl.ws_maskext) + align256(pl.ws_sched);
        if (phases & 4) {
            const hipError_t e = launch_q8_to_f16(kp.kv, kp.kv_nb1, kp.kv_nb3, a->n_kv, copy, pl.kvcopy_rows, st);
            if (e != hipSuccess) return (int) e;
        }
        kp.kv = copy; kp.kv_nb1 = ROW_BYTES; kp.kv_nb3 = kp.kv_nb3 ? a->n_kv * ROW_BYTES : 0;
        kp.rows_contig = 1; kp.q_as_q8 = 1;
        kv_type = MLA_TYPE_F16;
    }
    const bool scan_mask = !(a->flags & MLA_FLAG_MASK_EXTENTS_VALID);
    if (pl.variant == 0 && kp.mask_ext && (phases & 4) && scan_mask) {
        const hipError_t e = launch_mask_extent(kp, st);
        if (e != hipSuccess) return (int) e;
    }
    auto combine = [&](int dv) -> int {
        const int splits_per_row = pl.balanced ? (pl.n_wg + pl.n_units - 1) / pl.n_units : pl.n_splits;
        if (pl.part_f32 && splits_per_row > 32) {   // (one or two sequences: the waves of a block share the walk over a row's splits)
            dim3 gw((unsigned) kp.n_rows, (unsigned) ((dv / 4 + 63) / 64), (unsigned) a->n_seq);
            hipLaunchKernelGGL(mla_attn_combine_f32_wide_kernel, gw, dim3(256), 0, st, kp);
            return (int) hipGetLastError();
        }
        if (pl.part_f32) {
            const int groups = dv / 4, rows_per_block = 256 / groups;   // 128 -> 2 rows, 144 -> 1 row
            dim3 g((unsigned) ((kp.n_rows + rows_per_block - 1) / rows_per_block), 1, (unsigned) a->n_seq);
            hipLaunchKernelGGL(mla_attn_combine_f32_kernel, g, dim3(256), 0, st, kp, groups);
            return (int) hipGetLastError();
        }
        // rows with many splits (few long sequences): four lanes share the walk over a row's splits
        if (splits_per_row > 128) {   // (sixteen lanes pay from about 200 splits on: 256 splits 72.1 -> 67.7 us per step, 128 splits 64.1 -> 67.8)
            dim3 gw((unsigned) ((kp.n_rows + 3) / 4), (unsigned) ((dv + 31) / 32), (unsigned) a->n_seq);
            hipLaunchKernelGGL(mla_attn_combine_wide_kernel<16>, gw, dim3(256), 0, st, kp);
            return (int) hipGetLastError();
        }
        if (splits_per_row > 16) {
            dim3 gw((unsigned) ((kp.n_rows + 15) / 16), (unsigned) ((dv + 31) / 32), (unsigned) a->n_seq);
            hipLaunchKernelGGL(mla_attn_combine_wide_kernel<4>, gw, dim3(256), 0, st, kp);
            return (int) hipGetLastError();
        }
        dim3 g((unsigned) ((kp.n_rows + 15) / 16), (unsigned) ((dv + 255) / 256), (unsigned) a->n_seq);
        hipLaunchKernelGGL(mla_attn_combine_kernel, g, dim3(256), 0, st, kp);
        return (int) hipGetLastError();
    };
    if (pl.variant == 2) {
        // the pipelined kernel produces 512 columns per pass; a 576-wide V (V := K, the form ggml-cpu accepts) takes a second
        // pass with V = columns 64 .. 575 of the rows, whose results land on columns 64 .. 575 of dst (64 .. 511 twice, with
        // the same values: the same P and the same accumulation order).  Each pass has its own combine.
        kp.dv_total = 512;
        for (int pass = 0; pass < pl.n_passes; pass++) {
            kp.v_col0 = pass * 64;
            if (phases & 1) {
                kt.v_col0 = kp.v_col0; kt.dv_total = kp.dv_total;
                const hipError_t e = launch_decode_fast(kp, kv_type, grid, st, (phases & 4) != 0 && pass == 0, pl.dual ? &kt : nullptr, scan_mask);
                if (e != hipSuccess) return (int) e;
            }
            // the partials of a pass are consumed before the next pass overwrites them; a combine-only call finishes the last pass
            const bool last = pass + 1 == pl.n_passes;
            if (pl.n_splits > 1 && ((phases & 1) ? (!last || (phases & 2)) : (last && (phases & 2)))) {
                const int rc2 = combine(512);
                if (rc2) return rc2;
            }
        }
        return 0;
    }
    for (int pass = 0; pass < pl.n_passes && (phases & 1); pass++) {
        kp.d_off = pass * pl.ndb * 32;
        hipError_t e;
        switch (a->kv_type) {
            case MLA_TYPE_BF16: e = launch_tile_src<SRC_BF16>(pl, kp, grid, st); break;
            case MLA_TYPE_F16:  e = launch_tile_src<SRC_F16>(pl, kp, grid, st); break;
            default:            e = launch_tile_src<SRC_Q8>(pl, kp, grid, st); break;
        }
        if (e != hipSuccess) return (int) e;
    }
    if (pl.n_splits > 1 && (phases & 2)) return combine(a->dv);
    return 0;
}

int mla_attn_launch(const mla_attn_args * a, void * stream) { return launch_phases(a, stream, 7); }

// mla_attn_launch for callers that cannot allocate a workspace: the split-K partials, the Q operand image, the mask extents
// and the schedule live in a file-scope device array.  Each device holds its own copy of the array at its own address, which
// hipGetSymbolAddress returns with that device current (looked up once per device, on the first call there); the kernels get
// that address exactly as they get a caller's workspace.  Nothing in the array has to start at zero: every kernel writes what a
// later kernel of the same call reads.  Calls that overlap in time on one device share the array and race.
int mla_attn_launch_static(const mla_attn_args * a, void * stream) {
    if (!a) return MLA_ERR_NULL;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int) e;
    if (dev < 0 || dev >= MLA_MAX_DEVICES) return (int) hipErrorInvalidDevice;
    void * ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {   // (two threads that get here together look up the same address)
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int) e;
        if (!ptr) return (int) hipErrorInvalidSymbol;
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    mla_attn_args b = *a;
    b.workspace      = nullptr;
    b.workspace_size = 0;
    Plan pl;
    const int rc = make_plan(&b, &pl);
    if (rc) return rc;
    if (plan_ws(pl) > MLA_ATTN_STATIC_WORKSPACE_MAX) return MLA_ERR_TOO_LARGE;
    b.workspace      = ptr;
    b.workspace_size = MLA_ATTN_STATIC_WORKSPACE_MAX;
    return launch_phases(&b, stream, 7);
}
int mla_attn_launch_partials(const mla_attn_args * a, void * stream) { return launch_phases(a, stream, 5); }
int mla_attn_launch_kernel(const mla_attn_args * a, void * stream) { return launch_phases(a, stream, 1); }
int mla_attn_launch_combine(const mla_attn_args * a, void * stream) { return launch_phases(a, stream, 2); }

int mla_hbm_copy_launch(const void * src, void * dst, size_t n_bytes, void * stream) {
    if (!src || !dst) return MLA_ERR_NULL;
    if ((n_bytes & 15) || ((uintptr_t) src & 15) || ((uintptr_t) dst & 15)) return MLA_ERR_BAD_ALIGNMENT;
    if (n_bytes == 0) return 0;
    hipLaunchKernelGGL(mla_hbm_copy_kernel, dim3(2048), dim3(256), 0, (hipStream_t) stream, (const u32x4 *) src, (u32x4 *) dst, n_bytes / 16);
    return (int) hipGetLastError();
}

}  // extern "C"
