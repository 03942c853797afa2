// Workgroup bodies of the kernels either side of the attention node (rotary embedding, the absorb products at decode
// size, strided f32 copies, the cache write), each as a device function of (parameters, block index, LDS): the kernels of
// mla_front.hip and mla_kv_write.hip are these bodies under their own names, and mla_front_batch_kernel runs several
// independent ones in one dispatch, a range of workgroups each.  The host side that turns an argument block of the C ABI
// into a body's parameters and grid lives here too, so that a launch on its own and a launch inside a batch are the
// same work.
#pragma once

#include <math.h>

#include "mla_common.hpp"
#include "../../include/mla_front.h"
#include "../../include/mla_kv_write.h"

namespace mla {
namespace front {

struct Blk { unsigned x, y, z, gx; };   // the body's block index, and its grid's x extent

// Workgroups are handed to the 8 XCDs round-robin in dispatch order, and each XCD has its own L2.  The n tiles of a product that
// share their activation rows (the same y, z; consecutive x) would land on different XCDs, each of which fetches those rows for
// itself (the un-absorb product of a 128-head decode step: 50 MB fetched for 25 MB of operands).  With the grid's first block on
// XCD 0 and a block count that is a multiple of 8, block l runs on XCD l % 8: it takes the tuple number (l % 8) * G / 8 + l / 8, so
// that consecutive tuples -- the n tiles of one set of rows -- share an XCD.
__device__ __forceinline__ Blk xcd_grouped(const Blk b, unsigned gy, unsigned gz) {
    const unsigned G = b.gx * gy * gz;
    if ((G & 7) != 0 || b.gx == 1) return b;
    const unsigned l = (b.z * gy + b.y) * b.gx + b.x;
    const unsigned v = (l & 7) * (G >> 3) + (l >> 3);
    return Blk{ v % b.gx, (v / b.gx) % gy, v / (b.gx * gy), b.gx };
}

// ---------------------------------------------------------------- rotary embedding

constexpr int ROPE_MAX_PAIRS = 256;

// What the (cos, sin) pair of a (position, pair) depends on.
struct RopeC {
    const int32_t * pos; const float * ff;
    int   n_dims;
    float theta_scale, freq_scale, ext_factor, mscale, corr0, corr1;
};

struct RopeP {
    const char * src; char * dst;
    int64_t ne0, ne1;
    int64_t s_nb1, s_nb2, s_nb3, d_nb1, d_nb2, d_nb3;
    RopeC c;
    int   neox, heads_per_wg, vec2;
};

// theta of pair `pair` at position `pos`: the position multiplied by theta_scale once per pair, in f32, in order
// (ggml/src/ggml-cpu/ggml-cpu.c:10295-10307)
__device__ __forceinline__ float rope_theta(const RopeC & c, int pos, int pair) {
    float theta = (float) pos;
    for (int i = 0; i < pair; i++) theta = __fmul_rn(theta, c.theta_scale);
    return theta;
}

// (cos, sin) of a pair from its theta, with the YaRN blend and the magnitude scale (ggml-cpu.c:10272-10293)
__device__ __forceinline__ float2 rope_cs(const RopeC & c, float theta, int pair) {
    const float extrap = __fdiv_rn(theta, c.ff ? c.ff[pair] : 1.0f);
    const float interp = __fmul_rn(c.freq_scale, extrap);
    float       th     = interp;
    if (c.ext_factor != 0.0f) {
        const float y    = __fdiv_rn(__fsub_rn((float) pair, c.corr0), fmaxf(0.001f, __fsub_rn(c.corr1, c.corr0)));
        const float ramp = __fsub_rn(1.0f, fminf(1.0f, fmaxf(0.0f, y)));
        const float mix  = __fmul_rn(ramp, c.ext_factor);
        th = fmaf(interp, __fsub_rn(1.0f, mix), __fmul_rn(extrap, mix));
    }
    return make_float2(__fmul_rn(cosf(th), c.mscale), __fmul_rn(sinf(th), c.mscale));
}

__device__ __forceinline__ void rope_rotate(float x0, float x1, float2 c, float & y0, float & y1) {
    y0 = fmaf(x0, c.x, -__fmul_rn(x1, c.y));
    y1 = fmaf(x0, c.y, __fmul_rn(x1, c.x));
}

constexpr int ROPE_LDS = ROPE_MAX_PAIRS * 8;

__device__ __forceinline__ void rope_body(const RopeP & p, const Blk b, char * lds) {
    float2 * cs = (float2 *) lds;
    const int     n_pairs = p.c.n_dims / 2;
    const int64_t i2 = b.y, i3 = b.z;
    for (int pair = threadIdx.x; pair < n_pairs; pair += 256) cs[pair] = rope_cs(p.c, rope_theta(p.c, p.c.pos[i2], pair), pair);
    __syncthreads();
    const int64_t h0 = (int64_t) b.x * p.heads_per_wg;
    const int     nh = (int) min((int64_t) p.heads_per_wg, p.ne1 - h0);
    const char *  s  = p.src + i3 * p.s_nb3 + i2 * p.s_nb2 + h0 * p.s_nb1;
    char *        d  = p.dst + i3 * p.d_nb3 + i2 * p.d_nb2 + h0 * p.d_nb1;
    for (int idx = threadIdx.x; idx < nh * n_pairs; idx += 256) {
        const int    h = idx / n_pairs, pair = idx - h * n_pairs;
        const float2 c = cs[pair];
        const float * sr = (const float *) (s + h * p.s_nb1);
        float *       dr = (float *) (d + h * p.d_nb1);
        float x0, x1, y0, y1;
        const int a = p.neox ? pair : 2 * pair, bb = p.neox ? pair + n_pairs : 2 * pair + 1;
        if (p.vec2) { const float2 v = *(const float2 *) (sr + a); x0 = v.x; x1 = v.y; }
        else        { x0 = sr[a]; x1 = sr[bb]; }
        rope_rotate(x0, x1, c, y0, y1);
        if (p.vec2) *(float2 *) (dr + a) = make_float2(y0, y1);
        else        { dr[a] = y0; dr[bb] = y1; }
    }
    const int tail = (int) (p.ne0 - p.c.n_dims);  // channels past n_dims are copied (ggml-cpu.c:10535-10546)
    if (tail > 0 && p.src != p.dst)
        for (int idx = threadIdx.x; idx < nh * tail; idx += 256) {
            const int h = idx / tail, i = p.c.n_dims + idx - h * tail;
            ((float *) (d + h * p.d_nb1))[i] = ((const float *) (s + h * p.s_nb1))[i];
        }
}

// ---------------------------------------------------------------- absorb products, decode size

struct MmP {
    const char * w; const char * x; char * dst;
    int64_t K, N, M, ne2;
    int64_t w_nb1, w_nb2, w_nb3, x_nb1, x_nb2, x_nb3, d_nb1, d_nb2, d_nb3;
    int64_t r2, r3;
};

constexpr int MM_KC    = 128;              // K chunk
constexpr int MM_PITCH = MM_KC * 2 + 16;   // LDS row pitch of the rounded activations: 68 dwords, conflict-free b128 reads
template <int MB> constexpr int MM_LDS = MB * 32 * MM_PITCH;

template <bool F16, int MB>
__device__ __forceinline__ void mm_body(const MmP & p, const Blk b, char * lds) {
    const int     lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t i2 = b.z % p.ne2, i3 = b.z / p.ne2;
    const char *  W  = p.w + (i2 / p.r2) * p.w_nb2 + (i3 / p.r3) * p.w_nb3;
    const char *  X  = p.x + i2 * p.x_nb2 + i3 * p.x_nb3;
    char *        D  = p.dst + i2 * p.d_nb2 + i3 * p.d_nb3;
    const int64_t n0 = (int64_t) b.x * 128 + wave * 32, m0 = (int64_t) b.y * (32 * MB);
    const char *  wrow = W + min(n0 + (lane & 31), p.N - 1) * p.w_nb1 + (lane >> 5) * 16;
    const bool    wave_active = n0 < p.N;  // whole n block outside the matrix: still takes part in the barriers

    f32x16 acc[MB];
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
        for (int j = 0; j < 16; j++) acc[i][j] = 0.f;

    auto load_w = [&](u32x4 (&f)[MM_KC / 16], int64_t k0) {
#pragma unroll
        for (int ks = 0; ks < MM_KC / 16; ks++) {
            const int64_t k = min(k0 + ks * 16, p.K - 16);  // past the end: any valid address, the fragment is not used
            f[ks] = *(const u32x4 *) (wrow + k * 2);
        }
    };
    u32x4 wf[MM_KC / 16], wn[MM_KC / 16];
    if (wave_active) load_w(wf, 0);

    for (int64_t k0 = 0; k0 < p.K; k0 += MM_KC) {
        const int kc = (int) min((int64_t) MM_KC, p.K - k0), groups = kc / 8;
        __syncthreads();
        for (int g = threadIdx.x; g < MB * 32 * groups; g += 256) {
            const int     r = g / groups, kg = g - r * groups;
            const int64_t m = m0 + r;
            u32x4         v = { 0u, 0u, 0u, 0u };
            if (m < p.M) {
                const float4 * src = (const float4 *) (X + m * p.x_nb1 + (k0 + kg * 8) * 4);
                const float4   a = src[0], c = src[1];
                v[0] = pack2<F16>(a.x, a.y); v[1] = pack2<F16>(a.z, a.w);
                v[2] = pack2<F16>(c.x, c.y); v[3] = pack2<F16>(c.z, c.w);
            }
            *(u32x4 *) (lds + r * MM_PITCH + kg * 16) = v;
        }
        if (wave_active && k0 + MM_KC < p.K) load_w(wn, k0 + MM_KC);
        __syncthreads();
        if (wave_active) {
#pragma unroll
            for (int ks = 0; ks < MM_KC / 16; ks++)
                if (ks * 16 < kc) {
#pragma unroll
                    for (int mb = 0; mb < MB; mb++) {
                        const u32x4 af = *(const u32x4 *) (lds + (mb * 32 + (lane & 31)) * MM_PITCH + ks * 32 + (lane >> 5) * 16);
                        acc[mb] = mfma32<F16>(af, wf[ks], acc[mb]);
                    }
                }
#pragma unroll
            for (int ks = 0; ks < MM_KC / 16; ks++) wf[ks] = wn[ks];
        }
    }
    if (!wave_active) return;
    const int64_t n = n0 + (lane & 31);
    if (n >= p.N) return;
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const int64_t m = m0 + mb * 32 + (j >> 2) * 8 + (lane >> 5) * 4 + (j & 3);
            if (m < p.M) ((float *) (D + m * p.d_nb1))[n] = acc[mb][j];
        }
}

// Few rows m (a decode step) and too few 128-wide tiles to fill the chip: a workgroup owns 32 outputs n and 32 rows m, and
// both operands come through LDS.  Loading MFMA fragments straight from global memory fetches 16 bytes per lane from 32
// different rows per instruction, and the texture addresser takes those one row at a time (that form ran the un-absorb
// product of a 128-head layer at 32 tokens in 12.5 us, this one in 11.2); here the workgroup copies its 32 weight rows and
// its 32 activation rows chunk by chunk (256 k) with loads that run along the rows (a wave covers two whole 512-byte
// weight rows, or one 1 KB piece of an f32 activation row, per instruction), rounds the activations on the way, and the
// four waves take every fourth k-step of 16 out of LDS; their partial accumulators meet in LDS.  The grid is
// (N / 32) x (M / 32) x batches workgroups, enough to keep the weight stream of a 128-head layer in flight on every CU.
constexpr int MS_KC = 256, MS_PITCH = MS_KC * 2 + 16;
constexpr int MS_LDS = 2 * 32 * MS_PITCH + 4 * 16 * 64 * 4;

template <bool F16>
__device__ __forceinline__ void mm_small_body(const MmP & p, const Blk b, char * lds) {
    char * ws = lds;
    char * xs = lds + 32 * MS_PITCH;
    float (*red)[16][64] = (float (*)[16][64]) (lds + 2 * 32 * MS_PITCH);
    const int     lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t i2 = b.z % p.ne2, i3 = b.z / p.ne2;
    const int64_t n0 = (int64_t) b.x * 32, m0 = (int64_t) b.y * 32;
    const char *  W = p.w + (i2 / p.r2) * p.w_nb2 + (i3 / p.r3) * p.w_nb3;
    const char *  X = p.x + i2 * p.x_nb2 + i3 * p.x_nb3;
    f32x16 acc;
#pragma unroll
    for (int j = 0; j < 16; j++) acc[j] = 0.f;
    for (int64_t k0 = 0; k0 < p.K; k0 += MS_KC) {
        const int kc = (int) min((int64_t) MS_KC, p.K - k0), groups = kc / 8, units = 32 * groups;   // a unit: 8 values of one row
        u32x4  wv[4];
        float4 xa[4], xb[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int u = min((int) threadIdx.x + 256 * i, units - 1), row = u / groups, c = u - row * groups;
            wv[i] = *(const u32x4 *) (W + min(n0 + row, p.N - 1) * p.w_nb1 + (k0 + c * 8) * 2);
            const char * xr = X + min(m0 + row, p.M - 1) * p.x_nb1 + (k0 + c * 8) * 4;
            xa[i] = *(const float4 *) xr;
            xb[i] = *(const float4 *) (xr + 16);
        }
        if (k0) __syncthreads();   // every wave is done with the previous chunk
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int u = (int) threadIdx.x + 256 * i;
            if (u < units) {
                const int row = u / groups, c = u - row * groups;
                *(u32x4 *) (ws + row * MS_PITCH + c * 16) = wv[i];
                *(u32x4 *) (xs + row * MS_PITCH + c * 16) = u32x4{ pack2<F16>(xa[i].x, xa[i].y), pack2<F16>(xa[i].z, xa[i].w),
                                                                    pack2<F16>(xb[i].x, xb[i].y), pack2<F16>(xb[i].z, xb[i].w) };
            }
        }
        __syncthreads();
        for (int ks = wave; ks < kc / 16; ks += 4) {
            const int    off = (lane & 31) * MS_PITCH + ks * 32 + (lane >> 5) * 16;
            const u32x4 af = *(const u32x4 *) (xs + off), wf = *(const u32x4 *) (ws + off);
            acc = mfma32<F16>(af, wf, acc);
        }
    }
#pragma unroll
    for (int j = 0; j < 16; j++) red[wave][j][lane] = acc[j];
    __syncthreads();
    const int64_t n = n0 + (lane & 31);
    char * D = p.dst + i2 * p.d_nb2 + i3 * p.d_nb3;
#pragma unroll
    for (int jj = 0; jj < 4; jj++) {   // wave w finishes accumulator registers 4w .. 4w+3 (8 rows m)
        const int     j = wave * 4 + jj;
        const float   v = (red[0][j][lane] + red[1][j][lane]) + (red[2][j][lane] + red[3][j][lane]);
        const int64_t m = m0 + (j >> 2) * 8 + (lane >> 5) * 4 + (j & 3);
        if (m < p.M && n < p.N) ((float *) (D + m * p.d_nb1))[n] = v;
    }
}

// ---------------------------------------------------------------- strided f32 copies

struct CopyP {
    const char * src; char * dst;
    int64_t ne0, ne1, ne2, total;   // ne0 in units of `VEC` floats; total = units to copy
    int64_t s_nb1, s_nb2, s_nb3, d_nb1, d_nb2, d_nb3;
};

template <typename T>
__device__ __forceinline__ void copy_body(const CopyP & p, const Blk b) {
    for (int64_t i = (int64_t) b.x * 256 + threadIdx.x; i < p.total; i += (int64_t) b.gx * 256) {
        const int64_t i0 = i % p.ne0, r = i / p.ne0;
        const int64_t i1 = r % p.ne1, r2 = r / p.ne1;
        const int64_t i2 = r2 % p.ne2, i3 = r2 / p.ne2;
        ((T *) (p.dst + i3 * p.d_nb3 + i2 * p.d_nb2 + i1 * p.d_nb1))[i0] = ((const T *) (p.src + i3 * p.s_nb3 + i2 * p.s_nb2 + i1 * p.s_nb1))[i0];
    }
}

// ---------------------------------------------------------------- the cache write

struct WParams {
    const char * src; int64_t src_nb1;
    char * kv; int64_t kv_nb1, n_kv_rows, row0;
    const void * rows; int rows_i64;
    const int32_t * block_table; int64_t bt_stride;
    const int32_t * seq_ids; const int32_t * positions;
    int n_tok;
    // ROPE form: the last 64 values of a row come from `k_pe` (rows k_pe_nb1 bytes apart) and are rotated on the way
    const char * k_pe; int64_t k_pe_nb1;
    RopeC rope;
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

// One thread = 8 consecutive values of a row (72 threads per row): two 16-byte loads, one 16-byte store for the 16-bit
// types.  Q8_0: the 4 threads of a 32-value block (an aligned lane quad) agree on amax with two shuffles, then every
// thread writes its 8 int8 values and the quarter-0 thread the block scale, the way ggml-cpu's x86 quantizer does it
// (ggml-cpu-quants.c:855-900: d = amax/127 stored as f16, id = 127/amax, round half to even).
// KVT: SRC_BF16 / SRC_F16 / SRC_Q8.  CONVERT: source rows are f32; otherwise they already have the cache type.
// ROPE (with CONVERT): values 512 .. 575 of a row are the rotated k_pe of the token (adjacent pairs, 32 of them: a thread
// holds four) -- rope_ext(k_pe), concat(kv_compressed, k_pe) and the copy into the cache in one pass
// (src/llama-graph-deepseek2.cpp:226-236, src/llama-graph-attn.cpp:236-241), with the arithmetic of rope_body.
template <int KVT, bool CONVERT, bool ROPE>
__device__ __forceinline__ void kv_write_body(const WParams & p, const Blk b) {
    constexpr int GROUPS = CONVERT || KVT != SRC_Q8 ? 72 : 0;   // 8-value groups per row
    if constexpr (!CONVERT) {
        // raw row copy: 16-bit rows are 72 chunks of 16 bytes; Q8_0 rows are 153 words of 4 bytes
        constexpr int UNITS = KVT == SRC_Q8 ? Q8_ROW / 4 : 72;
        const int64_t gid = (int64_t) b.x * 256 + threadIdx.x;
        const int t = (int) (gid / UNITS), u = (int) (gid - (int64_t) t * UNITS);
        if (t >= p.n_tok) return;
        const int64_t r = dest_row(p, t);
        if (r < 0 || r >= p.n_kv_rows) return;
        if constexpr (KVT == SRC_Q8) *(unsigned *) (p.kv + r * p.kv_nb1 + 4 * u) = *(const unsigned *) (p.src + (int64_t) t * p.src_nb1 + 4 * u);
        else *(u32x4 *) (p.kv + r * p.kv_nb1 + 16 * u) = *(const u32x4 *) (p.src + (int64_t) t * p.src_nb1 + 16 * u);
        return;
    } else {
        const int64_t gid = (int64_t) b.x * 256 + threadIdx.x;
        const int t = (int) (gid / GROUPS), u = (int) (gid - (int64_t) t * GROUPS);
        const bool live = t < p.n_tok;
        const int tc = live ? t : p.n_tok - 1;
        const bool from_pe = ROPE && u >= 64;
        const float * s = from_pe ? (const float *) (p.k_pe + (int64_t) tc * p.k_pe_nb1) + 8 * (u - 64)
                                  : (const float *) (p.src + (int64_t) tc * p.src_nb1) + 8 * u;
        const f32x4 x0 = *(const f32x4 *) s, x1 = *(const f32x4 *) (s + 4);
        float x[8] = { x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w };
        if constexpr (ROPE) {
            if (from_pe) {
                const int pair0 = 4 * (u - 64);
                float theta = rope_theta(p.rope, p.rope.pos[tc], pair0);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float2 c = rope_cs(p.rope, theta, pair0 + i);
                    float y0, y1;
                    rope_rotate(x[2 * i], x[2 * i + 1], c, y0, y1);
                    x[2 * i] = y0; x[2 * i + 1] = y1;
                    theta = __fmul_rn(theta, p.rope.theta_scale);
                }
            }
        }
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
            const int bi = u >> 2, qt = u & 3;
            char * blk = p.kv + r * p.kv_nb1 + 34 * bi;
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

// ---------------------------------------------------------------- host: argument block -> parameters and grid

inline bool al16(const void * ptr) { return ((uintptr_t) ptr & 15) == 0; }

// host-side constants of the rotary embedding, evaluated as the reference evaluates them (ggml-cpu.c:10409-10412,
// ggml.c:3529-3541, ggml-cpu.c:10289)
inline void make_rope_consts(const mla_rope_args * a, RopeC * c) {
    c->pos = a->pos; c->ff = a->freq_factors;
    c->n_dims = a->n_dims;
    c->theta_scale = powf(a->freq_base, -2.0f / a->n_dims);
    const float two_log_base = 2 * logf(a->freq_base);
    const float start = floorf(a->n_dims * logf(a->n_ctx_orig / (a->beta_fast * 2 * (float) M_PI)) / two_log_base);
    const float end   = ceilf(a->n_dims * logf(a->n_ctx_orig / (a->beta_slow * 2 * (float) M_PI)) / two_log_base);
    c->corr0 = start > 0 ? start : 0;
    c->corr1 = end < a->n_dims - 1 ? end : (float) (a->n_dims - 1);
    c->freq_scale = a->freq_scale; c->ext_factor = a->ext_factor;
    c->mscale = a->attn_factor;
    // 1 + 0.1 log(1/s) as one fused multiply-add: what an FMA-enabled x86 build of the reference evaluates
    if (a->ext_factor != 0.0f) c->mscale *= fmaf(0.1f, logf(1.0f / a->freq_scale), 1.0f);
}

inline dim3 make_rope_params(const mla_rope_args * a, RopeP * p) {
    p->src = (const char *) a->src; p->dst = (char *) a->dst;
    p->ne0 = a->ne[0]; p->ne1 = a->ne[1];
    p->s_nb1 = a->src_nb[1]; p->s_nb2 = a->src_nb[2]; p->s_nb3 = a->src_nb[3];
    p->d_nb1 = a->dst_nb[1]; p->d_nb2 = a->dst_nb[2]; p->d_nb3 = a->dst_nb[3];
    make_rope_consts(a, &p->c);
    p->neox = a->mode == MLA_ROPE_MODE_NEOX;
    bool v2 = !p->neox && !((uintptr_t) a->src & 7) && !((uintptr_t) a->dst & 7);
    for (int i = 1; i < 4; i++) v2 = v2 && !(a->src_nb[i] & 7) && !(a->dst_nb[i] & 7);
    p->vec2 = v2;
    const int n_pairs = a->n_dims / 2;
    int hpw = 1024 / n_pairs;  // about four passes of the 256 threads
    if (hpw < 1) hpw = 1;
    p->heads_per_wg = hpw;
    return dim3((unsigned) ((a->ne[1] + hpw - 1) / hpw), (unsigned) a->ne[2], (unsigned) a->ne[3]);
}

// The forms of the product kernels.  MM_STREAM (prefill chunks) and MM_TILE with more than 32 rows per workgroup have
// no body here: they run as launches of their own.
enum { MM_SMALL = 0, MM_TILE1 = 1, MM_TILE2 = 2, MM_TILE4 = 4, MM_STREAM = 8 };

inline int make_mm_params(const mla_mul_mat_args * a, MmP * p, dim3 * grid) {
    p->w = (const char *) a->w; p->x = (const char *) a->x; p->dst = (char *) a->dst;
    p->K = a->K; p->N = a->N; p->M = a->M; p->ne2 = a->ne2;
    p->w_nb1 = a->w_nb1; p->w_nb2 = a->w_nb2; p->w_nb3 = a->w_nb3;
    p->x_nb1 = a->x_nb1; p->x_nb2 = a->x_nb2; p->x_nb3 = a->x_nb3;
    p->d_nb1 = a->d_nb1; p->d_nb2 = a->d_nb2; p->d_nb3 = a->d_nb3;
    p->r2 = a->ne2 / a->w_ne2; p->r3 = a->ne3 / a->w_ne3;
    const int64_t  batches = a->ne2 * a->ne3;
    const unsigned gx = (unsigned) ((p->N + 127) / 128);
    if (p->M > 64 && (p->K == 128 || p->K == 256 || p->K == 512)) return MM_STREAM;
    if (p->M <= 64 && (int64_t) gx * ((p->M + 31) / 32) * batches < 512 && p->K >= 256) {
        // few rows and fewer than two workgroups per CU with 128-wide tiles: split n finer and K over the waves
        *grid = dim3((unsigned) ((p->N + 31) / 32), (unsigned) ((p->M + 31) / 32), (unsigned) batches);
        return MM_SMALL;
    }
    if (p->M <= 32) { *grid = dim3(gx, (unsigned) ((p->M + 31) / 32), (unsigned) batches); return MM_TILE1; }
    if (p->M <= 64) { *grid = dim3(gx, (unsigned) ((p->M + 63) / 64), (unsigned) batches); return MM_TILE2; }
    *grid = dim3(gx, (unsigned) ((p->M + 127) / 128), (unsigned) batches);
    return MM_TILE4;
}

inline bool make_copy_params(const mla_copy_args * a, CopyP * p, dim3 * grid) {   // returns: 16-byte vectors
    const int64_t n = a->ne[0] * a->ne[1] * a->ne[2] * a->ne[3];
    bool v4 = a->ne[0] % 4 == 0 && al16(a->src) && al16(a->dst);
    for (int i = 1; i < 4; i++) v4 = v4 && !(a->src_nb[i] & 15) && !(a->dst_nb[i] & 15);
    p->src = (const char *) a->src; p->dst = (char *) a->dst;
    p->ne0 = v4 ? a->ne[0] / 4 : a->ne[0]; p->ne1 = a->ne[1]; p->ne2 = a->ne[2];
    p->total = v4 ? n / 4 : n;
    p->s_nb1 = a->src_nb[1]; p->s_nb2 = a->src_nb[2]; p->s_nb3 = a->src_nb[3];
    p->d_nb1 = a->dst_nb[1]; p->d_nb2 = a->dst_nb[2]; p->d_nb3 = a->dst_nb[3];
    *grid = dim3((unsigned) min((p->total + 255) / 256, (int64_t) 8192));
    return v4;
}

inline dim3 make_kv_write_params(const mla_kv_write_args * a, WParams * p) {
    p->src = (const char *) a->src; p->src_nb1 = a->src_nb1;
    p->kv = (char *) a->kv; p->kv_nb1 = a->kv_nb1; p->n_kv_rows = a->n_kv_rows; p->row0 = a->row0;
    p->rows = a->rows; p->rows_i64 = a->rows_type;
    p->block_table = a->block_table; p->bt_stride = a->bt_stride; p->seq_ids = a->seq_ids; p->positions = a->positions;
    p->n_tok = a->n_tok;
    p->k_pe = nullptr; p->k_pe_nb1 = 0;
    p->rope = RopeC{};
    const bool convert = a->src_type == MLA_TYPE_F32;
    const int  units = convert || a->kv_type != MLA_TYPE_Q8_0 ? 72 : Q8_ROW / 4;
    return dim3((unsigned) (((int64_t) a->n_tok * units + 255) / 256));
}

inline dim3 make_kv_write_rope_params(const mla_kv_write_rope_args * a, WParams * p) {
    const dim3 grid = make_kv_write_params(&a->w, p);
    p->k_pe = (const char *) a->rope.src; p->k_pe_nb1 = a->rope.src_nb[2];
    make_rope_consts(&a->rope, &p->rope);
    return grid;
}

}  // namespace front
}  // namespace mla
