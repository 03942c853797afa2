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

#include "mla_common.hpp"
#include "../../include/mla_front.h"

using namespace mla;

namespace {

constexpr int ROPE_MAX_PAIRS = 256;

struct RopeP {
    const char * src; char * dst;
    int64_t ne0, ne1;
    int64_t s_nb1, s_nb2, s_nb3, d_nb1, d_nb2, d_nb3;
    const int32_t * pos; const float * ff;
    int   n_dims, neox, heads_per_wg, vec2;
    float theta_scale, freq_scale, ext_factor, mscale, corr0, corr1;
};

__global__ void __launch_bounds__(256) mla_rope_kernel(const RopeP p) {
    __shared__ float2 cs[ROPE_MAX_PAIRS];
    const int     n_pairs = p.n_dims / 2;
    const int64_t i2 = blockIdx.y, i3 = blockIdx.z;
    for (int pair = threadIdx.x; pair < n_pairs; pair += 256) {
        float theta = (float) p.pos[i2];
        for (int i = 0; i < pair; i++) theta = __fmul_rn(theta, p.theta_scale);
        const float extrap = __fdiv_rn(theta, p.ff ? p.ff[pair] : 1.0f);
        const float interp = __fmul_rn(p.freq_scale, extrap);
        float       th     = interp;
        if (p.ext_factor != 0.0f) {
            const float y    = __fdiv_rn(__fsub_rn((float) pair, p.corr0), fmaxf(0.001f, __fsub_rn(p.corr1, p.corr0)));
            const float ramp = __fsub_rn(1.0f, fminf(1.0f, fmaxf(0.0f, y)));
            const float mix  = __fmul_rn(ramp, p.ext_factor);
            th = fmaf(interp, __fsub_rn(1.0f, mix), __fmul_rn(extrap, mix));
        }
        cs[pair] = make_float2(__fmul_rn(cosf(th), p.mscale), __fmul_rn(sinf(th), p.mscale));
    }
    __syncthreads();
    const int64_t h0 = (int64_t) blockIdx.x * p.heads_per_wg;
    const int     nh = (int) min((int64_t) p.heads_per_wg, p.ne1 - h0);
    const char *  s  = p.src + i3 * p.s_nb3 + i2 * p.s_nb2 + h0 * p.s_nb1;
    char *        d  = p.dst + i3 * p.d_nb3 + i2 * p.d_nb2 + h0 * p.d_nb1;
    for (int idx = threadIdx.x; idx < nh * n_pairs; idx += 256) {
        const int    h = idx / n_pairs, pair = idx - h * n_pairs;
        const float2 c = cs[pair];
        const float * sr = (const float *) (s + h * p.s_nb1);
        float *       dr = (float *) (d + h * p.d_nb1);
        float x0, x1;
        const int a = p.neox ? pair : 2 * pair, b = p.neox ? pair + n_pairs : 2 * pair + 1;
        if (p.vec2) { const float2 v = *(const float2 *) (sr + a); x0 = v.x; x1 = v.y; }
        else        { x0 = sr[a]; x1 = sr[b]; }
        const float y0 = fmaf(x0, c.x, -__fmul_rn(x1, c.y));
        const float y1 = fmaf(x0, c.y, __fmul_rn(x1, c.x));
        if (p.vec2) *(float2 *) (dr + a) = make_float2(y0, y1);
        else        { dr[a] = y0; dr[b] = y1; }
    }
    const int tail = (int) (p.ne0 - p.n_dims);  // channels past n_dims are copied (ggml-cpu.c:10535-10546)
    if (tail > 0 && p.src != p.dst)
        for (int idx = threadIdx.x; idx < nh * tail; idx += 256) {
            const int h = idx / tail, i = p.n_dims + idx - h * tail;
            ((float *) (d + h * p.d_nb1))[i] = ((const float *) (s + h * p.s_nb1))[i];
        }
}

struct MmP {
    const char * w; const char * x; char * dst;
    int64_t K, N, M, ne2;
    int64_t w_nb1, w_nb2, w_nb3, x_nb1, x_nb2, x_nb3, d_nb1, d_nb2, d_nb3;
    int64_t r2, r3;
};

constexpr int MM_KC    = 128;              // K chunk
constexpr int MM_PITCH = MM_KC * 2 + 16;   // LDS row pitch of the rounded activations: 68 dwords, conflict-free b128 reads

template <bool F16, int MB>
__global__ void __launch_bounds__(256) mla_mul_mat_kernel(const MmP p) {
    __shared__ __attribute__((aligned(16))) char lds[MB * 32 * MM_PITCH];
    const int     lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t i2 = blockIdx.z % p.ne2, i3 = blockIdx.z / p.ne2;
    const char *  W  = p.w + (i2 / p.r2) * p.w_nb2 + (i3 / p.r3) * p.w_nb3;
    const char *  X  = p.x + i2 * p.x_nb2 + i3 * p.x_nb3;
    char *        D  = p.dst + i2 * p.d_nb2 + i3 * p.d_nb3;
    const int64_t n0 = (int64_t) blockIdx.x * 128 + wave * 32, m0 = (int64_t) blockIdx.y * (32 * MB);
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
                const float4   a = src[0], b = src[1];
                v[0] = pack2<F16>(a.x, a.y); v[1] = pack2<F16>(a.z, a.w);
                v[2] = pack2<F16>(b.x, b.y); v[3] = pack2<F16>(b.z, b.w);
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
template <bool F16>
__global__ void __launch_bounds__(256) mla_mul_mat_small_kernel(const MmP p) {
    __shared__ __attribute__((aligned(16))) char ws[32 * MS_PITCH];
    __shared__ __attribute__((aligned(16))) char xs[32 * MS_PITCH];
    __shared__ float red[4][16][64];
    const int     lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t i2 = blockIdx.z % p.ne2, i3 = blockIdx.z / p.ne2;
    const int64_t n0 = (int64_t) blockIdx.x * 32, m0 = (int64_t) blockIdx.y * 32;
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

template <bool F16>
hipError_t launch_mm(const MmP & p, int64_t batches, hipStream_t st) {
    if (p.M > 64 && (p.K == 128 || p.K == 256 || p.K == 512)) return launch_mm_stream<F16>(p, batches, st);
    const unsigned gx = (unsigned) ((p.N + 127) / 128);
    if (p.M <= 64 && (int64_t) gx * ((p.M + 31) / 32) * batches < 512 && p.K >= 256) {
        // few rows and fewer than two workgroups per CU with 128-wide tiles: split n finer and K over the waves
        hipLaunchKernelGGL((mla_mul_mat_small_kernel<F16>), dim3((unsigned) ((p.N + 31) / 32), (unsigned) ((p.M + 31) / 32), (unsigned) batches), dim3(256), 0, st, p);
    } else if (p.M <= 32) {
        hipLaunchKernelGGL((mla_mul_mat_kernel<F16, 1>), dim3(gx, (unsigned) ((p.M + 31) / 32), (unsigned) batches), dim3(256), 0, st, p);
    } else if (p.M <= 64) {
        hipLaunchKernelGGL((mla_mul_mat_kernel<F16, 2>), dim3(gx, (unsigned) ((p.M + 63) / 64), (unsigned) batches), dim3(256), 0, st, p);
    } else {
        hipLaunchKernelGGL((mla_mul_mat_kernel<F16, 4>), dim3(gx, (unsigned) ((p.M + 127) / 128), (unsigned) batches), dim3(256), 0, st, p);
    }
    return hipGetLastError();
}

struct CopyP {
    const char * src; char * dst;
    int64_t ne0, ne1, ne2, total;   // ne0 in units of `VEC` floats; total = units to copy
    int64_t s_nb1, s_nb2, s_nb3, d_nb1, d_nb2, d_nb3;
};

template <typename T>
__global__ void __launch_bounds__(256) mla_copy_kernel(const CopyP p) {
    for (int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x; i < p.total; i += (int64_t) gridDim.x * 256) {
        const int64_t i0 = i % p.ne0, r = i / p.ne0;
        const int64_t i1 = r % p.ne1, r2 = r / p.ne1;
        const int64_t i2 = r2 % p.ne2, i3 = r2 / p.ne2;
        ((T *) (p.dst + i3 * p.d_nb3 + i2 * p.d_nb2 + i1 * p.d_nb1))[i0] = ((const T *) (p.src + i3 * p.s_nb3 + i2 * p.s_nb2 + i1 * p.s_nb1))[i0];
    }
}

inline bool al16(const void * ptr) { return ((uintptr_t) ptr & 15) == 0; }

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
    p.src = (const char *) a->src; p.dst = (char *) a->dst;
    p.ne0 = a->ne[0]; p.ne1 = a->ne[1];
    p.s_nb1 = a->src_nb[1]; p.s_nb2 = a->src_nb[2]; p.s_nb3 = a->src_nb[3];
    p.d_nb1 = a->dst_nb[1]; p.d_nb2 = a->dst_nb[2]; p.d_nb3 = a->dst_nb[3];
    p.pos = a->pos; p.ff = a->freq_factors;
    p.n_dims = a->n_dims; p.neox = a->mode == MLA_ROPE_MODE_NEOX;
    // host-side constants, evaluated as the reference evaluates them (ggml-cpu.c:10409-10412, ggml.c:3529-3541, ggml-cpu.c:10289)
    p.theta_scale = powf(a->freq_base, -2.0f / a->n_dims);
    const float two_log_base = 2 * logf(a->freq_base);
    const float start = floorf(a->n_dims * logf(a->n_ctx_orig / (a->beta_fast * 2 * (float) M_PI)) / two_log_base);
    const float end   = ceilf(a->n_dims * logf(a->n_ctx_orig / (a->beta_slow * 2 * (float) M_PI)) / two_log_base);
    p.corr0 = start > 0 ? start : 0;
    p.corr1 = end < a->n_dims - 1 ? end : (float) (a->n_dims - 1);
    p.freq_scale = a->freq_scale; p.ext_factor = a->ext_factor;
    p.mscale = a->attn_factor;
    // 1 + 0.1 log(1/s) as one fused multiply-add: what an FMA-enabled x86 build of the reference evaluates
    if (a->ext_factor != 0.0f) p.mscale *= fmaf(0.1f, logf(1.0f / a->freq_scale), 1.0f);
    bool v2 = !p.neox && !((uintptr_t) a->src & 7) && !((uintptr_t) a->dst & 7);
    for (int i = 1; i < 4; i++) v2 = v2 && !(a->src_nb[i] & 7) && !(a->dst_nb[i] & 7);
    p.vec2 = v2;
    const int n_pairs = a->n_dims / 2;
    int hpw = 1024 / n_pairs;  // about four passes of the 256 threads
    if (hpw < 1) hpw = 1;
    p.heads_per_wg = hpw;
    const dim3 grid((unsigned) ((a->ne[1] + hpw - 1) / hpw), (unsigned) a->ne[2], (unsigned) a->ne[3]);
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
    MmP p;
    p.w = (const char *) a->w; p.x = (const char *) a->x; p.dst = (char *) a->dst;
    p.K = a->K; p.N = a->N; p.M = a->M; p.ne2 = a->ne2;
    p.w_nb1 = a->w_nb1; p.w_nb2 = a->w_nb2; p.w_nb3 = a->w_nb3;
    p.x_nb1 = a->x_nb1; p.x_nb2 = a->x_nb2; p.x_nb3 = a->x_nb3;
    p.d_nb1 = a->d_nb1; p.d_nb2 = a->d_nb2; p.d_nb3 = a->d_nb3;
    p.r2 = a->ne2 / a->w_ne2; p.r3 = a->ne3 / a->w_ne3;
    const hipError_t e = a->w_type == MLA_TYPE_F16 ? launch_mm<true>(p, a->ne2 * a->ne3, (hipStream_t) stream)
                                                   : launch_mm<false>(p, a->ne2 * a->ne3, (hipStream_t) stream);
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
    const int64_t n = a->ne[0] * a->ne[1] * a->ne[2] * a->ne[3];
    if (n == 0) return 0;
    bool v4 = a->ne[0] % 4 == 0 && al16(a->src) && al16(a->dst);
    for (int i = 1; i < 4; i++) v4 = v4 && !(a->src_nb[i] & 15) && !(a->dst_nb[i] & 15);
    CopyP p;
    p.src = (const char *) a->src; p.dst = (char *) a->dst;
    p.ne0 = v4 ? a->ne[0] / 4 : a->ne[0]; p.ne1 = a->ne[1]; p.ne2 = a->ne[2];
    p.total = v4 ? n / 4 : n;
    p.s_nb1 = a->src_nb[1]; p.s_nb2 = a->src_nb[2]; p.s_nb3 = a->src_nb[3];
    p.d_nb1 = a->dst_nb[1]; p.d_nb2 = a->dst_nb[2]; p.d_nb3 = a->dst_nb[3];
    const unsigned blocks = (unsigned) min((p.total + 255) / 256, (int64_t) 8192);
    if (v4) hipLaunchKernelGGL(mla_copy_kernel<float4>, dim3(blocks), dim3(256), 0, (hipStream_t) stream, p);
    else    hipLaunchKernelGGL(mla_copy_kernel<float>, dim3(blocks), dim3(256), 0, (hipStream_t) stream, p);
    return (int) hipGetLastError();
}
