/*
 * CPU oracle for GGML_OP_FLASH_ATTN_EXT as ggml-cpu computes it.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the GPU kernels are compared against and the
 * "port" CPU baseline that bench.py times.  Nothing in the product path (jittorinfer_amd/) may link,
 * import or call it.
 *
 * It restates, in plain C, the algorithm of the reference's
 *   ggml/src/ggml-cpu/ggml-cpu.c:11914-12124  ggml_compute_forward_flash_attn_ext_f16
 * for the K/V types the MLA path uses (F16, BF16, Q8_0) with Q given as F32:
 *   - Q row is first converted to K's vec_dot_type (ggml-cpu.c:11991-11993, 12034-12035; table :269-434):
 *       F16 K  -> Q rounded to f16,  BF16 K -> Q rounded to bf16,  Q8_0 K -> Q quantized to Q8_0
 *   - per key, in order: mask value (skip the key when it is -inf, :12041-12044), dot, scale,
 *     optional softcap, add mask, online softmax with running max M and sum S (:12059-12100)
 *   - V accumulator is f16 (rounded to f16 after every scale / multiply-add) when V is F16
 *     (:12066-12080, vec ops :1788-1818, :1904-1929, x86 F16C forms :621-659, :718-765), f32 otherwise
 *     (:12081-12098, :1756-1786, :1873-1902)
 *   - final 1/S scaling and the permuted store dst[((i3*n_tok + i1)*n_head + i2) * ne0 ...] (:12109-12122)
 *   - ALiBi slope from max_bias (:11985-11989, :12006-12008)
 * Conversions follow ggml/src/ggml-impl.h:553-568 (bf16 RNE, quiet NaN) and IEEE binary16 RNE
 * (ggml/include/ggml.h:337-342 with F16C semantics).  Q8_0 follows ggml/src/ggml-common.h:217-224,
 * ggml/src/ggml-quants.c:202-226 (reference quantizer, roundf) and :357-373 (dequantize), and the AVX
 * form of the CPU-backend quantizer ggml/src/ggml-cpu/ggml-cpu-quants.c:855-900 (id = 127/amax,
 * round-half-even), which is the one flash_attn_ext calls for Q on an x86 host.  The Q8_0 x Q8_0 dot is
 * the per-block integer dot times d_x*d_y summed in f32 (ggml-cpu-quants.c:3814-4241).
 *
 * One deliberate generalisation: V may be narrower than K (DV <= DK, e.g. the first 512 of 576 columns);
 * the reference asserts DV == DK (ggml-cpu.c:11943) and output columns are independent, so with DV == DK
 * this is the reference's computation and with DV < DK it is its first DV output columns.
 *
 * Pinning: see tests/test_oracle.py (closed forms, brute force, exhaustive conversions, and the
 * differential against the reference's own compiled ggml-cpu when oracle/_ref is built) and
 * tests/test_golden.py (the vectors in tests/golden/, produced by the compiled reference).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define MLA_TYPE_F32 0
#define MLA_TYPE_F16 1
#define MLA_TYPE_Q8_0 8
#define MLA_TYPE_BF16 30

#define QK8_0 32
typedef struct {
    uint16_t d;          /* fp16 scale */
    int8_t   qs[QK8_0];  /* quants */
} oracle_block_q8_0;     /* 34 bytes, ggml-common.h:217-224 */

typedef struct {
    int32_t     type;
    int32_t     _pad;
    int64_t     ne[4];
    int64_t     nb[4]; /* byte strides */
    const void *data;
} mla_oracle_tensor;

/* ---------------------------------------------------------------- conversions */

static inline float u32_as_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_as_u32(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

float mla_oracle_bf16_to_f32(uint16_t h) { return u32_as_f32((uint32_t) h << 16); }

uint16_t mla_oracle_f32_to_bf16(float s) {
    uint32_t i = f32_as_u32(s);
    if ((i & 0x7fffffffu) > 0x7f800000u) return (uint16_t) ((i >> 16) | 64); /* quiet NaN */
    return (uint16_t) ((i + (0x7fffu + ((i >> 16) & 1u))) >> 16);
}

float mla_oracle_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t) (h & 0x8000u) << 16;
    uint32_t exp  = (h >> 10) & 0x1fu;
    uint32_t man  = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return u32_as_f32(sign);
        /* subnormal: man * 2^-24 */
        float f = (float) man * (1.0f / 16777216.0f);
        return (sign ? -f : f);
    }
    if (exp == 31) return u32_as_f32(sign | 0x7f800000u | (man << 13));
    return u32_as_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* IEEE binary32 -> binary16, round to nearest even (what F16C vcvtps2ph imm=0 does) */
uint16_t mla_oracle_f32_to_f16(float f) {
    uint32_t x    = f32_as_u32(f);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax   = x & 0x7fffffffu;
    if (ax > 0x7f800000u) return (uint16_t) (sign | 0x7e00u | ((ax >> 13) & 0x3ffu)); /* NaN, quieted */
    if (ax >= 0x47800000u) {                                                           /* >= 65536 or inf */
        return (uint16_t) (sign | 0x7c00u);
    }
    if (ax < 0x38800000u) { /* below 2^-14: subnormal or zero in f16 */
        if (ax < 0x33000000u) return (uint16_t) sign; /* < 2^-25 rounds to zero (2^-25 itself ties to even = 0) */
        uint32_t e     = ax >> 23;                    /* biased f32 exponent, 102..112 */
        uint32_t m     = (ax & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126u - e;                    /* 14..24 */
        uint32_t r     = m >> shift;
        uint32_t rem   = m & ((1u << shift) - 1u);
        uint32_t half  = 1u << (shift - 1u);
        if (rem > half || (rem == half && (r & 1u))) r++;
        return (uint16_t) (sign | r);
    }
    {
        uint32_t r   = ((ax >> 13) - (112u << 10));
        uint32_t rem = ax & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) r++;
        return (uint16_t) (sign | r); /* carry into exponent (and to inf at 65520) is the right result */
    }
}

void mla_oracle_f32_to_bf16_row(const float *x, uint16_t *y, int64_t n) { for (int64_t i = 0; i < n; i++) y[i] = mla_oracle_f32_to_bf16(x[i]); }
void mla_oracle_f32_to_f16_row(const float *x, uint16_t *y, int64_t n)  { for (int64_t i = 0; i < n; i++) y[i] = mla_oracle_f32_to_f16(x[i]); }
void mla_oracle_bf16_to_f32_row(const uint16_t *x, float *y, int64_t n) { for (int64_t i = 0; i < n; i++) y[i] = mla_oracle_bf16_to_f32(x[i]); }
void mla_oracle_f16_to_f32_row(const uint16_t *x, float *y, int64_t n)  { for (int64_t i = 0; i < n; i++) y[i] = mla_oracle_f16_to_f32(x[i]); }

/* ---------------------------------------------------------------- Q8_0 */

/* mode 0: reference quantizer (ggml-quants.c:202-226): id = 1/d, roundf (half away from zero)
 * mode 1: x86 CPU-backend quantizer (ggml-cpu-quants.c:855-900): id = 127/amax, round half to even */
void mla_oracle_quantize_row_q8_0(const float *x, void *vy, int64_t k, int mode) {
    oracle_block_q8_0 *y  = (oracle_block_q8_0 *) vy;
    const int64_t      nb = k / QK8_0;
    for (int64_t i = 0; i < nb; i++) {
        float amax = 0.0f;
        for (int j = 0; j < QK8_0; j++) {
            const float v = fabsf(x[i * QK8_0 + j]);
            if (v > amax) amax = v;
        }
        const float d = amax / 127.0f;
        y[i].d        = mla_oracle_f32_to_f16(d);
        if (mode == 0) {
            const float id = d ? 1.0f / d : 0.0f;
            for (int j = 0; j < QK8_0; j++) y[i].qs[j] = (int8_t) roundf(x[i * QK8_0 + j] * id);
        } else {
            const float id = (amax != 0.0f) ? 127.0f / amax : 0.0f;
            for (int j = 0; j < QK8_0; j++) y[i].qs[j] = (int8_t) nearbyintf(x[i * QK8_0 + j] * id); /* RNE in default mode */
        }
    }
}

void mla_oracle_dequantize_row_q8_0(const void *vx, float *y, int64_t k) {
    const oracle_block_q8_0 *x  = (const oracle_block_q8_0 *) vx;
    const int64_t            nb = k / QK8_0;
    for (int64_t i = 0; i < nb; i++) {
        const float d = mla_oracle_f16_to_f32(x[i].d);
        for (int j = 0; j < QK8_0; j++) y[i * QK8_0 + j] = (float) x[i].qs[j] * d;
    }
}

static float dot_q8_0_q8_0(int64_t n, const oracle_block_q8_0 *x, const oracle_block_q8_0 *y) {
    const int64_t nb   = n / QK8_0;
    float         sumf = 0.0f;
    for (int64_t ib = 0; ib < nb; ib++) {
        int32_t sumi = 0;
        for (int j = 0; j < QK8_0; j++) sumi += (int32_t) x[ib].qs[j] * (int32_t) y[ib].qs[j];
        sumf += (float) sumi * (mla_oracle_f16_to_f32(x[ib].d) * mla_oracle_f16_to_f32(y[ib].d));
    }
    return sumf;
}

/* ---------------------------------------------------------------- row helpers */

static void row_to_f32(int type, const void *src, float *dst, int64_t n) {
    switch (type) {
        case MLA_TYPE_F16:  mla_oracle_f16_to_f32_row((const uint16_t *) src, dst, n); break;
        case MLA_TYPE_BF16: mla_oracle_bf16_to_f32_row((const uint16_t *) src, dst, n); break;
        case MLA_TYPE_Q8_0: mla_oracle_dequantize_row_q8_0(src, dst, n); break;
        default:            memcpy(dst, src, (size_t) n * sizeof(float)); break;
    }
}

/* 16 running partial sums, the shape a SIMD dot has; the final reduction order is not the reference's
 * (that one depends on the host ISA, ggml-cpu.c:1586-1698) -- differences are at the 1e-7 relative level. */
static float dot_f32(int64_t n, const float *a, const float *b) {
    float acc[16] = { 0 };
    int64_t i = 0;
    for (; i + 16 <= n; i += 16)
        for (int j = 0; j < 16; j++) acc[j] += a[i + j] * b[i + j];
    double sum = 0.0;
    for (int j = 0; j < 16; j++) sum += (double) acc[j];
    for (; i < n; i++) sum += (double) (a[i] * b[i]);
    return (float) sum;
}

static size_t type_row_size(int type, int64_t n) {
    switch (type) {
        case MLA_TYPE_F32:  return (size_t) n * 4;
        case MLA_TYPE_F16:
        case MLA_TYPE_BF16: return (size_t) n * 2;
        case MLA_TYPE_Q8_0: return (size_t) (n / QK8_0) * sizeof(oracle_block_q8_0);
        default:            return 0;
    }
}

/* ---------------------------------------------------------------- the op */

/*
 * q    F32   [DK, n_tok, n_head, n3]
 * k    F16|BF16|Q8_0 [DK, n_kv, n_head_kv, n3k]
 * v    same type as k, [DV, n_kv, n_head_kv, n3v], DV <= DK
 * mask F16   [n_kv, >= n_tok] or NULL (shared by heads and by ne3, ggml-cpu.c:12024)
 * dst  F32   rows of dst_ne0 floats at ((i3*n_tok + i1)*n_head + i2); DV floats of each row are written
 * q8_mode: quantizer used for Q when K is Q8_0 (see mla_oracle_quantize_row_q8_0)
 * returns 0, or a negative code for an argument the reference would have asserted on.
 */
int mla_oracle_flash_attn_ext(const mla_oracle_tensor *q, const mla_oracle_tensor *k, const mla_oracle_tensor *v,
                              const mla_oracle_tensor *mask, float *dst, int64_t dst_ne0, float scale, float max_bias,
                              float logit_softcap, int q8_mode, int n_threads) {
    const int64_t DK = q->ne[0], N = q->ne[1], H = q->ne[2], B3 = q->ne[3];
    const int64_t DV = v->ne[0];
    const int64_t n_kv = k->ne[1];
    if (q->type != MLA_TYPE_F32) return -1;
    if (k->type != MLA_TYPE_F16 && k->type != MLA_TYPE_BF16 && k->type != MLA_TYPE_Q8_0) return -2;
    if (v->type != k->type) return -3;
    if (k->ne[0] != DK || DV > DK || DV > dst_ne0 || v->ne[1] != n_kv) return -4;
    if (k->type == MLA_TYPE_Q8_0 && (DK % QK8_0 || DV % QK8_0)) return -5;
    if (k->ne[2] == 0 || k->ne[3] == 0 || H % k->ne[2] || B3 % k->ne[3] || H % v->ne[2] || B3 % v->ne[3]) return -6;
    if (mask && (mask->type != MLA_TYPE_F16 || mask->ne[0] < n_kv || mask->ne[1] < N)) return -7;

    const int64_t rk2 = H / k->ne[2], rk3 = B3 / k->ne[3];
    const int64_t rv2 = H / v->ne[2], rv3 = B3 / v->ne[3];

    if (logit_softcap != 0.0f) scale /= logit_softcap;

    const uint32_t n_head      = (uint32_t) H;
    const uint32_t n_head_log2 = 1u << (uint32_t) floor(log2((double) n_head));
    const float    m0          = powf(2.0f, -(max_bias) / n_head_log2);
    const float    m1          = powf(2.0f, -(max_bias / 2.0f) / n_head_log2);

    const int64_t nr = N * H * B3;
    if (n_threads < 1) n_threads = 1;
    int err = 0;

#pragma omp parallel num_threads(n_threads)
    {
#ifdef _OPENMP
        const int ith = omp_get_thread_num(), nth = omp_get_num_threads();
#else
        const int ith = 0, nth = 1;
#endif
        /* rows split statically, as the reference does (ggml-cpu.c:11961-11971) */
        const int64_t dr  = (nr + nth - 1) / nth;
        const int64_t ir0 = dr * ith;
        const int64_t ir1 = (ir0 + dr < nr) ? ir0 + dr : nr;

        float    *VKQ32 = (float *) malloc(sizeof(float) * (size_t) DK * 4);
        float    *Vf    = VKQ32 + DK;      /* f32 image of the current V row */
        float    *Qf    = VKQ32 + 2 * DK;  /* f32 image of the rounded Q row (f16/bf16 K) */
        float    *Kf    = VKQ32 + 3 * DK;  /* f32 image of the current K row */
        uint16_t *VKQ16 = (uint16_t *) malloc(sizeof(uint16_t) * (size_t) DK);
        void     *Qq    = malloc(type_row_size(MLA_TYPE_Q8_0, (DK + QK8_0 - 1) / QK8_0 * QK8_0) + 64);
        if (!VKQ32 || !VKQ16 || !Qq) {
            err = -100;
        } else
        for (int64_t ir = ir0; ir < ir1; ir++) {
            const int64_t iq3 = ir / (H * N);
            const int64_t iq2 = (ir - iq3 * H * N) / N;
            const int64_t iq1 = ir - iq3 * H * N - iq2 * N;

            const uint32_t h = (uint32_t) iq2;
            const float slope = (max_bias > 0.0f) ? (h < n_head_log2 ? powf(m0, (float) (h + 1)) : powf(m1, (float) (2 * (h - n_head_log2) + 1))) : 1.0f;

            float S = 0.0f;
            float M = -INFINITY;

            if (v->type == MLA_TYPE_F16) memset(VKQ16, 0, (size_t) DV * sizeof(uint16_t));
            else                         memset(VKQ32, 0, (size_t) DV * sizeof(float));

            const uint16_t *mp = mask ? (const uint16_t *) ((const char *) mask->data + iq1 * mask->nb[1]) : NULL;

            const int64_t ik3 = iq3 / rk3, ik2 = iq2 / rk2;
            const int64_t iv3 = iq3 / rv3, iv2 = iq2 / rv2;

            const float *pq = (const float *) ((const char *) q->data + iq1 * q->nb[1] + iq2 * q->nb[2] + iq3 * q->nb[3]);
            /* Q -> vec_dot_type of K */
            if (k->type == MLA_TYPE_F16) {
                for (int64_t d = 0; d < DK; d++) Qf[d] = mla_oracle_f16_to_f32(mla_oracle_f32_to_f16(pq[d]));
            } else if (k->type == MLA_TYPE_BF16) {
                for (int64_t d = 0; d < DK; d++) Qf[d] = mla_oracle_bf16_to_f32(mla_oracle_f32_to_bf16(pq[d]));
            } else {
                mla_oracle_quantize_row_q8_0(pq, Qq, DK, q8_mode);
            }

            for (int64_t ic = 0; ic < n_kv; ic++) {
                const float mv = mp ? slope * mla_oracle_f16_to_f32(mp[ic]) : 0.0f;
                if (mv == -INFINITY) continue;

                const char *k_data = (const char *) k->data + ic * k->nb[1] + ik2 * k->nb[2] + ik3 * k->nb[3];
                float s;
                if (k->type == MLA_TYPE_Q8_0) {
                    s = dot_q8_0_q8_0(DK, (const oracle_block_q8_0 *) k_data, (const oracle_block_q8_0 *) Qq);
                } else {
                    row_to_f32(k->type, k_data, Kf, DK);
                    s = dot_f32(DK, Kf, Qf);
                }
                s = s * scale;
                if (logit_softcap != 0.0f) s = logit_softcap * tanhf(s);
                s += mv;

                const float Mold = M;
                float ms = 1.0f, vs = 1.0f;

                const char *v_data = (const char *) v->data + ic * v->nb[1] + iv2 * v->nb[2] + iv3 * v->nb[3];

                if (v->type == MLA_TYPE_F16) {
                    const uint16_t *vh = (const uint16_t *) v_data;
                    if (s > M) {
                        M  = s;
                        ms = expf(Mold - M);
                        for (int64_t d = 0; d < DV; d++) VKQ16[d] = mla_oracle_f32_to_f16(mla_oracle_f16_to_f32(VKQ16[d]) * ms);
                    } else {
                        vs = expf(s - M);
                    }
                    for (int64_t d = 0; d < DV; d++)
                        VKQ16[d] = mla_oracle_f32_to_f16(fmaf(mla_oracle_f16_to_f32(vh[d]), vs, mla_oracle_f16_to_f32(VKQ16[d])));
                } else {
                    if (s > M) {
                        M  = s;
                        ms = expf(Mold - M);
                        for (int64_t d = 0; d < DV; d++) VKQ32[d] *= ms;
                    } else {
                        vs = expf(s - M);
                    }
                    row_to_f32(v->type, v_data, Vf, DV);
                    for (int64_t d = 0; d < DV; d++) VKQ32[d] = fmaf(Vf[d], vs, VKQ32[d]);
                }
                S = S * ms + vs;
            }

            if (v->type == MLA_TYPE_F16)
                for (int64_t d = 0; d < DV; d++) VKQ32[d] = mla_oracle_f16_to_f32(VKQ16[d]);

            const float S_inv = 1.0f / S;
            for (int64_t d = 0; d < DV; d++) VKQ32[d] *= S_inv;

            /* permute(0,2,1,3): row index (i3*n_tok + i1)*n_head + i2 */
            memcpy(dst + ((iq3 * N + iq1) * H + iq2) * dst_ne0, VKQ32, (size_t) DV * sizeof(float));
        }
        free(VKQ32); free(VKQ16); free(Qq);
    }
    return err;
}

/* f64 evaluation of the same function on the same (already rounded) inputs: the mathematical value
 * softmax(scale*q.k + mask) . v with no intermediate rounding.  Used to report how far both the oracle and
 * the GPU kernel are from the exact answer. */
int mla_oracle_flash_attn_ext_f64(const mla_oracle_tensor *q, const mla_oracle_tensor *k, const mla_oracle_tensor *v,
                                  const mla_oracle_tensor *mask, float *dst, int64_t dst_ne0, float scale, int q8_mode,
                                  int n_threads) {
    const int64_t DK = q->ne[0], N = q->ne[1], H = q->ne[2], B3 = q->ne[3];
    const int64_t DV = v->ne[0], n_kv = k->ne[1];
    if (k->ne[0] != DK || DV > DK || DV > dst_ne0) return -4;
    const int64_t rk2 = H / k->ne[2], rk3 = B3 / k->ne[3];
    const int64_t rv2 = H / v->ne[2], rv3 = B3 / v->ne[3];
    const int64_t nr = N * H * B3;
    if (n_threads < 1) n_threads = 1;
#pragma omp parallel for num_threads(n_threads) schedule(static)
    for (int64_t ir = 0; ir < nr; ir++) {
        const int64_t iq3 = ir / (H * N);
        const int64_t iq2 = (ir - iq3 * H * N) / N;
        const int64_t iq1 = ir - iq3 * H * N - iq2 * N;
        float  *Qf = (float *) malloc(sizeof(float) * (size_t) DK * 2);
        float  *Kf = Qf + DK;
        double *acc = (double *) calloc((size_t) DV, sizeof(double));
        double *sc  = (double *) malloc(sizeof(double) * (size_t) n_kv);
        void   *Qq  = malloc(type_row_size(MLA_TYPE_Q8_0, (DK + QK8_0 - 1) / QK8_0 * QK8_0) + 64);
        const float *pq = (const float *) ((const char *) q->data + iq1 * q->nb[1] + iq2 * q->nb[2] + iq3 * q->nb[3]);
        if (k->type == MLA_TYPE_F16)       for (int64_t d = 0; d < DK; d++) Qf[d] = mla_oracle_f16_to_f32(mla_oracle_f32_to_f16(pq[d]));
        else if (k->type == MLA_TYPE_BF16) for (int64_t d = 0; d < DK; d++) Qf[d] = mla_oracle_bf16_to_f32(mla_oracle_f32_to_bf16(pq[d]));
        else { mla_oracle_quantize_row_q8_0(pq, Qq, DK, q8_mode); mla_oracle_dequantize_row_q8_0(Qq, Qf, DK); }
        const uint16_t *mp = mask ? (const uint16_t *) ((const char *) mask->data + iq1 * mask->nb[1]) : NULL;
        double mx = -INFINITY;
        for (int64_t ic = 0; ic < n_kv; ic++) {
            const double mv = mp ? (double) mla_oracle_f16_to_f32(mp[ic]) : 0.0;
            const char *k_data = (const char *) k->data + ic * k->nb[1] + (iq2 / rk2) * k->nb[2] + (iq3 / rk3) * k->nb[3];
            row_to_f32(k->type, k_data, Kf, DK);
            double s = 0.0;
            for (int64_t d = 0; d < DK; d++) s += (double) Kf[d] * (double) Qf[d];
            sc[ic] = s * (double) scale + mv;
            if (sc[ic] > mx) mx = sc[ic];
        }
        double sum = 0.0;
        for (int64_t ic = 0; ic < n_kv; ic++) {
            if (sc[ic] == -INFINITY) continue;
            const double p = exp(sc[ic] - mx);
            sum += p;
            const char *v_data = (const char *) v->data + ic * v->nb[1] + (iq2 / rv2) * v->nb[2] + (iq3 / rv3) * v->nb[3];
            row_to_f32(v->type, v_data, Kf, DV);
            for (int64_t d = 0; d < DV; d++) acc[d] += p * (double) Kf[d];
        }
        float *o = dst + ((iq3 * N + iq1) * H + iq2) * dst_ne0;
        for (int64_t d = 0; d < DV; d++) o[d] = (float) (acc[d] / sum);
        free(Qf); free(acc); free(sc); free(Qq);
    }
    return 0;
}

/*
 * KV cache write as ggml-cpu performs ggml_cpy(kv_cur f32 [576, n_tok] -> typed cache rows)
 * (ggml/src/ggml-cpu/ggml-cpu.c:3965-4040 ggml_compute_forward_dup_f32: per source row, from_float of the destination
 * type, table :269-434): F16 -> ggml_fp32_to_fp16_row, BF16 -> ggml_fp32_to_bf16_row, Q8_0 -> the CPU backend's
 * quantize_row_q8_0 (q8_mode 1 = its x86 form, 0 = the reference form of ggml-quants.c:202-226).
 * Destination rows are given explicitly (dest_rows[i], skipped when outside [0, n_kv_rows)), which also covers
 * ggml_scatter_update's dst[indices[i]] = updates[i] (ggml/src/ggml.c:3203-3223, aclnn_ops.cpp:6052-6129) and a block table
 * resolved by the caller.  src_type F32 converts; src_type == kv_type copies the row bytes.
 * Pinned by tests/test_kv_write.py: conversions are the functions above (exhaustive tests), the row placement is checked
 * against numpy indexing, and the whole against the reference's compiled ggml_cpy when oracle/_ref is built.
 */
int mla_oracle_kv_write(const void *src, int src_type, int64_t src_nb1, int64_t n_tok, void *kv, int kv_type, int64_t kv_nb1,
                        int64_t n_kv_rows, const int64_t *dest_rows, int q8_mode) {
    const size_t rs = type_row_size(kv_type, 576);
    if (rs == 0 || (src_type != 0 && src_type != kv_type)) return -2;
    for (int64_t t = 0; t < n_tok; t++) {
        const int64_t r = dest_rows[t];
        if (r < 0 || r >= n_kv_rows) continue;
        const char *s = (const char *) src + t * src_nb1;
        char *d = (char *) kv + r * kv_nb1;
        if (src_type != 0) { memcpy(d, s, rs); continue; }
        if (kv_type == 1)       mla_oracle_f32_to_f16_row((const float *) s, (uint16_t *) d, 576);
        else if (kv_type == 30) mla_oracle_f32_to_bf16_row((const float *) s, (uint16_t *) d, 576);
        else                    mla_oracle_quantize_row_q8_0((const float *) s, d, 576, q8_mode);
    }
    return 0;
}
