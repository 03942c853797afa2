/*
 * CPU oracle for the ggml nodes either side of the MLA attention node, as ggml-cpu computes them.
 *
 * TEST INFRASTRUCTURE ONLY (same rule as mla_oracle.c): nothing in the product path may link, import or call it.
 *
 * mla_oracle_rope       GGML_OP_ROPE on f32 rows (ggml_rope_ext of q_pe / k_pe, src/llama-graph-deepseek2.cpp:218-233):
 *                       ggml/src/ggml-cpu/ggml-cpu.c:10361-10552 (ggml_compute_forward_rope_f32, forward, the "normal"
 *                       and the NeoX pairing; not mrope / vision), the cos/sin cache of :10295-10307
 *                       (theta = pos, then theta *= theta_scale per pair, theta_scale = powf(freq_base, -2/n_dims)),
 *                       YaRN of :10272-10293 (ramp over the correction dims, theta = interp*(1-mix) + extrap*mix,
 *                       mscale *= 1 + 0.1*logf(1/freq_scale) when ext_factor != 0), correction dims of
 *                       ggml/src/ggml.c:3529-3541, channels past n_dims copied (:10535-10546).
 *                       The sums of products (blend, magnitude scale, rotation) are written with explicit fmaf in the form gcc -O3 -mfma contracts
 *                       them to on the reference's build (checked bit for bit against the compiled reference in
 *                       tests/test_front_vs_ref.py), and this file is compiled with -ffp-contract=off.
 * mla_oracle_mul_mat    GGML_OP_MUL_MAT with an F16 / BF16 / F32 src0 and an F32 src1 (the absorb products
 *                       q_nope x wk_b and wv_b x kqv, src/llama-graph-attn.cpp:269-275, :307-317):
 *                       ggml/src/ggml-cpu/ggml-cpu.c:8431-8700 (ggml_compute_forward_mul_mat): src1 rows are converted
 *                       to src0's vec_dot_type (table :269-434: F16 -> f16, BF16 -> bf16, F32 -> f32), dst[i0,i1,i2,i3] =
 *                       dot(src0[:, i0, i2/r2, i3/r3], src1[:, i1, i2, i3]) with broadcast factors r2 = ne12/ne02,
 *                       r3 = ne13/ne03.  The dot is evaluated here in double on the rounded operands; the reference's
 *                       f32 lane accumulators (:1586-1698) differ from that by summation order only, which the tests
 *                       bound (1e-5 relative to sum |a||b|).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define MLA_TYPE_F32 0
#define MLA_TYPE_F16 1
#define MLA_TYPE_BF16 30

uint16_t mla_oracle_f32_to_bf16(float f);
uint16_t mla_oracle_f32_to_f16(float f);
float    mla_oracle_bf16_to_f32(uint16_t h);
float    mla_oracle_f16_to_f32(uint16_t h);

typedef struct {
    int32_t n_dims, mode, n_ctx_orig;
    float   freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow;
} mla_oracle_rope_params;

#define ROPE_NEOX 2

static float yarn_corr_dim(int n_dims, int n_ctx_orig, float n_rot, float base) { /* ggml.c:3529-3531 */
    return n_dims * logf(n_ctx_orig / (n_rot * 2 * (float) M_PI)) / (2 * logf(base));
}

void mla_oracle_rope_corr_dims(int n_dims, int n_ctx_orig, float freq_base, float beta_fast, float beta_slow, float dims[2]) {
    float start = floorf(yarn_corr_dim(n_dims, n_ctx_orig, beta_fast, freq_base)); /* ggml.c:3533-3541 */
    float end   = ceilf(yarn_corr_dim(n_dims, n_ctx_orig, beta_slow, freq_base));
    dims[0] = start > 0 ? start : 0;
    dims[1] = end < n_dims - 1 ? end : n_dims - 1;
}

/* cos/sin of one pair (ggml-cpu.c:10272-10293) */
static void yarn_pair(float theta_extrap, float freq_scale, const float corr[2], int64_t i0, float ext_factor, float mscale,
                      float *c, float *s) {
    float theta_interp = freq_scale * theta_extrap;
    float theta        = theta_interp;
    if (ext_factor != 0.0f) {
        float d = corr[1] - corr[0];
        float y = ((int) i0 / 2 - corr[0]) / (d > 0.001f ? d : 0.001f);
        float ramp = 1 - (y < 0 ? 0 : (y > 1 ? 1 : y));
        float mix  = ramp * ext_factor;
        theta  = fmaf(theta_interp, 1 - mix, theta_extrap * mix);
        mscale *= fmaf(0.1f, logf(1.0f / freq_scale), 1.0f);
    }
    *c = cosf(theta) * mscale;
    *s = sinf(theta) * mscale;
}

/* src, dst: f32 [ne0, ne1 (heads), ne2 (tokens), ne3]; nb / dnb byte strides (nb[0] = 4); pos[ne2]; freq_factors or NULL */
int mla_oracle_rope(const void *src, const int64_t ne[4], const int64_t nb[4], void *dst, const int64_t dnb[4],
                    const int32_t *pos, const float *freq_factors, const mla_oracle_rope_params *p) {
    const int n_dims = p->n_dims;
    if (n_dims > ne[0] || n_dims % 2 || (p->mode & ~ROPE_NEOX)) return -1;
    const float theta_scale = powf(p->freq_base, -2.0f / n_dims);
    float corr[2];
    mla_oracle_rope_corr_dims(n_dims, p->n_ctx_orig, p->freq_base, p->beta_fast, p->beta_slow, corr);
    const int neox = p->mode & ROPE_NEOX;
    float *cache = (float *) malloc(sizeof(float) * (size_t) (ne[0] + 2));
    for (int64_t i3 = 0; i3 < ne[3]; i3++)
        for (int64_t i2 = 0; i2 < ne[2]; i2++) {
            float theta = (float) (int64_t) pos[i2];
            for (int64_t i0 = 0; i0 < ne[0]; i0 += 2) { /* ggml-cpu.c:10295-10307 */
                const float ff = freq_factors ? freq_factors[i0 / 2] : 1.0f;
                yarn_pair(theta / ff, p->freq_scale, corr, i0, p->ext_factor, p->attn_factor, &cache[i0], &cache[i0 + 1]);
                theta *= theta_scale;
            }
            for (int64_t i1 = 0; i1 < ne[1]; i1++) {
                const char *s = (const char *) src + i3 * nb[3] + i2 * nb[2] + i1 * nb[1];
                char *      d = (char *) dst + i3 * dnb[3] + i2 * dnb[2] + i1 * dnb[1];
                for (int64_t i0 = 0; i0 < n_dims; i0 += 2) {
                    const float c = cache[i0], sn = cache[i0 + 1];
                    const int64_t a = neox ? i0 / 2 : i0, b = neox ? i0 / 2 + n_dims / 2 : i0 + 1;
                    const float x0 = *(const float *) (s + a * 4), x1 = *(const float *) (s + b * 4);
                    *(float *) (d + a * 4) = fmaf(x0, c, -(x1 * sn));
                    *(float *) (d + b * 4) = fmaf(x0, sn, x1 * c);
                }
                for (int64_t i0 = n_dims; i0 < ne[0]; i0++) *(float *) (d + i0 * 4) = *(const float *) (s + i0 * 4);
            }
        }
    free(cache);
    return 0;
}

static double elem_as_dot_type(const char *row, int type, int64_t i) {
    if (type == MLA_TYPE_F16) return mla_oracle_f16_to_f32(((const uint16_t *) row)[i]);
    if (type == MLA_TYPE_BF16) return mla_oracle_bf16_to_f32(((const uint16_t *) row)[i]);
    return ((const float *) row)[i];
}
static double round_to_dot_type(float x, int type) {
    if (type == MLA_TYPE_F16) return mla_oracle_f16_to_f32(mla_oracle_f32_to_f16(x));
    if (type == MLA_TYPE_BF16) return mla_oracle_bf16_to_f32(mla_oracle_f32_to_bf16(x));
    return x;
}

/* src0: type0 [K, N, ne02, ne03] byte strides nb0[1..3]; src1: f32 [K, M, ne12, ne13] strides nb1[1..3];
 * dst: f32 [N, M, ne12, ne13] contiguous.  abs_out (optional, same shape): sum |a||b| per element, for error bounds. */
int mla_oracle_mul_mat(const void *src0, int type0, const int64_t ne0[4], const int64_t nb0[4], const void *src1,
                       const int64_t ne1[4], const int64_t nb1[4], float *dst, float *abs_out) {
    if (type0 != MLA_TYPE_F16 && type0 != MLA_TYPE_BF16 && type0 != MLA_TYPE_F32) return -1;
    if (ne0[0] != ne1[0] || ne1[2] % ne0[2] || ne1[3] % ne0[3]) return -2;
    const int64_t K = ne0[0], N = ne0[1], M = ne1[1];
    const int64_t r2 = ne1[2] / ne0[2], r3 = ne1[3] / ne0[3];
    double *b = (double *) malloc(sizeof(double) * (size_t) K);
    for (int64_t i3 = 0; i3 < ne1[3]; i3++)
        for (int64_t i2 = 0; i2 < ne1[2]; i2++)
            for (int64_t m = 0; m < M; m++) {
                const char *row1 = (const char *) src1 + i3 * nb1[3] + i2 * nb1[2] + m * nb1[1];
                for (int64_t k = 0; k < K; k++) b[k] = round_to_dot_type(((const float *) row1)[k], type0);
                for (int64_t n = 0; n < N; n++) {
                    const char *row0 = (const char *) src0 + (i3 / r3) * nb0[3] + (i2 / r2) * nb0[2] + n * nb0[1];
                    double acc = 0, aa = 0;
                    for (int64_t k = 0; k < K; k++) {
                        const double a = elem_as_dot_type(row0, type0, k);
                        acc += a * b[k];
                        aa += fabs(a * b[k]);
                    }
                    const int64_t o = ((i3 * ne1[2] + i2) * M + m) * N + n;
                    dst[o] = (float) acc;
                    if (abs_out) abs_out[o] = (float) aa;
                }
            }
    free(b);
    return 0;
}
