/*
 * Scalar C restatement of the fused W8A8 MoE kernel.  TEST INFRASTRUCTURE ONLY:
 * built into oracle/libmoe_oracle.so and loaded by tests/ alone; nothing shipped links it.
 *
 * Unlike moe_oracle.py (which de-interleaves w1 and then applies ordinary block scaling),
 * this file walks the operator's own INTERLEAVED layout with the indexing of the reference
 * kernel csrc/kernels/fused_moe_w8a8/fused_moe_w8a8_up_down_acc.cu ("K.cu"):
 *   - one work unit = (block of block_m sorted rows, 128-column slice bx of the intermediate)   K.cu:676-679,767
 *   - the unit's 256 w1 rows are [256*bx, 256*bx+256); within each 16-row chunk the first
 *     8 rows are gate and the next 8 are the matching up rows                                   K.cu:919-931
 *   - gate rows take w_scale row 2*bx, up rows take row 2*bx+1                                  K.cu:800-807
 *   - per 128-wide K block: fp32 dot, then (scale_w * scale_x) * dot                           K.cu:915-933
 *   - SwiGLU on bf16 gate/up, result to bf16, amax over the 128 columns, /448, clamp, RNE      K.cu:939-991
 *   - down: token_scale * dot * s_w with token_scale = s_a * topk_w * scaling_factor           K.cu:997-1003,1061
 *   - the result is ADDED into out                                                             K.cu:1085-1091
 * Departures (stricter than the reference): the K-block sum is kept in fp32 rather than bf16
 * (K.cu:740), and every row's amax is floored at 1e-10 (K.cu:940 floors only row 0).
 * The two restatements agreeing on random data pins the layout handling of both.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static float fp8_decode(uint8_t c)
{
    int e = (c >> 3) & 15, m = c & 7;
    float v;
    if (e == 15 && m == 7)
        v = NAN;
    else if (e == 0)
        v = ldexpf((float)m, -9);
    else
        v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return (c & 0x80) ? -v : v;
}

/* round-to-nearest-even, saturating at 448; v finite */
static uint8_t fp8_encode(float v)
{
    uint8_t sign = signbit(v) ? 0x80 : 0;
    float a = fabsf(v);
    if (a >= 448.0f)
        return sign | 0x7e;
    if (a < ldexpf(1.0f, -6)) {                    /* subnormal range: multiples of 2^-9 */
        int m = (int)nearbyintf(ldexpf(a, 9));     /* default rounding mode = ties to even */
        return sign | (uint8_t)m;                  /* m == 8 is code 0x08 = 2^-6: correct carry */
    }
    int e;
    float f = frexpf(a, &e);                       /* a = f * 2^e, f in [0.5,1) */
    int m = (int)nearbyintf(ldexpf(f, 4));         /* 1.mmm * 8 in [8,16] */
    e -= 1;
    if (m == 16) { m = 8; e += 1; }
    int code = ((e + 7) << 3) | (m - 8);
    if (code > 0x7e) code = 0x7e;
    return sign | (uint8_t)code;
}

static float bf16_to_float(uint16_t h)
{
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static uint16_t float_to_bf16(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u)
        return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static float round_bf16(float f) { return bf16_to_float(float_to_bf16(f)); }

uint8_t moe_oracle_fp8_encode(float v) { return fp8_encode(v); }
float moe_oracle_fp8_decode(uint8_t c) { return fp8_decode(c); }
uint16_t moe_oracle_float_to_bf16(float v) { return float_to_bf16(v); }

/*
 * Same arguments as the operator's C-level seam (K.cu:1258-1280) minus the tuning knobs that do
 * not change the result.  out is bf16 [M, K], updated in place: out = bf16(float(out) + sum of units).
 * Returns 0, or -1 on a shape the path does not define.
 */
int moe_oracle_fused(const uint8_t *x, const float *x_scale, const uint8_t *w, const float *w_scale,
                     const uint8_t *w2, const float *w2_scale, uint16_t *out, const int32_t *sorted_token_ids,
                     const int32_t *expert_ids, const int32_t *num_tokens_post_padded, const float *topk_weights,
                     int top_k, int M, int K, int N, int num_experts, int sorted_num, int block_m,
                     float scaling_factor)
{
    if (K % 128 || N % 256 || block_m <= 0 || top_k <= 0)
        return -1;
    const int I = N / 2, kblocks = K / 128, iblocks = I / 128;
    const int total = num_tokens_post_padded[0];
    float *acc = calloc((size_t)M * K, sizeof(float));
    float *dq_x = malloc(sizeof(float) * 128);
    uint8_t *q = malloc(128);
    if (!acc || !dq_x || !q)
        return -1;

    for (int b = 0; b * block_m < total && b * block_m < sorted_num; b++) {
        const int e = expert_ids[b];
        if (e < 0 || e >= num_experts)
            continue;
        for (int r = 0; r < block_m && b * block_m + r < sorted_num; r++) {
            const int id = sorted_token_ids[b * block_m + r];
            const int t = id / top_k;
            if (t >= M)
                continue;                                               /* padding row */
            for (int bx = 0; bx < iblocks; bx++) {
                float a[128];
                float amax = 1e-10f;
                for (int jj = 0; jj < 128; jj++) {
                    const int chunk = (128 * bx + jj) / 8, j = jj % 8;
                    const size_t row_g = (size_t)e * N + 16 * chunk + j;
                    const size_t row_u = row_g + 8;
                    float hg = 0.f, hu = 0.f;
                    for (int kb = 0; kb < kblocks; kb++) {
                        float dg = 0.f, du = 0.f;
                        for (int k = 0; k < 128; k++) {
                            float xv = fp8_decode(x[(size_t)t * K + kb * 128 + k]);
                            dg += fp8_decode(w[row_g * K + kb * 128 + k]) * xv;
                            du += fp8_decode(w[row_u * K + kb * 128 + k]) * xv;
                        }
                        const float sx = x_scale[(size_t)t * kblocks + kb];
                        const float sg = w_scale[((size_t)e * (N / 128) + 2 * bx) * kblocks + kb];
                        const float su = w_scale[((size_t)e * (N / 128) + 2 * bx + 1) * kblocks + kb];
                        hg += sg * sx * dg;
                        hu += su * sx * du;
                    }
                    hg = round_bf16(hg);
                    hu = round_bf16(hu);
                    a[jj] = round_bf16(hg / (1.0f + expf(-hg)) * hu);
                    if (fabsf(a[jj]) > amax)
                        amax = fabsf(a[jj]);
                }
                const float s_a = amax / 448.0f;
                for (int jj = 0; jj < 128; jj++) {
                    float v = a[jj] / s_a;
                    v = fminf(fmaxf(v, -448.0f), 448.0f);
                    q[jj] = fp8_encode(v);
                    dq_x[jj] = fp8_decode(q[jj]);
                }
                const float token_scale = s_a * (topk_weights[id] * scaling_factor);
                for (int c = 0; c < K; c++) {
                    float d = 0.f;
                    const uint8_t *w2row = w2 + ((size_t)e * K + c) * I + 128 * bx;
                    for (int jj = 0; jj < 128; jj++)
                        d += fp8_decode(w2row[jj]) * dq_x[jj];
                    const float s_w = w2_scale[((size_t)e * (K / 128) + c / 128) * iblocks + bx];
                    acc[(size_t)t * K + c] += token_scale * d * s_w;
                }
            }
        }
    }
    for (size_t i = 0; i < (size_t)M * K; i++)
        out[i] = float_to_bf16(bf16_to_float(out[i]) + acc[i]);
    free(acc);
    free(dq_x);
    free(q);
    return 0;
}
