/*
 * CPU oracle for the FP8 block-scale path (test infrastructure only, see fp8bs_oracle.h).
 *
 * Compile WITHOUT fast-math and without FMA contraction: every operation below is meant to
 * be one IEEE-754 binary32/binary64 operation with round-to-nearest-even, as torch's CPU
 * kernels perform it.  Denormals are kept (no FTZ/DAZ).
 *
 * Reference lines restated here (paths relative to the reference checkout):
 *   aiter/ops/quant.py:55-61    get_dtype_max           -> 448 for e4m3fn
 *   aiter/ops/quant.py:64-94    pertoken_quant          -> oracle_group_quant
 *   aiter/ops/quant.py:331-346  per_block_quant_wrapper -> the (-1, group) view
 *   op_tests/multigpu_tests/test_dispatch_combine.py:180-204 weight_per_128x128_quant
 *                                                       -> oracle_weight_block_quant
 *   op_tests/test_gemm_a8w8_blockscale.py:28-54 run_torch -> oracle_gemm_blockscale
 *   op_tests/test_rmsnorm2dFusedAddQuant.py:23-55 run_torch -> oracle_rmsnorm_bf16,
 *                                                       oracle_add_rmsnorm_bf16
 */
#include "fp8bs_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

static inline uint32_t f2u(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float u2f(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* ---------------------------------------------------------------- 16-bit floats */

float oracle_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

uint16_t oracle_f32_to_bf16(float f)
{
    uint32_t u = f2u(f);
    if((u & 0x7fffffffu) > 0x7f800000u) /* NaN: keep sign, force a quiet payload */
        return (uint16_t)((u >> 16) | 0x0040u);
    /* add half of the dropped field, minus one when the kept LSB is even */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

float oracle_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    int      e    = (h >> 10) & 0x1f;
    uint32_t m    = h & 0x3ffu;
    if(e == 0x1f)
        return u2f(sign | 0x7f800000u | (m << 13));
    if(e == 0)
    {
        /* zero or subnormal: value = m * 2^-24 exactly */
        float v = ldexpf((float)m, -24);
        return u2f(f2u(v) | sign);
    }
    return u2f(sign | ((uint32_t)(e - 15 + 127) << 23) | (m << 13));
}

/* ---------------------------------------------------------------- e4m3fn
 * OCP FP8 E4M3 "fn": 1 sign, 4 exponent (bias 7), 3 mantissa; no infinities; S.1111.111 is
 * NaN; largest finite 448 = 1.75 * 2^8; smallest subnormal 2^-9.
 * Conversion = round to nearest, ties to even, on the real value; anything that would round
 * to the 480 slot (|f| > 464, or |f| == 464 rounding up - it does not, 464 ties to even 448)
 * becomes the NaN code, as does inf/NaN input (torch: f_bits >= bits(480) -> 0x7f, and the
 * rounding carry into 0x7f for 464 < |f| < 480).
 */
uint8_t oracle_f32_to_e4m3fn(float f)
{
    uint32_t u    = f2u(f);
    uint8_t  sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a    = u & 0x7fffffffu;
    if(a > 0x7f800000u || a >= 0x43f00000u) /* NaN, inf, >= 480 */
        return sign | 0x7f;
    if(a == 0)
        return sign;
    float mag = u2f(a);
    /* quantum of the target grid at this magnitude: 2^(e-3) for normals (e >= -6), 2^-9 below */
    int e;
    (void)frexpf(mag, &e); /* mag = m * 2^e, m in [0.5,1) -> true exponent e-1 */
    int texp = e - 1;
    if(texp < -6)
        texp = -6;
    /* scaled = mag / 2^(texp-3) is exact (power-of-two scaling, no underflow: result >= 0) */
    float scaled = ldexpf(mag, -(texp - 3));
    /* round to nearest even integer: scaled < 2^24 so nearbyintf in the default mode is exact RNE */
    float    r = nearbyintf(scaled);
    uint32_t q = (uint32_t)r; /* 0..16 */
    uint32_t code;
    if(texp == -6 && q < 8)
        code = q; /* subnormal (or zero) */
    else
    {
        if(q == 16) /* mantissa carry */
        {
            q = 8;
            texp += 1;
        }
        code = ((uint32_t)(texp + 7) << 3) | (q - 8);
    }
    if(code >= 0x7f)
        code = 0x7f; /* rounded into the 480 slot */
    return sign | (uint8_t)code;
}

float oracle_e4m3fn_to_f32(uint8_t c)
{
    uint32_t sign = (uint32_t)(c & 0x80u) << 24;
    int      e    = (c >> 3) & 0xf;
    int      m    = c & 7;
    float    v;
    if(e == 0xf && m == 7)
        return u2f(sign | 0x7fc00000u);
    if(e == 0)
        v = ldexpf((float)m, -9);
    else
        v = ldexpf((float)(8 + m), e - 7 - 3);
    return u2f(f2u(v) | sign);
}

void oracle_f32_to_e4m3fn_n(const float* f, uint8_t* c, int64_t n)
{
    for(int64_t i = 0; i < n; ++i)
        c[i] = oracle_f32_to_e4m3fn(f[i]);
}

void oracle_e4m3fn_to_f32_n(const uint8_t* c, float* f, int64_t n)
{
    for(int64_t i = 0; i < n; ++i)
        f[i] = oracle_e4m3fn_to_f32(c[i]);
}

/* ---------------------------------------------------------------- group quant */

static inline float load_as_f32(const void* x, int in_dtype, int64_t i)
{
    switch(in_dtype)
    {
    case 0: return oracle_bf16_to_f32(((const uint16_t*)x)[i]);
    case 1: return oracle_f16_to_f32(((const uint16_t*)x)[i]);
    default: return ((const float*)x)[i];
    }
}

/* torch.max(|x|) along the group: NaN wins over every number (first NaN seen is returned) */
static float group_amax(const float* v, int n)
{
    float best = -1.0f;
    for(int i = 0; i < n; ++i)
    {
        float a = fabsf(v[i]);
        if(a != a)
            return a;
        if(a > best)
            best = a;
    }
    return best;
}

/* quant.py:64-94 with dtypeMax = 448: scale = amax / 448 (one fp32 division), exact zero
 * scale replaced by 1, y = fp8(x / scale) (one fp32 division, then the e4m3fn rounding). */
static void quant_one_group(const float* v, int n, uint8_t* y, float* scale)
{
    float amax = group_amax(v, n);
    float s    = amax / 448.0f;
    if(s == 0.0f)
        s = 1.0f;
    for(int i = 0; i < n; ++i)
        y[i] = oracle_f32_to_e4m3fn(v[i] / s);
    *scale = s;
}

void oracle_group_quant(const void* x, int in_dtype, int64_t n_groups, int group_size,
                        uint8_t* y, float* scale)
{
    float* v = (float*)malloc(sizeof(float) * (size_t)group_size);
    for(int64_t g = 0; g < n_groups; ++g)
    {
        for(int i = 0; i < group_size; ++i)
            v[i] = load_as_f32(x, in_dtype, g * group_size + i);
        quant_one_group(v, group_size, y + g * group_size, scale + g);
    }
    free(v);
}

/* test_dispatch_combine.py:180-204: each 128x128 block is flattened and handed to
 * pertoken_quant as one row.  A ragged edge block simply holds fewer elements. */
void oracle_weight_block_quant(const uint16_t* w, int64_t N, int64_t K, int block_n,
                               int block_k, uint8_t* wq, float* scale)
{
    int64_t nb = (N + block_n - 1) / block_n, kb = (K + block_k - 1) / block_k;
    float*  v = (float*)malloc(sizeof(float) * (size_t)block_n * (size_t)block_k);
    uint8_t* q = (uint8_t*)malloc((size_t)block_n * (size_t)block_k);
    for(int64_t bi = 0; bi < nb; ++bi)
        for(int64_t bj = 0; bj < kb; ++bj)
        {
            int64_t n0 = bi * block_n, k0 = bj * block_k;
            int64_t rn = (N - n0 < block_n) ? N - n0 : block_n;
            int64_t rk = (K - k0 < block_k) ? K - k0 : block_k;
            int     cnt = 0;
            for(int64_t r = 0; r < rn; ++r)
                for(int64_t c = 0; c < rk; ++c)
                    v[cnt++] = oracle_bf16_to_f32(w[(n0 + r) * K + k0 + c]);
            quant_one_group(v, cnt, q, scale + bi * kb + bj);
            cnt = 0;
            for(int64_t r = 0; r < rn; ++r)
                for(int64_t c = 0; c < rk; ++c)
                    wq[(n0 + r) * K + k0 + c] = q[cnt++];
        }
    free(v);
    free(q);
}

/* ---------------------------------------------------------------- RMSNorm
 * F.rms_norm on bf16 input, as the reference test calls it: statistics and arithmetic in
 * fp32, one rounding to bf16 at the end:  bf16( (x * rstd) * w ),  rstd = 1/sqrt(mean(x^2)+eps).
 * The sum of squares is taken exactly here (each bf16 square is exact in fp64; a compensated
 * fp64 sum keeps the total exact far below fp32 resolution), so the result does not depend on
 * summation order.
 */
static double exact_sum_sq(const float* v, int64_t n)
{
    double s = 0.0, comp = 0.0;
    for(int64_t i = 0; i < n; ++i)
    {
        double p = (double)v[i] * (double)v[i];
        double t = s + p;
        if(fabs(s) >= fabs(p))
            comp += (s - t) + p;
        else
            comp += (p - t) + s;
        s = t;
    }
    return s + comp;
}

static void rmsnorm_row(const float* xf, const uint16_t* w, float eps, int64_t cols,
                        int gemma_norm, uint16_t* out)
{
    double ss   = exact_sum_sq(xf, cols);
    float  mean = (float)(ss / (double)cols);
    float  var  = mean + eps;
    float  rstd = 1.0f / sqrtf(var);
    for(int64_t c = 0; c < cols; ++c)
    {
        float wf = oracle_bf16_to_f32(w[c]);
        if(gemma_norm)
            wf = 1.0f + wf;
        float t = xf[c] * rstd;
        float u = t * wf;
        out[c]  = oracle_f32_to_bf16(u);
    }
}

void oracle_rmsnorm_bf16(const uint16_t* x, const uint16_t* w, float eps, int64_t rows,
                         int64_t cols, int gemma_norm, uint16_t* out)
{
    float* xf = (float*)malloc(sizeof(float) * (size_t)cols);
    for(int64_t r = 0; r < rows; ++r)
    {
        for(int64_t c = 0; c < cols; ++c)
            xf[c] = oracle_bf16_to_f32(x[r * cols + c]);
        rmsnorm_row(xf, w, eps, cols, gemma_norm, out + r * cols);
    }
    free(xf);
}

void oracle_add_rmsnorm_bf16(const uint16_t* x, const uint16_t* res_in, const uint16_t* w,
                             float eps, int64_t rows, int64_t cols, int gemma_norm,
                             uint16_t* res_out, uint16_t* out)
{
    float* xf = (float*)malloc(sizeof(float) * (size_t)cols);
    for(int64_t r = 0; r < rows; ++r)
    {
        for(int64_t c = 0; c < cols; ++c)
        {
            float    a = oracle_bf16_to_f32(x[r * cols + c]);
            float    b = oracle_bf16_to_f32(res_in[r * cols + c]);
            uint16_t s = oracle_f32_to_bf16(a + b);
            res_out[r * cols + c] = s;
            xf[c]                 = oracle_bf16_to_f32(s);
        }
        rmsnorm_row(xf, w, eps, cols, gemma_norm, out + r * cols);
    }
    free(xf);
}

/* ---------------------------------------------------------------- block-scale GEMM
 * test_gemm_a8w8_blockscale.py:28-54: x_deq = fp32(xq) * x_scale (per 1x128), w_deq =
 * fp32(wq) * w_scale (per 128x128), out = F.linear(x_deq, w_deq) in fp32, cast to bf16.
 */
void oracle_gemm_blockscale(const uint8_t* xq, const uint8_t* wq, const float* xs,
                            const float* ws, int64_t M, int64_t N, int64_t K, int64_t lda,
                            int64_t ldb, int accumulate, float* out_f32, uint16_t* out_bf16)
{
    const int64_t G  = 128;
    int64_t       kb = (K + G - 1) / G;
    float         lut[256];
    for(int i = 0; i < 256; ++i)
        lut[i] = oracle_e4m3fn_to_f32((uint8_t)i);
    float* a = (float*)malloc(sizeof(float) * (size_t)K);
    float* b = (float*)malloc(sizeof(float) * (size_t)N * (size_t)K);
    for(int64_t n = 0; n < N; ++n)
        for(int64_t k = 0; k < K; ++k)
            b[n * K + k] = lut[wq[n * ldb + k]] * ws[(n / G) * kb + k / G];
    for(int64_t m = 0; m < M; ++m)
    {
        for(int64_t k = 0; k < K; ++k)
            a[k] = lut[xq[m * lda + k]] * xs[m * kb + k / G];
        for(int64_t n = 0; n < N; ++n)
        {
            const float* bn = b + n * K;
            float        r;
            if(accumulate == 0)
            {
                double acc = 0.0;
                for(int64_t k = 0; k < K; ++k)
                    acc += (double)a[k] * (double)bn[k];
                r = (float)acc;
            }
            else
            {
                float acc = 0.0f;
                for(int64_t k = 0; k < K; ++k)
                {
                    float p = a[k] * bn[k];
                    acc     = acc + p;
                }
                r = acc;
            }
            out_f32[m * N + n] = r;
            if(out_bf16)
                out_bf16[m * N + n] = oracle_f32_to_bf16(r);
        }
    }
    free(a);
    free(b);
}
