/*
 * CPU oracle for the FP8 block-scale path.  TEST INFRASTRUCTURE ONLY: nothing that ships
 * (the package, the C-ABI library) may include, link or call this.  Only tests, the smoke
 * check and the CPU-baseline leg of the benchmark use it, and only as the checker.
 *
 * Every function is a scalar restatement of the reference's torch semantics for the path;
 * the reference lines each one follows are cited at its definition in fp8bs_oracle.c.
 *
 * Pinning status (what independent evidence fixes each function, see tests/test_oracle_*.py):
 *   oracle_f32_to_e4m3fn      pinned: torch CPU .to(float8_e4m3fn) on 4M structured inputs
 *                             (every rounding boundary +-1 ulp) + known answers
 *   oracle_e4m3fn_to_f32      pinned: all 256 codes vs torch CPU, closed form
 *   oracle_bf16_* / f16       pinned: all 65536 codes vs torch CPU
 *   oracle_group_quant_*      pinned: torch CPU restatement of pertoken_quant (bitwise),
 *                             closed forms (amax->448, zero group->scale 1), invariants
 *   oracle_weight_block_quant pinned: same, via pertoken_quant on [nblocks,16384] views
 *   oracle_gemm_blockscale_*  pinned: fp64 textbook matmul on dequantised operands,
 *                             one-hot isolation of single scale products, torch F.linear
 *   oracle_rmsnorm_*          pinned to tolerance only: torch CPU F.rms_norm sums squares in
 *                             an unspecified fp32 order, so agreement is <=1 bf16 ulp with
 *                             >99.99% identical codes; closed form for constant rows.
 *                             Bitwise parity with torch for the norm: parity unpinned.
 */
#ifndef FP8BS_ORACLE_H
#define FP8BS_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* scalar conversions */
float    oracle_bf16_to_f32(uint16_t h);
uint16_t oracle_f32_to_bf16(float f);          /* round to nearest even, NaN kept quiet */
float    oracle_f16_to_f32(uint16_t h);
uint8_t  oracle_f32_to_e4m3fn(float f);        /* OCP e4m3fn, RNE, |f|>464 -> NaN code */
float    oracle_e4m3fn_to_f32(uint8_t c);

/* bulk versions (n elements) so the Python side can check millions of values quickly */
void oracle_f32_to_e4m3fn_n(const float* f, uint8_t* c, int64_t n);
void oracle_e4m3fn_to_f32_n(const uint8_t* c, float* f, int64_t n);

/* 1 x group_size dynamic quant of n_groups contiguous groups.
 * in_dtype: 0 = bf16, 1 = fp16 (both passed as raw 16-bit codes), 2 = fp32. */
void oracle_group_quant(const void* x, int in_dtype, int64_t n_groups, int group_size,
                        uint8_t* y, float* scale);

/* 128 x 128 block quant of a row-major [N,K] bf16 weight (ragged last blocks allowed);
 * scale is [ceil(N/128), ceil(K/128)] row-major. */
void oracle_weight_block_quant(const uint16_t* w, int64_t N, int64_t K, int block_n,
                               int block_k, uint8_t* wq, float* scale);

/* RMSNorm of row-major [rows, cols] bf16 with bf16 weight -> bf16 codes.
 * gemma_norm != 0 multiplies by (1 + w) instead of w. */
void oracle_rmsnorm_bf16(const uint16_t* x, const uint16_t* w, float eps, int64_t rows,
                         int64_t cols, int gemma_norm, uint16_t* out);

/* residual add (bf16 + bf16 -> bf16, one rounding) then RMSNorm as above; res_out gets the sum */
void oracle_add_rmsnorm_bf16(const uint16_t* x, const uint16_t* res_in, const uint16_t* w,
                             float eps, int64_t rows, int64_t cols, int gemma_norm,
                             uint16_t* res_out, uint16_t* out);

/* Block-scale GEMM: out[m,n] = sum_kb (sum_{k in kb} xq[m,k]*wq[n,k]) * xs[m,kb] * ws[n/128,kb].
 * accumulate == 0: dequantise both operands to fp32 first (one rounding each, as the reference
 *                  test does), accumulate products in fp64, round once to fp32.
 * accumulate == 1: same dequantised operands, plain fp32 running sum in k order.
 * out_f32 receives the fp32 result; out_bf16 (may be NULL) its bf16 rounding. */
void oracle_gemm_blockscale(const uint8_t* xq, const uint8_t* wq, const float* xs,
                            const float* ws, int64_t M, int64_t N, int64_t K, int64_t lda,
                            int64_t ldb, int accumulate, float* out_f32, uint16_t* out_bf16);

#ifdef __cplusplus
}
#endif
#endif
