// Types and device helpers shared by the block-scale GEMM kernels.
#pragma once

#include "fp8bs_launch.h"
#include "workspace.h"

namespace fp8bs {

typedef int      i32x8 __attribute__((ext_vector_type(8)));
typedef int      i32x4 __attribute__((ext_vector_type(4)));
typedef float    f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ f32x4 mfma_16x16x128_fp8(const i32x8& a, const i32x8& b, const f32x4& c)
{
    // cbsz = blgp = 0 selects e4m3 for both operands; zero scale operands select the
    // unscaled instruction
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

template <In16 DT>
__device__ __forceinline__ uint32_t pack2(float lo, float hi)
{
    if constexpr(DT == In16::bf16)
    {
        __bf16 a = (__bf16)lo, b = (__bf16)hi;
        return (uint32_t)__builtin_bit_cast(unsigned short, a) |
               ((uint32_t)__builtin_bit_cast(unsigned short, b) << 16);
    }
    else
    {
        _Float16 a = (_Float16)lo, b = (_Float16)hi;
        return (uint32_t)__builtin_bit_cast(unsigned short, a) |
               ((uint32_t)__builtin_bit_cast(unsigned short, b) << 16);
    }
}

struct GemmKernelParams
{
    const uint8_t* xq;
    const uint8_t* wq;
    const float*   xs;
    const float*   ws;
    uint16_t*      out;
    int32_t        M, N, K;
    int64_t        lda, ldb;
    int32_t        kblocks; // K / 128
    // x_scale element (m, kb) lives at xs[m * xs_m + kb * xs_k]: (K/128, 1) for the row-major
    // layout of gemm_a8w8_blockscale, (1, M) for the column-major one of the pre-shuffled entry
    int64_t        xs_m, xs_k;
    // weights pre-shuffled with layout (16,16) (aiter/ops/shuffle.py:192-205): per 16-row tile
    // and 32-byte K chunk, the 16 rows' first 16 bytes, then the 16 rows' second 16 bytes
    int32_t        w_shuffled;
};

// address of the 16-byte chunk c (0..7) of K block kb of weight row n, in either layout
__device__ __forceinline__ const uint8_t* w_chunk_ptr(const GemmKernelParams& p, int n, int kb, int c)
{
    if(p.w_shuffled)
        return p.wq + (size_t)(n >> 4) * 16 * (size_t)p.K + (size_t)(kb * 4 + (c >> 1)) * 512 +
               (size_t)(c & 1) * 256 + (size_t)(n & 15) * 16;
    return p.wq + (size_t)n * p.ldb + (size_t)kb * 128 + (size_t)c * 16;
}

// LDS tile: rows of 128 bytes (one K block); the 16-byte chunk c of row r lives at chunk
// c ^ lds_swizzle(r).  A fragment read is a ds_read_b128 in which lane (kg, l16) takes chunk 2 kg
// (or 2 kg + 1) of row l16.  The LDS serves such a read in four groups of 16 lanes -- lanes
// {0-3, 12-15, 20-23, 24-27}, {4-7, 8-11, 16-19, 28-31} and the same plus 32 -- and a group runs at
// full rate (256 bytes per clock) only if its 16 chunks fall on 16 different 16-byte bank groups
// of the 256-byte bank period.  A group holds rows {0-3, 12-15} of one kg and rows {4-11} of the
// neighbouring kg (chunks that differ by 2), so the term must send the even rows of
// {0,2,12,14 | 4,6,8,10 with bit 1 flipped} to eight different values, and the odd rows likewise:
// bit 0 = row bit 1, bits 1 and 2 = row bit 3 does (measured 4.3 clocks per read against 8.1 for
// c ^ (r & 7) or c ^ (r >> 1)).
__device__ __forceinline__ uint32_t lds_swizzle(uint32_t row) { return ((row >> 1) & 1u) | (((row >> 3) & 1u) * 6u); }

__device__ __forceinline__ uint32_t lds_off(uint32_t row, uint32_t chunk)
{
    return row * 128u + ((chunk ^ lds_swizzle(row)) << 4);
}


// launchers living in their own translation units
// K ranges per tile that the prefill kernel would choose on `cus` compute units, and the modelled
// duration (us) with them
struct PrefillPlan
{
    int   splits;
    float us;
    int   tile_n; // 256, 192 or 128 columns per tile
};
PrefillPlan gemm_prefill_plan(const GemmKernelParams& p, int cus);
// want_splits: K ranges per tile; 0 lets the launcher choose, 1 keeps a tile in one workgroup.
// want_tile_n: 256, 192 or 128 columns per tile; 0 lets the launcher choose (together with the K ranges).
hipError_t launch_gemm_prefill(const GemmKernelParams& p, In16 out_dtype, const LaunchCtx& ctx, int want_splits,
                               int want_tile_n = 0);
bool       gemm_prefill_supports(const GemmKernelParams& p);
hipError_t launch_gemm_decode(const GemmKernelParams& p, In16 out_dtype, int split_k_log2, const LaunchCtx& ctx,
                              const char* tuning = nullptr);
bool       gemm_decode_supports(const GemmKernelParams& p);
float      gemm_decode_estimate_us(const GemmKernelParams& p);
hipError_t launch_gemm_mid(const GemmKernelParams& p, In16 out_dtype, int split_k_log2, const LaunchCtx& ctx,
                           int tile = 0, int splits = 0);
bool       gemm_mid_supports(const GemmKernelParams& p);
// modelled duration (us) of the best mid_* tiling, for the choice between kernel families
void       gemm_mid_describe(const GemmKernelParams& g, char* buf, size_t n);
float      gemm_mid_estimate_us(const GemmKernelParams& p);
} // namespace fp8bs
