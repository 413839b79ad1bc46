// Types and device helpers shared by the block-scale GEMM kernels.
#pragma once

#include "fp8bs_launch.h"

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
};

// LDS tile: rows of 128 bytes (one K block); the 16-byte chunk c of row r lives at chunk
// c ^ (r & 7) so that the 16 rows a quarter-wave reads with one ds_read_b128 spread over banks.
__device__ __forceinline__ uint32_t lds_off(uint32_t row, uint32_t chunk)
{
    return row * 128u + ((chunk ^ (row & 7u)) << 4);
}


// launchers living in their own translation units
hipError_t launch_gemm_prefill(const GemmKernelParams& p, In16 out_dtype, hipStream_t stream);
bool       gemm_prefill_supports(const GemmKernelParams& p);
hipError_t launch_gemm_decode(const GemmKernelParams& p, In16 out_dtype, int split_k_log2, int device_id,
                              hipStream_t stream, const char* tuning = nullptr);
bool       gemm_decode_supports(const GemmKernelParams& p);

} // namespace fp8bs
