// Internal interface between the C-ABI entry points (abi.hip) and the kernel launchers.
// Launchers receive operands the entry points have already validated; they only enqueue work.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fp8bs {

enum class In16 : int
{
    bf16 = 0,
    fp16 = 1
};

struct QuantArgs
{
    const void* x;        // 16-bit floats, n_groups * group contiguous
    uint8_t*    y;        // fp8 codes, same element order as x
    float*      scale;    // n_groups floats
    int64_t     rows;     // rows of the original [rows, K] view
    int32_t     groups_per_row; // K / group
    int32_t     group;    // 32, 64 or 128
    bool        transpose_scale; // scale[g_in_row * rows + row] instead of row-major
    const int32_t* num_rows;     // optional device scalar limiting the rows processed
    int32_t     num_rows_factor;
    In16        dtype;
    int32_t     scale_row_stride = 0; // row-major scales with this many floats between rows (0: groups_per_row)
};
hipError_t launch_group_quant(const QuantArgs& a, hipStream_t stream);

struct WeightQuantArgs
{
    const void* w;     // [N, K] 16-bit floats, row stride ldw elements
    uint8_t*    q;     // [N, K] fp8 codes, row stride ldq elements
    float*      scale; // [ceil(N/128), K/128]
    int64_t     N, K, ldw, ldq;
    In16        dtype;
};
hipError_t launch_weight_block_quant(const WeightQuantArgs& a, hipStream_t stream);

struct NormArgs
{
    const void* x;          // [rows, hidden] 16-bit, row stride x_stride (elements)
    const void* residual_in;  // optional, same layout, stride res_in_stride
    void*       residual_out; // optional (required with residual_in), stride res_out_stride
    const void* weight;     // [hidden] 16-bit
    void*       out16;      // 16-bit output (plain norm) or nullptr
    uint8_t*    out8;       // fp8 output (fused quant) or nullptr, contiguous rows
    float*      scale;      // [rows, hidden/group] (fused quant)
    int64_t     rows;
    int32_t     hidden;
    int64_t     x_stride, res_in_stride, res_out_stride, out_stride;
    float       eps;
    int32_t     group;      // 32/64/128 when out8 != nullptr
    bool        transpose_scale;
    bool        gemma_norm;
    In16        dtype;
};
hipError_t launch_rmsnorm(const NormArgs& a, hipStream_t stream);

struct GemmArgs
{
    const uint8_t* xq;  // [M, K] fp8, row stride lda bytes
    const uint8_t* wq;  // [N, K] fp8, row stride ldb bytes
    const float*   xs;  // [M, K/128]
    const float*   ws;  // [ceil(N/128), K/128]
    void*          out; // [M, N] 16-bit, contiguous
    int64_t        M, N, K, lda, ldb;
    In16           out_dtype;
    int            split_k_log2; // -1 = choose
    const char*    kernel_name;  // nullptr / "" = choose
    int            device_id;
    bool           w_shuffled;   // wq holds shuffle_weight(w, (16,16)); needs N % 16 == 0, ldb == K
    bool           xs_col_major; // xs holds [K/128][M] instead of [M][K/128]
    bool           static_scratch = false; // split-K scratch from the static buffer: the call allocates nothing
};
// Returns hipSuccess, or hipErrorInvalidValue with *why set to a static message.
hipError_t launch_gemm_blockscale(const GemmArgs& a, hipStream_t stream, const char** why);
// out[m][n] += bias[n] on a stored, contiguous [M][N] result of 16-bit values (N a multiple of 4)
hipError_t launch_gemm_bias_add(void* out, In16 dtype, const float* bias, int64_t M, int64_t N, hipStream_t stream);
const char* gemm_kernel_names();
// the kernel (and, for the mid_* family, K range count) taken for contiguous operands of this shape when none is named
void gemm_describe_choice(int64_t M, int64_t N, int64_t K, bool shuffled, char* buf, size_t n);
// what a call's (kernelName, splitK) pair resolves to, as "<kernel>;splitK=<n>"; false + *why for an unknown name
bool gemm_describe_request(int64_t M, int64_t N, int64_t K, bool shuffled, int split_k_log2, const char* kernel_name,
                           char* buf, size_t n, const char** why);

} // namespace fp8bs
