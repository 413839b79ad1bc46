// Internal interface between the C-ABI entry points and the mixture-of-experts launchers.
#pragma once

#include "fp8bs_launch.h"
#include "workspace.h"

namespace fp8bs {

struct TopkSoftmaxArgs
{
    const void* gating; // [tokens][experts], contiguous
    int         gating_dtype; // 0 bf16, 1 fp16, 2 fp32
    float*      weights; // [tokens][topk], row stride w_stride
    int32_t*    ids;     // [tokens][topk], row stride id_stride
    int32_t*    src_rows; // optional [tokens][topk]: slot * tokens + token
    int32_t     tokens, experts, topk;
    int64_t     w_stride, id_stride;
    bool        renorm;
};
hipError_t launch_topk_softmax(const TopkSoftmaxArgs& a, hipStream_t stream);

struct MoeSortArgs
{
    const int32_t* topk_ids;
    const float*   topk_weights;
    const int32_t* expert_mask;      // optional [experts]
    const int32_t* num_local_tokens; // optional device scalar
    int32_t*       sorted_ids;        // [max_padded]
    float*         sorted_weights;    // [max_padded]
    int32_t*       sorted_expert_ids; // [max_blocks]
    int32_t*       num_valid_ids;     // [2]
    void*          moe_buf;           // zeroed (may be null)
    size_t         moe_buf_bytes;     // multiple of 16
    int32_t        M, topk, experts, unit, max_padded, max_blocks;
    int32_t        w_rows;            // rows of topk_weights, <= M
    int64_t        id_stride, w_stride;
    int            device_id;
};
// *why receives a static message when scratch memory cannot be had
hipError_t launch_moe_sorting(const MoeSortArgs& a, hipStream_t stream, const char** why);

struct MoeArgs
{
    const uint8_t* xq;  // [M][dim] fp8 (row stride lda), or null when x16 is given
    const float*   xs;  // [dim/128][M]
    const void*    x16; // [M][dim] bf16/fp16 contiguous: quantised inside
    In16           x16_dtype;
    const uint8_t* w1;       // [experts][2*inter][dim] fp8, shuffled (16,16)
    const float*   w1_scale; // [experts][2*inter/128][dim/128]
    const uint8_t* w2;       // [experts][dim][inter] fp8, shuffled (16,16)
    const float*   w2_scale; // [experts][dim/128][inter/128]
    const int32_t* sorted_ids;
    const float*   sorted_weights;
    const int32_t* sorted_expert_ids;
    const int32_t* num_valid;
    void*          out; // [M][dim] 16-bit, row stride out_stride; accumulated into
    In16           out_dtype;
    int32_t        M, dim, inter, experts, topk, max_padded, max_blocks;
    // The kernels walk the sorted rows in blocks of block_rows (32; 16 when the arrays were sorted in
    // blocks of 16); max_blocks and max_padded count those.  A block's expert is
    // sorted_expert_ids[block >> expert_shift] (arrays sorted in blocks of 64 or 128: shift 1 or 2).
    int32_t        block_rows, expert_shift;
    int32_t        activation; // 0 silu, 1 gelu
    int32_t        gate_tiles; // first GEMM: 16-column tiles per workgroup (1, 2, 4), 0 = choose
    int32_t        down_waves; // second GEMM: waves per workgroup (2, 4, 8), 0 = choose
    int32_t        down_wave_cols; // second GEMM: columns per wave (64, 128), 0 = choose
    int32_t        down_mode;      // second GEMM: 1 = rows through memory + separate sum, 2 = per-token sum in LDS
    int32_t        pair_blocks;    // consecutive blocks of one expert multiplied in pairs: 1 / 0, -1 = choose
    int32_t        fine_tail;      // first GEMM: 0 = no narrow workgroups at the end of the launch, else choose
    int32_t        down_staged;    // second GEMM: 0 = 16-bit rows stored straight from the lanes, else through LDS as whole lines
    int32_t        gate_ring;      // first GEMM, pairs of blocks: 0 = every K block requested and waited for in turn, else weights two K blocks ahead through LDS
                                   // (where its tables fit); 0 = choose
    int64_t        lda, out_stride;
    int            device_id;
};
hipError_t launch_fmoe_blockscale(const MoeArgs& a, hipStream_t stream, const char** why);

} // namespace fp8bs
