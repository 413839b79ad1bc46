/*
 * C ABI of libaiter_fp8bs.so: the gfx950 (MI355X) implementation of the DeepSeek-style FP8
 * block-scale path -- 1x128 dynamic FP8 group quant, RMSNorm (+residual add) fused with that
 * quant, and the 1x128 / 128x128 block-scale FP8 GEMM with bf16/fp16 output.
 *
 * Calling convention (the reference's ctypes flavour, aiter/jit/core.py:1306-1323 and
 * :1595-1612): every tensor is a BORROWED descriptor (`aiter_tensor_t*`, the caller owns the
 * memory and keeps it alive until the stream has run the work); `Optional[Tensor]` is NULL;
 * `int` is int64_t, `bool` is int, `float` is float, `str` is const char*; the caller's HIP
 * stream is the last argument.  Functions only enqueue work on that stream and can be captured
 * into a HIP graph.
 * Scratch memory: the GEMM entry points (when K is split across workgroups) and the
 * mixture-of-experts entry points use scratch buffers that the library owns.  Eager calls take
 * them per (device, stream), allocated (hipMalloc) on the first call on that stream that needs
 * a larger one: calls on different streams never share scratch, and host threads may call
 * concurrently (the launches of calls that use scratch are serialised by a lock).  A buffer that
 * has been handed out is never freed, so graphs captured earlier stay valid.  A call whose
 * stream is capturing allocates, clears and synchronises nothing: it uses a per-device buffer
 * reserved for graphs, which every eager call keeps at least as large as its own need (up to
 * 256 MiB of split-K partial tiles, 1 GiB of expert-layer intermediates).  So: run a call once
 * eagerly, on any stream of the device, before recording it; a call recorded without that fails
 * with a message.  Calls recorded on forked streams of ONE capture may run side by side when the
 * graph is replayed: each stream of a capture that records a scratch-using call gets a part (lane)
 * of the graph buffer to itself, and there are as many lanes (at most four) as streams of the
 * device have run scratch-using calls eagerly -- a warm-up that forks side streams the way the
 * capture will prepares them; a capture that forks wider is refused with a message (status -1,
 * the capture stays valid).  Graphs of one device share the graph buffer with each other (never
 * with eager work): do not replay two of them concurrently.  An eager call that has to allocate
 * while another host thread is capturing a graph allocates with its own thread's capture mode
 * set to relaxed (hipThreadExchangeStreamCaptureMode), which does not invalidate that capture;
 * if the runtime refuses the allocation all the same, the call returns -1 with a message that
 * says so.  When more than 1024 (device, stream) pairs have held scratch, the pair used longest
 * ago hands its buffers on (after a device synchronisation).  Nothing else allocates, and
 * nothing else synchronises.
 * Return value: 0 on success, -1 on failure with the message available from
 * aiter_get_last_error() (thread local).  No C++ exception crosses this boundary.
 *
 * Descriptor layout follows csrc/include/aiter_tensor.h:8-17 (160 bytes) and the dtype codes
 * follow csrc/include/aiter_enum.h:34-51 of the reference, so that the reference's own ctypes
 * marshalling (aiter/utility/aiter_types.py:68-87, aiter/utility/dtypes.py:101-129) can be
 * pointed at this library unchanged.
 */
#ifndef AITER_FP8BS_H
#define AITER_FP8BS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* csrc/include/aiter_enum.h:34-51 */
typedef enum
{
    AITER_DTYPE_fp8 = 0, /* OCP e4m3fn on gfx950 */
    AITER_DTYPE_fp8_e8m0,
    AITER_DTYPE_fp16,
    AITER_DTYPE_bf16,
    AITER_DTYPE_fp32,
    AITER_DTYPE_i4x2,
    AITER_DTYPE_fp4x2,
    AITER_DTYPE_u32,
    AITER_DTYPE_i32,
    AITER_DTYPE_i16,
    AITER_DTYPE_i8,
    AITER_DTYPE_u8,
    AITER_DTYPE_i64,
    AITER_DTYPE_u64
} AiterDtype;

/* csrc/include/aiter_tensor.h:8-17 */
typedef struct aiter_tensor_t
{
    void*   ptr;        /* device pointer */
    size_t  numel_;     /* number of elements */
    int     ndim;       /* 0..8 */
    int64_t shape[8];
    int64_t strides[8]; /* in elements */
    int     dtype_;     /* AiterDtype */
    int     device_id;  /* GPU ordinal, -1 = host memory */
} aiter_tensor_t;

/* hipStream_t without pulling the HIP headers into C callers */
typedef void* aiter_stream_t;

/* ---- error / version plumbing: csrc/include/aiter_ctypes_error.h:59-70 ---- */
int         aiter_ctypes_abi_version(void); /* == 2 */
const char* aiter_get_last_error(void);     /* NULL when no error is pending */
void        aiter_clear_last_error(void);

/*
 * 1 x G dynamic group quant (G = input.shape[-1] in {32, 64, 128}).
 * Replaces aiter::dynamic_per_token_scaled_quant, csrc/include/quant.h:18-24 (group branch of
 * csrc/kernels/quant_kernels.cu:738-804) as bound by aiter/ops/quant.py:754-763.
 *   out      fp8 [..., K] contiguous                (K = out.shape[-1], K % G == 0)
 *   input    bf16|fp16, the same memory viewed [-1, G], contiguous
 *   scales   fp32, numel == input.numel / G; written row-major [rows, K/G], or
 *            [K/G, rows] when shuffle_scale != 0   (rows = numel(out) / K)
 *   scale_ub must be NULL (unused by the group branch of the reference)
 *   num_rows optional int32[1] on the device: only the first num_rows[0]*num_rows_factor rows
 *            are quantised, the rest of out/scales is left untouched
 * Arithmetic follows the reference's torch definition (aiter/ops/quant.py:64-94), bit for bit:
 * scale = amax/448 (exact zero -> 1), code = e4m3fn_rne(x / scale), both IEEE fp32 divisions.
 */
int dynamic_per_token_scaled_quant(aiter_tensor_t* out, aiter_tensor_t* input,
                                   aiter_tensor_t* scales, aiter_tensor_t* scale_ub,
                                   int shuffle_scale, aiter_tensor_t* num_rows,
                                   int64_t num_rows_factor, aiter_stream_t stream);

/*
 * RMSNorm -> bf16|fp16.  Replaces aiter::rmsnorm, csrc/include/rmsnorm_quant.h:37-41
 * (binding aiter/ops/rmsnorm.py:625-632).
 *   out, input [rows, hidden] same 16-bit dtype, last dim contiguous; weight [hidden] same dtype
 *   out = round16( (x * rstd) * w ), rstd = 1/sqrt(mean(x^2) + epsilon), fp32 arithmetic;
 *   gemma_norm != 0 uses (1 + w).
 */
int rmsnorm(aiter_tensor_t* out, aiter_tensor_t* input, aiter_tensor_t* weight, float epsilon,
            int gemma_norm, aiter_stream_t stream);

/*
 * RMSNorm fused with the 1 x group_size FP8 quant of its (16-bit rounded) result.
 * Replaces aiter::rmsnorm_quant, csrc/include/rmsnorm_quant.h:28-35 (binding
 * aiter/ops/rmsnorm.py:612-622; caller aiter/ops/rmsnorm.py:506-532).
 *   out fp8 [rows, hidden]; scale fp32 [rows, hidden/group_size] (or transposed when
 *   shuffle_scale != 0); group_size in {32, 64, 128}; hidden % group_size == 0; hidden <= 8192.
 * The result is bit-identical to rmsnorm() followed by dynamic_per_token_scaled_quant().
 */
int rmsnorm_quant(aiter_tensor_t* out, aiter_tensor_t* input, aiter_tensor_t* scale,
                  aiter_tensor_t* weight, float epsilon, int64_t group_size, int shuffle_scale,
                  int gemma_norm, aiter_stream_t stream);

/*
 * Residual-add variants: residual_out = round16(input + residual_in), then as above on
 * residual_out.  Replace aiter::add_rmsnorm / aiter::add_rmsnorm_quant,
 * csrc/include/rmsnorm_quant.h:9-26 (bindings aiter/ops/rmsnorm.py:585-609).
 */
int add_rmsnorm(aiter_tensor_t* out, aiter_tensor_t* input, aiter_tensor_t* residual_in,
                aiter_tensor_t* residual_out, aiter_tensor_t* weight, float epsilon,
                int gemma_norm, aiter_stream_t stream);

int add_rmsnorm_quant(aiter_tensor_t* out, aiter_tensor_t* input, aiter_tensor_t* residual_in,
                      aiter_tensor_t* residual_out, aiter_tensor_t* scale,
                      aiter_tensor_t* weight, float epsilon, int64_t group_size,
                      int shuffle_scale, int gemma_norm, aiter_stream_t stream);

/*
 * Weight-side quantiser: one fp32 scale per 128x128 block of a [N, K] weight matrix, fp8 codes by
 * the same definition as the activation quant (scale = amax/448, zero block -> 1, code =
 * e4m3fn(w / scale), true divisions).  The reference performs this offline step with torch ops,
 * op_tests/multigpu_tests/test_dispatch_combine.py:180-204 (pertoken_quant,
 * aiter/ops/quant.py:64-94, on [n_blocks, 128*128] views); this is the same arithmetic on the GPU.
 *   input  bf16|fp16 [N, K], K % 128 == 0, row stride honoured; rows past N in the last block
 *          count as zeros
 *   out    fp8 [N, K], row stride honoured
 *   scales fp32 [ceil(N/128), K/128] contiguous
 */
int weight_per_128x128_quant(aiter_tensor_t* out, aiter_tensor_t* input, aiter_tensor_t* scales,
                             aiter_stream_t stream);

/*
 * Block-scale FP8 GEMM.  Replaces gemm_a8w8_blockscale,
 * csrc/ck_gemm_a8w8_blockscale/gemm_a8w8_blockscale.cu:82-114 (binding
 * aiter/ops/gemm_op_a8w8.py:285-298).
 *   XQ      fp8 [M, K], row stride honoured (last dim contiguous)
 *   WQ      fp8 [N, K], row stride honoured (last dim contiguous)
 *   x_scale fp32 [M, K/128] contiguous
 *   w_scale fp32 [ceil(N/128), K/128] contiguous
 *   Out     bf16|fp16 [M, N] contiguous
 *   Out[m,n] = round16( sum_kb  dot(XQ[m, kb], WQ[n, kb]) * x_scale[m,kb] * w_scale[n/128,kb] )
 *   with exact fp8 products, fp32 accumulation and one final rounding.  K % 128 == 0.
 *   kernelName: "" or NULL lets the library choose; one of aiter_fp8bs_gemm_kernel_names() asks
 *   for that kernel; a name of the reference's own zoo ("a8w8_blockscale_...", as its tuned tables
 *   carry them) is accepted and dropped together with the splitK that came with it.
 *   splitK (-1..30, log2 of the number of K partitions in the reference) is a hint and never a
 *   reason to fail: with no kernelName, <= 0 lets the library choose and > 0 asks the chosen
 *   kernel for 2^splitK K ranges, clamped to what the problem allows and ignored by kernels that
 *   keep a tile's K in one workgroup; with one of this library's names, 0 keeps K in one range.
 *   aiter_fp8bs_gemm_resolve reports what a pair resolves to.  Results are deterministic for a
 *   given (shape, kernelName, splitK).
 */
int gemm_a8w8_blockscale(aiter_tensor_t* XQ, aiter_tensor_t* WQ, aiter_tensor_t* x_scale,
                         aiter_tensor_t* w_scale, aiter_tensor_t* Out, int64_t splitK,
                         const char* kernelName, aiter_stream_t stream);

/*
 * gemm_a8w8_blockscale for callers that cannot allocate device memory (code under HIP graph
 * capture that was never run eagerly, tight serving loops, harnesses that forbid hipMalloc).  It
 * has no counterpart in the reference.  Same operands, same kernels, same results bit for bit;
 * the split-K scratch (fp32 partial tiles, tickets) comes from a fixed buffer in device memory
 * that the library's code object carries: 32 MiB of partial tiles and 4 MiB of counters and exchange slots per GPU, held
 * until the process ends.  The call allocates nothing (no hipMalloc, hipFree or allocating
 * library routine).  A problem whose kernel needs more than the buffer holds is rejected with a
 * message (status -1).  Every call on a GPU uses that GPU's one buffer: calls that overlap on one
 * GPU (different streams, or a graph replay beside eager calls) race; calls on one stream are
 * ordered and safe.  Where the library chooses the K ranges itself (no count named by kernelName or
 * splitK), it takes the best plan whose partial tiles fit the buffer.
 */
int gemm_a8w8_blockscale_noalloc(aiter_tensor_t* XQ, aiter_tensor_t* WQ, aiter_tensor_t* x_scale,
                                 aiter_tensor_t* w_scale, aiter_tensor_t* Out, int64_t splitK,
                                 const char* kernelName, aiter_stream_t stream);

/*
 * The same GEMM on pre-shuffled weights.  Replaces gemm_a8w8_blockscale_bpreshuffle,
 * csrc/ck_gemm_a8w8_blockscale_bpreshuffle/gemm_a8w8_blockscale_bpreshuffle.cu:64-89 (declared
 * include/gemm_a8w8_blockscale_bpreshuffle.h:7-13, binding aiter/ops/gemm_op_a8w8.py:318-330).
 *   WQ      fp8 [N, K] contiguous, holding shuffle_weight(w, layout=(16,16))
 *           (aiter/ops/shuffle.py:192-205): per 16-row tile and 32-byte K chunk, the 16 rows'
 *           first 16 bytes, then their second 16 bytes.  N % 16 == 0.
 *   x_scale fp32, M*K/128 values stored column-major: element (m, kb) at kb*M + m.  Accepted
 *           as a contiguous buffer of any shape with that many elements or as an [M, K/128]
 *           view with strides (1, M) (op_tests/test_gemm_a8w8_blockscale.py:112-125).
 *   XQ, w_scale, Out, kernelName and the arithmetic are those of gemm_a8w8_blockscale.
 */
int gemm_a8w8_blockscale_bpreshuffle(aiter_tensor_t* XQ, aiter_tensor_t* WQ, aiter_tensor_t* x_scale,
                                     aiter_tensor_t* w_scale, aiter_tensor_t* Out,
                                     const char* kernelName, aiter_stream_t stream);

/*
 * The entry point of the reference's hand-scheduled gfx950 kernel for the same operands.  Replaces
 * gemm_a8w8_blockscale_bpreshuffle_asm, csrc/py_itfs_cu/asm_a8w8_blockscale_bpreshuffle.cu:253-266
 * (binding aiter/ops/gemm_op_a8w8.py:371-430; note the argument order: out third).
 *   A, B, A_scale, B_scale, out: XQ, WQ, x_scale, w_scale, Out of gemm_a8w8_blockscale_bpreshuffle,
 *           without that kernel's M >= 16, K >= 512, bf16 limits.
 *   bias    optional fp32 [N] or [1, N]: out[m][n] = round16(float(round16(acc[m][n])) + bias[n]),
 *           added by a second launch onto the stored result (two roundings; N % 4 == 0).
 *   splitK, kernelName: tuning of the reference's kernel, not interpreted.  bpreshuffle must be
 *           non-zero.  zero_bias_buf (the zeros that kernel reads when there is no bias) is ignored.
 */
int gemm_a8w8_blockscale_bpreshuffle_asm(aiter_tensor_t* A, aiter_tensor_t* B, aiter_tensor_t* out,
                                         aiter_tensor_t* A_scale, aiter_tensor_t* B_scale, aiter_tensor_t* bias,
                                         int splitK, const char* kernelName, int bpreshuffle,
                                         aiter_tensor_t* zero_bias_buf, aiter_stream_t stream);

/* Comma-separated list of the tile kernels gemm_a8w8_blockscale can be asked for by name
 * (the counterpart of the reference's generated kernel zoo,
 * csrc/ck_gemm_a8w8_blockscale/gemm_a8w8_blockscale_instance.py:73-117). */
const char* aiter_fp8bs_gemm_kernel_names(void);

/* The kernel the library takes for contiguous operands of shape M x N x K when kernelName is empty,
 * written to `out` (at least 32 characters) in the form kernelName accepts, e.g. "decode_stream",
 * "prefill_256x256", "prefill_256x256:s=2", "mid_128x128:s=2" (":s=" = K ranges per tile).  Host-only: no device is touched.  The counterpart of the
 * reference's lookup in its tuned tables, get_CKGEMM_config (aiter/ops/gemm_op_a8w8.py:448-490):
 * here the choice is a shape rule inside the library. */
int aiter_fp8bs_gemm_choice(int64_t M, int64_t N, int64_t K, int preshuffled, char* out, int64_t out_len);

/* What the pair (kernelName, splitK) of a gemm_a8w8_blockscale call resolves to for contiguous
 * operands of shape M x N x K, written to `out` (at least 64 characters) as
 * "<kernel>;splitK=<n>" with <kernel> in the form kernelName accepts and n = -1 when the kernel
 * chooses its K ranges.  Host-only.  Fails (-1) for a kernelName that is neither one of this
 * library's nor one of the reference's zoo, as the GEMM entry points do. */
int aiter_fp8bs_gemm_resolve(int64_t M, int64_t N, int64_t K, int preshuffled, int64_t splitK, const char* kernelName,
                             char* out, int64_t out_len);

/*
 * ---- block-scale mixture of experts (gated experts, fp8 e4m3fn, 1x128 / 128x128 scales) ----
 *
 * Softmax over the experts, top-k, optional renormalisation of the k weights.
 * Replaces aiter::topk_softmax as bound by aiter/ops/moe_op.py:29-66 (used by fused_topk,
 * aiter/fused_moe.py:4058-4130).
 *   topk_weights fp32 [tokens, topk]; topk_indices int32 [tokens, topk] (rows may be strided);
 *   token_expert_indices optional int32 [tokens, topk] (slot * tokens + token);
 *   gating_output bf16|fp16|fp32 [tokens, experts] contiguous, experts <= 1024, topk <= 32.
 * Ties go to the lower expert index.
 */
int topk_softmax(aiter_tensor_t* topk_weights, aiter_tensor_t* topk_indices,
                 aiter_tensor_t* token_expert_indices, aiter_tensor_t* gating_output, int need_renorm,
                 aiter_stream_t stream);

/*
 * Sort the routed (token, slot) pairs by expert into blocks of unit_size rows and zero moe_buf.
 * Replaces moe_sorting_fwd, csrc/include/moe_sorting.h:6-17 as bound by
 * aiter/ops/moe_sorting.py:11-25; layout as in op_tests/test_moe_sorting.py:44-105:
 *   sorted_token_ids  int32 [tokens*topk + num_experts*unit_size - topk]: per local expert its
 *                     pairs as (slot << 24 | token), ascending, padded with (topk << 24 | tokens)
 *   sorted_weights    fp32, same length: the pairs' routing weights
 *   sorted_expert_ids int32 [ceil(that length / unit_size)]: local expert id per block, -1 beyond
 *   num_valid_ids     int32 [2]: {padded total, tokens sorted}
 *   moe_buf           optional, any dtype, contiguous: set to zero
 *   local_expert_mask optional int32 [num_experts]: experts with 0 are skipped and the others
 *                     renumbered; num_local_tokens optional int32 device scalar: only that many
 *                     rows of topk_ids take part.  dispatch_policy is accepted and ignored.
 */
int moe_sorting_fwd(aiter_tensor_t* topk_ids, aiter_tensor_t* topk_weights, aiter_tensor_t* sorted_token_ids,
                    aiter_tensor_t* sorted_weights, aiter_tensor_t* sorted_expert_ids,
                    aiter_tensor_t* num_valid_ids, aiter_tensor_t* moe_buf, int64_t num_experts,
                    int64_t unit_size, aiter_tensor_t* local_expert_mask, aiter_tensor_t* num_local_tokens,
                    int64_t dispatch_policy, aiter_stream_t stream);

/*
 * Gated experts on sorted tokens: out[token] += sum_k weight_k * down_e(act(gate_e x) * up_e x).
 * Replaces fmoe_fp8_blockscale_g1u1, csrc/py_itfs_cu/asm_fmoe.cu:893-958 as bound by
 * aiter/ops/moe_op.py:224-244 and called by op_tests/test_moe_blockscale.py:130-162.
 *   out    bf16|fp16 [tokens, dim], accumulated into (moe_sorting_fwd zeroes it)
 *   input  fp8 [tokens, dim] with input_scale fp32 [dim/128, tokens] (the transposed scales of
 *          the 1x128 quant), or bf16|fp16 [tokens, dim] with input_scale NULL (quantised inside)
 *   gate   fp8 [experts, 2*inter_dim, dim]: gate rows then up rows, each expert pre-shuffled
 *          with layout (16,16) (aiter/ops/shuffle.py:192-205); fc1_scale fp32
 *          [experts, 2*inter_dim/128 * dim/128]
 *   down   fp8 [experts, dim, inter_dim], pre-shuffled likewise; fc2_scale fp32
 *          [experts, dim/128 * inter_dim/128]
 *   the four sorted arrays as moe_sorting_fwd writes them with unit_size = block_size_M
 *   activation 0 = silu, 1 = gelu; fc_scale_blkn = fc_scale_blkk = 128; block_size_M = 16, 32, 64
 *   (the sizes the reference has kernels for: hsa/gfx950/fmoe/silu/fmoe_bf16_blockscaleFp8_g1u1_silu.csv,
 *   column subGU_m) or 128;
 *   fc2_smooth_scale must be NULL; kernel_name names the reference's tuned kernels and is only a
 *   tuning hint here ("nt=1|2|4", "dw=2|4|8", "dc=2|4|8", "down=rows", "down=cols"; anything
 *   else: choose).
 * The product of the first GEMM is quantised 1x128 to fp8 for the second.  Each token's k
 * contributions are added in a fixed order (sorted order while the per-token tables of the second GEMM fit
 * the LDS, about 280 tokens at inter = 256; slot order beyond):
 * results do not depend on timing.  Scratch memory: see the top of this file.
 */
int fmoe_fp8_blockscale_g1u1(aiter_tensor_t* out, aiter_tensor_t* input, aiter_tensor_t* gate, aiter_tensor_t* down,
                             aiter_tensor_t* sorted_token_ids, aiter_tensor_t* sorted_weights,
                             aiter_tensor_t* sorted_expert_ids, aiter_tensor_t* num_valid_ids, int64_t topk,
                             aiter_tensor_t* input_scale, aiter_tensor_t* fc1_scale, aiter_tensor_t* fc2_scale,
                             const char* kernel_name, int64_t fc_scale_blkn, int64_t fc_scale_blkk,
                             aiter_tensor_t* fc2_smooth_scale, int64_t activation, int64_t block_size_M,
                             aiter_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* AITER_FP8BS_H */
