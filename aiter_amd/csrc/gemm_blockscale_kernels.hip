// Block-scale FP8 GEMM for gfx950:  Out[m,n] = sum_kb dot(XQ[m,kb], WQ[n,kb]) * xs[m,kb] * ws[n/128,kb]
//
// Replaces the CK / CK-Tile device ops behind gemm_a8w8_blockscale
// (csrc/ck_gemm_a8w8_blockscale/include/gemm_a8w8_blockscale_common.cuh:97-176,
//  ..._cktile_common.cuh:121-140); semantics as in
// aiter/ops/triton/_triton_kernels/gemm/basic/gemm_a8w8_blockscale.py:160-190:
// one exact fp8 dot product per 128-wide K block, scaled in fp32 and accumulated in fp32.
//
// MFMA mapping.  v_mfma_f32_16x16x128_f8f6f4 consumes one whole 128-wide K block, so one
// instruction yields exactly the unscaled partial product of a 16x16 output tile for one
// scale block.  The weight rows play the MFMA "A" role and the activation rows the "B" role:
// a lane then owns 4 consecutive n for one m, which makes (a) the scale of its 4 accumulators
// one scalar per lane, xs[m,kb]*ws[nb,kb], and (b) its output 4 consecutive 16-bit values.
#include "fp8bs_launch.h"
#include "gemm_common.h"
#include <cstdio>

#include <string.h>

namespace fp8bs {

// ---------------------------------------------------------------- generic tile kernel
// BM x BN output tile per block (m = activation rows, n = weight rows), WAVES_M x WAVES_N
// waves, single-buffered LDS.  Handles every shape (ragged M and N); used for small and odd
// problems and as the always-available fallback.
template <In16 DT, int BM, int BN, int WAVES_M, int WAVES_N>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_tile_kernel(GemmKernelParams p)
{
    constexpr int T  = 64 * WAVES_M * WAVES_N;
    constexpr int TM = BM / WAVES_M, TN = BN / WAVES_N;
    constexpr int MT = TM / 16, NT = TN / 16;
    static_assert(TM % 16 == 0 && TN % 16 == 0, "wave tile must be a multiple of 16x16");

    __shared__ __attribute__((aligned(16))) uint8_t sW[BN * 128];
    __shared__ __attribute__((aligned(16))) uint8_t sX[BM * 128];

    const int t    = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int wm = (wave % WAVES_M) * TM, wn = (wave / WAVES_M) * TN;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int l16 = lane & 15, kg = lane >> 4;

    f32x4 acc[NT][MT];
#pragma unroll
    for(int i = 0; i < NT; ++i)
#pragma unroll
        for(int j = 0; j < MT; ++j)
            acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // rows of x_scale this lane needs (one per m tile), clamped for ragged M
    int mrow[MT];
#pragma unroll
    for(int j = 0; j < MT; ++j)
    {
        int m   = m0 + wm + j * 16 + l16;
        mrow[j] = m < p.M ? m : p.M - 1;
    }
    int nblk[NT];
#pragma unroll
    for(int i = 0; i < NT; ++i)
    {
        int n   = n0 + wn + i * 16;
        n       = n < p.N ? n : p.N - 1;
        nblk[i] = n >> 7;
    }

    for(int kb = 0; kb < p.kblocks; ++kb)
    {
        // global -> LDS, 16-byte chunks; 8 consecutive lanes cover one 128-byte row segment
        for(int q = t; q < BN * 8; q += T)
        {
            int row = q >> 3, c = q & 7;
            int n   = n0 + row;
            n       = n < p.N ? n : p.N - 1;
            u32x4 d = *(const u32x4*)w_chunk_ptr(p, n, kb, c);
            *(u32x4*)(sW + lds_off(row, c)) = d;
        }
        for(int q = t; q < BM * 8; q += T)
        {
            int row = q >> 3, c = q & 7;
            int m   = m0 + row;
            m       = m < p.M ? m : p.M - 1;
            u32x4 d = *(const u32x4*)(p.xq + (size_t)m * p.lda + (size_t)kb * 128 + c * 16);
            *(u32x4*)(sX + lds_off(row, c)) = d;
        }
        __syncthreads();

        i32x8 bx[MT];
#pragma unroll
        for(int j = 0; j < MT; ++j)
        {
            uint32_t row = wm + j * 16 + l16;
            i32x4    lo  = *(const i32x4*)(sX + lds_off(row, 2 * kg));
            i32x4    hi  = *(const i32x4*)(sX + lds_off(row, 2 * kg + 1));
            bx[j]        = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
        float sc[MT];
#pragma unroll
        for(int j = 0; j < MT; ++j)
            sc[j] = p.xs[(size_t)mrow[j] * p.xs_m + (size_t)kb * p.xs_k];

#pragma unroll
        for(int i = 0; i < NT; ++i)
        {
            uint32_t row = wn + i * 16 + l16;
            i32x4    lo  = *(const i32x4*)(sW + lds_off(row, 2 * kg));
            i32x4    hi  = *(const i32x4*)(sW + lds_off(row, 2 * kg + 1));
            i32x8    aw  = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            float    wsc = p.ws[(size_t)nblk[i] * p.kblocks + kb];
#pragma unroll
            for(int j = 0; j < MT; ++j)
            {
                f32x4 part = mfma_16x16x128_fp8(aw, bx[j], f32x4{0.f, 0.f, 0.f, 0.f});
                float s    = sc[j] * wsc;
#pragma unroll
                for(int r = 0; r < 4; ++r)
                    acc[i][j][r] = __builtin_fmaf(part[r], s, acc[i][j][r]);
            }
        }
        __syncthreads();
    }

    // epilogue: lane holds out[m][n .. n+3]
#pragma unroll
    for(int j = 0; j < MT; ++j)
    {
        int m = m0 + wm + j * 16 + l16;
        if(m >= p.M)
            continue;
#pragma unroll
        for(int i = 0; i < NT; ++i)
        {
            int       n   = n0 + wn + i * 16 + kg * 4;
            uint16_t* dst = p.out + (size_t)m * p.N + n;
            if(n + 3 < p.N && (p.N & 3) == 0)
            {
                u32x2 v = u32x2{pack2<DT>(acc[i][j][0], acc[i][j][1]),
                                pack2<DT>(acc[i][j][2], acc[i][j][3])};
                *(u32x2*)dst = v;
            }
            else
            {
#pragma unroll
                for(int r = 0; r < 4; ++r)
                    if(n + r < p.N)
                        dst[r] = (uint16_t)(pack2<DT>(acc[i][j][r], 0.f) & 0xffffu);
            }
        }
    }
}

// ---------------------------------------------------------------- dispatch

template <In16 DT, int BM, int BN, int WAVES_M, int WAVES_N>
static hipError_t launch_tile(const GemmKernelParams& p, hipStream_t stream)
{
    dim3 grid((p.N + BN - 1) / BN, (p.M + BM - 1) / BM);
    hipLaunchKernelGGL((gemm_tile_kernel<DT, BM, BN, WAVES_M, WAVES_N>), grid,
                       dim3(64 * WAVES_M * WAVES_N), 0, stream, p);
    return hipGetLastError();
}

static const char* const kKernelNames =
    "tile_16x256,tile_64x128,tile_128x128,mid_64x64,mid_64x128,mid_128x128,prefill_256x256,prefill_256x192,prefill_256x128,"
    "decode_stream";

const char* gemm_kernel_names() { return kKernelNames; }

// The kernel family taken when the caller names none.
// Up to 64 activation rows the weight-streaming kernel or the mid_* tilings, whichever is modelled
// faster: the streaming kernel where N / 16 row tiles with one K step per wave cover the chip
// ((1 ... 64, 7168, 2048): 6.0 ... 8.6 us against 8.8 ... 10.0), the tilings from 17 rows on where K
// is long or very short or N is large ((64, 24576, 1536): 12.6 us against 15.0; (64, 32768, 512): 7.1
// against 17.5; (32, 4608, 7168): 11.8 against 17.3; (8, 4096, 11008): 13.9 against 17.9; from one row
// on where the weights are large: (1, 16384, 4096) 16.2 against 18.2, (1, 32768, 512) 6.2 against 6.9).
// Above 64 rows, the 256-row
// tiling or the mid_* tilings, whichever is modelled faster.  Measured on the DeepSeek shapes, a
// 256x256 iteration over one K block takes 1.7 us while the tiles of a round cover up to 56 % of
// the compute units and up to 2.1 us when they cover all of them, against 0.8 us for a quarter of
// the area: it wins once its tiles cover about half of the chip.  Near a tie it is preferred: it
// gains more when the weights are still in the last-level cache.
static const char* automatic_choice(const GemmKernelParams& p)
{
    const float prefill_us = gemm_prefill_plan(p, 256).us; // fitted on a 256-CU part, like the mid model
    if(p.M <= 64 && gemm_decode_supports(p) && (!gemm_mid_supports(p) || gemm_mid_estimate_us(p) >= gemm_decode_estimate_us(p)))
        return "decode_stream";
    if(gemm_mid_supports(p) && (!gemm_prefill_supports(p) || gemm_mid_estimate_us(p) * 1.03f < prefill_us))
        return "mid_auto";
    if(gemm_prefill_supports(p))
    {
        const int bn = gemm_prefill_plan(p, 256).tile_n;
        return bn == 128 ? "prefill_256x128" : bn == 192 ? "prefill_256x192" : "prefill_256x256";
    }
    return "tile_128x128";
}

// Names of the reference's own kernel zoo ("a8w8_blockscale_1x128x128_256x16x128x256_..."), as
// its tuned tables hand them out (aiter/configs/model_configs/a8w8_blockscale_tuned_gemm_ds_v3.csv),
// say nothing about the kernels here.
static bool foreign_kernel_name(const char* name) { return strncmp(name, "a8w8_blockscale_", 16) == 0; }

// What a call's (kernelName, splitK) pair asks for.  splitK is a hint, never a reason to fail:
//  * a foreign name is dropped together with its splitK (tuned for that kernel): the library chooses;
//  * no name and splitK <= 0: the library chooses kernel and K ranges (the reference's default
//    splitK = 0 with no name means "nothing tuned", csrc/ck_gemm_a8w8_blockscale/gemm_a8w8_blockscale.cu:82-114);
//  * no name and splitK > 0: the automatic kernel with 2^splitK K ranges where that kernel can
//    split K (clamped to what the problem allows), ignored where it cannot;
//  * one of this library's names: that kernel; splitK = 0 keeps K in one range, > 0 as above.
struct KernelRequest
{
    const char* name;         // one of this library's names, never null
    int         split_k_log2; // -1 = choose
};
static KernelRequest resolve_request(const GemmArgs& a, const GemmKernelParams& p)
{
    const bool named = a.kernel_name && a.kernel_name[0] && !foreign_kernel_name(a.kernel_name);
    if(named)
        return KernelRequest{a.kernel_name, a.split_k_log2};
    const bool foreign = a.kernel_name && a.kernel_name[0];
    return KernelRequest{automatic_choice(p), (foreign || a.split_k_log2 <= 0) ? -1 : a.split_k_log2};
}

// One of this library's kernel names, taken apart.
enum class Family
{
    tile,
    decode,
    mid,
    prefill
};
struct ParsedKernel
{
    Family      family;
    int         tile;   // tile: 16256 / 64128 / 128128; mid: 0 (choose) / 64 / 64128 / 128
    int         splits; // ":s=<n>" of mid_* and prefill_*, 0 when absent
    const char* tuning; // what follows "decode_stream:", or null
};
static const char* const kUnknownName = "unknown kernelName (see aiter_fp8bs_gemm_kernel_names())";

static bool parse_kernel_name(const char* name, ParsedKernel* out)
{
    *out = ParsedKernel{Family::tile, 0, 0, nullptr};
    if(strcmp(name, "tile_16x256") == 0 || strcmp(name, "tile_64x128") == 0 || strcmp(name, "tile_128x128") == 0)
    {
        out->tile = name[5] == '1' ? (name[6] == '6' ? 16256 : 128128) : 64128;
        return true;
    }
    // "decode_stream" alone, or "decode_stream:r=2,s=4,w=4,g=256" to pin its work split
    if(strncmp(name, "decode_stream", 13) == 0 && (name[13] == 0 || name[13] == ':'))
    {
        out->family = Family::decode;
        out->tuning = name[13] == ':' ? name + 14 : nullptr;
        return true;
    }
    const char*  colon = strchr(name, ':');
    const size_t len   = colon ? (size_t)(colon - name) : strlen(name);
    auto         is    = [&](const char* s) { return strlen(s) == len && strncmp(name, s, len) == 0; };
    // "mid_128x128" alone, or "mid_128x128:s=7" to pin the number of K ranges
    if(strncmp(name, "mid_", 4) == 0)
    {
        out->family = Family::mid;
        out->tile   = is("mid_128x128") ? 128 : is("mid_64x128") ? 64128 : is("mid_64x64") ? 64 : is("mid_auto") ? 0 : -1;
        if(colon && (sscanf(colon, ":s=%d", &out->splits) != 1 || out->splits < 1 || out->splits > 64))
            return false;
        return out->tile >= 0;
    }
    // "prefill_256x256" / "prefill_256x192" / "prefill_256x128", or "prefill_256x256:s=2" to pin the number of K ranges per tile
    if(is("prefill_256x256") || is("prefill_256x192") || is("prefill_256x128"))
    {
        out->family = Family::prefill;
        out->tile   = is("prefill_256x128") ? 128 : is("prefill_256x192") ? 192 : 256;
        if(colon && (sscanf(colon, ":s=%d", &out->splits) != 1 || out->splits < 1 || out->splits > 16))
            return false;
        return true;
    }
    return false;
}

template <In16 DT>
static hipError_t dispatch(const GemmArgs& a, const GemmKernelParams& p, hipStream_t stream,
                           const char** why)
{
    const KernelRequest req   = resolve_request(a, p);
    const bool          named = req.name == a.kernel_name;
    ParsedKernel        k;
    if(!parse_kernel_name(req.name, &k))
    {
        *why = kUnknownName;
        return hipErrorInvalidValue;
    }
    LaunchCtx ctx;
    ctx.device_id = a.device_id;
    ctx.stream      = stream;
    ctx.why         = why;
    ctx.static_only = a.static_scratch;
    switch(k.family)
    {
    case Family::tile:
        // (these keep a tile's K in one workgroup: splitK is a hint they have no use for)
        if(k.tile == 16256)
            return launch_tile<DT, 16, 256, 1, 4>(p, stream);
        if(k.tile == 64128)
            return launch_tile<DT, 64, 128, 2, 2>(p, stream);
        return launch_tile<DT, 128, 128, 2, 2>(p, stream);
    case Family::decode:
        if(!gemm_decode_supports(p))
        {
            *why = "decode_stream handles 1 <= M <= 512";
            return hipErrorInvalidValue;
        }
        return launch_gemm_decode(p, DT, req.split_k_log2, ctx, k.tuning);
    case Family::mid:
        if(!gemm_mid_supports(p))
        {
            *why = "the mid_* kernels need operand matrices below 4 GiB";
            return hipErrorInvalidValue;
        }
        return launch_gemm_mid(p, DT, req.split_k_log2, ctx, k.tile, k.splits);
    case Family::prefill:
        if(!gemm_prefill_supports(p))
        {
            *why = "the prefill_* kernels need N % 4 == 0 and operand matrices below 4 GiB";
            return hipErrorInvalidValue;
        }
        // by name it keeps every tile in one workgroup (bitwise the result of the tile_* kernels)
        // unless ":s=" pins the K ranges per tile; chosen automatically, the launcher decides.
        // splitK is a hint this kernel has no use for.
        return launch_gemm_prefill(p, DT, ctx, k.splits > 0 ? k.splits : (named ? 1 : 0), named ? k.tile : 0);
    }
    *why = kUnknownName;
    return hipErrorInvalidValue;
}

hipError_t launch_gemm_blockscale(const GemmArgs& a, hipStream_t stream, const char** why)
{
    *why = nullptr;
    if(a.M == 0 || a.N == 0)
        return hipSuccess;
    GemmKernelParams p;
    p.xq      = a.xq;
    p.wq      = a.wq;
    p.xs      = a.xs;
    p.ws      = a.ws;
    p.out     = (uint16_t*)a.out;
    p.M       = (int32_t)a.M;
    p.N       = (int32_t)a.N;
    p.K       = (int32_t)a.K;
    p.lda     = a.lda;
    p.ldb     = a.ldb;
    p.kblocks = (int32_t)(a.K / 128);
    p.xs_m       = a.xs_col_major ? 1 : a.K / 128;
    p.xs_k       = a.xs_col_major ? a.M : 1;
    p.w_shuffled = a.w_shuffled ? 1 : 0;
    return a.out_dtype == In16::bf16 ? dispatch<In16::bf16>(a, p, stream, why)
                                     : dispatch<In16::fp16>(a, p, stream, why);
}

void gemm_describe_choice(int64_t M, int64_t N, int64_t K, bool shuffled, char* buf, size_t n)
{
    GemmKernelParams p{};
    p.M          = (int32_t)M;
    p.N          = (int32_t)N;
    p.K          = (int32_t)K;
    p.lda        = K;
    p.ldb        = K;
    p.kblocks    = (int32_t)(K / 128);
    p.w_shuffled = shuffled ? 1 : 0;
    const char* name = automatic_choice(p);
    if(strcmp(name, "mid_auto") == 0)
        gemm_mid_describe(p, buf, n);
    else if(strncmp(name, "prefill_", 8) == 0 && gemm_prefill_plan(p, 256).splits > 1)
        snprintf(buf, n, "%s:s=%d", name, gemm_prefill_plan(p, 256).splits); // as on a 256-CU part
    else
        snprintf(buf, n, "%s", name);
}

// "<kernel>;splitK=<n>": what the pair (kernelName, splitK) of a call resolves to for contiguous
// operands of this shape (n = -1: the kernel chooses its K ranges).  False with *why set when the
// name is neither one of this library's nor one of the reference's zoo.
bool gemm_describe_request(int64_t M, int64_t N, int64_t K, bool shuffled, int split_k_log2, const char* kernel_name,
                           char* buf, size_t n, const char** why)
{
    GemmKernelParams p{};
    p.M          = (int32_t)M;
    p.N          = (int32_t)N;
    p.K          = (int32_t)K;
    p.lda        = K;
    p.ldb        = K;
    p.kblocks    = (int32_t)(K / 128);
    p.w_shuffled = shuffled ? 1 : 0;
    GemmArgs a{};
    a.kernel_name        = kernel_name;
    a.split_k_log2       = split_k_log2;
    const KernelRequest r = resolve_request(a, p);
    ParsedKernel        k;
    if(!parse_kernel_name(r.name, &k))
    {
        *why = kUnknownName;
        return false;
    }
    if(r.name != kernel_name) // chosen here: say which tiling and K ranges the choice means
    {
        char chosen[48];
        gemm_describe_choice(M, N, K, shuffled, chosen, sizeof chosen);
        if(r.split_k_log2 >= 0) // the caller's ranges replace the choice's
            if(char* colon = strchr(chosen, ':'))
                *colon = 0;
        snprintf(buf, n, "%s;splitK=%d", chosen, r.split_k_log2);
    }
    else
        snprintf(buf, n, "%s;splitK=%d", r.name, r.split_k_log2);
    return true;
}


namespace {
// out[m][n] = round16(float(out[m][n]) + bias[n]), four columns per thread
template <In16 DT>
__global__ __launch_bounds__(256) void gemm_bias_add_kernel(uint16_t* __restrict__ out, const float* __restrict__ bias,
                                                            int64_t quads, int32_t quads_per_row)
{
    const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if(q >= quads)
        return;
    const int   n = (int)(q % quads_per_row) * 4;
    const u32x2 v = *(const u32x2*)(out + q * 4);
    const f32x4 b = *(const f32x4*)(bias + n);
    float       f[4];
#pragma unroll
    for(int c = 0; c < 4; ++c)
    {
        const unsigned short h = (unsigned short)((v[c >> 1] >> (16 * (c & 1))) & 0xffffu);
        if constexpr(DT == In16::bf16)
            f[c] = __uint_as_float((uint32_t)h << 16) + b[c];
        else
            f[c] = (float)__builtin_bit_cast(_Float16, h) + b[c];
    }
    *(u32x2*)(out + q * 4) = u32x2{pack2<DT>(f[0], f[1]), pack2<DT>(f[2], f[3])};
}
} // namespace

// Adds a per-column fp32 bias onto a stored [M][N] result (N a multiple of 4, rows contiguous).
hipError_t launch_gemm_bias_add(void* out, In16 dtype, const float* bias, int64_t M, int64_t N, hipStream_t stream)
{
    const int64_t quads = M * N / 4;
    if(quads == 0)
        return hipSuccess;
    const dim3 grid((unsigned)((quads + 255) / 256));
    if(dtype == In16::bf16)
        hipLaunchKernelGGL(gemm_bias_add_kernel<In16::bf16>, grid, dim3(256), 0, stream, (uint16_t*)out, bias, quads,
                           (int32_t)(N / 4));
    else
        hipLaunchKernelGGL(gemm_bias_add_kernel<In16::fp16>, grid, dim3(256), 0, stream, (uint16_t*)out, bias, quads,
                           (int32_t)(N / 4));
    return hipGetLastError();
}

} // namespace fp8bs
