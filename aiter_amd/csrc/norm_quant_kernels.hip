// 1 x G dynamic FP8 group quant, and RMSNorm (optionally with residual add) with or without
// that quant fused behind it.  gfx950 only.
//
// Both kernels are HBM-bound streaming passes: every lane owns 16 consecutive elements of one
// group (two 16-byte loads of 16-bit floats in, one 16-byte store of fp8 codes out), so a
// G-element group is held by G/16 neighbouring lanes and its amax is reduced with DPP
// quad/row permutes -- no LDS, no cross-wave traffic in the quant stage.
//
// Reference behaviour replaced: csrc/kernels/quant_kernels.cu:27-167 (group quant kernel) and
// the absent csrc/kernels/rmsnorm_quant_kernels.cu (contract: csrc/include/rmsnorm_quant.h:9-41).
// Arithmetic follows the reference's torch definition aiter/ops/quant.py:64-94, not the
// reference kernel's multiply-by-reciprocal approximation.
#include "fp8bs_launch.h"
#include "fp8bs_math.h"

namespace fp8bs {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// ---------------------------------------------------------------- 16-bit <-> fp32

template <In16 DT>
__device__ __forceinline__ void unpack8(const u32x4& c, float* v)
{
#pragma unroll
    for(int i = 0; i < 4; ++i)
    {
        if constexpr(DT == In16::bf16)
        {
            v[2 * i]     = __uint_as_float(c[i] << 16);
            v[2 * i + 1] = __uint_as_float(c[i] & 0xffff0000u);
        }
        else
        {
            const uint32_t w = c[i]; // copy first: bit_cast straight from a vector element misreads
            f16x2 h      = __builtin_bit_cast(f16x2, w);
            v[2 * i]     = (float)h.x;
            v[2 * i + 1] = (float)h.y;
        }
    }
}

// round to nearest even to the 16-bit type; returns the raw code
template <In16 DT>
__device__ __forceinline__ uint32_t round16(float f)
{
    if constexpr(DT == In16::bf16)
    {
        __bf16 b = (__bf16)f;
        return (uint32_t)__builtin_bit_cast(unsigned short, b);
    }
    else
    {
        _Float16 h = (_Float16)f;
        return (uint32_t)__builtin_bit_cast(unsigned short, h);
    }
}

template <In16 DT>
__device__ __forceinline__ float widen16(uint32_t code)
{
    if constexpr(DT == In16::bf16)
        return __uint_as_float(code << 16);
    else
        return (float)__builtin_bit_cast(_Float16, (unsigned short)code);
}

// two floats rounded to nearest even to the 16-bit type, a in the low half
template <In16 DT>
__device__ __forceinline__ uint32_t round16_pk(float a, float b)
{
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    if constexpr(DT == In16::bf16)
    {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
    }
    else
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, f16x2));
}

// Largest magnitude among 16 packed 16-bit floats, as its 15-bit pattern: for both 16-bit types the
// order of the patterns is the order of the magnitudes, with inf above every finite value and the
// NaNs above inf -- so a group that holds a NaN or an inf shows in its maximum, and nothing has to
// be tested element by element.
__device__ __forceinline__ uint32_t absmax_pk16(const u32x4& lo, const u32x4& hi)
{
    typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
    auto           mx = [](uint32_t a, uint32_t b) {
        return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b)));
    };
    const uint32_t k = 0x7fff7fffu;
    const uint32_t a = mx(mx(mx(lo[0] & k, lo[1] & k), mx(lo[2] & k, lo[3] & k)),
                          mx(mx(hi[0] & k, hi[1] & k), mx(hi[2] & k, hi[3] & k)));
    return max(a & 0xffffu, a >> 16);
}

// ---------------------------------------------------------------- DPP reductions over a group

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
}

constexpr int kDppXor1       = 0xB1;  // quad_perm [1,0,3,2]
constexpr int kDppXor2       = 0x4E;  // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <- lane 7-i inside each 8 lanes
constexpr int kDppRowMirror  = 0x140; // lane i <- lane 15-i inside each 16 lanes

// all-reduce max over LPG (1,2,4,8,16) adjacent lanes; every lane ends with the group's value
template <int LPG>
__device__ __forceinline__ float group_max_f32(float v)
{
    if constexpr(LPG >= 2)
        v = fmaxf(v, __uint_as_float(dpp_u32<kDppXor1>(__float_as_uint(v))));
    if constexpr(LPG >= 4)
        v = fmaxf(v, __uint_as_float(dpp_u32<kDppXor2>(__float_as_uint(v))));
    if constexpr(LPG >= 8)
        v = fmaxf(v, __uint_as_float(dpp_u32<kDppHalfMirror>(__float_as_uint(v))));
    if constexpr(LPG >= 16)
        v = fmaxf(v, __uint_as_float(dpp_u32<kDppRowMirror>(__float_as_uint(v))));
    return v;
}

template <int LPG>
__device__ __forceinline__ uint32_t group_max_u32(uint32_t v)
{
    if constexpr(LPG >= 2)
        v = max(v, dpp_u32<kDppXor1>(v));
    if constexpr(LPG >= 4)
        v = max(v, dpp_u32<kDppXor2>(v));
    if constexpr(LPG >= 8)
        v = max(v, dpp_u32<kDppHalfMirror>(v));
    if constexpr(LPG >= 16)
        v = max(v, dpp_u32<kDppRowMirror>(v));
    return v;
}

// sum of a double over the 64 lanes of a wave, same value in every lane.  DPP permutes inside
// each row of 16 lanes (no LDS traffic, unlike ds_bpermute-based shuffles), then the four row
// sums are read with v_readlane and added in a fixed order.
__device__ __forceinline__ double dpp_add_f64(double v, int which)
{
    uint32_t lo = (uint32_t)__double2loint(v), hi = (uint32_t)__double2hiint(v);
    uint32_t plo, phi;
    switch(which)
    {
    case 0: plo = dpp_u32<kDppXor1>(lo); phi = dpp_u32<kDppXor1>(hi); break;
    case 1: plo = dpp_u32<kDppXor2>(lo); phi = dpp_u32<kDppXor2>(hi); break;
    case 2: plo = dpp_u32<kDppHalfMirror>(lo); phi = dpp_u32<kDppHalfMirror>(hi); break;
    default: plo = dpp_u32<kDppRowMirror>(lo); phi = dpp_u32<kDppRowMirror>(hi); break;
    }
    return v + __hiloint2double((int)phi, (int)plo);
}

__device__ __forceinline__ double wave_sum_f64(double v)
{
    v = dpp_add_f64(v, 0);
    v = dpp_add_f64(v, 1);
    v = dpp_add_f64(v, 2);
    v = dpp_add_f64(v, 3); // every lane now holds the sum of its row of 16
    const uint32_t lo = (uint32_t)__double2loint(v), hi = (uint32_t)__double2hiint(v);
    double         r[4];
#pragma unroll
    for(int k = 0; k < 4; ++k)
        r[k] = __hiloint2double((int)__builtin_amdgcn_readlane(hi, 16 * k),
                                (int)__builtin_amdgcn_readlane(lo, 16 * k));
    return (r[0] + r[1]) + (r[2] + r[3]);
}

// ---------------------------------------------------------------- the quant stage
// v[16]: this lane's 16 consecutive elements of its group (already widened to fp32).
// codes: their 16 e4m3fn codes in memory order.  scale: the group's scale (same in all lanes).

// Rare path: group holds NaN/inf, is all zero, or its amax is so small or large that the
// scale or its reciprocal leaves the normal range.  Everything is done with IEEE divisions and
// the software conversion.  NaN/inf follow what the host division does in the torch reference:
// a NaN element keeps its own sign, other elements of a NaN group get the (positive) NaN of
// the scale; inf/inf is the default NaN, which has the sign bit set on x86.
// Inlined on purpose: an out-of-line call would give the kernel a private (scratch) segment,
// and waves that need scratch are dispatched far more slowly than the HBM stream can be fed.
__device__ __forceinline__ uint32_t absmax_bits16(const float (&v)[16])
{
    uint32_t mm = 0;
#pragma unroll
    for(int i = 0; i < 16; ++i)
        mm = max(mm, __float_as_uint(v[i]) & 0x7fffffffu);
    return mm; // as integers: NaN > inf > every finite magnitude
}

// mm: the group's largest |x| as an integer (absmax_bits16 reduced over the group)
__device__ __forceinline__ void encode16_slow(const float (&v)[16], uint32_t mm, u32x4& codes, float& scale)
{
    float s;
    if(mm > 0x7f800000u)
        s = __uint_as_float(mm | 0x00400000u);
    else
    {
        s = __uint_as_float(mm) / 448.0f;
        if(s == 0.0f)
            s = 1.0f;
    }
    uint32_t out[4] = {0, 0, 0, 0};
#pragma unroll
    for(int i = 0; i < 16; ++i)
    {
        uint32_t xb = __float_as_uint(v[i]);
        uint32_t xa = xb & 0x7fffffffu;
        uint32_t sg = (xb >> 24) & 0x80u;
        uint32_t c;
        if(mm > 0x7f800000u)
            c = (xa > 0x7f800000u) ? (sg | 0x7fu) : 0x7fu;
        else if(mm == 0x7f800000u)
            c = (xa == 0x7f800000u) ? 0xffu : sg;
        else
            c = f32_to_e4m3fn_sw(v[i] / s);
        out[i >> 2] |= c << (8 * (i & 3));
    }
    codes = u32x4{out[0], out[1], out[2], out[3]};
    scale = s;
}

// largest |x| of 16 values as a float; a NaN (which fmaxf would drop) turns it into +inf, which
// sends the group to the slow path
__device__ __forceinline__ float amax16(const float (&v)[16])
{
    float m  = 0.0f;
    bool  un = false;
#pragma unroll
    for(int i = 0; i < 16; i += 2)
    {
        m = fmaxf(fmaxf(m, fabsf(v[i])), fabsf(v[i + 1]));
        un |= __builtin_isunordered(v[i], v[i + 1]);
    }
    return un ? __builtin_inff() : m;
}

// m: the group's amax, for which amax_allows_fast_path holds
__device__ __forceinline__ void encode16_fast(const float (&v)[16], float m, u32x4& codes, float& scale)
{
    const float s = amax_over_448(m); // = m / 448 as IEEE division gives it
    const float r = recip_in_range(s); // the correctly rounded reciprocal: s lies within 2^-89 .. 2^92 here
    uint32_t    out[4];
#pragma unroll
    for(int j = 0; j < 4; ++j)
    {
        int w = 0;
        w = __builtin_amdgcn_cvt_pk_fp8_f32(div_by_scale(v[4 * j], s, r), div_by_scale(v[4 * j + 1], s, r), w,
                                            false);
        w = __builtin_amdgcn_cvt_pk_fp8_f32(div_by_scale(v[4 * j + 2], s, r), div_by_scale(v[4 * j + 3], s, r),
                                            w, true);
        out[j] = (uint32_t)w;
    }
    codes = u32x4{out[0], out[1], out[2], out[3]};
    scale = s;
}

// lo, hi: the 16 values as packed 16-bit floats in memory order; v: the same values widened
template <In16 DT, int LPG>
__device__ __forceinline__ void quant16(const u32x4& lo, const u32x4& hi, const float (&v)[16], u32x4& codes,
                                        float& scale)
{
    const float m = widen16<DT>(group_max_u32<LPG>(absmax_pk16(lo, hi)));
    if(amax_allows_fast_path(__float_as_uint(m))) // false for inf and NaN, too
        encode16_fast(v, m, codes, scale);
    else
        encode16_slow(v, group_max_u32<LPG>(absmax_bits16(v)), codes, scale);
}

// ---------------------------------------------------------------- standalone group quant

struct QuantKernelParams
{
    const u32x4*   x;
    u32x4*         y;
    float*         scale;
    uint32_t       rows;
    uint32_t       groups_per_row;
    const int32_t* num_rows;
    int32_t        num_rows_factor;
    int32_t        transpose_scale;
    uint32_t       scale_row_stride; // 0: scales are contiguous
};

constexpr int kQuantBlock = 256;

template <In16 DT, int GS, int UNITS>
__global__ __launch_bounds__(kQuantBlock) void group_quant_kernel(QuantKernelParams p)
{
    constexpr int LPG = GS / 16;          // lanes per group
    constexpr int GPB = kQuantBlock / LPG; // groups per block per unit

    uint32_t rows = p.rows;
    if(p.num_rows != nullptr)
    {
        int64_t lim = (int64_t)(*p.num_rows) * p.num_rows_factor;
        lim         = lim < 0 ? 0 : lim;
        rows        = lim < (int64_t)rows ? (uint32_t)lim : rows;
    }
    const uint32_t n_groups = rows * p.groups_per_row;
    const uint32_t lig      = threadIdx.x % LPG;
    const uint32_t g0       = blockIdx.x * (GPB * UNITS) + threadIdx.x / LPG;
    __shared__ float block_scales[UNITS * GPB];
    const bool     contiguous_scales = !p.transpose_scale && p.scale_row_stride == 0; // uniform

    u32x4 c[UNITS][2];
#pragma unroll
    for(int u = 0; u < UNITS; ++u)
    {
        const uint32_t g = g0 + u * GPB;
        if(g < n_groups)
        {
            const u32x4* src = p.x + (size_t)g * (GS / 8) + lig * 2;
            c[u][0]          = __builtin_nontemporal_load(src);
            c[u][1]          = __builtin_nontemporal_load(src + 1);
        }
    }
#pragma unroll
    for(int u = 0; u < UNITS; ++u)
    {
        const uint32_t g = g0 + u * GPB;
        if(g < n_groups)
        {
            float v[16];
            unpack8<DT>(c[u][0], v);
            unpack8<DT>(c[u][1], v + 8);
            u32x4 codes;
            float s;
            quant16<DT, LPG>(c[u][0], c[u][1], v, codes, s);
            __builtin_nontemporal_store(codes, p.y + (size_t)g * (GS / 16) + lig);
            if(lig == 0 && contiguous_scales)
                block_scales[u * GPB + threadIdx.x / LPG] = s;
            else if(lig == 0)
            {
                size_t idx = g;
                if(p.transpose_scale)
                {
                    uint32_t row = g / p.groups_per_row;
                    uint32_t col = g - row * p.groups_per_row;
                    idx          = (size_t)col * rows + row;
                }
                else if(p.scale_row_stride)
                {
                    uint32_t row = g / p.groups_per_row;
                    uint32_t col = g - row * p.groups_per_row;
                    idx          = (size_t)row * p.scale_row_stride + col;
                }
                p.scale[idx] = s;
            }
        }
    }
    // Contiguous scales leave as whole lines: the block's GPB scales per unit go through LDS and GPB
    // neighbouring lanes store them (4 bytes each, 128 bytes for 1x128 groups).  Stored by the lanes that
    // computed them, every wave wrote 32 bytes of the line on its own, and those partial writes cost the
    // memory system far more than their bytes (16384 x 7168: 58.8 us; without any scale store 56.85; whole
    // lines 57.97, whole lines stored non-temporally 57.35).
    if(contiguous_scales)
    {
        __syncthreads();
#pragma unroll
        for(int u = 0; u < UNITS; ++u)
        {
            const uint32_t g = blockIdx.x * (GPB * UNITS) + u * GPB + threadIdx.x;
            if(threadIdx.x < GPB && g < n_groups)
                __builtin_nontemporal_store(block_scales[u * GPB + threadIdx.x], p.scale + g);
        }
    }
}

// Transposed scales ([groups per row][rows]) for 1x128 groups.  In the kernel above a wave's eight scales are
// eight 4-byte stores a column apart, and the 32 rows that share a 128-byte line of a scale column are
// quantised by workgroups that run at different times on different XCDs: every line is written in 32 pieces
// (16384 x 7168 in a replayed graph: 67.4 us per launch against 57.4 with row-major scales).  Here a workgroup of
// 512 lanes takes a tile of 32 rows x 4 groups, two rows per lane group (a wave: 2 rows x 1 KiB), parks the 128
// scales in LDS and stores each column's 32 scales as one line: 62.1 us.  Of the 4.7 us that remain, 4 are the
// tiles' strided reads (61.4 us without any scale store; tiles of 32 x 2 groups measure the same).  Same
// arithmetic, same results.
constexpr int kQuantTileRows = 32, kQuantTileCols = 4, kQuantTileUnits = 2;
constexpr int kQuantTileBlock = kQuantTileRows / kQuantTileUnits * kQuantTileCols * 8;
template <In16 DT>
__global__ __launch_bounds__(kQuantTileBlock) void group_quant_tiles_kernel(QuantKernelParams p, uint32_t col_tiles)
{
    constexpr int  LPG  = 8;
    constexpr int  kRowsPerUnit = kQuantTileRows / kQuantTileUnits;
    const uint32_t band = blockIdx.x / col_tiles, ct = blockIdx.x - band * col_tiles;
    const uint32_t pair = threadIdx.x / LPG, lig = threadIdx.x % LPG;
    const uint32_t col  = ct * kQuantTileCols + pair % kQuantTileCols;
    __shared__ float tile_scales[kQuantTileCols][kQuantTileRows];
    u32x4 c[kQuantTileUnits][2];
#pragma unroll
    for(int u = 0; u < kQuantTileUnits; ++u)
    {
        const uint32_t row = band * kQuantTileRows + u * kRowsPerUnit + pair / kQuantTileCols;
        if(row < p.rows && col < p.groups_per_row) // uniform over the 8 lanes of a group
        {
            const u32x4* src = p.x + ((size_t)row * p.groups_per_row + col) * 16 + lig * 2;
            c[u][0]          = __builtin_nontemporal_load(src);
            c[u][1]          = __builtin_nontemporal_load(src + 1);
        }
    }
#pragma unroll
    for(int u = 0; u < kQuantTileUnits; ++u)
    {
        const uint32_t r   = u * kRowsPerUnit + pair / kQuantTileCols;
        const uint32_t row = band * kQuantTileRows + r;
        if(row < p.rows && col < p.groups_per_row)
        {
            float v[16];
            unpack8<DT>(c[u][0], v);
            unpack8<DT>(c[u][1], v + 8);
            u32x4 codes;
            float s;
            quant16<DT, LPG>(c[u][0], c[u][1], v, codes, s);
            __builtin_nontemporal_store(codes, p.y + ((size_t)row * p.groups_per_row + col) * 8 + lig);
            if(lig == 0)
                tile_scales[pair % kQuantTileCols][r] = s;
        }
    }
    __syncthreads();
    if(threadIdx.x < kQuantTileCols * kQuantTileRows)
    {
        const uint32_t cc = threadIdx.x / kQuantTileRows, r = threadIdx.x % kQuantTileRows;
        const uint32_t orow = band * kQuantTileRows + r, ocol = ct * kQuantTileCols + cc;
        if(orow < p.rows && ocol < p.groups_per_row)
            __builtin_nontemporal_store(tile_scales[cc][r], p.scale + (size_t)ocol * p.rows + orow);
    }
}

template <In16 DT, int GS>
static hipError_t launch_group_quant_t(const QuantArgs& a, hipStream_t stream)
{
    constexpr int UNITS = 1;
    constexpr int LPG   = GS / 16;
    constexpr int GPB   = kQuantBlock / LPG * UNITS;
    QuantKernelParams p;
    p.x               = (const u32x4*)a.x;
    p.y               = (u32x4*)a.y;
    p.scale           = a.scale;
    p.rows            = (uint32_t)a.rows;
    p.groups_per_row  = (uint32_t)a.groups_per_row;
    p.num_rows        = a.num_rows;
    p.num_rows_factor = a.num_rows_factor;
    p.transpose_scale = a.transpose_scale ? 1 : 0;
    p.scale_row_stride = (uint32_t)a.scale_row_stride;
    const uint64_t n_groups = (uint64_t)a.rows * (uint64_t)a.groups_per_row;
    if(n_groups == 0)
        return hipSuccess;
    if constexpr(GS == 128)
    {
        // transposed scales of a whole matrix (no row count on the device): by tiles of 32 rows
        const uint64_t col_tiles = ((uint64_t)a.groups_per_row + kQuantTileCols - 1) / kQuantTileCols;
        const uint64_t tiles     = (((uint64_t)a.rows + kQuantTileRows - 1) / kQuantTileRows) * col_tiles;
        if(a.transpose_scale && a.num_rows == nullptr && a.rows >= kQuantTileRows && tiles < (1ull << 31))
        {
            hipLaunchKernelGGL((group_quant_tiles_kernel<DT>), dim3((uint32_t)tiles), dim3(kQuantTileBlock), 0, stream, p,
                               (uint32_t)col_tiles);
            return hipGetLastError();
        }
    }
    const uint32_t grid = (uint32_t)((n_groups + GPB - 1) / GPB);
    hipLaunchKernelGGL((group_quant_kernel<DT, GS, UNITS>), dim3(grid), dim3(kQuantBlock), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_group_quant(const QuantArgs& a, hipStream_t stream)
{
    const bool bf = a.dtype == In16::bf16;
    switch(a.group)
    {
    case 128:
        return bf ? launch_group_quant_t<In16::bf16, 128>(a, stream)
                  : launch_group_quant_t<In16::fp16, 128>(a, stream);
    case 64:
        return bf ? launch_group_quant_t<In16::bf16, 64>(a, stream)
                  : launch_group_quant_t<In16::fp16, 64>(a, stream);
    case 32:
        return bf ? launch_group_quant_t<In16::bf16, 32>(a, stream)
                  : launch_group_quant_t<In16::fp16, 32>(a, stream);
    default: return hipErrorInvalidValue;
    }
}

// ---------------------------------------------------------------- weight-side 128x128 block quant
// One workgroup per 128x128 block of a [N, K] weight matrix: one scale per block, codes by the
// same exact division as the activation quant.  Rows past N count as zeros (they do not move the
// amax), as in the torch formulation that zero-pads ragged blocks
// (op_tests/multigpu_tests/test_dispatch_combine.py:180-204 applies pertoken_quant,
// aiter/ops/quant.py:64-94, to [n_blocks, 128*128] views).  An offline step: built for
// exactness, not tuned.

struct WeightQuantKernelParams
{
    const uint16_t* w;
    uint8_t*        q;
    float*          scale;
    int32_t         N, K;
    int64_t         ldw, ldq; // row strides in elements
};

template <class T, class Op>
__device__ __forceinline__ T block256_reduce(T v, T* lds, Op op)
{
#pragma unroll
    for(int off = 32; off >= 1; off >>= 1)
        v = op(v, __shfl_xor(v, off, 64));
    const int wave = threadIdx.x >> 6;
    __syncthreads(); // lds may still be read from a previous reduction
    if((threadIdx.x & 63) == 0)
        lds[wave] = v;
    __syncthreads();
    return op(op(lds[0], lds[1]), op(lds[2], lds[3]));
}

template <In16 DT>
__global__ __launch_bounds__(256) void weight_block_quant_kernel(WeightQuantKernelParams p)
{
    __shared__ float    red_f[4];
    __shared__ uint32_t red_u[4];
    const int t = threadIdx.x;
    const int r = t >> 1, half = t & 1;      // block row, 64-element half of its 128 columns
    const int n = blockIdx.y * 128 + r;
    const int k0 = blockIdx.x * 128 + half * 64;
    const bool live = n < p.N;

    float v[4][16];
#pragma unroll
    for(int u = 0; u < 4; ++u)
#pragma unroll
        for(int i = 0; i < 16; ++i)
            v[u][i] = 0.0f;
    if(live)
    {
        const u32x4* src = (const u32x4*)(p.w + (size_t)n * p.ldw + k0);
#pragma unroll
        for(int u = 0; u < 4; ++u)
        {
            unpack8<DT>(src[2 * u], v[u]);
            unpack8<DT>(src[2 * u + 1], v[u] + 8);
        }
    }
    float m = 0.0f;
#pragma unroll
    for(int u = 0; u < 4; ++u)
        m = fmaxf(m, amax16(v[u])); // +inf when the unit holds a NaN
    m = block256_reduce(m, red_f, [](float a, float b) { return fmaxf(a, b); });

    u32x4 codes[4];
    float s = 1.0f;
    if(amax_allows_fast_path(__float_as_uint(m)))
    {
#pragma unroll
        for(int u = 0; u < 4; ++u)
            encode16_fast(v[u], m, codes[u], s);
    }
    else
    {
        uint32_t mm = 0;
#pragma unroll
        for(int u = 0; u < 4; ++u)
            mm = max(mm, absmax_bits16(v[u]));
        mm = block256_reduce(mm, red_u, [](uint32_t a, uint32_t b) { return max(a, b); });
#pragma unroll
        for(int u = 0; u < 4; ++u)
            encode16_slow(v[u], mm, codes[u], s);
    }
    if(live)
    {
        u32x4* dst = (u32x4*)(p.q + (size_t)n * p.ldq + k0);
#pragma unroll
        for(int u = 0; u < 4; ++u)
            dst[u] = codes[u];
    }
    if(t == 0)
        p.scale[(size_t)blockIdx.y * gridDim.x + blockIdx.x] = s;
}

hipError_t launch_weight_block_quant(const WeightQuantArgs& a, hipStream_t stream)
{
    if(a.N == 0 || a.K == 0)
        return hipSuccess;
    WeightQuantKernelParams p;
    p.w     = (const uint16_t*)a.w;
    p.q     = a.q;
    p.scale = a.scale;
    p.N     = (int32_t)a.N;
    p.K     = (int32_t)a.K;
    p.ldw   = a.ldw;
    p.ldq   = a.ldq;
    const dim3 grid((unsigned)(a.K / 128), (unsigned)((a.N + 127) / 128));
    if(a.dtype == In16::bf16)
        hipLaunchKernelGGL(weight_block_quant_kernel<In16::bf16>, grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(weight_block_quant_kernel<In16::fp16>, grid, dim3(256), 0, stream, p);
    return hipGetLastError();
}

// ---------------------------------------------------------------- RMSNorm (+add) (+quant)
// One block per row, one or two 16-element units per lane (hidden <= 8192).
// The sum of squares is accumulated in fp64 (each 16-bit float square is exact there), so the
// mean is the correctly rounded one regardless of reduction order up to ~2^-45 relative.

struct NormKernelParams
{
    const uint16_t* x;
    const uint16_t* res_in;
    uint16_t*       res_out;
    const uint16_t* weight;
    uint16_t*       out16;
    uint8_t*        out8;
    float*          scale;
    uint32_t        rows;
    int32_t         hidden;
    int64_t         x_stride, res_in_stride, res_out_stride, out_stride;
    float           eps;
    int32_t         transpose_scale;
    int32_t         gemma_norm;
    double          inv_hidden; // RN(1 / hidden), for div_by_count
};

template <In16 DT, bool ADD, int GS /* 0 = no quant */, int U /* 16-element units per lane */>
__global__ __launch_bounds__(512) void rmsnorm_kernel(NormKernelParams p)
{
    const uint32_t row = blockIdx.x;
    const int      t   = threadIdx.x;
    // unit j of this lane covers elements [e0[j], e0[j] + 16); consecutive lanes hold
    // consecutive units, so loads coalesce and the lanes of one quant group stay adjacent
    int  e0[U];
    bool act0[U], act1[U];
#pragma unroll
    for(int j = 0; j < U; ++j)
    {
        e0[j]   = (t + j * (int)blockDim.x) * 16;
        act0[j] = e0[j] < p.hidden;     // first 8 elements present
        act1[j] = e0[j] + 8 < p.hidden; // second 8 elements present
    }

    // every request of the lane (row, residual, weight) is issued before anything is consumed;
    // the weight would otherwise pay its latency a second time behind the reduction
    u32x4 xraw[U][2], rraw[U][2], wraw[U][2];
#pragma unroll
    for(int j = 0; j < U; ++j)
    {
        const u32x4 z = {0, 0, 0, 0};
        xraw[j][0] = xraw[j][1] = rraw[j][0] = rraw[j][1] = wraw[j][0] = wraw[j][1] = z;
        if(act0[j])
        {
            const u32x4* src = (const u32x4*)(p.x + (size_t)row * p.x_stride + e0[j]);
            xraw[j][0]       = src[0];
            if(act1[j])
                xraw[j][1] = src[1];
            if constexpr(ADD)
            {
                const u32x4* rs =
                    (const u32x4*)(p.res_in + (size_t)row * p.res_in_stride + e0[j]);
                rraw[j][0] = rs[0];
                if(act1[j])
                    rraw[j][1] = rs[1];
            }
            const u32x4* wsrc = (const u32x4*)(p.weight + e0[j]);
            wraw[j][0]        = wsrc[0];
            if(act1[j])
                wraw[j][1] = wsrc[1];
        }
    }

    float  v[U][16];
    double ss = 0.0, ss2 = 0.0; // two chains: an fp64 FMA does not wait for the one before it
#pragma unroll
    for(int j = 0; j < U; ++j)
    {
        unpack8<DT>(xraw[j][0], v[j]);
        unpack8<DT>(xraw[j][1], v[j] + 8);
        if constexpr(ADD)
        {
            float r[16];
            unpack8<DT>(rraw[j][0], r);
            unpack8<DT>(rraw[j][1], r + 8);
            u32x4 h[2];
#pragma unroll
            for(int i = 0; i < 8; ++i)
                h[i >> 2][i & 3] = round16_pk<DT>(v[j][2 * i] + r[2 * i], v[j][2 * i + 1] + r[2 * i + 1]);
            unpack8<DT>(h[0], v[j]);
            unpack8<DT>(h[1], v[j] + 8);
            // stored with the row's other outputs, behind the reduction: a block then reads, computes and
            // writes in turn (stored here, between the reads, the 16384-row case runs 6 % slower)
            rraw[j][0] = h[0];
            rraw[j][1] = h[1];
        }
#pragma unroll
        for(int i = 0; i < 16; i += 2)
        {
            ss  = __builtin_fma((double)v[j][i], (double)v[j][i], ss);
            ss2 = __builtin_fma((double)v[j][i + 1], (double)v[j][i + 1], ss2);
        }
    }
    ss += ss2;
    ss = wave_sum_f64(ss);

    // eight slots whatever the block size: the waves that do not exist contribute zeros, so the
    // read-back is four wide LDS loads and a fixed tree of seven additions
    __shared__ __attribute__((aligned(16))) double part[8];
    const int wave = t >> 6, n_waves = blockDim.x >> 6;
    if((t & 63) == 0)
        part[wave] = ss;
    if(t >= n_waves && t < 8)
        part[t] = 0.0;
    __syncthreads();
    double pr[8];
#pragma unroll
    for(int w = 0; w < 8; ++w)
        pr[w] = part[w];
    const double tot = ((pr[0] + pr[1]) + (pr[2] + pr[3])) + ((pr[4] + pr[5]) + (pr[6] + pr[7]));

    // every wave of the block repeats this: the quotient and the reciprocal take the short forms that
    // give the IEEE results (tot / hidden as correctly rounded; 1 / root inside recip_in_range's range)
    const float    mean = (float)div_by_count(tot, (double)p.hidden, p.inv_hidden);
    const float    root = sqrtf(mean + p.eps); // correctly rounded
    const uint32_t rb   = __float_as_uint(root);
    const float    rstd = rb >= kRecipMinBits && rb <= kRecipMaxBits ? recip_in_range(root) : 1.0f / root;

#pragma unroll
    for(int j = 0; j < U; ++j)
    {
        if(!act0[j])
            continue;
        float w[16];
        unpack8<DT>(wraw[j][0], w);
        unpack8<DT>(wraw[j][1], w + 8);
        if(p.gemma_norm) // uniform branch: the common case pays nothing for it
        {
#pragma unroll
            for(int i = 0; i < 16; ++i)
                w[i] = 1.0f + w[i];
        }
        if constexpr(ADD)
        {
            u32x4* ro = (u32x4*)(p.res_out + (size_t)row * p.res_out_stride + e0[j]);
            ro[0]     = rraw[j][0];
            if(act1[j])
                ro[1] = rraw[j][1];
        }
        u32x4 h[2];
#pragma unroll
        for(int i = 0; i < 8; ++i)
            h[i >> 2][i & 3] = round16_pk<DT>((v[j][2 * i] * rstd) * w[2 * i], (v[j][2 * i + 1] * rstd) * w[2 * i + 1]);
        if constexpr(GS == 0)
        {
            u32x4* o = (u32x4*)(p.out16 + (size_t)row * p.out_stride + e0[j]);
            o[0]     = h[0];
            if(act1[j])
                o[1] = h[1];
        }
        else
        {
            constexpr int LPG = GS / 16;
            u32x4         codes;
            float         s;
            unpack8<DT>(h[0], v[j]);
            unpack8<DT>(h[1], v[j] + 8);
            quant16<DT, LPG>(h[0], h[1], v[j], codes, s);
            // the codes are not read again by this kernel: past the caches (plain stores: 12.3 us against 11.0 at
            // 2048 x 7168); rows, residuals and the 16-bit outputs go with the default policy, which measured
            // faster for them
            __builtin_nontemporal_store(codes, (u32x4*)(p.out8 + (size_t)row * p.out_stride + e0[j]));
            const int unit = e0[j] >> 4;
            if(unit % LPG == 0)
            {
                const uint32_t gpr = (uint32_t)p.hidden / GS;
                const uint32_t col = (uint32_t)unit / LPG;
                size_t         idx =
                    p.transpose_scale ? (size_t)col * p.rows + row : (size_t)row * gpr + col;
                p.scale[idx] = s;
            }
        }
    }
}

// Rows of more than 2048 elements give each lane two units: the whole problem then fits the
// chip in one round of blocks at the usual row counts, instead of two dependent rounds.
template <In16 DT, bool ADD, int GS>
static hipError_t launch_rmsnorm_t(const NormKernelParams& p, hipStream_t stream)
{
    const int units = (p.hidden + 15) / 16;
    if(units > 128)
    {
        const int threads = ((units + 1) / 2 + 63) / 64 * 64;
        hipLaunchKernelGGL((rmsnorm_kernel<DT, ADD, GS, 2>), dim3(p.rows), dim3(threads), 0,
                           stream, p);
    }
    else
    {
        const int threads = (units + 63) / 64 * 64;
        hipLaunchKernelGGL((rmsnorm_kernel<DT, ADD, GS, 1>), dim3(p.rows), dim3(threads), 0,
                           stream, p);
    }
    return hipGetLastError();
}

template <In16 DT, bool ADD>
static hipError_t launch_rmsnorm_g(const NormKernelParams& p, int group, hipStream_t stream)
{
    switch(group)
    {
    case 0: return launch_rmsnorm_t<DT, ADD, 0>(p, stream);
    case 32: return launch_rmsnorm_t<DT, ADD, 32>(p, stream);
    case 64: return launch_rmsnorm_t<DT, ADD, 64>(p, stream);
    case 128: return launch_rmsnorm_t<DT, ADD, 128>(p, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_rmsnorm(const NormArgs& a, hipStream_t stream)
{
    if(a.rows == 0)
        return hipSuccess;
    NormKernelParams p;
    p.x               = (const uint16_t*)a.x;
    p.res_in          = (const uint16_t*)a.residual_in;
    p.res_out         = (uint16_t*)a.residual_out;
    p.weight          = (const uint16_t*)a.weight;
    p.out16           = (uint16_t*)a.out16;
    p.out8            = a.out8;
    p.scale           = a.scale;
    p.rows            = (uint32_t)a.rows;
    p.hidden          = a.hidden;
    p.x_stride        = a.x_stride;
    p.res_in_stride   = a.res_in_stride;
    p.res_out_stride  = a.res_out_stride;
    p.out_stride      = a.out_stride;
    p.eps             = a.eps;
    p.transpose_scale = a.transpose_scale ? 1 : 0;
    p.gemma_norm      = a.gemma_norm ? 1 : 0;
    p.inv_hidden      = 1.0 / (double)a.hidden;
    const int  group  = a.out8 ? a.group : 0;
    const bool add    = a.residual_in != nullptr;
    if(a.dtype == In16::bf16)
        return add ? launch_rmsnorm_g<In16::bf16, true>(p, group, stream)
                   : launch_rmsnorm_g<In16::bf16, false>(p, group, stream);
    return add ? launch_rmsnorm_g<In16::fp16, true>(p, group, stream)
               : launch_rmsnorm_g<In16::fp16, false>(p, group, stream);
}

} // namespace fp8bs
