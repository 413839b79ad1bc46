// Measurement aids of bench.py (`--workload stream`, `--workload ceiling`): kernels that carry one
// ingredient of a product kernel with everything else taken out, so that what the chip gives that
// ingredient can be put beside the product kernel's own figure.  Built into libbench_probes.so, which
// only bench.py loads; nothing here is part of the product library or its C ABI.
//
//   probe_stream   the 1 x 128 quant kernel's memory skeleton (same grid, same 32 bytes read and 16
//                  bytes written per lane, same non-temporal accesses) without its arithmetic
//   probe_mfma     the prefill GEMM's arithmetic (v_mfma_f32_16x16x128_f8f6f4 on fp8 codes, four
//                  v_fmac_f32 per MFMA that fold the product into fp32 accumulators with a scale, in
//                  the product kernel's issue order) on operands that stay in registers: no LDS, no
//                  global memory inside the loop, no barriers; also with the 32 x 32 x 64 shape of
//                  the matrix instruction
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int      i32x8 __attribute__((ext_vector_type(8)));
typedef float    f32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int kQuantBlock = 256;

template <int MODE>
__global__ __launch_bounds__(kQuantBlock) void stream_probe_kernel(const u32x4* __restrict__ x, u32x4* __restrict__ y,
                                                                   uint32_t n_units)
{
    const uint32_t i = blockIdx.x * kQuantBlock + threadIdx.x;
    if(i >= n_units)
        return;
    u32x4 o = u32x4{i, i, i, i};
    if constexpr(MODE != 1)
    {
        const u32x4 a = __builtin_nontemporal_load(x + 2 * (size_t)i);
        const u32x4 b = __builtin_nontemporal_load(x + 2 * (size_t)i + 1);
        o             = a ^ b;
    }
    if constexpr(MODE == 0)
    {
        if((o[0] ^ o[1] ^ o[2] ^ o[3]) == 0x9e3779b9u && (o[0] + o[1]) == 0x7f4a7c15u) // practically never: keeps the loads alive
            y[0] = o;
    }
    else
        __builtin_nontemporal_store(o, y + i);
}

// One wave = the product kernel's wave: 8 weight fragments x 4 activation fragments = 32 MFMA
// tiles per pass over the loop body ("K block"), 128 fp32 accumulators per lane.  FMAS = 4 folds
// every product into its accumulators two MFMA slots after the MFMA that made it, as the product
// kernel does; FMAS = 0 leaves the matrix instructions alone.
template <int FMAS, int THREADS>
__global__ __launch_bounds__(THREADS) void mfma_ceiling_kernel(const i32x8* __restrict__ wcodes,
                                                               const i32x8* __restrict__ xcodes,
                                                               const float* __restrict__ scales,
                                                               float* __restrict__ sink, int iters)
{
    extern __shared__ uint8_t holds_the_compute_unit[]; // sized by the launcher so that one workgroup fills a compute unit
    const int t = threadIdx.x;
    i32x8     aw[8], bx[4];
    float     sc[4];
#pragma unroll
    for(int i = 0; i < 8; ++i)
        aw[i] = wcodes[i * THREADS + t];
#pragma unroll
    for(int j = 0; j < 4; ++j)
    {
        bx[j] = xcodes[j * THREADS + t];
        sc[j] = scales[j * THREADS + t];
    }
    float acc[8][4][4];
#pragma unroll
    for(int i = 0; i < 8; ++i)
#pragma unroll
        for(int j = 0; j < 4; ++j)
#pragma unroll
            for(int r = 0; r < 4; ++r)
                acc[i][j][r] = 0.f;
    f32x4 P[4];
#pragma unroll
    for(int q = 0; q < 4; ++q)
        P[q] = f32x4{0.f, 0.f, 0.f, 0.f};
    // operands settled in their registers before the first matrix instruction reads them
#pragma unroll
    for(int i = 0; i < 8; ++i)
        asm volatile("" : "+v"(aw[i]));
#pragma unroll
    for(int j = 0; j < 4; ++j)
        asm volatile("" : "+v"(bx[j]), "+v"(sc[j]));
#pragma unroll
    for(int q = 0; q < 4; ++q)
        asm volatile("" : "+v"(P[q]));
    asm volatile("s_nop 7" ::: "memory");

#define PROBE_MFMA(Pq, A, B) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0" : "=&v"(Pq) : "v"(A), "v"(B))
#define PROBE_FMA4(ACC, Pq, S)                                                         \
    do                                                                                 \
    {                                                                                  \
        asm volatile("v_fmac_f32 %0, %1, %2" : "+v"((ACC)[0]) : "v"((Pq)[0]), "v"(S)); \
        asm volatile("v_fmac_f32 %0, %1, %2" : "+v"((ACC)[1]) : "v"((Pq)[1]), "v"(S)); \
        asm volatile("v_fmac_f32 %0, %1, %2" : "+v"((ACC)[2]) : "v"((Pq)[2]), "v"(S)); \
        asm volatile("v_fmac_f32 %0, %1, %2" : "+v"((ACC)[3]) : "v"((Pq)[3]), "v"(S)); \
    } while(0)
    for(int it = 0; it < iters; ++it)
    {
#pragma unroll
        for(int q = 0; q < 32; ++q)
        {
            PROBE_MFMA(P[q & 3], aw[q >> 2], bx[q & 3]);
            if constexpr(FMAS == 4)
            {
                // the product issued two slots ago is written back by now (the matrix pipe takes the
                // instructions in order, 32 clocks each): no wait states
                const int tq = (q + 30) & 31;
                PROBE_FMA4(acc[tq >> 2][tq & 3], P[tq & 3], sc[tq & 3]);
            }
        }
    }
#undef PROBE_MFMA
#undef PROBE_FMA4
    asm volatile("s_nop 15\n s_nop 15\n s_nop 15" ::: "memory");
    float s = P[0][0] + P[1][1] + P[2][2] + P[3][3];
#pragma unroll
    for(int i = 0; i < 8; ++i)
#pragma unroll
        for(int j = 0; j < 4; ++j)
#pragma unroll
            for(int r = 0; r < 4; ++r)
                s += acc[i][j][r];
    sink[(size_t)blockIdx.x * THREADS + t] = s;
}


// The same arithmetic with v_mfma_f32_32x32x64_f8f6f4: a wave's 128 x 64 block is 4 x 2 tiles of
// 32 x 32, each the sum of two chained matrix instructions per K block (64 of the 128 K values each),
// folded into 16 accumulators per lane by 16 FMAs.  Same flops, same FMAs per flop, half as many
// matrix instructions, twice as long each.  Tiles go in pairs (first halves of both, then second
// halves), so a chained instruction never follows the one it depends on; a tile's FMAs trail its
// second half by two slots.
typedef float f32x16 __attribute__((ext_vector_type(16)));
template <int FMAS, int THREADS>
__global__ __launch_bounds__(THREADS) void mfma32_ceiling_kernel(const i32x8* __restrict__ wcodes,
                                                                 const i32x8* __restrict__ xcodes,
                                                                 const float* __restrict__ scales,
                                                                 float* __restrict__ sink, int iters)
{
    extern __shared__ uint8_t holds_the_compute_unit[];
    const int t = threadIdx.x;
    i32x8     aw[3], bx[2];
    float     sc[2];
#pragma unroll
    for(int i = 0; i < 3; ++i)
        aw[i] = wcodes[i * THREADS + t];
#pragma unroll
    for(int j = 0; j < 2; ++j)
    {
        bx[j] = xcodes[j * THREADS + t];
        sc[j] = scales[j * THREADS + t];
    }
    f32x16 acc[8], P[4];
#pragma unroll
    for(int i = 0; i < 8; ++i)
#pragma unroll
        for(int r = 0; r < 16; ++r)
            acc[i][r] = 0.f;
#pragma unroll
    for(int q = 0; q < 4; ++q)
#pragma unroll
        for(int r = 0; r < 16; ++r)
            P[q][r] = 0.f;
#pragma unroll
    for(int i = 0; i < 3; ++i)
        asm volatile("" : "+v"(aw[i]));
#pragma unroll
    for(int j = 0; j < 2; ++j)
        asm volatile("" : "+v"(bx[j]), "+v"(sc[j]));
#pragma unroll
    for(int q = 0; q < 4; ++q)
        asm volatile("" : "+v"(P[q]));
    asm volatile("s_nop 7" ::: "memory");

    for(int it = 0; it < iters; ++it)
    {
#pragma unroll
        for(int s = 0; s < 16; ++s)
        {
            const int pair = s >> 2, tile = 2 * pair + (s & 1); // tile = (n tile i = tile >> 1, m tile j = tile & 1)
            if((s & 2) == 0) // first half of the K block
                asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, 0" : "=&v"(P[tile & 3]) : "v"(aw[(tile >> 1) % 3]), "v"(bx[tile & 1]));
            else             // second half, onto the first (other fragments: the codes differ as in a real K block)
                asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0" : "+v"(P[tile & 3]) : "v"(aw[((tile >> 1) + 1) % 3]), "v"(bx[(tile & 1) ^ 1]));
            if constexpr(FMAS == 4)
            {
                // the tile whose second half was issued two slots ago: tile - 2 (the previous pair) for
                // the slots of first halves
                if((s & 2) == 0)
                {
                    const int done = (tile + 6) & 7;
#pragma unroll
                    for(int r = 0; r < 16; ++r)
                        asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(acc[done][r]) : "v"(P[done & 3][r]), "v"(sc[done & 1]));
                }
            }
        }
    }
    asm volatile("s_nop 15\n s_nop 15\n s_nop 15\n s_nop 15\n s_nop 15" ::: "memory");
    float sum = P[0][0] + P[1][1] + P[2][2] + P[3][3];
#pragma unroll
    for(int i = 0; i < 8; ++i)
#pragma unroll
        for(int r = 0; r < 16; ++r)
            sum += acc[i][r];
    sink[(size_t)blockIdx.x * THREADS + t] = sum;
}

template <int FMAS, int THREADS, bool WIDE>
hipError_t launch_mfma(const void* wcodes, const void* xcodes, const float* scales, float* sink, int iters,
                       int workgroups, hipStream_t stream)
{
    auto kernel = WIDE ? mfma32_ceiling_kernel<FMAS, THREADS> : mfma_ceiling_kernel<FMAS, THREADS>;
    // 96 KiB of the 160 KiB of LDS: a second workgroup does not fit beside this one
    constexpr int kLds = 96 * 1024;
    hipError_t    e    = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if(e != hipSuccess)
        return e;
    hipLaunchKernelGGL(kernel, dim3(workgroups), dim3(THREADS), kLds, stream, (const i32x8*)wcodes,
                       (const i32x8*)xcodes, scales, sink, iters);
    return hipGetLastError();
}

} // namespace

extern "C" {

// mode 2: dst[i] <- f(src[2i], src[2i+1]) in 16-byte units; mode 0: src is read and nothing written;
// mode 1: dst is written and nothing read.  src spans 32 n_units bytes, dst 16 n_units, both 16-byte
// aligned device memory.  Returns a hipError_t (0 = success).
int probe_stream(int mode, const void* src, void* dst, uint64_t n_units, void* stream)
{
    if(n_units == 0 || n_units >= (1ull << 32))
        return (int)hipErrorInvalidValue;
    const dim3  grid((unsigned)((n_units + kQuantBlock - 1) / kQuantBlock)), block(kQuantBlock);
    hipStream_t s = (hipStream_t)stream;
    switch(mode)
    {
    case 0: hipLaunchKernelGGL(stream_probe_kernel<0>, grid, block, 0, s, (const u32x4*)src, (u32x4*)dst, (uint32_t)n_units); break;
    case 1: hipLaunchKernelGGL(stream_probe_kernel<1>, grid, block, 0, s, (const u32x4*)src, (u32x4*)dst, (uint32_t)n_units); break;
    case 2: hipLaunchKernelGGL(stream_probe_kernel<2>, grid, block, 0, s, (const u32x4*)src, (u32x4*)dst, (uint32_t)n_units); break;
    default: return (int)hipErrorInvalidValue;
    }
    return (int)hipGetLastError();
}

// `workgroups` workgroups of `threads` (256 or 512) lanes, one per compute unit, each wave running
// `iters` passes of 32 matrix instructions (+ 128 FMAs with fmas = 4, none with fmas = 0); with
// wide != 0, 16 instructions of the 32 x 32 x 64 shape per pass instead (512 lanes only).
//   wcodes  8 * threads fragments of 32 bytes (fp8 codes), xcodes 4 * threads fragments,
//   scales  4 * threads floats, sink workgroups * threads floats (written once at the end).
// Flops per launch: workgroups * threads / 64 * iters * 32 * 65536.  Returns a hipError_t.
int probe_mfma(int fmas, int threads, int wide, const void* wcodes, const void* xcodes, const float* scales, float* sink,
               int iters, int workgroups, void* stream)
{
    hipStream_t s = (hipStream_t)stream;
    if(iters < 1 || workgroups < 1)
        return (int)hipErrorInvalidValue;
    if(wide && fmas == 4 && threads == 512)
        return (int)launch_mfma<4, 512, true>(wcodes, xcodes, scales, sink, iters, workgroups, s);
    if(wide && fmas == 0 && threads == 512)
        return (int)launch_mfma<0, 512, true>(wcodes, xcodes, scales, sink, iters, workgroups, s);
    if(wide)
        return (int)hipErrorInvalidValue;
    if(fmas == 4 && threads == 512)
        return (int)launch_mfma<4, 512, false>(wcodes, xcodes, scales, sink, iters, workgroups, s);
    if(fmas == 0 && threads == 512)
        return (int)launch_mfma<0, 512, false>(wcodes, xcodes, scales, sink, iters, workgroups, s);
    if(fmas == 4 && threads == 256)
        return (int)launch_mfma<4, 256, false>(wcodes, xcodes, scales, sink, iters, workgroups, s);
    if(fmas == 0 && threads == 256)
        return (int)launch_mfma<0, 256, false>(wcodes, xcodes, scales, sink, iters, workgroups, s);
    return (int)hipErrorInvalidValue;
}

} // extern "C"
