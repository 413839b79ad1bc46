// Decode-shape block-scale FP8 GEMM (M <= 64): weight streaming, HBM-bound.
//
// The weight matrix is read exactly once, straight from global memory into registers in the
// MFMA "A" operand layout (lane = weight row l%16, 32 bytes of one 128-wide K block), with every
// load of a wave's share issued before anything is consumed, so a wave keeps up to 32 KiB in
// flight and the whole matrix is requested from HBM at once.  The (small) activation matrix and
// its scales are staged once per workgroup in LDS and shared by its 4 waves.
//
// Work split: a workgroup owns 64 weight rows (16 per wave) and one K chunk.  When N alone gives
// too few workgroups to keep the memory system busy, K is split across workgroups as well; the
// fp32 partial tiles go to a workspace and the last workgroup to finish a row block (an atomic
// ticket) adds them in a fixed order, so results do not depend on arrival order.
#include "gemm_common.h"

namespace fp8bs {

namespace {

constexpr int kRowsPerWave = 16, kWaves = 4, kRowsPerBlock = kRowsPerWave * kWaves;
constexpr int kThreads   = 64 * kWaves;
constexpr int kMaxChunkKb = 16; // K blocks per chunk: 16 x 2 loads x 16 B = 512 B in flight per lane

struct DecodeParams
{
    GemmKernelParams g;
    int32_t  m_tiles;      // ceil(M / 16), 1..4
    int32_t  chunk_kb;     // K blocks per workgroup chunk
    int32_t  chunk_kb_pad; // chunk_kb rounded up to a multiple of 8 (LDS row pitch)
    int32_t  splits;       // number of K chunks
    float*   partial;      // [splits][n_blocks * 64][m_tiles * 16] fp32 when splits > 1
    uint32_t* tickets;     // [n_blocks] zero between launches
};

__device__ __forceinline__ uint32_t x_lds_off(uint32_t row, uint32_t kb, uint32_t chunk, uint32_t row_bytes)
{
    return row * row_bytes + kb * 128u + ((chunk ^ (row & 7u)) << 4);
}

template <In16 DT, int MT, int KBMAX>
__global__ __launch_bounds__(kThreads) void gemm_decode_kernel(DecodeParams p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const GemmKernelParams& g = p.g;

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int l16 = lane & 15, kg = lane >> 4;
    const int nblk  = blockIdx.x;            // 64-row block of the weight
    const int split = blockIdx.y;
    const int kb0   = split * p.chunk_kb;
    const int nkb   = min(p.chunk_kb, g.kblocks - kb0);
    const int n_row = nblk * kRowsPerBlock + wave * kRowsPerWave + l16;
    const int n_ld  = n_row < g.N ? n_row : g.N - 1; // ragged N: load a valid row, never store it

    // ---- 1. activations for this K chunk -> LDS with LDS-direct loads (no registers, all in
    // flight at once).  One instruction moves one activation row x 8 K blocks (1 KiB): lane p
    // fills LDS chunk p of that KiB = K block p/8, stored chunk p%8, which must hold the row's
    // logical chunk (p%8) ^ (row&7).  Rows and K blocks past the end are clamped (re-fetched,
    // never used).  Issued before the weight loads so that they are the oldest in the queue.
    const uint32_t x_row_bytes = (uint32_t)p.chunk_kb_pad * 128u;
    uint8_t*       sX          = smem;
    float*         sS          = (float*)(smem + (size_t)MT * 16 * x_row_bytes);
    {
        typedef uint8_t __attribute__((address_space(3)))* lds_byte_ptr;
        const uint32_t lds0   = (uint32_t)(uintptr_t)(lds_byte_ptr)smem;
        const int      groups = p.chunk_kb_pad >> 3;          // 8-K-block groups per row
        const int      units  = MT * 16 * groups;             // 1 KiB units in the chunk
        for(int u = wave; u < units; u += kWaves)
        {
            const int row = u / groups, grp = u - row * groups;
            const int m   = row < g.M ? row : g.M - 1;
            int       kb  = grp * 8 + (lane >> 3);
            kb            = kb < nkb ? kb : nkb - 1;
            const uint32_t c    = (uint32_t)(lane & 7) ^ (uint32_t)(row & 7);
            const uint32_t voff = (uint32_t)m * (uint32_t)g.lda + (uint32_t)(kb0 + kb) * 128u + c * 16u;
            const uint32_t dst  = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)row * x_row_bytes + (uint32_t)grp * 1024u);
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                         :
                         : "s"(dst), "v"(voff), "s"(g.xq)
                         : "memory");
        }
    }
    // x_scale of the chunk: at most 4 values per thread, all requested before any is used
    float sval[4];
    {
        const int total = MT * 16 * nkb;
#pragma unroll
        for(int i = 0; i < 4; ++i)
        {
            const int q   = t + i * kThreads;
            const int qq  = q < total ? q : total - 1;
            const int row = qq / nkb, k = qq - row * nkb;
            const int m   = row < g.M ? row : g.M - 1;
            sval[i]       = g.xs[(size_t)m * g.kblocks + kb0 + k];
        }
    }

    // w_scale of this wave's rows: one 128-row block (16 | 128, so a wave never straddles two).
    // The block index is wave-uniform; saying so turns these into scalar loads that are all
    // issued here instead of one dependent vector load per K block inside the multiply loop.
    const int nb = __builtin_amdgcn_readfirstlane(
        min((nblk * kRowsPerBlock + wave * kRowsPerWave) >> 7, (g.N + 127) / 128 - 1));
    const float* ws_row = g.ws + (size_t)nb * g.kblocks + kb0;
    float        wsv[KBMAX];
#pragma unroll
    for(int k = 0; k < KBMAX; ++k)
        wsv[k] = ws_row[k < nkb ? k : nkb - 1];

    // ---- 2. every weight load of this wave, up front and unconditional: the kernel is
    // instantiated for chunk capacities of 4, 8, 12 and 16 K blocks, and the (at most 3) slots
    // past the end of a shorter chunk re-read its last K block (a cache hit, never used).
    // Straight-line loads let the compiler count them, so each K block below waits only for its
    // own two loads and the multiply overlaps the arrival of the rest.
    u32x4 wlo[KBMAX], whi[KBMAX];
    {
        const uint8_t* wp = g.wq + (size_t)n_ld * g.ldb + (size_t)kb0 * 128 + kg * 32;
#pragma unroll
        for(int k = 0; k < KBMAX; ++k)
        {
            const int kk = k < nkb ? k : nkb - 1;
            wlo[k]       = __builtin_nontemporal_load((const u32x4*)(wp + kk * 128));
            whi[k]       = __builtin_nontemporal_load((const u32x4*)(wp + kk * 128 + 16));
        }
    }
    {
        // Using the scale values makes the compiler wait for their loads; loads return in
        // order, so the older LDS-direct loads of this wave have landed by then as well.
        const int total = MT * 16 * nkb;
#pragma unroll
        for(int i = 0; i < 4; ++i)
        {
            const int q = t + i * kThreads;
            if(q < total)
            {
                const int row = q / nkb, k = q - row * nkb;
                sS[row * p.chunk_kb + k] = sval[i];
            }
        }
    }
    __syncthreads();

    // ---- 3. multiply: one MFMA per (K block, m tile), scaled into fp32 accumulators
    f32x4 acc[MT];
#pragma unroll
    for(int j = 0; j < MT; ++j)
        acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
    for(int k = 0; k < KBMAX; ++k)
    {
        if(k < nkb)
        {
            // activation fragments and scales of this K block first (LDS), then the weights
            i32x8 bx[MT];
            float sc[MT];
#pragma unroll
            for(int j = 0; j < MT; ++j)
            {
                const uint32_t row = j * 16 + l16;
                const i32x4    lo  = *(const i32x4*)(sX + x_lds_off(row, k, 2 * kg, x_row_bytes));
                const i32x4    hi  = *(const i32x4*)(sX + x_lds_off(row, k, 2 * kg + 1, x_row_bytes));
                bx[j]              = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                sc[j]              = sS[row * p.chunk_kb + k] * wsv[k];
            }
            const i32x8 aw = i32x8{(int)wlo[k][0], (int)wlo[k][1], (int)wlo[k][2], (int)wlo[k][3],
                                   (int)whi[k][0], (int)whi[k][1], (int)whi[k][2], (int)whi[k][3]};
            f32x4 part[MT];
#pragma unroll
            for(int j = 0; j < MT; ++j)
                part[j] = mfma_16x16x128_fp8(aw, bx[j], f32x4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
            for(int j = 0; j < MT; ++j)
#pragma unroll
                for(int r = 0; r < 4; ++r)
                    acc[j][r] = __builtin_fmaf(part[j][r], sc[j], acc[j][r]);
        }
    }

    // lane owns out[m = j*16 + l16][n .. n+3], n = block row base + wave*16 + kg*4
    const int n_out = nblk * kRowsPerBlock + wave * kRowsPerWave + kg * 4;

    auto store_out = [&](const f32x4 (&v)[MT]) {
#pragma unroll
        for(int j = 0; j < MT; ++j)
        {
            const int m = j * 16 + l16;
            if(m >= g.M)
                continue;
            uint16_t* dst = g.out + (size_t)m * g.N + n_out;
            if(n_out + 3 < g.N && (g.N & 3) == 0)
                *(u32x2*)dst = u32x2{pack2<DT>(v[j][0], v[j][1]), pack2<DT>(v[j][2], v[j][3])};
            else
            {
#pragma unroll
                for(int r = 0; r < 4; ++r)
                    if(n_out + r < g.N)
                        dst[r] = (uint16_t)(pack2<DT>(v[j][r], 0.f) & 0xffffu);
            }
        }
    };

    if(p.splits == 1)
    {
        store_out(acc);
        return;
    }

    // ---- 4. split K: park the partial tile, take a ticket, last one in adds them up.
    // The workgroups of one row block run on different XCDs, whose L2 caches are not coherent
    // with each other.  Instead of device-wide fences (which write back and invalidate a whole
    // L2, once per workgroup), every access to the exchanged data is itself device-coherent:
    // partials are written with agent-scope stores (write-through) and waited for (vmcnt 0)
    // before this workgroup's ticket is taken with an agent-scope atomic; the last workgroup
    // reads them back with agent-scope loads, which cannot be served from a stale L2 line.
    const size_t n_pad   = (size_t)gridDim.x * kRowsPerBlock;
    const size_t m_pad   = (size_t)MT * 16;
    const size_t plane   = n_pad * m_pad; // one split's partials, laid out [m][n_pad]
    float*       my_part = p.partial + (size_t)split * plane;
#pragma unroll
    for(int j = 0; j < MT; ++j)
    {
        float* dst = my_part + (size_t)(j * 16 + l16) * n_pad + n_out;
#pragma unroll
        for(int r = 0; r < 4; ++r)
            __hip_atomic_store(dst + r, acc[j][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): the stores above have reached memory
    __shared__ uint32_t s_ticket;
    __syncthreads();
    if(t == 0)
        s_ticket = __hip_atomic_fetch_add(p.tickets + nblk, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if(s_ticket != (uint32_t)p.splits - 1)
        return;
    if(t == 0) // leave the ticket ready for the next launch
        __hip_atomic_store(p.tickets + nblk, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    f32x4 sum[MT];
#pragma unroll
    for(int j = 0; j < MT; ++j)
        sum[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    for(int s = 0; s < p.splits; ++s) // fixed order: independent of which workgroup came last
    {
        const float* part = p.partial + (size_t)s * plane;
#pragma unroll
        for(int j = 0; j < MT; ++j)
        {
            const float* src = part + (size_t)(j * 16 + l16) * n_pad + n_out;
#pragma unroll
            for(int r = 0; r < 4; ++r)
                sum[j][r] += __hip_atomic_load(src + r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    store_out(sum);
}

// workspace for split-K partials and tickets, one per device, grown on demand and kept for the
// life of the process.  Calls that need it on the same device must not overlap.
struct Workspace
{
    float*    partial      = nullptr;
    size_t    partial_size = 0;
    uint32_t* tickets      = nullptr;
    size_t    n_tickets    = 0;
};
constexpr int kMaxDevices = 64;
Workspace     g_ws[kMaxDevices];

hipError_t ensure_workspace(int dev, size_t partial_floats, size_t n_tickets, hipStream_t stream,
                            Workspace** out)
{
    if(dev < 0 || dev >= kMaxDevices)
        return hipErrorInvalidDevice;
    Workspace& w = g_ws[dev];
    if(w.partial_size < partial_floats)
    {
        if(w.partial)
            (void)hipFree(w.partial);
        w.partial      = nullptr;
        w.partial_size = 0;
        hipError_t e   = hipMalloc((void**)&w.partial, partial_floats * sizeof(float));
        if(e != hipSuccess)
            return e;
        w.partial_size = partial_floats;
    }
    if(w.n_tickets < n_tickets)
    {
        if(w.tickets)
            (void)hipFree(w.tickets);
        w.tickets   = nullptr;
        w.n_tickets = 0;
        size_t n    = n_tickets < 4096 ? 4096 : n_tickets;
        hipError_t e = hipMalloc((void**)&w.tickets, n * sizeof(uint32_t));
        if(e != hipSuccess)
            return e;
        e = hipMemsetAsync(w.tickets, 0, n * sizeof(uint32_t), stream);
        if(e != hipSuccess)
            return e;
        w.n_tickets = n;
    }
    *out = &w;
    return hipSuccess;
}

} // namespace

bool gemm_decode_supports(const GemmKernelParams& p) { return p.M >= 1 && p.M <= 64 && p.kblocks >= 1; }

// split_k_log2 < 0: choose.  Otherwise 2^split_k_log2 chunks (rounded so chunks hold <= 16 K blocks).
hipError_t launch_gemm_decode(const GemmKernelParams& g, In16 out_dtype, int split_k_log2, int device_id,
                              hipStream_t stream)
{
    DecodeParams p{};
    p.g       = g;
    p.m_tiles = (g.M + 15) / 16;
    const int n_blocks = (g.N + kRowsPerBlock - 1) / kRowsPerBlock;

    int splits;
    if(split_k_log2 >= 0)
        splits = 1 << split_k_log2;
    else
    {
        // Splitting K costs an fp32 round trip of the output tile through device-coherent
        // stores and loads, which measured slower than it gains unless N alone leaves most of the
        // chip idle: split only while fewer than ~100 workgroups exist.
        splits = 1;
        while(n_blocks * splits < 100 && splits * 2 <= g.kblocks)
            splits *= 2;
    }
    if(splits > g.kblocks)
        splits = g.kblocks;
    int chunk_kb = (g.kblocks + splits - 1) / splits;
    if(chunk_kb > kMaxChunkKb)
    {
        chunk_kb = kMaxChunkKb;
    }
    splits     = (g.kblocks + chunk_kb - 1) / chunk_kb;
    p.chunk_kb = chunk_kb;
    p.chunk_kb_pad = (chunk_kb + 7) / 8 * 8;
    p.splits   = splits;

    if(splits > 1)
    {
        Workspace* w = nullptr;
        size_t     partial_floats = (size_t)splits * n_blocks * kRowsPerBlock * p.m_tiles * 16;
        hipError_t e = ensure_workspace(device_id, partial_floats, (size_t)n_blocks, stream, &w);
        if(e != hipSuccess)
            return e;
        p.partial = w->partial;
        p.tickets = w->tickets;
    }

    const size_t smem = (size_t)p.m_tiles * 16 * p.chunk_kb_pad * 128 + (size_t)p.m_tiles * 16 * chunk_kb * 4;
    dim3         grid(n_blocks, splits);
    const bool   bf = out_dtype == In16::bf16;
#define FP8BS_LAUNCH_DECODE(MT, KB)                                                               \
    {                                                                                             \
        auto       kernel = bf ? gemm_decode_kernel<In16::bf16, MT, KB>                           \
                               : gemm_decode_kernel<In16::fp16, MT, KB>;                          \
        hipError_t e      = hipFuncSetAttribute((const void*)kernel,                              \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); \
        if(e != hipSuccess)                                                                       \
            return e;                                                                             \
        hipLaunchKernelGGL(kernel, grid, dim3(kThreads), smem, stream, p);                        \
    }
#define FP8BS_LAUNCH_DECODE_KB(MT)                     \
    if(chunk_kb <= 4)                                  \
        FP8BS_LAUNCH_DECODE(MT, 4)                     \
    else if(chunk_kb <= 8)                             \
        FP8BS_LAUNCH_DECODE(MT, 8)                     \
    else if(chunk_kb <= 12)                            \
        FP8BS_LAUNCH_DECODE(MT, 12)                    \
    else                                               \
        FP8BS_LAUNCH_DECODE(MT, 16)
    switch(p.m_tiles)
    {
    case 1: FP8BS_LAUNCH_DECODE_KB(1) break;
    case 2: FP8BS_LAUNCH_DECODE_KB(2) break;
    case 3: FP8BS_LAUNCH_DECODE_KB(3) break;
    default: FP8BS_LAUNCH_DECODE_KB(4) break;
    }
#undef FP8BS_LAUNCH_DECODE_KB
#undef FP8BS_LAUNCH_DECODE
    return hipGetLastError();
}

} // namespace fp8bs
