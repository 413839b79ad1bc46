// Mid-size block-scale FP8 GEMM: problems too tall for the weight-streaming kernel and too small
// to cover the chip with 256x256 tiles.
//
// BM (m) x BN (n) output tile per workgroup, 128x128, 64x128 or 64x64, picked at launch so that
// the tiles alone give every compute unit work: splitting K across workgroups instead costs an
// fp32 round trip of the tile through memory, which measured far dearer than the extra operand
// traffic of smaller tiles.  4 waves laid out 2 (n) x 2 (m).  Both operand slabs of a K block and
// the block's x_scale column come in with direct global->LDS loads into a four-stage ring: three
// K blocks are in flight while one is multiplied.  The 64x64 tile leaves room for two workgroups
// per compute unit.
//
// K can still be split across workgroups (very few tiles, long K): fp32 partial tiles go to a
// workspace (lane-major, 16-byte accesses that bypass the per-XCD L2) and the last workgroup to
// finish a tile, found with an atomic ticket, adds them in split order, so results never depend
// on timing.
//
// The MFMAs of a K block and the FMAs that fold their products into the accumulators are an
// explicit instruction stream, as in the 256x256 kernel: left to the compiler, every MFMA writes
// the same accumulator quad and waits for the previous product to be read out, which alone takes
// 1 us per K block.
#include "gemm_common.h"

namespace fp8bs {

namespace {

constexpr int kThreads = 256;

// s_waitcnt immediate for vmcnt(n) alone (expcnt and lgkmcnt left at their maxima)
constexpr int vmcnt_imm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }

struct MidParams
{
    GemmKernelParams g;
    int32_t   tiles_m, tiles_n;
    int32_t   splits, kb_per_split;
    int32_t   bf16_out;
    float*    partial; // [splits][tiles][4 waves x TI*TJ tiles][64 lanes] x 4 fp32
    uint32_t  partial_bytes;
    uint32_t* tickets; // [tiles], zero between launches
};

template <int BM, int BN>
struct MidShape
{
    static constexpr int kWBytes = BN * 128, kXBytes = BM * 128;
    static constexpr int kStageBytes = kWBytes + kXBytes + BM * 4;
    static constexpr int TI = BN / 32, TJ = BM / 32;       // MFMA tiles per wave along n and m
    static constexpr int NQ = TI * TJ;                      // tiles per wave and K block
    static constexpr int kWUnits = BN / 32, kXUnits = BM / 32; // 1-KiB units per wave and stage
    static constexpr int kLoadsPerStage = kWUnits + kXUnits + 1;
    // four stages: three K blocks in flight while one is multiplied (deeper rings measured no
    // faster); the 64x64 tile then leaves room for two workgroups per compute unit
    static constexpr int kStages = 4;
    static constexpr int kSmem = kStages * kStageBytes;
    static constexpr int kOccupancy = kSmem <= 72 * 1024 ? 2 : 1;
    static_assert(NQ % 4 == 0, "the product rotation below assumes a multiple of four tiles");
};

// waits until at most `ahead` stages' worth of this wave's loads are still in flight
template <int A, int LPS>
__device__ __forceinline__ void wait_ahead(int ahead)
{
    if(ahead >= A)
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(A * LPS));
    else if constexpr(A > 0)
        wait_ahead<A - 1, LPS>(ahead);
}

// The two instruction forms of the multiply stream, as non-template functions: inside the kernel
// template their operands would be value-dependent, the statements would be rebuilt per
// instantiation, and the host pass (which knows no 'v' register class of this width) would then
// drop the kernel's launch stub without a word.
__device__ __forceinline__ void mfma_asm(f32x4& product, const i32x8& a, const i32x8& b)
{
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0" : "=&v"(product) : "v"(a), "v"(b));
}
__device__ __forceinline__ void fma4_asm(float (&acc)[4], const f32x4& product, float s)
{
    asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(acc[0]) : "v"(product[0]), "v"(s));
    asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(acc[1]) : "v"(product[1]), "v"(s));
    asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(acc[2]) : "v"(product[2]), "v"(s));
    asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(acc[3]) : "v"(product[3]), "v"(s));
}

template <int BM, int BN, bool SHUF, int OCC>
__global__ __launch_bounds__(kThreads, OCC) void gemm_mid_kernel(MidParams p)
{
    using S = MidShape<BM, BN>;
    constexpr int TI = S::TI, TJ = S::TJ, NQ = S::NQ;
    constexpr int kWBytes = S::kWBytes, kXBytes = S::kXBytes, kStageBytes = S::kStageBytes;
    constexpr int kLoadsPerStage = S::kLoadsPerStage, kStages = S::kStages;

    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    const GemmKernelParams& g = p.g;

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int l16 = lane & 15, kg = lane >> 4;
    const int wn = wave & 1, wm = wave >> 1;

    // ---- which tile and K range: workgroups go round-robin over the 8 XCDs, so give each XCD
    // a contiguous run of (split, tile) pairs, tiles m-fastest: neighbours share weight slabs
    const int tiles = p.tiles_m * p.tiles_n, total = tiles * p.splits;
    int       v     = blockIdx.x;
    if((total & 7) == 0)
        v = (v & 7) * (total >> 3) + (v >> 3);
    const int split = v / tiles, tile = v - split * tiles;
    const int tn = tile / p.tiles_m, tm = tile - tn * p.tiles_m;
    const int m0 = tm * BM, n0 = tn * BN;
    const int kb_lo = split * p.kb_per_split;
    const int kb_hi = min(kb_lo + p.kb_per_split, g.kblocks);

    typedef const volatile i32x4 __attribute__((address_space(3)))* lds_vvec_ptr;
    typedef const float __attribute__((address_space(3)))*          lds_f32_ptr;
    typedef uint8_t __attribute__((address_space(3)))*              lds_byte_ptr;
    const lds_byte_ptr smem3 = (lds_byte_ptr)smem;

    // ---- global -> LDS plan: a stage is BN/8 + BM/8 units of 1 KiB (8 rows each); wave w moves
    // units 4 i + w of either slab.  Lane p of a unit fills LDS chunk p: stage row 8 u + p/8,
    // stored chunk p%8, which must hold the row's logical chunk (p%8) ^ ((row>>1)&7).
    // Pre-shuffled weights: unit u is half of 16-row tile u/2's K block, copied as it lies.
    uint32_t goff_w[S::kWUnits], goff_x[S::kXUnits];
#pragma unroll
    for(int i = 0; i < S::kWUnits; ++i)
    {
        const uint32_t u = 4u * i + wave;
        const uint32_t r = 8u * u + (lane >> 3);
        const uint32_t c = (lane & 7u) ^ ((r >> 1) & 7u);
        if(SHUF)
        {
            uint32_t tl = ((uint32_t)n0 >> 4) + (u >> 1);
            tl          = min(tl, ((uint32_t)g.N >> 4) - 1u);
            goff_w[i]   = tl * 16u * (uint32_t)g.K + (u & 1u) * 1024u + (uint32_t)lane * 16u;
        }
        else
        {
            const uint32_t n = min((uint32_t)n0 + r, (uint32_t)g.N - 1u);
            goff_w[i]        = n * (uint32_t)g.ldb + c * 16u;
        }
    }
#pragma unroll
    for(int i = 0; i < S::kXUnits; ++i)
    {
        const uint32_t u = 4u * i + wave;
        const uint32_t r = 8u * u + (lane >> 3);
        const uint32_t c = (lane & 7u) ^ ((r >> 1) & 7u);
        const uint32_t m = min((uint32_t)m0 + r, (uint32_t)g.M - 1u);
        goff_x[i]        = m * (uint32_t)g.lda + c * 16u;
    }
    // LDS-direct loads (lane p's bytes land at M0 + 16 p / M0 + 4 p).  Issued from asm: the
    // compiler models the builtin as a flat access that may touch LDS and from then on waits for
    // every outstanding LDS read in full.  They are invisible to the compiler's wait counts, so
    // the waits for them are counted by hand below.
    auto dma16 = [](uint32_t lds_dst, uint32_t voff, const uint8_t* sbase) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(lds_dst), "v"(voff), "s"(sbase)
                     : "memory");
    };
    auto dma4 = [](uint32_t lds_dst, uint32_t voff, const void* sbase) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                     :
                     : "s"(lds_dst), "v"(voff), "s"(sbase)
                     : "memory");
    };
    // x_scale of the tile's BM rows: wave w, lanes 0 .. BM/4-1 -> rows (BM/4) w + lane
    constexpr int kXsLanes = BM / 4;
    uint32_t      xs_goff;
    {
        const uint32_t m = min((uint32_t)m0 + (uint32_t)kXsLanes * wave + (lane % kXsLanes), (uint32_t)g.M - 1u);
        xs_goff          = m * (uint32_t)g.xs_m * 4u;
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)smem3;
    auto fill_stage = [&](int stage, int kb) {
        const uint32_t base = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)stage * kStageBytes);
        const size_t   koff = (size_t)kb * 128, koff_w = SHUF ? (size_t)kb * 2048 : koff;
#pragma unroll
        for(int i = 0; i < S::kWUnits; ++i)
            dma16(__builtin_amdgcn_readfirstlane(base + (4u * i + wave) * 1024u), goff_w[i], g.wq + koff_w);
#pragma unroll
        for(int i = 0; i < S::kXUnits; ++i)
            dma16(__builtin_amdgcn_readfirstlane(base + (uint32_t)kWBytes + (4u * i + wave) * 1024u), goff_x[i],
                  g.xq + koff);
        if(lane < kXsLanes) // every wave issues the same number of loads per stage: the waits count them
            dma4(__builtin_amdgcn_readfirstlane(base + (uint32_t)(kWBytes + kXBytes) +
                                                (uint32_t)wave * (uint32_t)kXsLanes * 4u),
                 xs_goff + (uint32_t)kb * (uint32_t)g.xs_k * 4u, g.xs);
    };

    // ---- w_scale of this wave's BN/2 weight rows (one 128-row block): 64 consecutive K blocks
    // live in one VGPR (lane = K block) and are picked with v_readlane.  The window is a vector
    // load the compiler waits for with vmcnt(0) at its first use, which also drains the ring of
    // LDS-direct loads it cannot see: once at the first K block and once every 64 after that.
    uint32_t nb = (uint32_t)(n0 + wn * (BN / 2)) >> 7;
    nb          = min(nb, (uint32_t)((g.N + 127) / 128 - 1));
    const float* ws_row = g.ws + (size_t)nb * g.kblocks;
    auto load_ws_window = [&](int kb0) -> float {
        const int k = kb0 + lane;
        return ws_row[k < g.kblocks ? k : g.kblocks - 1];
    };
    float ws_vec = load_ws_window(kb_lo & ~63);
    auto  ws_at  = [&](int kb) -> float {
        return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(ws_vec), kb & 63));
    };

    // ---- LDS read offsets of this lane's fragment halves (tile rows start at multiples of 16,
    // so the swizzle term depends on l16 only)
    const uint32_t sw      = (uint32_t)(l16 >> 1) & 7u;
    const uint32_t lo_off  = (uint32_t)l16 * 128u + (((2u * kg) ^ sw) << 4);
    const uint32_t hi_off  = (uint32_t)l16 * 128u + (((2u * kg + 1u) ^ sw) << 4);
    const uint32_t wlo_off = SHUF ? (uint32_t)kg * 512u + (uint32_t)l16 * 16u : lo_off;
    const uint32_t whi_off = SHUF ? wlo_off + 256u : hi_off;
    const uint32_t w_base  = (uint32_t)wn * (uint32_t)(BN / 2) * 128u;
    const uint32_t x_base  = (uint32_t)kWBytes + (uint32_t)wm * (uint32_t)(BM / 2) * 128u;
    const uint32_t xs_lds  = (uint32_t)(kWBytes + kXBytes) + ((uint32_t)wm * (uint32_t)(BM / 2) + (uint32_t)l16) * 4u;

    float acc[TI][TJ][4]; // plain floats: the FMAs below name single elements as asm operands
#pragma unroll
    for(int i = 0; i < TI; ++i)
#pragma unroll
        for(int j = 0; j < TJ; ++j)
#pragma unroll
            for(int c = 0; c < 4; ++c)
                acc[i][j][c] = 0.f;

    f32x4 P[4];
#pragma unroll
    for(int q = 0; q < 4; ++q)
        P[q] = f32x4{0.f, 0.f, 0.f, 0.f};
    float scp[TJ]; // scales of the previous K block, per m tile
#pragma unroll
    for(int j = 0; j < TJ; ++j)
        scp[j] = 0.f;

    // ---- K loop.  Stage s of the ring holds K block kb_lo + s (mod kStages); kStages - 1 stages
    // are requested ahead.  Per iteration: wait until this wave's share of the current stage has
    // landed (loads return in order, so that is a count of the younger ones still allowed in
    // flight), barrier (every wave's share has landed, and every wave is done with the stage read
    // in the previous iteration), refill that previous stage, multiply.
    const int nkb = kb_hi - kb_lo;
#pragma unroll
    for(int s0 = 0; s0 < kStages - 1; ++s0)
        if(s0 < nkb)
            fill_stage(s0, kb_lo + s0);

    for(int it = 0; it < nkb; ++it)
    {
        const int kb    = kb_lo + it;
        const int ahead = min(nkb - 1 - it, kStages - 2); // younger stages already requested
        wait_ahead<kStages - 2, kLoadsPerStage>(ahead);
        __syncthreads();
        // (the scale is picked before the refill is issued: where the compiler drains the ring
        // for the window load, the stage requested below is not yet part of it)
        if((kb & 63) == 0 && it != 0)
            ws_vec = load_ws_window(kb);
        const float wsc = ws_at(kb);
        asm volatile("" ::"s"(wsc));
        if(it + kStages - 1 < nkb)
            fill_stage((it + kStages - 1) % kStages, kb + kStages - 1);

        const uint32_t stage = (uint32_t)(it % kStages) * kStageBytes;
        // Fragment reads are volatile so that they stay where they are written: the activation
        // fragments and the first weight fragment ahead of the first MFMA, each further weight
        // fragment one row of tiles ahead of its use (the compiler would hoist every read to the
        // top and leave the matrix pipe idle while they travel).
        auto read_w = [&](int i) -> i32x8 {
            const i32x4 lo = *(lds_vvec_ptr)(smem3 + stage + w_base + i * 2048 + wlo_off);
            const i32x4 hi = *(lds_vvec_ptr)(smem3 + stage + w_base + i * 2048 + whi_off);
            return i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        };
        i32x8 bx[TJ], aw[TI];
        float sc[TJ];
        aw[0] = read_w(0);
#pragma unroll
        for(int j = 0; j < TJ; ++j)
        {
            const i32x4 lo = *(lds_vvec_ptr)(smem3 + stage + x_base + j * 2048 + lo_off);
            const i32x4 hi = *(lds_vvec_ptr)(smem3 + stage + x_base + j * 2048 + hi_off);
            bx[j]          = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            sc[j]          = *(lds_f32_ptr)(smem3 + stage + xs_lds + j * 64) * wsc;
        }
        // Tile q = (i, j) = (q / TJ, q % TJ).  The product of tile q is folded in behind the MFMA
        // of tile q + 2: it has been written back by then (two MFMAs of 8 passes each), so no
        // wait states are needed.  Products rotate through four register quads; the last two
        // tiles of a K block are folded in behind the first two MFMAs of the next one.
#pragma unroll
        for(int q = 0; q < NQ; ++q)
        {
            if(q % TJ == 0 && q / TJ + 1 < TI)
                aw[q / TJ + 1] = read_w(q / TJ + 1);
            mfma_asm(P[q & 3], aw[q / TJ], bx[q % TJ]);
            if(q < 2)
                fma4_asm(acc[(NQ - 2 + q) / TJ][(NQ - 2 + q) % TJ], P[(NQ - 2 + q) & 3], scp[(NQ - 2 + q) % TJ]);
            else
                fma4_asm(acc[(q - 2) / TJ][(q - 2) % TJ], P[(q - 2) & 3], sc[(q - 2) % TJ]);
        }
#pragma unroll
        for(int j = 0; j < TJ; ++j)
            scp[j] = sc[j];
    }
    // drain the two products still in flight (>= 11 wait states after the last MFMA)
    asm volatile("s_nop 15\n s_nop 15\n s_nop 15" ::: "memory");
    fma4_asm(acc[(NQ - 2) / TJ][(NQ - 2) % TJ], P[(NQ - 2) & 3], scp[(NQ - 2) % TJ]);
    fma4_asm(acc[(NQ - 1) / TJ][(NQ - 1) % TJ], P[(NQ - 1) & 3], scp[(NQ - 1) % TJ]);

    // ---- epilogue: lane owns out[m][n .. n+3] for each of its TI x TJ tiles
    auto store_tile = [&](int i, int j, const float(&a)[4]) {
        const int m = m0 + wm * (BM / 2) + j * 16 + l16;
        const int n = n0 + wn * (BN / 2) + i * 16 + kg * 4;
        if(m >= g.M || n >= g.N)
            return;
        uint16_t*   dst = g.out + (size_t)m * g.N + n;
        const u32x2 o   = p.bf16_out ? u32x2{pack2<In16::bf16>(a[0], a[1]), pack2<In16::bf16>(a[2], a[3])}
                                     : u32x2{pack2<In16::fp16>(a[0], a[1]), pack2<In16::fp16>(a[2], a[3])};
        if(n + 3 < g.N && (g.N & 3) == 0)
            *(u32x2*)dst = o;
        else
        {
#pragma unroll
            for(int c = 0; c < 4; ++c)
                if(n + c < g.N)
                    dst[c] = (uint16_t)((o[c >> 1] >> (16 * (c & 1))) & 0xffffu);
        }
    };
    if(p.splits == 1)
    {
#pragma unroll
        for(int j = 0; j < TJ; ++j)
#pragma unroll
            for(int i = 0; i < TI; ++i)
                store_tile(i, j, acc[i][j]);
        return;
    }

    // ---- K split across workgroups: park the partial tile set, take a ticket, last one in adds
    // them up in split order.  The workgroups of one tile run on different XCDs, whose L2 caches
    // are not coherent with each other, so every access to the exchanged data bypasses them (sc1)
    // and the stores are waited for before the ticket is taken.
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(p.partial, 0, (int)p.partial_bytes, 0x00020000);
    constexpr int kCoherent = 16;
    auto part_off = [&](int sp, int i, int j) -> uint32_t {
        return (uint32_t)(((((size_t)sp * tiles + tile) * 4 + wave) * NQ + i * TJ + j) * 64 + lane) * 16u;
    };
#pragma unroll
    for(int i = 0; i < TI; ++i)
#pragma unroll
        for(int j = 0; j < TJ; ++j)
            __builtin_amdgcn_raw_buffer_store_b128(
                u32x4{__float_as_uint(acc[i][j][0]), __float_as_uint(acc[i][j][1]), __float_as_uint(acc[i][j][2]),
                      __float_as_uint(acc[i][j][3])},
                rsrc,
                                                   part_off(split, i, j), 0, kCoherent);
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0)); // the stores above have reached memory
    __shared__ uint32_t s_ticket;
    __syncthreads();
    if(t == 0)
        s_ticket = __hip_atomic_fetch_add(p.tickets + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if(s_ticket != (uint32_t)p.splits - 1)
        return;
    if(t == 0) // leave the ticket ready for the next launch
        __hip_atomic_store(p.tickets + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for(int j = 0; j < TJ; ++j)
#pragma unroll
        for(int i = 0; i < TI; ++i)
        {
            f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
            for(int sp = 0; sp < p.splits; ++sp) // split order, whoever arrived last
                s += __builtin_bit_cast(
                    f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, part_off(sp, i, j), 0, kCoherent));
            const float sum[4] = {s[0], s[1], s[2], s[3]};
            store_tile(i, j, sum);
        }
}

template <int BM, int BN>
hipError_t launch_shape(MidParams& p, int split_k_log2, int device_id, hipStream_t stream)
{
    using S = MidShape<BM, BN>;
    const GemmKernelParams& g = p.g;
    p.tiles_m = (g.M + BM - 1) / BM;
    p.tiles_n = (g.N + BN - 1) / BN;
    const int tiles = p.tiles_m * p.tiles_n;

    int splits = 1;
    if(split_k_log2 >= 0)
        splits = 1 << split_k_log2;
    else
    {
        // Splitting K costs an fp32 round trip of the tile through memory: taken only when even
        // the smallest tile leaves most of the chip idle, and never below 8 K blocks per split.
        while(tiles * splits * 2 <= 160 && g.kblocks / (splits * 2) >= 8)
            splits *= 2;
    }
    if(splits > g.kblocks)
        splits = g.kblocks;
    p.kb_per_split = (g.kblocks + splits - 1) / splits;
    splits         = (g.kblocks + p.kb_per_split - 1) / p.kb_per_split;
    p.splits       = splits;

    if(splits > 1)
    {
        const size_t bytes = (size_t)splits * tiles * 4 * S::NQ * 64 * 16;
        if(bytes >= ((size_t)1 << 31))
            return hipErrorInvalidValue;
        hipError_t e = gemm_split_workspace(device_id, bytes, (size_t)tiles, stream, &p.partial, &p.tickets);
        if(e != hipSuccess)
            return e;
        p.partial_bytes = (uint32_t)bytes;
    }

    auto        kernel = g.w_shuffled ? gemm_mid_kernel<BM, BN, true, S::kOccupancy>
                                      : gemm_mid_kernel<BM, BN, false, S::kOccupancy>;
    static bool raised[2][64]; // dynamic LDS above the default limit needs opting in, once
    const int   which = g.w_shuffled ? 1 : 0;
    if(device_id >= 0 && device_id < 64 && !raised[which][device_id])
    {
        hipError_t e =
            hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, S::kSmem);
        if(e != hipSuccess)
            return e;
        raised[which][device_id] = true;
    }
    hipLaunchKernelGGL(kernel, dim3(tiles * splits), dim3(kThreads), S::kSmem, stream, p);
    return hipGetLastError();
}

} // namespace

bool gemm_mid_supports(const GemmKernelParams& p)
{
    // 32-bit byte offsets inside the operand matrices
    return p.kblocks >= 1 && (uint64_t)p.N * (uint64_t)p.ldb < (1ull << 32) &&
           (uint64_t)p.M * (uint64_t)p.lda < (1ull << 32) && (uint64_t)p.M * (uint64_t)p.kblocks < (1ull << 30);
}

// split_k_log2 < 0: choose.  tile: 0 = choose, else 128 (128x128), 64128 (64x128) or 64 (64x64).
hipError_t launch_gemm_mid(const GemmKernelParams& g, In16 out_dtype, int split_k_log2, int device_id,
                           hipStream_t stream, int tile)
{
    MidParams p{};
    p.g        = g;
    p.bf16_out = out_dtype == In16::bf16 ? 1 : 0;
    if(tile == 0)
    {
        // 128x128 once that gives most compute units a workgroup, else 64x64 (measured: the
        // iteration costs about the same for either tile, so few large tiles lose to many small
        // ones until the chip is covered)
        const int64_t big = (int64_t)((g.M + 127) / 128) * ((g.N + 127) / 128);
        tile              = big >= 160 ? 128 : 64;
    }
    switch(tile)
    {
    case 128: return launch_shape<128, 128>(p, split_k_log2, device_id, stream);
    case 64128: return launch_shape<64, 128>(p, split_k_log2, device_id, stream);
    case 64: return launch_shape<64, 64>(p, split_k_log2, device_id, stream);
    default: return hipErrorInvalidValue;
    }
}

} // namespace fp8bs
