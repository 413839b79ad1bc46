// Mid-size block-scale FP8 GEMM: problems too tall for the weight-streaming kernel and too small
// to cover the chip with 256x256 tiles.
//
// BM (m) x BN (n) output tile per workgroup, 128x128, 64x128 or 64x64, and a number of K ranges,
// picked together at launch from a small cost model so that every compute unit has work.
// 4 waves laid out 2 (n) x 2 (m) multiply; 4 more issue the loads.  Both operand slabs of a K
// block and the block's x_scale column come in with direct global->LDS loads into a four-stage
// ring: three K blocks are in flight while one is multiplied.  The 64x64 tile leaves room for two workgroups
// per compute unit; when there are no more workgroups than compute units it runs a six-stage ring
// instead, filled two K blocks at a time.
//
// K split across workgroups (few tiles, long K): each range's fp32 partial tile goes to a
// workspace and a second, chip-wide launch adds the ranges in order and converts, so results never
// depend on timing.
//
// The MFMAs of a K block and the FMAs that fold their products into the accumulators are an
// explicit instruction stream, as in the 256x256 kernel: left to the compiler, every MFMA writes
// the same accumulator quad and waits for the previous product to be read out, which alone takes
// 1 us per K block.
#include "gemm_common.h"

#include <atomic>
#include <cstdio>

namespace fp8bs {

namespace {

constexpr int kThreads = 512; // four waves that multiply, four that fetch
constexpr size_t kMaxPartialBytes = (size_t)2 << 30; // what the arenas serve for partial tiles

// s_waitcnt immediate for vmcnt(n) alone (expcnt and lgkmcnt left at their maxima)
constexpr int vmcnt_imm(int n) { return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8); }

struct MidParams
{
    GemmKernelParams g;
    int32_t   tiles_m, tiles_n;
    int32_t   splits, kb_per_split;
    int32_t   bf16_out;
    float*    partial; // [splits][M][N] fp32
};

template <int BM, int BN, bool PAIR = false>
struct MidShape
{
    static constexpr int kWBytes = BN * 128, kXBytes = BM * 128;
    static constexpr int kStageBytes = kWBytes + kXBytes + BM * 4;
    static constexpr int TI = BN / 32, TJ = BM / 32;       // MFMA tiles per wave along n and m
    static constexpr int NQ = TI * TJ;                      // tiles per wave and K block
    static constexpr int kWUnits = BN / 32, kXUnits = BM / 32; // 1-KiB units per wave and stage
    static constexpr int kLoadsPerStage = kWUnits + kXUnits + 1;
    // four stages: three K blocks in flight while one is multiplied (deeper rings filled one K
    // block at a time measured no faster); the 64x64 tile then leaves room for two workgroups per
    // compute unit.  PAIR: six stages, filled in pairs every other iteration.
    static constexpr int kStages = PAIR ? 6 : 4;
    static constexpr int kSmem = kStages * kStageBytes;
    // Row-major x_scale in windows of four K blocks (16 bytes per row and load instead of 4: a wave's load of
    // one scale per row touches as many lines as the rows it covers, and fetched per K block these loads are a
    // third of the kernel's line requests).  A ring of four windows behind the stages: the stages in flight
    // and the one being multiplied (at most seven consecutive K blocks) never span more than three.
    static constexpr int kWindowBytes = BM * 16, kWindows = 4;
    static constexpr int kSmemWindows = kSmem + kWindows * kWindowBytes;
    static constexpr int kOccupancy = kSmemWindows <= 72 * 1024 ? 2 : 1;
    static_assert(NQ % 4 == 0, "the product rotation below assumes a multiple of four tiles");
};

// waits until at most `ahead` stages' worth of this wave's loads (and `extra` single loads: 0 or 1)
// are still in flight
template <int A, int LPS>
__device__ __forceinline__ void wait_ahead(int ahead, int extra = 0)
{
    if(ahead >= A)
    {
        if(extra)
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(A * LPS + 1));
        else
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(A * LPS));
    }
    else if constexpr(A > 0)
        wait_ahead<A - 1, LPS>(ahead, extra);
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

// 16-byte store that is written through to memory instead of lingering dirty in this XCD's L2:
// the end of the kernel then has less to write back before the reduction launch can start
__device__ __forceinline__ void store_through(float* dst, const f32x4& v)
{
    asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(dst), "v"(v) : "memory");
}

// XS4: x_scale is row-major with 16-byte aligned rows and comes in windows of four K blocks.
template <int BM, int BN, bool SHUF, int OCC, bool PAIR, bool XS4>
__global__ __launch_bounds__(kThreads, OCC) void gemm_mid_kernel(MidParams p)
{
    using S = MidShape<BM, BN, PAIR>;
    constexpr int TI = S::TI, TJ = S::TJ, NQ = S::NQ;
    constexpr int kWBytes = S::kWBytes, kXBytes = S::kXBytes, kStageBytes = S::kStageBytes;
    // XS4: a stage's loads are its slab units, plus the window's load in front of them when the stage opens a
    // window; the waits count the windows opened by the younger stages on top of their slab units.
    constexpr int kLoadsPerStage = XS4 ? S::kLoadsPerStage - 1 : S::kLoadsPerStage, kStages = S::kStages;
    constexpr uint32_t kWindowsAt = (uint32_t)S::kSmem;

    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    const GemmKernelParams& g = p.g;

    // Waves 0-3 multiply, waves 4-7 issue the ring's loads.  A wave that issues loads is held at
    // the issue while the memory pipeline's queue is full (a compute unit takes in about 40 KB/us
    // from HBM), so a wave that did both would start its LDS reads and MFMAs only after its share
    // of the next stage had been accepted: fetch and arithmetic of a K block would add up instead
    // of overlapping (0.19 us of 0.5 us per K block in the 64x64 tile).
    const int  t = threadIdx.x, lane = t & 63, wave = (t >> 6) & 3;
    const bool fetches = __builtin_amdgcn_readfirstlane(t >> 8) != 0;
    const int  l16 = lane & 15, kg = lane >> 4;
    const int  wn = wave & 1, wm = wave >> 1;

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
    // stored chunk p%8, which must hold the row's logical chunk (p%8) ^ lds_swizzle(row).
    // Pre-shuffled weights: unit u is half of 16-row tile u/2's K block, copied as it lies.
    uint32_t goff_w[S::kWUnits], goff_x[S::kXUnits];
#pragma unroll
    for(int i = 0; i < S::kWUnits; ++i)
    {
        const uint32_t u = 4u * i + wave;
        const uint32_t r = 8u * u + (lane >> 3);
        const uint32_t c = (lane & 7u) ^ lds_swizzle(r);
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
        const uint32_t c = (lane & 7u) ^ lds_swizzle(r);
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
        if constexpr(XS4)
        {
            // the first stage of a window (or of the K range) brings the window, ahead of its own slabs
            if(((kb & 3) == 0 || kb == kb_lo) && lane < kXsLanes)
                dma16(__builtin_amdgcn_readfirstlane(lds0 + kWindowsAt + (uint32_t)((kb >> 2) & 3) * S::kWindowBytes +
                                                     (uint32_t)wave * (uint32_t)kXsLanes * 16u),
                      xs_goff + (uint32_t)(kb & ~3) * 4u, (const uint8_t*)g.xs);
        }
#pragma unroll
        for(int i = 0; i < S::kWUnits; ++i)
            dma16(__builtin_amdgcn_readfirstlane(base + (4u * i + wave) * 1024u), goff_w[i], g.wq + koff_w);
#pragma unroll
        for(int i = 0; i < S::kXUnits; ++i)
            dma16(__builtin_amdgcn_readfirstlane(base + (uint32_t)kWBytes + (4u * i + wave) * 1024u), goff_x[i],
                  g.xq + koff);
        if(!XS4 && lane < kXsLanes) // every wave issues the same number of loads per stage: the waits count them
            dma4(__builtin_amdgcn_readfirstlane(base + (uint32_t)(kWBytes + kXBytes) +
                                                (uint32_t)wave * (uint32_t)kXsLanes * 4u),
                 xs_goff + (uint32_t)kb * (uint32_t)g.xs_k * 4u, g.xs);
    };

    // ---- w_scale of this wave's BN/2 weight rows (one 128-row block): 64 consecutive K blocks
    // live in one VGPR (lane = K block) and are picked with v_readlane.  The window is a vector
    // load the compiler waits for with vmcnt(0) at its first use: in the waves that multiply,
    // which have no LDS-direct loads of their own in flight.
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
    const uint32_t sw      = lds_swizzle((uint32_t)l16);
    const uint32_t lo_off  = (uint32_t)l16 * 128u + (((2u * kg) ^ sw) << 4);
    const uint32_t hi_off  = (uint32_t)l16 * 128u + (((2u * kg + 1u) ^ sw) << 4);
    const uint32_t wlo_off = SHUF ? (uint32_t)kg * 512u + (uint32_t)l16 * 16u : lo_off;
    const uint32_t whi_off = SHUF ? wlo_off + 256u : hi_off;
    const uint32_t w_base  = (uint32_t)wn * (uint32_t)(BN / 2) * 128u;
    const uint32_t x_base  = (uint32_t)kWBytes + (uint32_t)wm * (uint32_t)(BM / 2) * 128u;
    // (XS4: this lane's row in window 0, first K block of the window)
    const uint32_t xs_lds  = XS4 ? kWindowsAt + ((uint32_t)wm * (uint32_t)(BM / 2) + (uint32_t)l16) * 16u
                                 : (uint32_t)(kWBytes + kXBytes) + ((uint32_t)wm * (uint32_t)(BM / 2) + (uint32_t)l16) * 4u;

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
    // XS4: where this lane's x_scale of K block kb lies (window (kb / 4) & 3, block kb & 3 of its row).  The
    // address of the next K block is worked out behind the multiply stream, not between the barrier and the
    // first reads of the next iteration.
    auto xs_window_addr = [&](int kb) -> uint32_t {
        return (uint32_t)(((kb >> 2) & 3) * S::kWindowBytes + (kb & 3) * 4) + xs_lds;
    };
    uint32_t xs_addr = XS4 ? xs_window_addr(kb_lo) : 0u;

    const int nkb = kb_hi - kb_lo;
    constexpr int kAhead = PAIR ? 4 : kStages - 2; // most stages in flight behind the one waited for
    if(fetches)
    {
#pragma unroll
        for(int s0 = 0; s0 < (PAIR ? 4 : kStages - 1); ++s0)
            if(s0 < nkb)
                fill_stage(s0, kb_lo + s0);
    }

    for(int it = 0; it < nkb; ++it)
    {
        const int kb    = kb_lo + it;
        // younger stages already requested
        const int ahead = min(nkb - 1 - it, PAIR ? ((it & 1) ? 4 : 3) : kStages - 2);
        // (XS4: a K block among the `ahead` younger ones that is a multiple of four came with a window's load;
        // there is at most one, as ahead <= 4)
        if(fetches)
            wait_ahead<kAhead, kLoadsPerStage>(ahead, XS4 ? ((kb & 3) + ahead) >> 2 : 0);
        __syncthreads();
        if(fetches)
        {
            if constexpr(PAIR)
            {
                // two K blocks are requested together every other iteration: a weight row's 256
                // consecutive bytes then reach the memory controller side by side
                if((it & 1) == 0)
                {
                    if(it + 4 < nkb)
                        fill_stage((it + 4) % kStages, kb + 4);
                    if(it + 5 < nkb)
                        fill_stage((it + 5) % kStages, kb + 5);
                }
            }
            else if(it + kStages - 1 < nkb)
                fill_stage((it + kStages - 1) % kStages, kb + kStages - 1);
            continue;
        }
        if((kb & 63) == 0 && it != 0)
            ws_vec = load_ws_window(kb);
        const float wsc = ws_at(kb);
        asm volatile("" ::"s"(wsc));

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
            sc[j]          = (XS4 ? *(lds_f32_ptr)(smem3 + xs_addr + j * 256)
                                  : *(lds_f32_ptr)(smem3 + stage + xs_lds + j * 64)) *
                             wsc;
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
        if constexpr(XS4)
        {
            xs_addr = xs_window_addr(kb + 1);
            asm volatile("" : "+v"(xs_addr)); // here, behind the last MFMA
        }
    }
    // One K range, 16-byte aligned output rows: the tile goes through LDS so that all eight waves
    // store whole 128-byte (or longer) row segments, 16 bytes per lane; otherwise the waves that
    // multiplied store their fragments as they hold them (8 bytes per lane, 32 per row and instruction).
    const bool staged = p.splits == 1 && (g.N & 7) == 0 && ((uintptr_t)g.out & 15) == 0;
    if(fetches && !staged)
        return;
    if(!fetches)
    {
        // drain the two products still in flight (>= 11 wait states after the last MFMA)
        asm volatile("s_nop 15\n s_nop 15\n s_nop 15" ::: "memory");
        fma4_asm(acc[(NQ - 2) / TJ][(NQ - 2) % TJ], P[(NQ - 2) & 3], scp[(NQ - 2) % TJ]);
        fma4_asm(acc[(NQ - 1) / TJ][(NQ - 1) % TJ], P[(NQ - 1) & 3], scp[(NQ - 1) % TJ]);
    }
    if(staged)
    {
        constexpr int kPitch = BN * 2 + 16; // bytes between two rows of the staged tile
        static_assert(BM * kPitch <= S::kSmem, "the staged tile takes the ring's place");
        __syncthreads(); // every wave is done with the ring's last stage
        if(!fetches)
        {
#pragma unroll
            for(int j = 0; j < TJ; ++j)
#pragma unroll
                for(int i = 0; i < TI; ++i)
                {
                    const float(&a)[4] = acc[i][j];
                    const u32x2 o = p.bf16_out ? u32x2{pack2<In16::bf16>(a[0], a[1]), pack2<In16::bf16>(a[2], a[3])}
                                               : u32x2{pack2<In16::fp16>(a[0], a[1]), pack2<In16::fp16>(a[2], a[3])};
                    const int r = wm * (BM / 2) + j * 16 + l16, c = wn * (BN / 2) + i * 16 + kg * 4;
                    *(u32x2*)(smem + r * kPitch + c * 2) = o;
                }
        }
        __syncthreads();
        constexpr int kChunks = BN / 8, kRowsPerPass = kThreads / kChunks; // 16-byte chunks per row
#pragma unroll
        for(int r0 = 0; r0 < BM; r0 += kRowsPerPass)
        {
            const int r = r0 + t / kChunks, c = t % kChunks;
            const int m = m0 + r, n = n0 + c * 8;
            if(m < g.M && n < g.N) // N is a multiple of 8: the chunk is inside the row
                *(u32x4*)(g.out + (size_t)m * g.N + n) = *(const u32x4*)(smem + r * kPitch + c * 16);
        }
        return;
    }

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

    // ---- K split across workgroups: this range's fp32 partial tile goes to the workspace,
    // row-major [split][M][N]; the reduction kernel launched behind this one adds the ranges in
    // order (results never depend on timing) and converts.  A second launch costs a few
    // microseconds but spreads the sum over the whole chip: leaving it to the last workgroup of
    // each tile serialises splits x tile bytes behind one compute unit's loads.
    float* const part = p.partial + (size_t)split * (size_t)g.M * (size_t)g.N;
#pragma unroll
    for(int j = 0; j < TJ; ++j)
#pragma unroll
        for(int i = 0; i < TI; ++i)
        {
            const int m = m0 + wm * (BM / 2) + j * 16 + l16;
            const int n = n0 + wn * (BN / 2) + i * 16 + kg * 4;
            if(m < g.M && n < g.N) // N % 4 == 0 on this path
                store_through(part + (size_t)m * g.N + n, f32x4{acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]});
        }
}

// out[m][n .. n+3] = sum over the K ranges, in range order, of the fp32 partial tiles
template <int SPLITS>
__global__ __launch_bounds__(256) void gemm_mid_reduce_kernel(const float* __restrict__ partial,
                                                              uint16_t* __restrict__ out, uint32_t quads,
                                                              uint32_t splits, int bf16_out)
{
    const uint32_t q = blockIdx.x * 256u + threadIdx.x;
    if(q >= quads)
        return;
    const f32x4* src = (const f32x4*)partial + q;
    f32x4        v[SPLITS];
#pragma unroll
    for(int sp = 0; sp < SPLITS; ++sp)
        v[sp] = src[(size_t)sp * quads];
    f32x4 sum = v[0];
#pragma unroll
    for(int sp = 1; sp < SPLITS; ++sp)
        sum += v[sp];
    for(uint32_t sp = SPLITS; sp < splits; ++sp) // more ranges than the unrolled count
        sum += src[(size_t)sp * quads];
    const u32x2 o = bf16_out ? u32x2{pack2<In16::bf16>(sum[0], sum[1]), pack2<In16::bf16>(sum[2], sum[3])}
                             : u32x2{pack2<In16::fp16>(sum[0], sum[1]), pack2<In16::fp16>(sum[2], sum[3])};
    *((u32x2*)out + q) = o;
}

template <int BM, int BN, bool PAIR = false>
hipError_t launch_shape(MidParams& p, int split_k_log2, int want_splits, const LaunchCtx& ctx)
{
    using S = MidShape<BM, BN, PAIR>;
    const GemmKernelParams& g = p.g;
    p.tiles_m = (g.M + BM - 1) / BM;
    p.tiles_n = (g.N + BN - 1) / BN;
    const int tiles = p.tiles_m * p.tiles_n;

    int splits = 1;
    if(want_splits > 0)
        splits = want_splits;
    else if(split_k_log2 >= 0)
        splits = 1 << split_k_log2;
    if((g.N & 3) != 0 || ((uintptr_t)g.out & 7) != 0) // the reduction works on quads of n
        splits = 1;
    if(splits > g.kblocks)
        splits = g.kblocks;
    // The fp32 partial tiles (ranges x M x N x 4 bytes) stay within kMaxPartialBytes, and the
    // reduction indexes quads of n with 32 bits: a larger request gets fewer ranges.
    const size_t range_bytes = (size_t)g.M * (size_t)g.N * 4;
    if(range_bytes / 16 >= ((size_t)1 << 32))
        splits = 1;
    while(!ctx.static_only && splits > 1 && (size_t)splits * range_bytes > kMaxPartialBytes)
        --splits;
    p.kb_per_split = (g.kblocks + splits - 1) / splits;
    splits         = (g.kblocks + p.kb_per_split - 1) / p.kb_per_split;
    p.splits       = splits;

    const int         device_id = ctx.device_id;
    const hipStream_t stream    = ctx.stream;
    WorkspaceLock     lock(splits > 1); // from the request to the reduction's launch
    if(splits > 1)
    {
        void*      partial = nullptr;
        hipError_t e = workspace_acquire(ctx, lock, WsKind::split_partial, (size_t)splits * range_bytes, false, &partial);
        if(e != hipSuccess)
            return e;
        p.partial = (float*)partial;
    }

    // x_scale in windows of four K blocks: row-major, whole windows, 16-byte aligned rows.  With the weights
    // coming from HBM: 1024 x 2112 x 7168 44.8 -> 39.2 us, 512 x 4608 x 7168 44.9 -> 39.5, 128 x 16384 x 4096
    // 25.9 -> 22.9, 96 x 36864 x 7168 86.6 -> 79.3; loops of 8 to 16 K blocks gain 0 to 5 %.  (With weights
    // that a benchmark loop leaves in the last-level cache a single round of workgroups measures 0 to 7 %
    // slower with windows; that is not the case the kernel is built for.)
    const bool  xs4    = !g.w_shuffled && g.xs_k == 1 && g.xs_m == g.kblocks && (g.kblocks & 3) == 0 &&
                         ((uintptr_t)g.xs & 15) == 0;
    auto        kernel = g.w_shuffled ? gemm_mid_kernel<BM, BN, true, S::kOccupancy, PAIR, false>
                         : xs4        ? gemm_mid_kernel<BM, BN, false, S::kOccupancy, PAIR, true>
                                      : gemm_mid_kernel<BM, BN, false, S::kOccupancy, PAIR, false>;
    const int   smem   = xs4 ? S::kSmemWindows : S::kSmem;
    static std::atomic<bool> raised[3][64]; // dynamic LDS above the default limit needs opting in, once
    const int   which = g.w_shuffled ? 1 : xs4 ? 2 : 0;
    if(device_id >= 0 && device_id < 64 && !raised[which][device_id])
    {
        hipError_t e =
            hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if(e != hipSuccess)
            return e;
        raised[which][device_id] = true;
    }
    hipLaunchKernelGGL(kernel, dim3(tiles * splits), dim3(kThreads), smem, stream, p);
    hipError_t e = hipGetLastError();
    if(e != hipSuccess || splits == 1)
        return e;
    const uint32_t quads = (uint32_t)((size_t)g.M * (size_t)g.N / 4);
    const dim3     rgrid((quads + 255) / 256);
    switch(splits)
    {
    case 2: hipLaunchKernelGGL(gemm_mid_reduce_kernel<2>, rgrid, dim3(256), 0, stream, p.partial, g.out, quads, (uint32_t)splits, p.bf16_out); break;
    case 3: hipLaunchKernelGGL(gemm_mid_reduce_kernel<3>, rgrid, dim3(256), 0, stream, p.partial, g.out, quads, (uint32_t)splits, p.bf16_out); break;
    case 4: hipLaunchKernelGGL(gemm_mid_reduce_kernel<4>, rgrid, dim3(256), 0, stream, p.partial, g.out, quads, (uint32_t)splits, p.bf16_out); break;
    case 5: hipLaunchKernelGGL(gemm_mid_reduce_kernel<5>, rgrid, dim3(256), 0, stream, p.partial, g.out, quads, (uint32_t)splits, p.bf16_out); break;
    case 6: hipLaunchKernelGGL(gemm_mid_reduce_kernel<6>, rgrid, dim3(256), 0, stream, p.partial, g.out, quads, (uint32_t)splits, p.bf16_out); break;
    case 7: hipLaunchKernelGGL(gemm_mid_reduce_kernel<7>, rgrid, dim3(256), 0, stream, p.partial, g.out, quads, (uint32_t)splits, p.bf16_out); break;
    default: hipLaunchKernelGGL(gemm_mid_reduce_kernel<8>, rgrid, dim3(256), 0, stream, p.partial, g.out, quads, (uint32_t)splits, p.bf16_out); break;
    }
    return hipGetLastError();
}

} // namespace

bool gemm_mid_supports(const GemmKernelParams& p)
{
    // 32-bit byte offsets inside the operand matrices
    return p.kblocks >= 1 && (uint64_t)p.N * (uint64_t)p.ldb < (1ull << 32) &&
           (uint64_t)p.M * (uint64_t)p.lda < (1ull << 32) && (uint64_t)p.M * (uint64_t)p.kblocks < (1ull << 30);
}

// Rough duration (us) of one tiling on a 256-CU part, fitted to event timings of every tiling and
// K range count at M = 16 ... 1536 on the DeepSeek-V3 projection shapes and nine more, with the
// weights coming from HBM (9 % off on average; the tiling it picks is 1 % slower than the best one
// on average).  A launch costs a fixed share
// (first wave running, first stage landing: about 2 us from HBM, output stores draining, end of
// kernel) plus an iteration per K block whose cost is set by what a compute unit can pull in
// (about 40 KB/us, so it hardly depends on how many workgroups run).  K ranges beyond the first
// add the partial tiles' write-back and the reduction launch.  Only the order of the candidates
// matters.
struct MidPlan
{
    int   tile, splits;
    float cost;
};
static MidPlan plan_cost(const GemmKernelParams& g, int tile, int splits)
{
    const int   bm = tile == 128 ? 128 : 64, bn = tile == 64 ? 64 : 128;
    const int   occupancy = tile == 64 ? 2 : 1;
    const float fixed     = tile == 64 ? 3.1f : tile == 64128 ? 3.67f : 4.31f;
    const float iter1     = tile == 64 ? 0.f : tile == 64128 ? 0.075f : 0.128f;
    // a single row of tiles (M <= BM): no second workgroup asks for the same weight slab
    const float solo      = tile == 64 ? 0.049f : tile == 64128 ? 0.12f : 0.f;
    const int   tiles_m   = (g.M + bm - 1) / bm;
    const int   tiles     = tiles_m * ((g.N + bn - 1) / bn);
    const int   wgs = tiles * splits, slots = 256 * occupancy;
    // (64x64 with a compute unit per workgroup runs the six-stage ring)
    const float iter0 = tile == 64 ? (wgs <= 256 ? 0.367f : 0.535f) : tile == 64128 ? 0.422f : 0.555f;
    const int   rounds    = (wgs + slots - 1) / slots;
    const float per_cu    = (float)(wgs < slots ? wgs : slots) / 256.f;
    const int   iters     = (g.kblocks + splits - 1) / splits;
    float       iter      = iter0 + (iter1 + (tiles_m == 1 ? solo : 0.f)) * per_cu;
    // row-major weights with long rows: a slab's 128-byte pieces lie further apart (more DRAM pages per K
    // block); 64x128 tiles on (7168, 16384) and (7168, 16256) take 0.8 us per K block where 7168-byte rows take 0.6
    if(!g.w_shuffled && g.ldb > 8192)
        iter *= 1.f + 0.35f * (g.ldb >= 16384 ? 1.f : (float)(g.ldb - 8192) / 8192.f);
    float cost = fixed + (float)rounds * (float)iters * iter + (float)(rounds - 1) * (fixed - 2.4f);
    if(splits > 1)
    {
        // the second launch, and the partial tiles written and read back
        const float launch = tile == 64 ? 2.19f : tile == 64128 ? 1.78f : 1.97f;
        const float rate   = tile == 128 ? 2.92e6f : 2.0e6f; // bytes per us
        cost += launch + (float)splits * (float)g.M * (float)g.N * 4.f / rate;
    }
    return MidPlan{tile, splits, cost};
}
// partial_cap: the most bytes of fp32 partial tiles (ranges x M x N x 4) a plan may use; 0 = no limit
static MidPlan best_plan(const GemmKernelParams& g, int tile, size_t partial_cap = 0)
{
    const int  tiles_to_try[3] = {128, 64128, 64};
    const bool can_split       = (g.N & 3) == 0 && ((uintptr_t)g.out & 7) == 0;
    MidPlan    best{0, 1, 1e30f};
    for(int t : tiles_to_try)
    {
        if(tile != 0 && t != tile)
            continue;
        // (more than eight K ranges never measured best; the model is not fitted beyond)
        const int max_splits = can_split ? (g.kblocks / 4 < 8 ? g.kblocks / 4 : 8) : 1;
        for(int sp = 1; sp <= (max_splits < 1 ? 1 : max_splits); ++sp)
        {
            if(sp > 1 && partial_cap != 0 && (size_t)sp * (size_t)g.M * (size_t)g.N * 4 > partial_cap)
                break;
            const MidPlan c = plan_cost(g, t, sp);
            if(c.cost < best.cost * 0.98f) // ties go to the earlier candidate (fewer ranges)
                best = c;
        }
    }
    return best;
}

float gemm_mid_estimate_us(const GemmKernelParams& g) { return best_plan(g, 0).cost; }

// split_k_log2 < 0: choose.  tile: 0 = choose, else 128 (128x128), 64128 (64x128) or 64 (64x64).
// splits > 0 pins the number of K ranges (any count, not only powers of two).
hipError_t launch_gemm_mid(const GemmKernelParams& g, In16 out_dtype, int split_k_log2, const LaunchCtx& ctx,
                           int tile, int splits)
{
    MidParams p{};
    p.g        = g;
    p.bf16_out = out_dtype == In16::bf16 ? 1 : 0;
    if(tile != 0 && tile != 128 && tile != 64128 && tile != 64)
        return hipErrorInvalidValue;
    if(splits <= 0 && split_k_log2 >= 0)
        splits = 1 << split_k_log2;
    if(tile == 0 || splits <= 0)
    {
        // a caller that may not allocate gets the best plan whose partial tiles fit the fixed buffer
        // (a count of K ranges that the caller named is an error there instead)
        MidPlan plan = splits > 0 ? MidPlan{0, splits, 0.f} : best_plan(g, tile, ctx.static_only ? kStaticPartialBytes : 0);
        if(splits > 0) // ranges pinned, tile free: best tile for that count
        {
            plan.cost = 1e30f;
            for(int t : {128, 64128, 64})
            {
                const MidPlan c = plan_cost(g, t, splits);
                if(c.cost < plan.cost)
                    plan = c;
            }
        }
        tile   = plan.tile;
        splits = plan.splits;
    }
    // 64x64 tiles that leave every workgroup a compute unit of its own: the six-stage ring with
    // K blocks requested in pairs (about 0.06 us per K block faster; with two workgroups per
    // compute unit the four-stage ring wins, and the 64x128 tile gains nothing from pairs)
    if(tile == 64 && ((g.M + 63) / 64) * ((g.N + 63) / 64) * splits <= 256)
        return launch_shape<64, 64, true>(p, -1, splits, ctx);
    switch(tile)
    {
    case 128: return launch_shape<128, 128>(p, -1, splits, ctx);
    case 64128: return launch_shape<64, 128>(p, -1, splits, ctx);
    default: return launch_shape<64, 64>(p, -1, splits, ctx);
    }
}

// "mid_128x128:s=2": the tiling and K range count the automatic choice takes for this problem
void gemm_mid_describe(const GemmKernelParams& g, char* buf, size_t n)
{
    const MidPlan pl = best_plan(g, 0);
    snprintf(buf, n, "%s:s=%d", pl.tile == 128 ? "mid_128x128" : pl.tile == 64128 ? "mid_64x128" : "mid_64x64",
             pl.splits);
}

} // namespace fp8bs
