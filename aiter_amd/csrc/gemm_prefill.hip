// Prefill-shape block-scale FP8 GEMM (large M): MFMA-bound.
//
// 256 (m) x 256 (n) output tile per workgroup, one 128-wide K block per step, 8 waves laid out
// 2 (n) x 4 (m) so that each wave owns 128 n x 64 m = 8 x 4 MFMA tiles (128 fp32 accumulators
// per lane).  Both operand slabs are brought in with direct global->LDS loads
// (global_load_lds_dwordx4: no VGPR staging, no ds_write) into a two-stage ring, so the loads of
// K block kb+1 fly while block kb is multiplied.  Per K block every 16x16 tile costs one
// v_mfma_f32_16x16x128_f8f6f4 (32 cycles) plus 4 fp32 FMAs that fold the unscaled product into
// the accumulators with the scale xs[m,kb]*ws[n/128,kb].
//
// Workgroups are renumbered so that the 32 tiles resident on one XCD at a time form a compact
// 8 (m) x 4 (n) patch: each XCD's L2 then serves every operand slab to several CUs.
#include "gemm_common.h"

#include <atomic>
#include <algorithm>

namespace fp8bs {

namespace {

constexpr int kBM = 256, kThreads = 512;
constexpr int kStages = 2;
constexpr int kGroupN = 4; // n tiles swept together by consecutive workgroups
// The tile is 256 (m) x NW * 32 (n): NW = 8 weight fragments per wave for the 256 x 256 tile, 4 for the
// 256 x 128 one (twice the workgroups where the wide tiles leave compute units idle), 6 for the
// 256 x 192 one (N = 2112 = 11 x 192: no ragged last column of tiles).
constexpr int tile_n(int nw) { return nw * 32; }
constexpr int slab_bytes(int nw) { return (kBM + tile_n(nw)) * 128; } // weight rows, then 256 activation rows
constexpr int stage_bytes(int nw) { return slab_bytes(nw) + kBM * 4; } // + this K block's x_scale for the 256 rows
constexpr uint32_t epi_pitch(int nw) { return (uint32_t)nw * 32u + 16u; } // bytes per row of a wave's 64 x NW*16 output block in LDS
// Row-major x_scale ([M][K/128]): a lane's scale of one K block is 4 bytes of a line that holds 32 K
// blocks of its row, and a wave's load of 64 such scales touches 64 lines.  Fetched per K block these
// loads are a third of all line requests of the kernel for 1.5 % of its bytes (8192 x 36864 x 7168:
// 1865 us, against 1775 us with the same scales stored column-major).  Where the rows allow 16-byte
// loads the scales therefore come four K blocks at a time: a quarter of the requests, into two
// windows of 16 bytes per row behind the stages.
constexpr int kWindowBytes = kBM * 16;

// 16-byte chunk c of stage row r is stored at chunk c ^ lds_swizzle(r): every group of 16 lanes
// that the LDS serves together in a fragment read then falls on 16 different 16-byte bank groups.
__device__ __forceinline__ uint32_t swz(uint32_t row, uint32_t chunk) { return lds_off(row, chunk); }

__device__ __forceinline__ i32x8 read_frag(const uint8_t* base, uint32_t row, uint32_t kg)
{
    i32x4 lo = *(const i32x4*)(base + swz(row, 2 * kg));
    i32x4 hi = *(const i32x4*)(base + swz(row, 2 * kg + 1));
    return i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

// SHUF: weights pre-shuffled (16,16).  A 16-row tile's K block is then 2 KiB of contiguous global
// memory already in fragment order; the weight slab in LDS is a straight copy of it (tile after
// tile), and a lane's fragment halves sit at kg*512 + l16*16 and 256 bytes further.
// XS4: x_scale is row-major with 16-byte aligned rows and comes in windows of four K blocks.
template <In16 DT, bool SHUF, int NW, bool XS4>
__global__ __launch_bounds__(kThreads) void gemm_prefill_kernel(GemmKernelParams p, int tiles_m,
                                                                int tiles_n, int splits,
                                                                int kb_per_split, float* partial,
                                                                uint32_t partial_bytes,
                                                                uint32_t* tickets)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    constexpr int      kBN = tile_n(NW), kSlabBytes = slab_bytes(NW), kStageBytes = stage_bytes(NW);
    constexpr uint32_t kEpiPitch = epi_pitch(NW);
    constexpr int      kLoads    = (kBM + kBN) / 64; // slab loads per wave and stage: 8 rows each, weights first
    constexpr int      kWLoads   = kBN / 64;
    constexpr uint32_t kWindows  = (uint32_t)(kStages * kStageBytes); // the two x_scale windows (XS4)

    typedef const volatile i32x4 __attribute__((address_space(3)))* lds_vec_ptr;
    typedef uint8_t __attribute__((address_space(3)))*              lds_byte_ptr;
    const lds_byte_ptr smem3 = (lds_byte_ptr)smem;

    // The workgroup walks tiles blockIdx.x, blockIdx.x + gridDim.x, ... (one workgroup per compute
    // unit when there are more tiles than compute units): a tile's output stores drain, and the
    // next tile's first slabs arrive, behind one wait instead of a workgroup's end and start.
    // With fewer tiles than compute units the K blocks of a tile are shared out over `splits`
    // workgroups (item = split * tiles + tile); see the epilogue for how their sums meet.
    const int total = tiles_m * tiles_n;
    __shared__ uint32_t s_ticket;
    for(int item = blockIdx.x; item < total * splits; item += gridDim.x)
    {
    const int split = item / total, tile = item - split * total;
    const int kb_lo = split * kb_per_split, kb_hi = min(p.kblocks, kb_lo + kb_per_split);
    // Everything derived from the lane index is derived again for every tile (the empty asm
    // hides that it is the same value): kept live across the K loop it would not fit the registers.
    int t = threadIdx.x;
    asm volatile("" : "+v"(t));
    const int lane = t & 63, wave = t >> 6;
    const int l16 = lane & 15, kg = lane >> 4;
    const int wn = wave & 1, wm = wave >> 1; // n half (NW * 16 rows), m quarter (64 rows)

    // ---- tile choice: XCD-aware renumbering, then n-groups swept m-fastest
    int       v     = tile;
    if((total & 7) == 0)
        v = (v & 7) * (total >> 3) + (v >> 3); // workgroups go round-robin over the 8 XCDs
    const int group  = v / (kGroupN * tiles_m);
    const int within = v - group * (kGroupN * tiles_m);
    const int gn     = min(kGroupN, tiles_n - group * kGroupN);
    const int tm     = within / gn;
    const int tn     = group * kGroupN + (within - tm * gn);
    const int m0 = tm * kBM, n0 = tn * kBN;

    // ---- global -> LDS plan: per stage 8 * kLoads units of 8 rows (1 KiB); wave w moves units i*8+w.
    // Lane p of a unit fills LDS chunk p, i.e. stage row 8u + p/8, stored chunk p%8, which must
    // hold the row's logical chunk (p%8) ^ lds_swizzle(row).
    uint32_t goff[kLoads];
#pragma unroll
    for(int i = 0; i < kLoads; ++i)
    {
        const uint32_t r = 64u * i + 8u * wave + (lane >> 3);
        const uint32_t c = (lane & 7u) ^ lds_swizzle(r);
        if(i < kWLoads && SHUF)
        {
            // unit U = 8 i + wave is half of tile U/2's K block: 1 KiB, copied as it lies
            const uint32_t U    = 8u * i + wave;
            uint32_t       tile = ((uint32_t)n0 >> 4) + (U >> 1);
            tile                = min(tile, ((uint32_t)p.N >> 4) - 1u);
            goff[i]             = tile * 16u * (uint32_t)p.K + (U & 1u) * 1024u + (uint32_t)lane * 16u;
        }
        else if(i < kWLoads)
        {
            uint32_t n = n0 + r;
            n          = n < (uint32_t)p.N ? n : (uint32_t)p.N - 1;
            goff[i]    = n * (uint32_t)p.ldb + c * 16u;
        }
        else
        {
            uint32_t m = m0 + (r - (uint32_t)kBN);
            m          = m < (uint32_t)p.M ? m : (uint32_t)p.M - 1;
            goff[i]    = m * (uint32_t)p.lda + c * 16u;
        }
    }
    // One LDS-direct load (global_load_lds_dwordx4): lane p's 16 bytes land at M0 + 16 p.
    // Written as asm on purpose: the compiler models the builtin as a flat access that may touch
    // LDS and from then on waits for every outstanding LDS read in full.  The loads are not
    // visible to the compiler's wait-count bookkeeping, so every consumer sits behind an
    // explicit s_waitcnt vmcnt(0) and a workgroup barrier.
    auto dma16 = [](uint32_t lds_dst, uint32_t voff, const uint8_t* sbase) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(lds_dst), "v"(voff), "s"(sbase)
                     : "memory");
    };

    // x_scale of K block kb for the tile's 256 rows: one 4-byte LDS-direct load per 64 rows
    // (waves 0..3), lane l -> row 64 w + l, landing behind the operand slabs of the stage.
    auto dma4 = [](uint32_t lds_dst, uint32_t voff, const void* sbase) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                     :
                     : "s"(lds_dst), "v"(voff), "s"(sbase)
                     : "memory");
    };
    uint32_t xs_goff; // byte offset of this lane's x_scale row (waves 0..3 only)
    {
        uint32_t m = m0 + 64u * (wave & 3) + lane;
        m          = m < (uint32_t)p.M ? m : (uint32_t)p.M - 1;
        xs_goff    = m * (uint32_t)p.xs_m * 4u;
    }

    // ---- scales: x_scale comes through LDS with each stage, w_scale: one block per wave, or (six
    // fragments: a wave's 96 columns can straddle a block boundary) two, the second from fragment
    // `ws_split` on.  Fragments share a scale in pairs: group g = fragment / 2.
    constexpr int  kScaleGroups = NW == 6 ? 3 : 1;
    const uint32_t n_wave  = (uint32_t)(n0 + wn * (NW * 16));
    const uint32_t nb_last = (uint32_t)((p.N + 127) / 128 - 1);
    const uint32_t nb      = min(n_wave >> 7, nb_last);
    const float* ws_row  = p.ws + (size_t)nb * p.kblocks;
    const float* ws_row2 = p.ws + (size_t)min(nb + 1u, nb_last) * p.kblocks;
    const int    ws_split = __builtin_amdgcn_readfirstlane((int)((128u - (n_wave & 127u)) >> 4)); // 8, 6, 4 or 2

    // ---- LDS read addresses.  A fragment is 32 bytes of one row: logical chunks 2kg and 2kg+1.
    // Tile rows start at multiples of 16, so the swizzle term depends on l16 only and every
    // tile is reached with an immediate offset from these four per-lane bases.
    const uint32_t sw     = lds_swizzle((uint32_t)l16);
    const uint32_t lo_off = (uint32_t)l16 * 128u + (((2u * kg) ^ sw) << 4);
    const uint32_t hi_off = (uint32_t)l16 * 128u + (((2u * kg + 1u) ^ sw) << 4);
    const uint32_t wlo_off = SHUF ? (uint32_t)kg * 512u + (uint32_t)l16 * 16u : lo_off;
    const uint32_t whi_off = SHUF ? wlo_off + 256u : hi_off;
    const uint32_t w_base = (uint32_t)wn * ((uint32_t)(NW * 16) * 128u);
    const uint32_t x_base = (uint32_t)kBN * 128u + (uint32_t)wm * (64u * 128u);

    float acc[NW][4][4];
#pragma unroll
    for(int i = 0; i < NW; ++i)
#pragma unroll
        for(int j = 0; j < 4; ++j)
#pragma unroll
            for(int r = 0; r < 4; ++r)
                acc[i][j][r] = 0.f;

    // The K loop is written as an explicit instruction stream.  Every 16x16 tile costs one MFMA
    // (32 cycles in the matrix pipe) and 4 FMAs that fold its unscaled product into the
    // accumulators.  To keep the matrix pipe fed from a single wave, the FMAs of tile t-2 are
    // issued behind the MFMA of tile t: by then the older product has been written back, so no
    // wait states are needed, and the in-order issue never parks on a result that is still in
    // flight.  Products rotate through four register quads; the last two tiles of a K block are
    // folded in after the first two MFMAs of the next one.  `asm volatile` keeps this order; the
    // LDS reads are volatile loads so they stay where they are written (ahead of their use) while
    // the compiler still derives their wait counts.
#define FP8BS_MFMA(P, A, B) \
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0" : "=&v"(P) : "v"(A), "v"(B))
#define FP8BS_FMA4(ACC, P, S)                                                              \
    do                                                                                     \
    {                                                                                      \
        asm volatile("v_fmac_f32 %0, %1, %2" : "+v"((ACC)[0]) : "v"((P)[0]), "v"(S));      \
        asm volatile("v_fmac_f32 %0, %1, %2" : "+v"((ACC)[1]) : "v"((P)[1]), "v"(S));      \
        asm volatile("v_fmac_f32 %0, %1, %2" : "+v"((ACC)[2]) : "v"((P)[2]), "v"(S));      \
        asm volatile("v_fmac_f32 %0, %1, %2" : "+v"((ACC)[3]) : "v"((P)[3]), "v"(S));      \
    } while(0)

    auto read_frag_w = [&](uint32_t stage_off, uint32_t tile_off) -> i32x8 {
        const i32x4 lo = *(lds_vec_ptr)(smem3 + stage_off + wlo_off + tile_off);
        const i32x4 hi = *(lds_vec_ptr)(smem3 + stage_off + whi_off + tile_off);
        return i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };
    auto read_frag_v = [&](uint32_t stage_off, uint32_t tile_off) -> i32x8 {
        const i32x4 lo = *(lds_vec_ptr)(smem3 + stage_off + lo_off + tile_off);
        const i32x4 hi = *(lds_vec_ptr)(smem3 + stage_off + hi_off + tile_off);
        return i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };

    // w_scale of this wave's n block for 64 consecutive K blocks lives in one VGPR (lane = K
    // block) and is picked with v_readlane: a scalar load inside the loop would share the LGKM
    // counter with the LDS reads and force them to be waited for in full.
    auto load_ws_window = [&](const float* row, int kb0) -> float {
        const int k = kb0 + lane;
        return row[k < p.kblocks ? k : p.kblocks - 1];
    };
    float ws_vec  = load_ws_window(ws_row, kb_lo & ~63);
    float ws_vec2 = kScaleGroups > 1 ? load_ws_window(ws_row2, kb_lo & ~63) : 0.f;
    auto  ws_at   = [&](float vec, int kb) -> float {
        return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(vec), kb & 63));
    };

    {
        const uint32_t dst0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(smem3 + wave * 1024));
#pragma unroll
        for(int i = 0; i < kLoads; ++i)
            dma16(dst0 + i * 8192, goff[i],
                  i < kWLoads ? p.wq + (size_t)kb_lo * (SHUF ? 2048 : 128) : p.xq + (size_t)kb_lo * 128);
        if(wave < 4 && XS4) // the window that holds K block kb_lo: lane l's 16 bytes are row 64 w + l's
            dma16(__builtin_amdgcn_readfirstlane(
                      (uint32_t)(uintptr_t)(smem3 + kWindows + ((kb_lo >> 2) & 1) * kWindowBytes + wave * 1024)),
                  xs_goff + (uint32_t)(kb_lo & ~3) * 4u, (const uint8_t*)p.xs);
        else if(wave < 4)
            dma4(__builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(smem3 + kSlabBytes + wave * 256)),
                 xs_goff + (uint32_t)kb_lo * (uint32_t)p.xs_k * 4u, p.xs);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): this wave's LDS-direct loads have landed
    __syncthreads();
    // LDS address of this lane's x_scale for m tile 0 (tile j sits 64 bytes further)
    // (XS4: of this lane's row in window 0, K block 0 of the window; tile j sits 256 bytes further)
    const uint32_t xs_lds = XS4 ? kWindows + ((uint32_t)wm * 64u + (uint32_t)l16) * 16u
                                : (uint32_t)kSlabBytes + ((uint32_t)wm * 64u + (uint32_t)l16) * 4u;

    // ---- the K loop, skewed by a quarter of a K block.
    // Issue order of one iteration (4 NW MFMA slots; the numbers are those of NW = 8):
    //   slots 0..7   the last 8 tiles (weight fragments NW - 2 and NW - 1) of the PREVIOUS K block, whose
    //                operands are already in registers.  They keep the matrix pipe busy while
    //                the first fragments of this K block travel from LDS, which would otherwise
    //                be dead time right after the barrier (every wave reads at once).
    //   slots 8..31  tiles of weight fragments 0..5 of this K block.
    // The FMAs that fold a product into the accumulators trail their MFMA by two slots (the
    // product is written back by then: no wait states), also across the iteration boundary.
    // Registers: weight fragments rotate through 4 buffers (fragment i lives in buffer i & 3,
    // so 6 and 7 of one K block and 0 and 1 of the next never collide); an activation fragment
    // is replaced by the next K block's as soon as its two deferred tiles have been issued.
    f32x4 P[4];
#pragma unroll
    for(int q = 0; q < 4; ++q)
        P[q] = f32x4{0.f, 0.f, 0.f, 0.f};
    // weight fragment i lives in buffer BUF(i): four buffers in rotation, or one per fragment
    constexpr int kBufs = NW == 6 ? 6 : 4;
#define FP8BS_BUF(i) (NW == 6 ? (i) : ((i)&3))
    i32x8 bx[4], aw[kBufs];
#pragma unroll
    for(int q = 0; q < 4; ++q) // first iteration: the "previous K block" is all zero codes with zero scales
        bx[q] = i32x8{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for(int q = 0; q < kBufs; ++q)
        aw[q] = i32x8{0, 0, 0, 0, 0, 0, 0, 0};
    // x_scale * w_scale of the previous K block, per scale group and m tile
    float scp[kScaleGroups][4];
#pragma unroll
    for(int g = 0; g < kScaleGroups; ++g)
#pragma unroll
        for(int j = 0; j < 4; ++j)
            scp[g][j] = 0.f;
#define FP8BS_GROUP(i) (NW == 6 ? (i) >> 1 : 0)
    // The zero fragments must sit in their registers before the first MFMA reads them: a vector
    // move followed at once by a matrix instruction that reads its result needs wait states, and
    // nothing inserts them around inline asm (a stale register read as fp8 codes can hold NaN
    // codes, and NaN x the zero scale stays NaN).  Opaque to the compiler, so that it cannot
    // re-create the zeros right in front of the first MFMA.
#pragma unroll
    for(int q = 0; q < 4; ++q)
        asm volatile("" : "+v"(bx[q]));
#pragma unroll
    for(int q = 0; q < kBufs; ++q)
        asm volatile("" : "+v"(aw[q]));
    asm volatile("s_nop 7" ::: "memory");

    typedef const volatile float __attribute__((address_space(3)))* lds_f32_ptr;

    // XS4: where this lane's x_scale of K block kb lies (window (kb / 4) & 1, block kb & 3 of its row).  The
    // address of the next K block is worked out in the middle of the multiply stream, not between the barrier
    // and the first reads of the next iteration.
    auto xs_window_addr = [&](int kb) -> uint32_t {
        return (uint32_t)(((kb >> 2) & 1) * kWindowBytes + (kb & 3) * 4) + xs_lds;
    };
    uint32_t xs_addr = XS4 ? xs_window_addr(kb_lo) : 0u;

    for(int kb = kb_lo; kb < kb_hi; ++kb)
    {
        const int      cur      = (kb - kb_lo) & 1;
        const uint32_t stage    = (uint32_t)cur * kStageBytes;
        const int      kn       = kb + 1 < kb_hi ? kb + 1 : kb; // last pass re-fetches, unused
        const uint32_t dma_dst  = __builtin_amdgcn_readfirstlane(
            (uint32_t)(uintptr_t)(smem3 + (cur ^ 1) * kStageBytes + wave * 1024));
        const size_t   dma_koff   = (size_t)kn * 128;
        const size_t   dma_koff_w = SHUF ? (size_t)kn * 2048 : dma_koff;

        if((kb & 63) == 0 && kb != kb_lo)
        {
            ws_vec = load_ws_window(ws_row, kb);
            if(kScaleGroups > 1)
                ws_vec2 = load_ws_window(ws_row2, kb);
        }
        float wsc[kScaleGroups];
        wsc[0] = ws_at(ws_vec, kb);
        if constexpr(kScaleGroups > 1)
        {
            const float second = ws_at(ws_vec2, kb);
            wsc[1]             = ws_split <= 2 ? second : wsc[0]; // fragments 2, 3
            wsc[2]             = ws_split <= 4 ? second : wsc[0]; // fragments 4, 5
        }

        aw[0] = read_frag_w(stage, w_base); // weight fragment 0 of this K block
        float sc[kScaleGroups][4];
#pragma unroll
        for(int j = 0; j < 4; ++j)
        {
            const float xsv = XS4 ? *(lds_f32_ptr)(smem3 + xs_addr + j * 256)
                                  : *(lds_f32_ptr)(smem3 + stage + xs_lds + j * 64);
#pragma unroll
            for(int g = 0; g < kScaleGroups; ++g)
                sc[g][j] = xsv * wsc[g];
        }

#pragma unroll
        for(int q = 0; q < 4 * NW; ++q)
        {
            if(q == 2)
                aw[1] = read_frag_w(stage, w_base + 1 * 2048);

            if(q < 8) // deferred tile (NW - 2 + (q & 1), q >> 1) of the previous K block
                FP8BS_MFMA(P[q & 3], aw[FP8BS_BUF(NW - 2 + (q & 1))], bx[q >> 1]);
            else      // tile ((q - 8) >> 2, (q - 8) & 3) of this K block
                FP8BS_MFMA(P[q & 3], aw[FP8BS_BUF((q - 8) >> 2)], bx[(q - 8) & 3]);

            // LDS reads that the slot just issued has made room for
            if(q < 8 && (q & 1))
                bx[q >> 1] = read_frag_v(stage, x_base + (q >> 1) * 2048);
            if(q == 6)
                aw[2] = read_frag_w(stage, w_base + 2 * 2048);
            if(q == 7)
                aw[3] = read_frag_w(stage, w_base + 3 * 2048);
            if(q >= 11 && ((q - 11) & 3) == 0 && 4 + ((q - 11) >> 2) < NW) // fragments 4 .. NW - 1 at slots 11, 15, 19, 23
                aw[FP8BS_BUF(4 + ((q - 11) >> 2))] = read_frag_w(stage, w_base + (4 + ((q - 11) >> 2)) * 2048);

            // next stage: the slab loads and the x_scale column, in the first half of the slots
            if((q & 1) == 1 && q < 2 * kLoads)
            {
                const int u = q >> 1;
                dma16(dma_dst + u * 8192, goff[u], u < kWLoads ? p.wq + dma_koff_w : p.xq + dma_koff);
            }
            if(q == 2 * kLoads && wave < 4)
            {
                if constexpr(XS4)
                {
                    // the next K block opens a window: into the one that was last read four K blocks ago
                    if((kn & 3) == 0 && kn != kb)
                        dma16(__builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(
                                  smem3 + kWindows + ((kn >> 2) & 1) * kWindowBytes + wave * 1024)),
                              xs_goff + (uint32_t)kn * 4u, (const uint8_t*)p.xs);
                }
                else
                    dma4(__builtin_amdgcn_readfirstlane(dma_dst - wave * 1024 + kSlabBytes + wave * 256),
                         xs_goff + (uint32_t)kn * (uint32_t)p.xs_k * 4u, p.xs);
            }

            if(XS4 && q == 2 * NW)
            {
                xs_addr = xs_window_addr(kb + 1);
                asm volatile("" : "+v"(xs_addr)); // here, between two slots
            }

            // fold in the product issued two slots ago
            if(q == 0)
                FP8BS_FMA4(acc[NW - 3][2], P[2], scp[FP8BS_GROUP(NW - 3)][2]);
            else if(q == 1)
                FP8BS_FMA4(acc[NW - 3][3], P[3], scp[FP8BS_GROUP(NW - 3)][3]);
            else if(q < 10)
                FP8BS_FMA4(acc[NW - 2 + ((q - 2) & 1)][(q - 2) >> 1], P[(q - 2) & 3],
                           scp[FP8BS_GROUP(NW - 2)][(q - 2) >> 1]);
            else
                FP8BS_FMA4(acc[(q - 10) >> 2][(q - 10) & 3], P[(q - 2) & 3],
                           sc[FP8BS_GROUP((q - 10) >> 2)][(q - 10) & 3]);
        }
#pragma unroll
        for(int g = 0; g < kScaleGroups; ++g)
#pragma unroll
            for(int j = 0; j < 4; ++j)
                scp[g][j] = sc[g][j];

        // vmcnt(0): this wave's share of the next stage is in LDS; the barrier (which also
        // waits for this wave's outstanding LDS reads) publishes it and retires the stage just read
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
    }
    // tail: the 8 deferred tiles of the last K block, then drain the two products in flight
#pragma unroll
    for(int q = 0; q < 8; ++q)
    {
        FP8BS_MFMA(P[q & 3], aw[FP8BS_BUF(NW - 2 + (q & 1))], bx[q >> 1]);
        if(q == 0)
            FP8BS_FMA4(acc[NW - 3][2], P[2], scp[FP8BS_GROUP(NW - 3)][2]);
        else if(q == 1)
            FP8BS_FMA4(acc[NW - 3][3], P[3], scp[FP8BS_GROUP(NW - 3)][3]);
        else
            FP8BS_FMA4(acc[NW - 2 + ((q - 2) & 1)][(q - 2) >> 1], P[(q - 2) & 3],
                       scp[FP8BS_GROUP(NW - 2)][(q - 2) >> 1]);
    }
    asm volatile("s_nop 15\n s_nop 15\n s_nop 15" ::: "memory"); // >= 11 wait states after the last MFMA
    FP8BS_FMA4(acc[NW - 2][3], P[2], scp[FP8BS_GROUP(NW - 2)][3]);
    FP8BS_FMA4(acc[NW - 1][3], P[3], scp[FP8BS_GROUP(NW - 1)][3]);
#undef FP8BS_MFMA
#undef FP8BS_FMA4
#undef FP8BS_BUF
#undef FP8BS_GROUP

    // ---- K shared out over workgroups: every workgroup parks its fp32 accumulators in the
    // workspace exactly as its lanes hold them (item slot x 4 NW MFMA tiles x 512 lanes x 16 bytes:
    // every store and load is 1 KiB contiguous per wave), takes a ticket, and the one that draws
    // the last ticket of the tile adds the slots in split order (so the result does not depend on
    // who came last) and carries on into the ordinary epilogue.  The workgroups of a tile run on
    // different XCDs, whose L2 caches are not coherent with each other: the parked tiles are
    // written and read past them (sc1), and the stores are waited for before the ticket is taken.
    bool writes_out = true;
    if(splits > 1)
    {
        const __amdgpu_buffer_rsrc_t rsrc =
            __builtin_amdgcn_make_buffer_rsrc(partial, 0, (int)partial_bytes, 0x00020000);
        constexpr int kCoherent = 16;
        constexpr uint32_t kTilesPerWave = 4u * NW;
        const uint32_t mine     = ((uint32_t)(tile * splits + split) * kTilesPerWave * 512u + (uint32_t)t) * 16u;
#pragma unroll
        for(int i = 0; i < NW; ++i)
#pragma unroll
            for(int j = 0; j < 4; ++j)
                __builtin_amdgcn_raw_buffer_store_b128(
                    __builtin_bit_cast(u32x4, f32x4{acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]}),
                    rsrc, mine + (uint32_t)(i * 4 + j) * (512u * 16u), 0, kCoherent);
        __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): the stores above have reached memory
        __syncthreads();
        if(t == 0)
            s_ticket = __hip_atomic_fetch_add(tickets + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        writes_out = s_ticket == (uint32_t)splits - 1u;
        if(writes_out)
        {
            if(t == 0) // leave the ticket ready for the next launch
                __hip_atomic_store(tickets + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for(int i = 0; i < NW; ++i)
#pragma unroll
                for(int j = 0; j < 4; ++j)
                {
                    // 0 + p0 + p1 + ... whoever is last; its own term comes from its registers
                    // (the same bits it parked), the others from the workspace
                    const f32x4 own = f32x4{acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
                    f32x4       sum = f32x4{0.f, 0.f, 0.f, 0.f};
                    for(int sp = 0; sp < splits; ++sp)
                    {
                        const uint32_t off =
                            ((uint32_t)(tile * splits + sp) * kTilesPerWave * 512u + (uint32_t)t) * 16u +
                            (uint32_t)(i * 4 + j) * (512u * 16u);
                        if(sp == split) // uniform
                            sum += own;
                        else
                            sum += __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, kCoherent));
                    }
#pragma unroll
                    for(int r = 0; r < 4; ++r)
                        acc[i][j][r] = sum[r];
                }
        }
    }

    // ---- epilogue.  A lane owns out[m][n .. n+3] for each of its NW x 4 tiles: stored from there,
    // one instruction would touch 16 rows with 32 bytes each.  The wave's 64 x NW*16 block goes
    // through its own LDS region instead (the stage buffers are free after the loop's last
    // barrier; rows padded by 16 bytes so the 16 rows of one write fall on different banks) and
    // leaves as 16-byte stores, 2 NW lanes per row piece (256 or 128 bytes), 4 or 8 rows per
    // instruction.  LDS operations of one wave complete in order, so no barrier stands between
    // write and read.
    if(writes_out) // uniform
    {
        const uint32_t ebase = (uint32_t)wave * (64u * kEpiPitch);
        typedef u32x2 __attribute__((address_space(3)))*       lds_u2_ptr;
        typedef const u32x4 __attribute__((address_space(3)))* lds_u4_ptr;
#pragma unroll
        for(int j = 0; j < 4; ++j)
#pragma unroll
            for(int i = 0; i < NW; ++i)
                *(lds_u2_ptr)(smem3 + ebase + (uint32_t)(j * 16 + l16) * kEpiPitch +
                              (uint32_t)(i * 16 + kg * 4) * 2u) =
                    u32x2{pack2<DT>(acc[i][j][0], acc[i][j][1]), pack2<DT>(acc[i][j][2], acc[i][j][3])};

        constexpr int kRowLanes = 2 * NW;          // lanes that store one row piece
        constexpr int kRowsPer  = 64 / kRowLanes;  // rows per store instruction (lanes beyond them idle)
        const int  rl     = lane / kRowLanes;
        const int  col    = (lane - rl * kRowLanes) * 8;
        const int  n      = n0 + wn * (NW * 16) + col;
        const bool vec_ok = (p.N & 7) == 0 && ((uintptr_t)p.out & 15) == 0 && n + 8 <= p.N;
#pragma unroll
        for(int c = 0; c < (64 + kRowsPer - 1) / kRowsPer; ++c)
        {
            const int row = c * kRowsPer + rl;
            if(rl >= kRowsPer || row >= 64)
                continue;
            const int   m   = m0 + wm * 64 + row;
            const u32x4 vv  = *(lds_u4_ptr)(smem3 + ebase + (uint32_t)row * kEpiPitch + (uint32_t)col * 2u);
            if(m >= p.M)
                continue;
            uint16_t* dst = p.out + (size_t)m * p.N + n;
            if(vec_ok)
            {
                *(u32x4*)dst = vv;
            }
            else
            {
#pragma unroll
                for(int r = 0; r < 8; ++r)
                    if(n + r < p.N)
                        dst[r] = (uint16_t)((vv[r >> 1] >> ((r & 1) * 16)) & 0xffffu);
            }
        }
    }
    // the next tile's first slabs must not land in LDS while another wave still reads its block
    __syncthreads();
    } // items of this workgroup
}

} // namespace

bool gemm_prefill_supports(const GemmKernelParams& p)
{
    // 32-bit byte offsets inside the operand matrices, 8-byte aligned output rows
    return p.kblocks >= 1 && (uint64_t)p.N * (uint64_t)p.ldb < (1ull << 32) &&
           (uint64_t)p.M * (uint64_t)p.lda < (1ull << 32) &&
           (uint64_t)p.M * (uint64_t)p.kblocks < (1ull << 30) && (p.N % 4) == 0;
}

// Duration model (us) on `cus` compute units, fitted to event timings with weights from HBM:
// a round of workgroups costs 8 us (first slabs, output tile) plus, per K block, 1.36 us while
// the workgroups of a round cover up to 44 % of the compute units, rising to 1.79 us from 62 % on
// (8192 x 36864 x 7168: 18 rounds x (8 + 56 x 1.79) = 1948 us, measured 1950; 2048 x 4608 x 7168,
// 144 workgroups: 100 us; 1536 x 7168 x 2048, 168 workgroups: 36 us).  K
// ranges over s workgroups per tile cost 4 us plus the parked tiles' traffic, (2 s - 1) x 256 KiB
// per tile at about 5 TB/s (2048 x 4096 x 7168: 89.8 us as one range, 77-80 us as two).
// 256 x 128 tiles: 6 us per round and 1.2 us per K block, rising to 1.4 us when the workgroups of a round
// cover all compute units (a compute unit takes in its 48 KiB per K block no faster than the wide
// tile's 64 KiB: what the narrow tile buys is workgroups, not speed; 1024 x 7168 x 2048: 26.4 us
// against 34.4, 256 x 24576 x 1536: 22.5 against 30.9, 2048 x 4096 x 7168: 84.0 against 78.8 with
// the wide tile's K ranges).
constexpr float kFixed128 = 6.f, kIter128 = 1.2f;

static float plan_cost(const GemmKernelParams& p, int cus, int bn, int s)
{
    const int   tiles  = ((p.M + kBM - 1) / kBM) * ((p.N + bn - 1) / bn);
    const int   items  = tiles * s;
    const int   rounds = (items + cus - 1) / cus;
    const float share  = (float)items / (float)(rounds * cus);
    const int   kb     = (p.kblocks + s - 1) / s;
    if(bn == 128)
        return (float)rounds * (kFixed128 + (float)kb * (kIter128 + (share > 0.44f ? (share - 0.44f) * 0.35f : 0.f)));
    if(bn == 192) // 56 KiB and 24 MFMA slots per K block: 1.4 us (4096 x 2112 x 7168, 176 workgroups: 86.9 us;
                  // 2048 x 2112 x 7168 as 88 tiles x 2 K ranges: 60.3 us against 73.1 with the wide tile),
                  // 1.5 us with a workgroup on every compute unit (8192 x 1536 x 7168, 256 tiles: 93 us)
        return (float)rounds * (7.f + (float)kb * (1.4f + (share > 0.75f ? (share - 0.75f) * 0.4f : 0.f))) +
               (s > 1 ? 4.f + (float)tiles * (float)(2 * s - 1) * 0.0375f : 0.f);
    const float iter = std::min(1.79f, 1.36f + (share > 0.44f ? (share - 0.44f) * 2.4f : 0.f));
    return (float)rounds * (8.f + (float)kb * iter) +
           (s > 1 ? 4.f + (float)tiles * (float)(2 * s - 1) * 0.05f : 0.f);
}

PrefillPlan gemm_prefill_plan(const GemmKernelParams& p, int cus)
{
    const int tiles = ((p.M + kBM - 1) / kBM) * ((p.N + 255) / 256);
    cus             = std::max(cus, 1);
    PrefillPlan best{1, plan_cost(p, cus, 256, 1), 256};
    for(int s = 2; s <= 3; ++s)
    {
        // (below 64 tiles the model is off: 1024 x 2112 x 7168, 36 tiles x 3, takes 67 us where it
        // says 47, and the mid_* kernels need 51)
        if(tiles < 64 || tiles * s > cus || p.kblocks / s < 8 || (p.N & 3) != 0)
            break;
        const float c = plan_cost(p, cus, 256, s);
        if(c < best.us * 0.97f)
            best = PrefillPlan{s, c, 256};
    }
    // half-width tiles where the wide ones leave at least half of the compute units without a workgroup
    if(tiles * 2 <= cus)
    {
        const float c = plan_cost(p, cus, 128, 1);
        if(c < best.us * 0.97f)
            best = PrefillPlan{1, c, 128};
    }
    // 192-wide tiles: no ragged last column where they divide N and 256 does not (N = 2112: a
    // ninth column of tiles that is three quarters empty against eleven full ones), and often a better
    // fit of whole rounds (1024 x 24576 x 1536: 512 tiles in two full rounds, 48 us,
    // against 384 wide ones in one and a half, 59 us; 512 x 24576 x 1536: 26 us against 32;
    // 2048 x 4608 x 7168: 192 tiles, 88 us, against 144 wide ones, 100 us; 1536 x 7168 x 2048: 228
    // tiles, the last column a third full, 30 us against 36).  At most two K ranges:
    // three (2048 x 1536 x 7168, 64 tiles) take 53 us where the model says 50 and mid_128x128 needs 49.
    {
        const int t192 = ((p.M + kBM - 1) / kBM) * ((p.N + 191) / 192);
        for(int s = 1; s <= 2; ++s)
        {
            if(s > 1 && (t192 < 64 || t192 * s > cus || p.kblocks / s < 8)) // (as above: few tiles, model off)
                break;
            const float c = plan_cost(p, cus, 192, s);
            if(c < best.us * 0.97f)
                best = PrefillPlan{s, c, 192};
        }
    }
    return best;
}

template <int NW>
static hipError_t launch_prefill_nw(const GemmKernelParams& p, In16 out_dtype, const LaunchCtx& ctx, int splits,
                                    bool splits_chosen_here, int device, int cus)
{
    constexpr int     kBN    = tile_n(NW);
    const hipStream_t stream = ctx.stream;
    const int    tiles_m = (p.M + kBM - 1) / kBM, tiles_n = (p.N + kBN - 1) / kBN;
    // the two stages, or the eight waves' output blocks of the epilogue, whichever is larger
    // x_scale in windows of four K blocks: row-major, whole windows, 16-byte aligned rows
    const bool   xs4     = !p.w_shuffled && p.xs_k == 1 && p.xs_m == p.kblocks && (p.kblocks & 3) == 0 &&
                           ((uintptr_t)p.xs & 15) == 0;
    const size_t smem    = std::max((size_t)kStages * stage_bytes(NW) + (xs4 ? 2 * kWindowBytes : 0),
                                    (size_t)8 * 64 * epi_pitch(NW));
    const bool   bf      = out_dtype == In16::bf16;
    auto         kernel  = p.w_shuffled ? (bf ? gemm_prefill_kernel<In16::bf16, true, NW, false> : gemm_prefill_kernel<In16::fp16, true, NW, false>)
                           : xs4        ? (bf ? gemm_prefill_kernel<In16::bf16, false, NW, true> : gemm_prefill_kernel<In16::fp16, false, NW, true>)
                                        : (bf ? gemm_prefill_kernel<In16::bf16, false, NW, false> : gemm_prefill_kernel<In16::fp16, false, NW, false>);
    // Per device and instantiation, once: the opt-in to more than 64 KiB of LDS.  (Racing first
    // calls repeat the same idempotent set-up.)
    constexpr int kMaxDevices = 64;
    static std::atomic<bool> ready[kMaxDevices][6];
    const int inst = (p.w_shuffled ? 2 : xs4 ? 4 : 0) + (bf ? 0 : 1);
    hipError_t e;
    if(device < 0 || device >= kMaxDevices || !ready[device][inst])
    {
        if((e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)smem)) != hipSuccess)
            return e;
        if(device >= 0 && device < kMaxDevices)
            ready[device][inst] = true;
    }
    // one workgroup fills a compute unit (LDS, registers); with more tiles than compute units the
    // workgroups walk the tiles.  A multiple of 8 keeps a workgroup's tiles on one XCD's patch order.
    const int total = tiles_m * tiles_n;
    if(total * splits > 4096) // 32-bit byte offsets into the parked tiles
        splits = 1;
    // a caller that may not allocate gets one K range per tile where the library's own choice of more
    // would not fit the fixed buffer (a count asked for by name is an error there instead)
    if(ctx.static_only && splits_chosen_here && (size_t)total * splits * (4 * NW) * 512 * 16 > kStaticPartialBytes)
        splits = 1;
    splits                 = std::max(1, std::min(splits, (int)p.kblocks));
    const int kb_per_split = (p.kblocks + splits - 1) / splits;
    splits                 = (p.kblocks + kb_per_split - 1) / kb_per_split;
    float*    partial = nullptr;
    uint32_t* tickets = nullptr;
    size_t    bytes   = 0;
    WorkspaceLock lock(splits > 1);
    if(splits > 1)
    {
        bytes = (size_t)total * splits * (4 * NW) * 512 * 16;
        if((e = split_workspace(ctx, lock, bytes, (size_t)total, &partial, &tickets)) != hipSuccess)
            return e;
    }
    const int items = total * splits;
    const int grid  = (items > cus && cus >= 8) ? (cus & ~7) : items;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), smem, stream, p, tiles_m, tiles_n, splits,
                       kb_per_split, partial, (uint32_t)bytes, tickets);
    return hipGetLastError();
}

hipError_t launch_gemm_prefill(const GemmKernelParams& p, In16 out_dtype, const LaunchCtx& ctx, int want_splits,
                               int want_tile_n)
{
    // the number of compute units, per device, once
    constexpr int kMaxDevices = 64;
    static std::atomic<int> cus_of[kMaxDevices];
    int           device = 0, cus = 0;
    hipError_t    e = hipGetDevice(&device);
    if(e != hipSuccess)
        return e;
    if(device >= 0 && device < kMaxDevices)
        cus = cus_of[device];
    if(cus == 0)
    {
        if((e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device)) != hipSuccess)
            return e;
        if(device >= 0 && device < kMaxDevices)
            cus_of[device] = cus;
    }
    // want_splits / want_tile_n: 0 = the plan's choice, otherwise as told
    const PrefillPlan plan = gemm_prefill_plan(p, cus);
    const int bn     = want_tile_n == 128 || want_tile_n == 192 || want_tile_n == 256
                           ? want_tile_n
                           : (want_splits > 0 ? 256 : plan.tile_n);
    const int splits = want_splits > 0 ? want_splits : (bn == plan.tile_n ? plan.splits : 1);
    const bool chosen = want_splits <= 0;
    return bn == 128   ? launch_prefill_nw<4>(p, out_dtype, ctx, splits, chosen, device, cus)
           : bn == 192 ? launch_prefill_nw<6>(p, out_dtype, ctx, splits, chosen, device, cus)
                       : launch_prefill_nw<8>(p, out_dtype, ctx, splits, chosen, device, cus);
}

} // namespace fp8bs
