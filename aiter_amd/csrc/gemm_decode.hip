// Decode-shape block-scale FP8 GEMM (M <= 64): weight streaming, bound by how fast a compute
// unit can pull bytes in.
//
// A compute unit keeps only a few tens of KiB of memory requests in flight, so the kernel is
// built to (a) spread the weight matrix over every compute unit of the chip, (b) bring each
// byte in exactly once, straight into registers in MFMA operand layout, and (c) keep the
// activations from multiplying that traffic.
//
// Work split.  A workgroup owns a group of R 16-row weight tiles and one K range; its waves
// split that K range between them, 4 K blocks (512 bytes of every row) per wave and step.
// A wave therefore needs only its own K slice of the activations, which it keeps in registers
// as MFMA "B" fragments for the life of the workgroup; no LDS staging, no re-reads.  The
// per-wave fp32 partial tiles are added through LDS in wave order.  A workgroup that owns
// several row groups walks them with the next group's weights already requested.
//
// When N alone gives too few workgroups to cover the chip, the K range is also split across
// workgroups; their fp32 partial tiles go to a workspace and the last workgroup to finish a
// row group (an atomic ticket) adds them in split order, so results never depend on timing.
#include "gemm_common.h"

#include <atomic>
#include <stdlib.h>
#include <string.h>

namespace fp8bs {

namespace {

constexpr int kStepKb = 4; // K blocks per wave and step
constexpr int kMaxDynamicLds = 128 * 1024;
constexpr int kDecodeMaxM    = 512; // 8 chunks of 64 activation rows

struct DecodeParams
{
    GemmKernelParams g;
    int32_t   n_tiles;      // ceil(N / 16)
    int32_t   n_groups;     // ceil(n_tiles / R)
    int32_t   kb_per_split; // K blocks per workgroup-level K range
    int32_t   splits;       // number of such ranges (grid.y)
    int32_t   bf16_out;
    int32_t   m_chunks;     // chunks of MT x 16 activation rows a workgroup walks per row group
    int32_t   grid_x, waves; // launch dimensions, passed explicitly: the implicit ones cost a dependent load
    int32_t   xs_vec4;      // x_scale rows can be read four K blocks at a time (16-byte aligned)
    float*    partial;      // [splits - 1][items][R * MT * 64] x 4 fp32 when splits > 1: all zero between launches
    uint32_t  partial_bytes;
};

__device__ __forceinline__ u32x2 pack4(const f32x4& v, bool bf)
{
    return bf ? u32x2{pack2<In16::bf16>(v[0], v[1]), pack2<In16::bf16>(v[2], v[3])}
              : u32x2{pack2<In16::fp16>(v[0], v[1]), pack2<In16::fp16>(v[2], v[3])};
}

template <int MT>
constexpr int decode_max_waves()
{
    return 4; // one wave per SIMD: each may use the whole 512-register file
}

// FULL: every step of every wave holds exactly 4 K blocks (K is a multiple of 512), which
// makes the multiply straight-line code; otherwise the block count of a step is a run-time value.
// SHUF: the weights are pre-shuffled (16,16): a lane's MFMA fragment is then two coalesced 16-byte
// loads and needs no transposition.
// CHUNKED (SINGLE only): more than 64 activation rows, walked in chunks of MT x 16 per row group.
// SPLIT: K is shared out over workgroups (p.splits > 1).  A template parameter so that the kernels
// without K ranges carry none of the exchange code: its mere presence cost them 2-5 %.
template <int MT, int R, bool SINGLE, bool FULL, bool SHUF, bool CHUNKED, bool SPLIT>
__global__ __launch_bounds__(64 * decode_max_waves<MT>()) void gemm_decode_kernel(DecodeParams p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const GemmKernelParams& g = p.g;

    // Kernel arguments arrive through scalar loads, which the compiler places per basic block:
    // three dependent round trips before the first weight request.  Naming every argument
    // here puts all of them into the entry block, behind a single wait.
#define FP8BS_TOUCH(x) asm volatile("" ::"s"(x))
    FP8BS_TOUCH(g.xq); FP8BS_TOUCH(g.wq); FP8BS_TOUCH(g.xs); FP8BS_TOUCH(g.ws); FP8BS_TOUCH(g.out);
    FP8BS_TOUCH(g.M); FP8BS_TOUCH(g.N); FP8BS_TOUCH(g.lda); FP8BS_TOUCH(g.ldb); FP8BS_TOUCH(g.kblocks);
    FP8BS_TOUCH(g.K); FP8BS_TOUCH(g.xs_m); FP8BS_TOUCH(g.xs_k);
    FP8BS_TOUCH(p.n_tiles); FP8BS_TOUCH(p.n_groups); FP8BS_TOUCH(p.kb_per_split); FP8BS_TOUCH(p.splits);
    FP8BS_TOUCH(p.bf16_out); FP8BS_TOUCH(p.xs_vec4); FP8BS_TOUCH(p.partial); FP8BS_TOUCH(p.partial_bytes);
    FP8BS_TOUCH(p.grid_x); FP8BS_TOUCH(p.waves); FP8BS_TOUCH(p.m_chunks);
#undef FP8BS_TOUCH

    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int nw   = p.waves;
    const int l16 = lane & 15, kg = lane >> 4;
    const int split = blockIdx.y;
    const int kb_lo = split * p.kb_per_split;
    const int kb_hi = min(kb_lo + p.kb_per_split, g.kblocks);
    constexpr int E = R * MT * 64; // f32x4 elements of a workgroup's output tile set

    // Global loads are issued row-segment-wise: 8 consecutive lanes fetch one 128-byte K block of
    // one row, so a load instruction touches 8 cache lines in full.  (Fetching straight into the
    // MFMA layout, 16 rows x 16 bytes per quarter wave, costs a tag lookup per 16 bytes and
    // caps a compute unit far below what the memory system delivers.)  The wave then turns each
    // 16-row x 128-byte unit into MFMA fragments through a private 2 KiB LDS slot: written as
    // loaded, read back fragment-wise; the bank swizzle of that slot is applied on the global
    // side, by which 16-byte chunk of its row a lane fetches.
    const int crow = lane >> 3;
    const int cchunk[2] = {(int)((lane & 7) ^ lds_swizzle(crow)), (int)((lane & 7) ^ lds_swizzle(8 + crow))};
    uint8_t*  slot = smem + (size_t)wave * 2048;
    auto      as_fragment = [&](const u32x4(&raw)[2]) -> i32x8 {
        return i32x8{(int)raw[0][0], (int)raw[0][1], (int)raw[0][2], (int)raw[0][3],
                     (int)raw[1][0], (int)raw[1][1], (int)raw[1][2], (int)raw[1][3]};
    };
    auto      settle = [&](const u32x4(&raw)[2]) -> i32x8 {
        *(u32x4*)(slot + lane * 16)        = raw[0];
        *(u32x4*)(slot + 1024 + lane * 16) = raw[1];
        const i32x4 lo = *(const i32x4*)(slot + lds_off(l16, 2 * kg));
        const i32x4 hi = *(const i32x4*)(slot + lds_off(l16, 2 * kg + 1));
        return i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };

    // K block i of a step that starts at kb0 and holds nk (1..4) blocks; slots past the end
    // re-read the last block (a cache hit) and are never multiplied
    auto kslot = [&](int kb0, int nk, int i) { return FULL ? kb0 + i : kb0 + (i < nk ? i : nk - 1); };

    // Requests go out row by row with a row's K blocks back to back (512 contiguous bytes per
    // row close together in time suits the DRAM pages), weights first: they come from furthest
    // away.  Loads return in order, so the activation tiles, requested last, can be multiplied
    // one m tile at a time while the later ones are still on their way.
    auto issue_w = [&](int grp, int kb0, int nk, u32x4(&raw)[R][kStepKb][2], float(&s)[R][kStepKb]) {
#pragma unroll
        for(int r = 0; r < R; ++r)
        {
            const int    tile = min(grp * R + r, p.n_tiles - 1);
            const float* wsp  = g.ws + (size_t)((tile * 16) >> 7) * g.kblocks; // wave-uniform
            if constexpr(SHUF)
            {
                // lane (l16, kg) of K block kk: 16 bytes at chunk (4 kk + kg), row l16, both halves
                const uint8_t* wp = g.wq + (size_t)tile * 16 * (size_t)g.K + (size_t)kg * 512 + l16 * 16;
#pragma unroll
                for(int i = 0; i < kStepKb; ++i)
#pragma unroll
                    for(int h = 0; h < 2; ++h)
                        raw[r][i][h] = __builtin_nontemporal_load(
                            (const u32x4*)(wp + (size_t)kslot(kb0, nk, i) * 2048 + h * 256));
            }
            else
            {
#pragma unroll
                for(int h = 0; h < 2; ++h)
                {
                    const int      n  = min(tile * 16 + h * 8 + crow, g.N - 1);
                    const uint8_t* wp = g.wq + (size_t)n * g.ldb + cchunk[h] * 16;
#pragma unroll
                    for(int i = 0; i < kStepKb; ++i)
                        raw[r][i][h] = __builtin_nontemporal_load(
                            (const u32x4*)(wp + (size_t)kslot(kb0, nk, i) * 128));
                }
            }
#pragma unroll
            for(int i = 0; i < kStepKb; ++i)
                s[r][i] = wsp[kslot(kb0, nk, i)];
        }
    };

    // Long K (several steps per wave): the workgroup's first weight requests go out before anything
    // else is set up (activation addresses, the reduction's bookkeeping: a few hundred instructions,
    // which the requests' latency then covers; (16, 2112, 7168): 8.0 -> 7.5 us).  With one step per
    // wave the requests of the first group, the activations and the second group stay together
    // further down (hoisted, (1, 7168, 2048) ran 3 % slower).
    // No branch around the requests: values that flow out of a branch get copied, and a copy waits
    // for its load.  A wave whose step lies beyond the K range requests the row's last blocks and
    // never uses them.
    u32x4 raw_h[SINGLE ? 1 : R][kStepKb][2];
    float ws_h[SINGLE ? 1 : R][kStepKb];
    if constexpr(!SINGLE)
    {
        const int first_kb0 = kb_lo + wave * kStepKb;
        const int first_nk  = max(0, min(kStepKb, kb_hi - first_kb0));
        issue_w(blockIdx.x, min(first_kb0, FULL ? g.kblocks - kStepKb : g.kblocks - 1), max(first_nk, 1), raw_h, ws_h);
        __builtin_amdgcn_sched_barrier(0);
    }

    // activation rows this lane fetches (two per m tile: rows crow and 8 + crow of the tile) and
    // the row whose scales it needs (rows past M re-read the last one, never stored), for the
    // chunk of 64 rows that starts at m_base
    const uint8_t* xrow[MT][2];
    const float*   xsrow[MT];
    auto           set_chunk = [&](int m_base) {
#pragma unroll
        for(int j = 0; j < MT; ++j)
        {
#pragma unroll
            for(int h = 0; h < 2; ++h)
                xrow[j][h] =
                    g.xq + (size_t)min(m_base + j * 16 + h * 8 + crow, g.M - 1) * g.lda + cchunk[h] * 16;
            xsrow[j] = g.xs + (size_t)min(m_base + j * 16 + l16, g.M - 1) * g.xs_m;
        }
    };
    set_chunk(0);

    i32x8 bx[MT][kStepKb];
    float xsv[MT][kStepKb];
    f32x4 acc[R][MT];

    auto issue_x = [&](int kb0, int nk, u32x4(&raw)[MT][kStepKb][2], float(&xs_out)[MT][kStepKb], int j_lo,
                       int j_hi) {
#pragma unroll
        for(int j = 0; j < MT; ++j)
        {
            if(j < j_lo || j >= j_hi) // compile-time bounds at every call site
                continue;
#pragma unroll
            for(int h = 0; h < 2; ++h)
#pragma unroll
                for(int i = 0; i < kStepKb; ++i)
                    raw[j][i][h] = *(const u32x4*)(xrow[j][h] + (size_t)kslot(kb0, nk, i) * 128);
            if((FULL || nk == kStepKb) && p.xs_vec4) // the four scales of the step in one load
            {
                const f32x4 v = *(const f32x4*)(xsrow[j] + kb0);
#pragma unroll
                for(int i = 0; i < kStepKb; ++i)
                    xs_out[j][i] = v[i];
            }
            else
            {
#pragma unroll
                for(int i = 0; i < kStepKb; ++i)
                    xs_out[j][i] = xsrow[j][(size_t)kslot(kb0, nk, i) * g.xs_k];
            }
        }
    };

    auto settle_x = [&](const u32x4(&raw)[MT][kStepKb][2]) {
#pragma unroll
        for(int j = 0; j < MT; ++j)
#pragma unroll
            for(int i = 0; i < kStepKb; ++i)
                bx[j][i] = settle(raw[j][i]);
    };
    // first row group of a workgroup: weight fragments are ready, activation fragments are formed
    // (and kept) one m tile at a time, each multiplied at once
    auto multiply_first = [&](int nk, const i32x8(&aw)[R][kStepKb], const float(&s)[R][kStepKb],
                              const u32x4(&xraw)[MT][kStepKb][2], int j_lo, int j_hi) {
#pragma unroll
        for(int j = 0; j < MT; ++j)
        {
            if(j < j_lo || j >= j_hi) // compile-time bounds at every call site
                continue;
#pragma unroll
            for(int i = 0; i < kStepKb; ++i)
                bx[j][i] = settle(xraw[j][i]);
#pragma unroll
            for(int i = 0; i < kStepKb; ++i)
            {
                if(FULL || i < nk) // wave-uniform
                {
#pragma unroll
                    for(int r = 0; r < R; ++r)
                    {
                        const f32x4 part = mfma_16x16x128_fp8(aw[r][i], bx[j][i], f32x4{0.f, 0.f, 0.f, 0.f});
                        const float sc   = xsv[j][i] * s[r][i];
#pragma unroll
                        for(int c = 0; c < 4; ++c)
                            acc[r][j][c] = __builtin_fmaf(part[c], sc, acc[r][j][c]);
                    }
                }
            }
        }
    };
    // one weight unit at a time: fragments out of the raw registers, then its MT tile products,
    // scaled and accumulated
    auto multiply = [&](int nk, const u32x4(&wraw)[R][kStepKb][2], const float(&s)[R][kStepKb]) {
#pragma unroll
        for(int r = 0; r < R; ++r)
#pragma unroll
            for(int i = 0; i < kStepKb; ++i)
            {
                if(FULL || i < nk) // wave-uniform
                {
                    const i32x8 w = SHUF ? as_fragment(wraw[r][i]) : settle(wraw[r][i]);
#pragma unroll
                    for(int j = 0; j < MT; ++j)
                    {
                        const f32x4 part = mfma_16x16x128_fp8(w, bx[j][i], f32x4{0.f, 0.f, 0.f, 0.f});
                        const float sc   = xsv[j][i] * s[r][i];
#pragma unroll
                        for(int c = 0; c < 4; ++c)
                            acc[r][j][c] = __builtin_fmaf(part[c], sc, acc[r][j][c]);
                    }
                }
            }
    };
    auto clear_acc = [&]() {
#pragma unroll
        for(int r = 0; r < R; ++r)
#pragma unroll
            for(int j = 0; j < MT; ++j)
                acc[r][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    };

    // element e of a group's tile set -> (row tile r, m tile j, lane ln): that lane's 4 outputs
    // A unit of output is an "item": row group grp x chunk c of 64 activation rows, numbered
    // grp * m_chunks + c (with M <= 64 there is one chunk and item == grp).
    auto store_out = [&](int item, int e, const f32x4& v) {
        const int grp = item / p.m_chunks, chunk = item - grp * p.m_chunks;
        const int r = e / (MT * 64), j = (e >> 6) % MT, ln = e & 63;
        const int tile = grp * R + r;
        const int m = chunk * (MT * 16) + j * 16 + (ln & 15), n = tile * 16 + (ln >> 4) * 4;
        if(tile >= p.n_tiles || m >= g.M)
            return;
        uint16_t* dst = g.out + (size_t)m * g.N + n;
        const u32x2 o = pack4(v, p.bf16_out != 0);
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

    const __amdgpu_buffer_rsrc_t part_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(p.partial, 0, SPLIT ? (int)p.partial_bytes : 0, 0x00020000);
    constexpr int kCoherent = 16; // cache-policy bit sc1: served by memory, not by a per-XCD L2

    // Per-wave partial tiles of a row group are parked in one of two LDS slots; they are added up
    // in wave order and stored while the workgroup waits for the next group's weights, so only
    // the last group's sum is left for the end.
    f32x4* const parked = (f32x4*)(smem + (size_t)nw * 2048);
    auto         park   = [&](int q) {
        f32x4* mine = parked + ((size_t)q * nw + wave) * E;
#pragma unroll
        for(int r = 0; r < R; ++r)
#pragma unroll
            for(int j = 0; j < MT; ++j)
                mine[(r * MT + j) * 64 + lane] = acc[r][j];
    };
    // sum over the waves of element e of a parked tile set, in wave order; all reads are issued
    // before the first addition (reads past the last wave repeat it and are not added)
    constexpr int kMaxWaves = decode_max_waves<MT>();
    auto          wave_sum  = [&](const f32x4* red, int e) -> f32x4 {
        f32x4 v[kMaxWaves];
#pragma unroll
        for(int w = 0; w < kMaxWaves; ++w)
            v[w] = red[(size_t)min(w, nw - 1) * E + e];
        f32x4 sum = v[0];
#pragma unroll
        for(int w = 1; w < kMaxWaves; ++w)
            sum = w < nw ? sum + v[w] : sum;
        return sum;
    };
    // K ranges of one item meet without a counter.  The workgroup of every range but the last
    // writes its tile set to the exchange buffer and is done; the workgroup of the LAST range
    // (dispatched after the others: it can only wait for workgroups that are already running or
    // finished) reads them in range order, adds its own on top and stores the output -- so the
    // result does not depend on timing.  The buffer is all zero between launches and a tile set
    // is written as the complement of its bits: a 16-byte piece that still reads zero in any of
    // its words has not arrived.  The reader polls lane by lane, past the caches, and puts the
    // zeros back once it has the value.  (A partial sum whose bits are all ones -- one particular
    // NaN, which no arithmetic here produces -- would read as zero for good: the wait is bounded,
    // and a piece that never turns up is taken as it stands, which is that NaN.)  The workgroups
    // of an item run on different XCDs, whose L2 caches are not coherent with each other: every
    // access to the exchanged tiles bypasses them (sc1).
    auto flush_group_split = [&](int grp /* item */, const f32x4* red) {
        const size_t n_items = (size_t)p.n_groups * p.m_chunks;
        const int    last    = p.splits - 1;
        if(split != last)
        {
            for(int e = t; e < E; e += (nw * 64))
            {
                const u32x4    s   = ~__builtin_bit_cast(u32x4, wave_sum(red, e));
                const uint32_t off = (uint32_t)(((size_t)split * n_items + grp) * E + e) * 16u;
                __builtin_amdgcn_raw_buffer_store_b128(s, part_rsrc, off, 0, kCoherent);
            }
            return;
        }
        constexpr int kPollCoherent = 17;      // sc0 | sc1: never served by a cache
        constexpr int kMaxPolls     = 1 << 16; // a tenth of a second, a thousand times a launch
        for(int e = t; e < E; e += (nw * 64))
        {
            const f32x4 own = wave_sum(red, e);
            f32x4       s   = f32x4{0.f, 0.f, 0.f, 0.f};
            for(int sp = 0; sp < last; ++sp) // range order, whenever they arrive
            {
                const uint32_t off = (uint32_t)(((size_t)sp * n_items + grp) * E + e) * 16u;
                u32x4          v   = __builtin_amdgcn_raw_buffer_load_b128(part_rsrc, off, 0, kPollCoherent);
                for(int polls = 0; (v[0] == 0u || v[1] == 0u || v[2] == 0u || v[3] == 0u) && polls < kMaxPolls; ++polls)
                {
                    __builtin_amdgcn_s_sleep(2);
                    v = __builtin_amdgcn_raw_buffer_load_b128(part_rsrc, off, 0, kPollCoherent);
                }
                __builtin_amdgcn_raw_buffer_store_b128(u32x4{0u, 0u, 0u, 0u}, part_rsrc, off, 0, kCoherent);
                s += __builtin_bit_cast(f32x4, ~v);
            }
            store_out(grp, e, s + own);
        }
    };
    // adds up and stores the group parked in `slot`; the barrier makes every wave's tiles visible
    // (and, one group later, guarantees that the other slot has been read before it is reused)
    auto flush_one = [&](int fgrp, int which) {
        __syncthreads();
        const f32x4* red = parked + (size_t)which * nw * E;
        if constexpr(!SPLIT)
        {
            // four elements per thread and pass, all LDS reads of a pass issued together
            const int T = (nw * 64);
            for(int base = t; base < E; base += 4 * T)
            {
                f32x4 sum[4];
#pragma unroll
                for(int u = 0; u < 4; ++u)
                    sum[u] = wave_sum(red, min(base + u * T, E - 1));
#pragma unroll
                for(int u = 0; u < 4; ++u)
                    if(base + u * T < E)
                        store_out(fgrp, base + u * T, sum[u]);
            }
        }
        else
            flush_group_split(fgrp, red);
    };

    const int stride = p.grid_x;
    int       grp = blockIdx.x, prev = -1, pslot = 0;
    // to be called between requesting the next group's weights and multiplying the current one
    auto flush_prev = [&]() {
        if(prev >= 0)
        {
            flush_one(prev, pslot);
            pslot ^= 1;
        }
    };
    auto park_current = [&](int item) {
        park(pslot);
        prev = item;
    };

    if constexpr(SINGLE)
    {
        // one step per wave covers the K range: activations stay in registers for the life of
        // the workgroup, and while a row group is multiplied the next one's weights are already
        // requested into the other of two register sets (no copies: reading a register that a
        // load is still to fill would wait for that load)
        const int kb0 = kb_lo + wave * kStepKb;
        const int nk  = max(0, min(kStepKb, kb_hi - kb0));
        if constexpr(CHUNKED)
        {
            {
                // More than 64 activation rows: the weights of a row group are turned into
                // fragments once and stay in registers while the workgroup walks the chunks
                // of MT x 16 rows; each chunk's activations are requested while the previous chunk
                // is multiplied, the next group's weights while the current group is walked.
                u32x4 xraw[MT][kStepKb][2];
                float xsn[MT][kStepKb];
                auto  issue_chunk = [&](int chunk) {
                    set_chunk(chunk * (MT * 16));
                    issue_x(kb0, nk, xraw, xsn, 0, MT);
                };
                u32x4 raw[R][kStepKb][2];
                float ws_next[R][kStepKb], ws_cur[R][kStepKb];
                if(nk > 0)
                {
                    issue_w(grp, kb0, nk, raw, ws_next);
                    issue_chunk(0);
                }
                for(; grp < p.n_groups; grp += stride)
                {
                    const bool more = grp + stride < p.n_groups;
                    i32x8      aw[R][kStepKb];
                    if(nk > 0)
                    {
#pragma unroll
                        for(int r = 0; r < R; ++r)
#pragma unroll
                            for(int i = 0; i < kStepKb; ++i)
                            {
                                aw[r][i]     = SHUF ? as_fragment(raw[r][i]) : settle(raw[r][i]);
                                ws_cur[r][i] = ws_next[r][i];
                            }
                    }
                    for(int chunk = 0; chunk < p.m_chunks; ++chunk)
                    {
                        float xsc[MT][kStepKb];
                        clear_acc();
                        if(nk > 0)
                        {
                            settle_x(xraw);
#pragma unroll
                            for(int j = 0; j < MT; ++j)
#pragma unroll
                                for(int i = 0; i < kStepKb; ++i)
                                    xsc[j][i] = xsn[j][i];
                            // what the next item needs goes out before this one is multiplied;
                            // the raw weight registers are free since the fragments were formed
                            if(chunk + 1 < p.m_chunks)
                                issue_chunk(chunk + 1);
                            else if(more)
                            {
                                issue_w(grp + stride, kb0, nk, raw, ws_next);
                                issue_chunk(0);
                            }
#pragma unroll
                            for(int j = 0; j < MT; ++j)
#pragma unroll
                                for(int i = 0; i < kStepKb; ++i)
                                {
                                    if(FULL || i < nk)
                                    {
#pragma unroll
                                        for(int r = 0; r < R; ++r)
                                        {
                                            const f32x4 part = mfma_16x16x128_fp8(aw[r][i], bx[j][i],
                                                                                  f32x4{0.f, 0.f, 0.f, 0.f});
                                            const float sc   = xsc[j][i] * ws_cur[r][i];
#pragma unroll
                                            for(int c = 0; c < 4; ++c)
                                                acc[r][j][c] = __builtin_fmaf(part[c], sc, acc[r][j][c]);
                                        }
                                    }
                                }
                        }
                        flush_prev();
                        park_current(grp * p.m_chunks + chunk);
                    }
                }
                flush_prev();
                return;
            }
        }
        u32x4     raw_a[R][kStepKb][2], raw_b[R][kStepKb][2];
        float     ws_a[R][kStepKb], ws_b[R][kStepKb];
        {
            u32x4      xraw[MT][kStepKb][2];
            const bool more = grp + stride < p.n_groups;
            clear_acc();
            if(nk > 0)
            {
                // Requests are throttled by the memory system, so the instruction stream does
                // useful work between them: the weight fragments are formed while the second
                // half of the activations is still being requested, and each m tile is
                // multiplied as soon as its own fragments are in.
                constexpr int kHalf = (MT + 1) / 2;
                issue_w(grp, kb0, nk, raw_a, ws_a);
                if constexpr(MT <= 2)
                {
                    // narrow activations leave registers to spare: the second group's weights
                    // are requested at once, behind the first group's and the activations
                    issue_x(kb0, nk, xraw, xsv, 0, MT);
                    if(more)
                    {
                        issue_w(grp + stride, kb0, nk, raw_b, ws_b);
                        settle_x(xraw);
                        multiply(nk, raw_a, ws_a);
                    }
                    else
                    {
                        settle_x(xraw);
                        multiply(nk, raw_a, ws_a);
                    }
                }
                else
                {
                    issue_x(kb0, nk, xraw, xsv, 0, kHalf);
                    i32x8 aw[R][kStepKb];
#pragma unroll
                    for(int r = 0; r < R; ++r)
#pragma unroll
                        for(int i = 0; i < kStepKb; ++i)
                            aw[r][i] = SHUF ? as_fragment(raw_a[r][i]) : settle(raw_a[r][i]);
                    issue_x(kb0, nk, xraw, xsv, kHalf, MT);
                    multiply_first(nk, aw, ws_a, xraw, 0, kHalf);
                    if(more) // the next group's weights, now that half of the raw registers are free
                    {
                        issue_w(grp + stride, kb0, nk, raw_b, ws_b);
                        multiply_first(nk, aw, ws_a, xraw, kHalf, MT);
                    }
                    else
                        multiply_first(nk, aw, ws_a, xraw, kHalf, MT);
                }
            }
            park_current(grp);
            grp += stride;
        }
        while(grp < p.n_groups) // raw_b holds this group
        {
            bool more = grp + stride < p.n_groups;
            clear_acc();
            if(nk > 0 && more)
            {
                issue_w(grp + stride, kb0, nk, raw_a, ws_a);
                flush_prev();
                multiply(nk, raw_b, ws_b);
            }
            else
            {
                flush_prev();
                if(nk > 0)
                    multiply(nk, raw_b, ws_b);
            }
            park_current(grp);
            grp += stride;
            if(grp >= p.n_groups)
                break;
            more = grp + stride < p.n_groups; // raw_a holds this group
            clear_acc();
            if(nk > 0 && more)
            {
                issue_w(grp + stride, kb0, nk, raw_b, ws_b);
                flush_prev();
                multiply(nk, raw_a, ws_a);
            }
            else
            {
                flush_prev();
                if(nk > 0)
                    multiply(nk, raw_a, ws_a);
            }
            park_current(grp);
            grp += stride;
        }
    }
    else
    {
        // long K: every wave takes several steps; activations are re-read per item
        bool first_step = true;
        for(; grp < p.n_groups; grp += stride)
            for(int chunk = 0; chunk < p.m_chunks; ++chunk)
            {
                if(p.m_chunks > 1)
                    set_chunk(chunk * (MT * 16));
                clear_acc();
                bool flushed = false;
                for(int kb0 = kb_lo + wave * kStepKb; kb0 < kb_hi; kb0 += nw * kStepKb)
                {
                    const int nk = min(kStepKb, kb_hi - kb0);
                    auto&     wraw = raw_h;
                    auto&     wsv  = ws_h;
                    u32x4     xraw[MT][kStepKb][2];
                    if(!first_step) // (the workgroup's first step was requested at the top)
                        issue_w(grp, kb0, nk, wraw, wsv);
                    first_step = false;
                    issue_x(kb0, nk, xraw, xsv, 0, MT);
                    if(!flushed) // the previous item's sum, behind this item's first requests
                    {
                        flush_prev();
                        flushed = true;
                    }
                    settle_x(xraw);
                    multiply(nk, wraw, wsv);
                }
                if(!flushed)
                    flush_prev();
                park_current(grp * p.m_chunks + chunk);
            }
    }
    flush_prev();
}

constexpr int kMaxDevices = 64;

// reads "key=value" integers out of a comma-separated tuning string; 0 when absent
int tuning_value(const char* tuning, const char* key)
{
    if(tuning == nullptr)
        return 0;
    const size_t klen = strlen(key);
    for(const char* s = tuning; *s;)
    {
        if(strncmp(s, key, klen) == 0 && s[klen] == '=')
            return atoi(s + klen + 1);
        const char* c = strchr(s, ',');
        if(c == nullptr)
            break;
        s = c + 1;
    }
    return 0;
}

template <int MT, int R, bool SINGLE, bool FULL, bool SHUF, bool CHUNKED, bool SPLIT>
hipError_t launch_split(const DecodeParams& p, dim3 grid, int waves, size_t smem, hipStream_t stream)
{
    auto        kernel = gemm_decode_kernel<MT, R, SINGLE, FULL, SHUF, CHUNKED, SPLIT>;
    static std::atomic<bool> raised[kMaxDevices]; // dynamic LDS above the default limit needs opting in, once
    int         dev = 0;
    (void)hipGetDevice(&dev);
    if(dev >= 0 && dev < kMaxDevices && !raised[dev])
    {
        hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           kMaxDynamicLds);
        if(e != hipSuccess)
            return e;
        raised[dev] = true;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(64 * waves), smem, stream, p);
    return hipGetLastError();
}

template <int MT, int R, bool SINGLE, bool FULL, bool SHUF, bool CHUNKED = false>
hipError_t launch_one(const DecodeParams& p, dim3 grid, int waves, size_t smem, hipStream_t stream)
{
    return p.splits > 1 ? launch_split<MT, R, SINGLE, FULL, SHUF, CHUNKED, true>(p, grid, waves, smem, stream)
                        : launch_split<MT, R, SINGLE, FULL, SHUF, CHUNKED, false>(p, grid, waves, smem, stream);
}

template <int MT, int R, bool SHUF>
hipError_t launch_mt_r(const DecodeParams& p, bool single, bool full, dim3 grid, int waves, size_t smem,
                       hipStream_t stream)
{
    if constexpr(MT == 2)
    {
        if(single && p.m_chunks > 1)
            return full ? launch_one<MT, R, true, true, SHUF, true>(p, grid, waves, smem, stream)
                        : launch_one<MT, R, true, false, SHUF, true>(p, grid, waves, smem, stream);
    }
    if(single)
        return full ? launch_one<MT, R, true, true, SHUF>(p, grid, waves, smem, stream)
                    : launch_one<MT, R, true, false, SHUF>(p, grid, waves, smem, stream);
    return full ? launch_one<MT, R, false, true, SHUF>(p, grid, waves, smem, stream)
                : launch_one<MT, R, false, false, SHUF>(p, grid, waves, smem, stream);
}

template <int MT>
hipError_t launch_mt(const DecodeParams& p, int rows, bool single, bool full, dim3 grid, int waves,
                     size_t smem, hipStream_t stream)
{
    if(p.g.w_shuffled)
        return rows == 2 ? launch_mt_r<MT, 2, true>(p, single, full, grid, waves, smem, stream)
                         : launch_mt_r<MT, 1, true>(p, single, full, grid, waves, smem, stream);
    return rows == 2 ? launch_mt_r<MT, 2, false>(p, single, full, grid, waves, smem, stream)
                     : launch_mt_r<MT, 1, false>(p, single, full, grid, waves, smem, stream);
}

} // namespace

bool gemm_decode_supports(const GemmKernelParams& p)
{
    return p.M >= 1 && p.M <= kDecodeMaxM && p.kblocks >= 1;
}

// How a problem is split over workgroups and waves.
struct DecodePlan
{
    int  mt;       // m tiles a wave holds at a time
    int  rows;     // 16-row weight tiles per group
    int  n_tiles, n_groups, steps;
    int  splits, steps_per_split, waves;
    bool single;   // one step per wave covers the workgroup's K range
    bool full;
    int  m_chunks, grid_x;
};

// split_k_log2 < 0: choose.  Otherwise 2^split_k_log2 K ranges (rounded to whole steps).
// `tuning` may override the choices: "r=<row tiles per group>,s=<K ranges>,w=<waves>,g=<grid.x>".
static DecodePlan plan_decode(const GemmKernelParams& g, int split_k_log2, const char* tuning)
{
    DecodePlan d{};
    d.n_tiles           = (g.N + 15) / 16;
    d.mt                = g.M > 64 ? 4 : (g.M + 15) / 16;
    const int max_waves = 4;
    d.steps             = (g.kblocks + kStepKb - 1) / kStepKb;
    const int kChipCus  = 256;

    // Two row tiles per group halve the activation traffic and double what a wave keeps in
    // flight: taken when the activations are wide (from 33 rows; their re-reads then cost more
    // than anything else).  Up to 32 rows single tiles are faster at every N measured, walked two
    // or three to a workgroup with the next tile's weights already requested ((1, 7168, 2048):
    // 5.8 us against 6.2, (1, 24576, 1536): 9.4 against 10.4, (32, 24576, 1536): 11.1 against 12.2).
    d.rows = tuning_value(tuning, "r");
    if(d.rows != 1 && d.rows != 2)
        d.rows = d.mt >= 3 ? 2 : 1;
    d.n_groups = (d.n_tiles + d.rows - 1) / d.rows;

    int splits = tuning_value(tuning, "s");
    if(splits <= 0)
    {
        if(split_k_log2 >= 0)
            splits = 1 << split_k_log2;
        else
        {
            // K ranges across workgroups while the row groups alone leave compute units idle.  Best
            // is one step per wave (four steps per range: every wave of a workgroup requests its whole
            // share at once and the waves finish together), as long as that keeps the launch within
            // about two workgroups per compute unit; otherwise as many ranges as that limit allows.
            // ((1, 512 ... 1536, 7168): four ranges 5.4 / 5.8 / 6.4 us against 6.0 / 5.8 / 6.7 with 7 / 4 / 2;
            // (1, 2112, 7168): three ranges 7.4 us against 8.5 with one; (1, 3072, 7168): two, 8.4 against 9.2;
            // (1, 1024, 4096): two, 4.7 against 5.1 with four; one step per range is never worth the exchange.)
            const int one_step_per_wave = (d.steps + max_waves - 1) / max_waves;
            if(d.n_groups * one_step_per_wave <= 2 * kChipCus - kChipCus / 4)
                splits = one_step_per_wave;
            else
                splits = std::min(one_step_per_wave, (2 * kChipCus) / d.n_groups);
            if(splits < 1)
                splits = 1;
        }
    }
    if(splits > d.steps)
        splits = d.steps;
    d.steps_per_split = (d.steps + splits - 1) / splits;
    d.splits          = (d.steps + d.steps_per_split - 1) / d.steps_per_split;

    d.waves = tuning_value(tuning, "w");
    if(d.waves <= 0 || d.waves > max_waves)
        d.waves = d.steps_per_split < max_waves ? d.steps_per_split : max_waves;
    d.single = d.steps_per_split <= d.waves;
    d.full   = (g.kblocks % kStepKb) == 0;
    // more than 64 rows are walked in chunks: 32 rows at a time when the weights stay in registers
    // across chunks (that path also stages the next chunk), else 64
    if(g.M > 64 && d.single)
        d.mt = 2;
    d.m_chunks = g.M > 64 ? (g.M + d.mt * 16 - 1) / (d.mt * 16) : 1;

    int gx = tuning_value(tuning, "g");
    if(gx <= 0)
    {
        gx = d.n_groups;
        if(d.single && d.rows == 1 && d.mt <= 2 && d.splits == 1 && d.n_groups >= 2 * (kChipCus - kChipCus / 8))
        {
            // single tiles, short K: at least two tiles per workgroup, at most two workgroups per
            // compute unit at a time
            int iters = (d.n_groups + 2 * kChipCus - 1) / (2 * kChipCus);
            iters     = iters < 2 ? 2 : iters;
            gx        = (d.n_groups + iters - 1) / iters;
        }
        else if(d.single && d.n_groups * d.splits > 2 * kChipCus)
        {
            const int per_split = (kChipCus + d.splits - 1) / d.splits;
            const int iters     = (d.n_groups + per_split - 1) / per_split;
            gx                  = (d.n_groups + iters - 1) / iters;
        }
    }
    d.grid_x = gx > d.n_groups ? d.n_groups : gx;
    return d;
}

// Rough duration (us) of the launch this file would choose, fitted per regime (one K step per
// workgroup; one step per wave; several steps per wave) to event timings of M = 16 ... 64 on
// fourteen weight shapes from 1.8 MB to 117 MB coming from HBM (about 10 % off on average).  Terms:
// the weights over the share of the chip the workgroups cover, the activation re-reads, the MFMA
// work (m tiles x weights), the parked partial tiles and the output.  Only used to decide between
// this kernel and the mid_* family.
float gemm_decode_estimate_us(const GemmKernelParams& g)
{
    const DecodePlan d = plan_decode(g, -1, nullptr);
    const float mb    = 1e-6f;
    const float w     = (float)g.N * (float)g.K * mb;
    const float a     = (float)(d.single ? d.grid_x : d.n_groups) * (float)g.M * (float)g.K * mb;
    const float wgs   = (float)d.grid_x * (float)d.splits;
    const float share = std::max(0.05f, std::min(1.f, wgs * (float)d.waves / 4.f / 256.f));
    const float part  = d.splits > 1 ? (float)d.splits * (float)g.M * (float)g.N * 4.f * mb : 0.f;
    const float out   = (float)g.M * (float)g.N * 2.f * mb;
    const float wide_split = (d.mt >= 3 && d.splits > 1) ? (float)d.splits : 0.f;
    const float mt    = (float)d.mt;
    if(d.waves == 1)
        return 2.53f + 0.096f * w / share + 0.028f * mt * w + 0.67f * out + 0.62f * mt;
    // K not a multiple of four K blocks: the multiply is not straight-line code ((8, 4096, 11008): 17.9 us
    // where the terms below say 13.4)
    const float ragged_k = d.full ? 1.f : 1.3f;
    if(d.single)
        return ragged_k * (3.59f + 0.107f * w / share + 0.038f * mt * w + 2.9f * part + 0.44f * wide_split + 0.10f * mt);
    // (K ranges that meet without a counter: 15 % below what the terms, fitted with a counter, say --
    // (1 ... 32, 4096, 7168) 8.8 ... 10.8 us against 10.1 ... 13.5)
    const float ranges = d.splits > 1 ? 0.85f : 1.f;
    return ragged_k * ranges *
           (4.67f + 0.141f * w / share + 0.021f * a + 0.029f * mt * w + 3.78f * out + 0.65f * wide_split + 0.38f * mt);
}

hipError_t launch_gemm_decode(const GemmKernelParams& g, In16 out_dtype, int split_k_log2, const LaunchCtx& ctx,
                                   const char* tuning)
{
    const hipStream_t stream = ctx.stream;
    DecodeParams p{};
    p.g           = g;
    p.bf16_out    = out_dtype == In16::bf16 ? 1 : 0;
    p.xs_vec4     = (g.xs_k == 1 && (g.xs_m & 3) == 0 && ((uintptr_t)g.xs & 15) == 0) ? 1 : 0;
    const DecodePlan d = plan_decode(g, split_k_log2, tuning);
    p.n_tiles      = d.n_tiles;
    p.n_groups     = d.n_groups;
    p.kb_per_split = d.steps_per_split * kStepKb;
    p.splits       = d.splits;
    p.m_chunks     = d.m_chunks;
    const int  mt = d.mt, rows = d.rows, splits = d.splits, waves = d.waves, gx = d.grid_x;
    const bool single = d.single, full = d.full;

    const size_t tile_set = (size_t)rows * mt * 64 * 16; // bytes of one group's fp32 tile set
    WorkspaceLock lock(splits > 1);
    if(splits > 1)
    {
        // the exchange buffer of the K ranges: zero between launches (the kernel puts the zeros back)
        const size_t bytes = (size_t)(splits - 1) * p.n_groups * p.m_chunks * tile_set;
        if(bytes >= ((size_t)1 << 31))
        {
            if(ctx.why)
                *ctx.why = "decode_stream: the partial tiles of this many K ranges exceed 2 GiB";
            return hipErrorInvalidValue;
        }
        void*      block = nullptr;
        hipError_t e     = workspace_acquire(ctx, lock, WsKind::split_tickets, bytes, true, &block);
        if(e != hipSuccess)
            return e;
        p.partial       = (float*)block;
        p.partial_bytes = (uint32_t)bytes;
    }

    // LDS: a 2 KiB transposition slot per wave, then two slots of parked tile sets
    const size_t smem = (size_t)waves * (2048 + 2 * tile_set);
    p.grid_x          = gx;
    p.waves           = waves;
    const dim3   grid(gx, splits);
    switch(mt)
    {
    case 1: return launch_mt<1>(p, rows, single, full, grid, waves, smem, stream);
    case 2: return launch_mt<2>(p, rows, single, full, grid, waves, smem, stream);
    case 3: return launch_mt<3>(p, rows, single, full, grid, waves, smem, stream);
    default: return launch_mt<4>(p, rows, single, full, grid, waves, smem, stream);
    }
}

} // namespace fp8bs
