// Block-scale FP8 mixture-of-experts: routing (softmax top-k), sorting of the routed
// (token, expert) pairs into per-expert blocks, and the two grouped GEMMs of a gated expert
//   h = act(x W_gate^T) * (x W_up^T),   y = h W_down^T,   out[token] += sum_k weight_k * y_k
// with fp8 e4m3fn operands, 1x128 activation scales and 128x128 weight scales.
//
// Semantics follow aiter/fused_moe.py (moe_sorting :341-416, fused_topk :4058-4130),
// op_tests/test_moe_sorting.py:44-105 (the sorted layout) and op_tests/test_moe_blockscale.py
// (torch_moe_blockscale :19-101, the arithmetic; asm_moe_test :130-162, the call).
//
// Layout of the sorted arrays: per expert, its (token, slot) pairs in ascending (token, slot)
// order as `slot << 24 | token`, padded with `topk << 24 | M` to a multiple of the block size;
// sorted_expert_ids holds one expert id per block; num_valid_ids = {padded total, M}.
//
// The GEMMs stream pre-shuffled (16,16) weights straight into MFMA operand registers: a 16-row
// tile's K block is 2 KiB of contiguous memory in fragment order, so no LDS staging is needed.
// A workgroup owns one block of 32 sorted rows (one expert).  First GEMM: 32 gate + 32 up
// columns, its 8 waves split K and add their partial tiles through LDS, the activation is applied
// and the product written as bf16; the 1x128 quantiser of the dense path then turns it into fp8.
// Second GEMM, up to 128 tokens: a workgroup owns 16 output columns of every expert and adds each
// token's weighted rows in LDS, in sorted order, then onto `out` (no intermediate rows at all).
// Beyond: waves x 128 columns, K = inter_dim; rows are written per sorted slot (one writer per
// element, fp32 while they take at most 32 MiB, else bf16), and a last kernel adds each token's
// slots in slot order, weighted, into `out`.  Both are deterministic, unlike atomic accumulation.
#include "gemm_common.h"
#include "moe_launch.h"

#include <algorithm>
#include <atomic>
#include <cmath>

namespace fp8bs {

namespace {

constexpr int kSortChunk = 4096;      // most (token, slot) pairs the one-workgroup sort takes
constexpr int kSortChunkMulti = 1024; // most pairs per workgroup (chunk) of the three-launch sort

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for(int o = 32; o > 0; o >>= 1)
        v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for(int o = 32; o > 0; o >>= 1)
        v += __shfl_xor(v, o);
    return v;
}

// ---------------------------------------------------------------------------------------------
// softmax + top-k, one wave per token.  Ties go to the lower expert index.
template <typename T>
__global__ __launch_bounds__(256) void topk_softmax_kernel(const T* __restrict__ gating, float* __restrict__ weights,
                                                           int32_t* __restrict__ ids, int32_t* __restrict__ src_rows,
                                                           int32_t tokens, int32_t experts, int32_t topk,
                                                           int64_t w_stride, int64_t id_stride, int renorm)
{
    constexpr int kMaxPerLane = 16; // experts <= 1024
    const int     lane = threadIdx.x & 63;
    const int     tok  = blockIdx.x * 4 + (threadIdx.x >> 6);
    if(tok >= tokens)
        return;
    const T* row = gating + (size_t)tok * experts;
    float    v[kMaxPerLane];
    float    mx = -INFINITY;
#pragma unroll
    for(int i = 0; i < kMaxPerLane; ++i)
    {
        const int e = i * 64 + lane;
        v[i]        = e < experts ? (float)row[e] : -INFINITY;
        mx          = fmaxf(mx, v[i]);
    }
    mx        = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for(int i = 0; i < kMaxPerLane; ++i)
    {
        v[i] = (i * 64 + lane) < experts ? expf(v[i] - mx) : -1.f; // -1: never selected
        sum += v[i] > 0.f ? v[i] : 0.f;
    }
    sum               = wave_sum(sum);
    const float inv   = 1.f / sum;
    float       picked = 0.f, my_w = 0.f;
    int         my_id = 0;
    for(int k = 0; k < topk; ++k)
    {
        float best = -1.f;
        int   bi   = 0x7fffffff;
#pragma unroll
        for(int i = 0; i < kMaxPerLane; ++i)
            if(v[i] > best) // ascending i = ascending expert index within a lane
            {
                best = v[i];
                bi   = i * 64 + lane;
            }
#pragma unroll
        for(int o = 32; o > 0; o >>= 1)
        {
            const float ob = __shfl_xor(best, o);
            const int   oi = __shfl_xor(bi, o);
            if(ob > best || (ob == best && oi < bi))
            {
                best = ob;
                bi   = oi;
            }
        }
        if((bi & 63) == lane)
        {
#pragma unroll
            for(int i = 0; i < kMaxPerLane; ++i)
                if(i == (bi >> 6))
                    v[i] = -1.f;
        }
        if(lane == k)
        {
            my_w  = best * inv;
            my_id = bi;
        }
        picked += best * inv;
    }
    if(lane < topk)
    {
        weights[(size_t)tok * w_stride + lane] = renorm ? my_w / picked : my_w;
        ids[(size_t)tok * id_stride + lane]    = my_id;
        if(src_rows)
            src_rows[(size_t)tok * topk + lane] = lane * tokens + tok;
    }
}

// ---------------------------------------------------------------------------------------------
// Sorting.  Three launches: per-chunk histograms; one workgroup that turns them into per-chunk
// write positions, block -> expert ids and the totals; a stable scatter, one wave per chunk, so
// that pairs keep their (token, slot) order.  Up to kSortChunk pairs one workgroup does it all.
struct SortParams
{
    const int32_t* topk_ids;     // [M][topk], row stride id_stride
    const float*   topk_weights; // [M][topk], row stride w_stride
    const int32_t* expert_mask;  // optional [experts], 0 = not local
    const int32_t* num_local_tokens; // optional device scalar: rows of topk_ids to sort
    int32_t*       sorted_ids;
    float*         sorted_weights;
    int32_t*       sorted_expert_ids;
    int32_t*       num_valid_ids;
    int32_t*       counts; // workspace [chunks][experts]: counts, then positions
    int32_t*       expert_begin; // workspace [experts + 1]: start of each expert's padded run
    int32_t        M, topk, experts, unit, chunks;
    int32_t        chunk_pairs; // pairs per chunk of the three-launch sort, <= kSortChunkMulti
    int32_t        w_rows; // rows of topk_weights (may be fewer than M when num_local_tokens says so)
    u32x4*         zero_dst;  // buffer to clear (may be null), by the workgroups behind the sorting ones
    size_t         zero_vecs; // its size in 16-byte units
    int32_t        max_padded, max_blocks;
    int64_t        id_stride, w_stride;
};

__device__ __forceinline__ int32_t sort_rows(const SortParams& p)
{
    int32_t rows = p.M;
    if(p.num_local_tokens)
    {
        const int32_t r = *p.num_local_tokens;
        rows            = r < 0 ? 0 : (r < rows ? r : rows);
    }
    return rows < p.w_rows ? rows : p.w_rows;
}

// The output buffer of the expert layer has to come back zeroed.  Rather than a launch of its own,
// the workgroups of the first sorting launch beyond the `first` that sort clear it.
__device__ __forceinline__ void zero_slice(const SortParams& p, int first)
{
    const size_t workers = (size_t)(gridDim.x - first) * blockDim.x;
    for(size_t i = (size_t)(blockIdx.x - first) * blockDim.x + threadIdx.x; i < p.zero_vecs; i += workers)
        p.zero_dst[i] = u32x4{0u, 0u, 0u, 0u};
}

__global__ __launch_bounds__(1024) void moe_sort_count_kernel(SortParams p)
{
    if((int)blockIdx.x >= p.chunks)
    {
        zero_slice(p, p.chunks);
        return;
    }
    extern __shared__ int32_t hist[];
    for(int e = threadIdx.x; e < p.experts; e += blockDim.x)
        hist[e] = 0;
    __syncthreads();
    const int64_t n = (int64_t)sort_rows(p) * p.topk;
    const int64_t lo = (int64_t)blockIdx.x * p.chunk_pairs;
    for(int i = threadIdx.x; i < p.chunk_pairs; i += blockDim.x)
    {
        const int64_t f = lo + i;
        if(f >= n)
            break;
        const int32_t e = p.topk_ids[(f / p.topk) * p.id_stride + (f % p.topk)];
        if(e >= 0 && e < p.experts)
            atomicAdd(&hist[e], 1);
    }
    __syncthreads();
    for(int e = threadIdx.x; e < p.experts; e += blockDim.x)
        p.counts[(size_t)blockIdx.x * p.experts + e] = hist[e];
}

// Exclusive scan over the experts (thread = expert, 1024 threads) of the padded run lengths and of
// the "is local" flags: where each expert's run starts (-1 if masked out), its local id, and the
// padded total.
struct ExpertSpan
{
    int32_t begin, local, total;
};
__device__ __forceinline__ ExpertSpan expert_spans(bool live, int32_t padded_len)
{
    __shared__ int64_t wave_total[16];
    int64_t       packed = ((int64_t)(live ? 1 : 0) << 40) | (int64_t)(live ? padded_len : 0);
    const int64_t mine   = packed;
#pragma unroll
    for(int o = 1; o < 64; o <<= 1)
    {
        const int64_t up = __shfl_up(packed, o);
        if((int)(threadIdx.x & 63) >= o)
            packed += up;
    }
    if((threadIdx.x & 63) == 63)
        wave_total[threadIdx.x >> 6] = packed;
    __syncthreads();
    int64_t base = 0, all = 0;
    for(int w = 0; w < 16; ++w)
    {
        if(w < (int)(threadIdx.x >> 6))
            base += wave_total[w];
        all += wave_total[w];
    }
    const int64_t excl = base + packed - mine;
    ExpertSpan    r;
    r.begin = live ? (int32_t)(excl & 0xffffffffffll) : -1;
    r.local = (int32_t)(excl >> 40);
    r.total = (int32_t)(all & 0xffffffffffll);
    return r;
}

__global__ __launch_bounds__(1024) void moe_sort_scan_kernel(SortParams p)
{
    const int e   = threadIdx.x;
    int32_t   run = 0;
    if(e < p.experts)
        for(int c0 = 0; c0 < p.chunks; c0 += 32) // 32 counts requested together: one round trip, not 32
        {
            int32_t n[32];
#pragma unroll
            for(int i = 0; i < 32; ++i)
                n[i] = c0 + i < p.chunks ? p.counts[(size_t)(c0 + i) * p.experts + e] : 0;
#pragma unroll
            for(int i = 0; i < 32; ++i)
                if(c0 + i < p.chunks)
                {
                    p.counts[(size_t)(c0 + i) * p.experts + e] = run; // position inside the expert's run
                    run += n[i];
                }
        }
    const bool       live = e < p.experts && !(p.expert_mask && p.expert_mask[e] == 0);
    const int32_t    len  = (run + p.unit - 1) / p.unit * p.unit;
    const ExpertSpan span = expert_spans(live, len);
    if(e == 0)
    {
        p.num_valid_ids[0] = span.total;
        p.num_valid_ids[1] = sort_rows(p);
    }
    const int32_t pad_id = (p.topk << 24) | p.M;
    if(e < p.experts)
    {
        p.expert_begin[e] = span.begin;
        if(live)
        {
            for(int b = 0; b < len / p.unit; ++b)
                p.sorted_expert_ids[span.begin / p.unit + b] = span.local;
            for(int i = run; i < len; ++i)
            {
                p.sorted_ids[span.begin + i]     = pad_id;
                p.sorted_weights[span.begin + i] = 0.f;
            }
        }
    }
    for(int b = span.total / p.unit + threadIdx.x; b < p.max_blocks; b += blockDim.x)
        p.sorted_expert_ids[b] = -1;
    for(int i = span.total + threadIdx.x; i < p.max_padded; i += blockDim.x)
    {
        p.sorted_ids[i]     = pad_id;
        p.sorted_weights[i] = 0.f;
    }
}

// Stable scatter of one chunk of (token, slot) pairs held in LDS, by one wave: 64 pairs at a time,
// a pair's rank among the earlier pairs of its expert comes from ballots over the bits of the
// expert id, and `running[e]` (LDS) carries the expert's fill level from one step to the next.
__device__ __forceinline__ void scatter_chunk(const SortParams& p, const int32_t* ids, const float* wts,
                                              const int32_t* begin, int32_t* running, int cnt, int64_t first)
{
    const int lane = threadIdx.x & 63;
    for(int base = 0; base < cnt; base += 64)
    {
        const int  i  = base + lane;
        const int  e  = i < cnt ? ids[i] : -1;
        const bool in = e >= 0 && e < p.experts && begin[e] >= 0;
        uint64_t   same = __ballot(in);
#pragma unroll
        for(int b = 0; b < 10; ++b)
        {
            const uint64_t bal = __ballot((e >> b) & 1);
            same &= ((e >> b) & 1) ? bal : ~bal;
        }
        if(in)
        {
            const int     rank = __popcll(same & ((1ull << lane) - 1ull));
            const int     n    = __popcll(same);
            const int32_t fill = running[e];
            const int32_t at   = begin[e] + fill + rank;
            const int64_t f    = first + i;
            p.sorted_ids[at]     = ((int32_t)(f % p.topk) << 24) | (int32_t)(f / p.topk);
            p.sorted_weights[at] = wts[i];
            if(rank == n - 1)
                running[e] = fill + n;
        }
    }
}

__global__ __launch_bounds__(64) void moe_sort_scatter_kernel(SortParams p)
{
    __shared__ int32_t ids[kSortChunkMulti];
    __shared__ float   wts[kSortChunkMulti];
    __shared__ int32_t begin[1024], running[1024];
    const int64_t      n  = (int64_t)sort_rows(p) * p.topk;
    const int64_t      lo = (int64_t)blockIdx.x * p.chunk_pairs;
    const int          cnt = (int)((n - lo) < p.chunk_pairs ? (n - lo > 0 ? n - lo : 0) : p.chunk_pairs);
    for(int i = threadIdx.x; i < cnt; i += blockDim.x)
    {
        const int64_t f = lo + i;
        ids[i]          = p.topk_ids[(f / p.topk) * p.id_stride + (f % p.topk)];
        wts[i]          = p.topk_weights[(f / p.topk) * p.w_stride + (f % p.topk)];
    }
    for(int e = threadIdx.x; e < p.experts; e += blockDim.x)
    {
        begin[e]   = p.expert_begin[e];
        running[e] = p.counts[(size_t)blockIdx.x * p.experts + e];
    }
    __syncthreads();
    scatter_chunk(p, ids, wts, begin, running, cnt, lo);
}

// All of it in one workgroup, for up to kSortChunk pairs (the decode regime).  The pairs are cut
// into kSortWaves contiguous runs, one per wave: histograms per run (LDS), a scan over the experts
// and, per expert, over the runs, then every wave scatters its own run, starting each expert at
// the fill level the earlier runs leave -- the (token, slot) order of the pairs is kept.
constexpr int kSortWaves = 8;
constexpr int kSortRunSteps = kSortChunk / kSortWaves / 64; // 64-pair steps of the longest run

// scatter_chunk for one run of the one-workgroup sort: the weights come from memory, all of the
// run's requested before the first step (they would otherwise cost a round trip per step)
__device__ __forceinline__ void scatter_run(const SortParams& p, const int32_t* ids, const int32_t* begin,
                                            int32_t* running, int cnt, int first)
{
    const int lane = threadIdx.x & 63;
    float     w[kSortRunSteps];
#pragma unroll
    for(int st = 0; st < kSortRunSteps; ++st)
    {
        const int f = first + st * 64 + lane;
        w[st]       = st * 64 + lane < cnt ? p.topk_weights[(size_t)(f / p.topk) * p.w_stride + (f % p.topk)] : 0.f;
    }
#pragma unroll
    for(int st = 0; st < kSortRunSteps; ++st)
    {
        if(st * 64 >= cnt)
            break;
        const int  i  = st * 64 + lane;
        const int  e  = i < cnt ? ids[i] : -1;
        const bool in = e >= 0 && e < p.experts && begin[e] >= 0;
        uint64_t   same = __ballot(in);
#pragma unroll
        for(int b = 0; b < 10; ++b)
        {
            const uint64_t bal = __ballot((e >> b) & 1);
            same &= ((e >> b) & 1) ? bal : ~bal;
        }
        if(in)
        {
            const int     rank = __popcll(same & ((1ull << lane) - 1ull));
            const int     n    = __popcll(same);
            const int32_t fill = running[e];
            const int32_t at   = begin[e] + fill + rank;
            const int     f    = first + i;
            p.sorted_ids[at]     = ((int32_t)(f % p.topk) << 24) | (int32_t)(f / p.topk);
            p.sorted_weights[at] = w[st];
            if(rank == n - 1)
                running[e] = fill + n;
        }
    }
}

__global__ __launch_bounds__(1024) void moe_sort_single_kernel(SortParams p)
{
    if(blockIdx.x > 0)
    {
        zero_slice(p, 1);
        return;
    }
    __shared__ int32_t ids[kSortChunk];
    __shared__ int32_t fill[kSortWaves][1024]; // per run: the expert's count, then its fill level
    __shared__ int32_t count[1024], begin[1024], local[1024];
    __shared__ int32_t s_total;
    const int rows = sort_rows(p);
    const int cnt  = rows * p.topk; // <= kSortChunk, checked at launch
    const int run_len = ((cnt + kSortWaves - 1) / kSortWaves + 63) / 64 * 64;
    for(int i = threadIdx.x; i < kSortWaves * 1024; i += blockDim.x)
        (&fill[0][0])[i] = 0;
    __syncthreads();
    for(int i = threadIdx.x; i < cnt; i += blockDim.x)
    {
        const int     r = i / p.topk, k = i - r * p.topk;
        const int32_t e = p.topk_ids[(size_t)r * p.id_stride + k];
        ids[i]          = e;
        if(e >= 0 && e < p.experts)
            atomicAdd(&fill[i / run_len][e], 1);
    }
    __syncthreads();
    if((int)threadIdx.x < p.experts)
    {
        int32_t run = 0;
#pragma unroll
        for(int w = 0; w < kSortWaves; ++w)
        {
            const int32_t n       = fill[w][threadIdx.x];
            fill[w][threadIdx.x] = run;
            run += n;
        }
        count[threadIdx.x] = run;
    }
    const bool       live_e = (int)threadIdx.x < p.experts && !(p.expert_mask && p.expert_mask[threadIdx.x] == 0);
    const int32_t    len_e  = (int)threadIdx.x < p.experts ? (count[threadIdx.x] + p.unit - 1) / p.unit * p.unit : 0;
    const ExpertSpan span   = expert_spans(live_e, len_e);
    const int32_t pad_id    = (p.topk << 24) | p.M;
    if((int)threadIdx.x < p.experts)
    {
        begin[threadIdx.x] = span.begin;
        if(span.begin >= 0)
        {
            for(int b = 0; b < len_e / p.unit; ++b)
                p.sorted_expert_ids[span.begin / p.unit + b] = span.local;
            for(int32_t at = span.begin + count[threadIdx.x]; at < span.begin + len_e; ++at)
            {
                p.sorted_ids[at]     = pad_id;
                p.sorted_weights[at] = 0.f;
            }
        }
    }
    if(threadIdx.x == 0)
    {
        s_total            = span.total;
        p.num_valid_ids[0] = span.total;
        p.num_valid_ids[1] = rows;
    }
    __syncthreads();
    const int32_t total = s_total;
    const int     wave  = threadIdx.x >> 6;
    if(wave < kSortWaves)
    {
        const int lo = wave * run_len;
        const int n  = cnt - lo < run_len ? cnt - lo : run_len;
        if(n > 0)
            scatter_run(p, ids + lo, begin, fill[wave], n, lo);
    }
    for(int b = total / p.unit + threadIdx.x; b < p.max_blocks; b += blockDim.x)
        p.sorted_expert_ids[b] = -1;
    for(int i = total + threadIdx.x; i < p.max_padded; i += blockDim.x)
    {
        p.sorted_ids[i]     = pad_id;
        p.sorted_weights[i] = 0.f;
    }
}


// ---------------------------------------------------------------------------------------------
// The two grouped GEMMs.

// What the second GEMM needs to know about a sorted row besides its activations, in one 32-byte
// record (one cache line touched instead of three): floats 0..3 the row's 1x128 scales (written by
// the quantiser), float 4 its routing weight, float 5 its token id as bits (written by the first
// GEMM).  Used while inter_dim / 128 <= 4.
constexpr int kRowInfo = 8;

struct MoeGemmParams
{
    const uint8_t* xq;   // first GEMM: [M][K] fp8 tokens (row stride lda); second: [slots][K] by sorted slot
    const float*   xs;   // first: [K/128][M]; second: [slots][xs_stride], a slot's K/128 scales first
    const uint8_t* w;    // [experts][N][K] fp8, pre-shuffled (16,16) per expert
    const float*   wsc;  // [experts][N/128][K/128]
    const int32_t* sorted_ids;
    const int32_t* sorted_expert_ids;
    const int32_t* num_valid;
    uint16_t*      out;  // first: [slots][inter] bf16; second: [slots][N] bf16 or fp32
    int32_t        M, K, N, inter, kblocks, n_groups, max_blocks, experts, activation;
    int32_t        out_f32; // second GEMM only: rows kept in fp32
    int32_t        topk;
    int32_t        waves;   // second GEMM only: waves per workgroup
    int32_t        wave_cols; // second GEMM only: columns per wave (64 or 128)
    int32_t        out_staged; // second GEMM only: 16-bit rows leave through LDS as whole 128-byte lines
    int32_t        gate_ring;  // first GEMM, pairs of blocks: weights two K blocks ahead through LDS (gate_up_ring_body)
    int32_t*       where;   // first GEMM only: [M][topk] sorted position of each (token, slot) pair
    uint32_t*      block_mask; // first GEMM only: [blocks] bit r set = row r of the block is a real pair
    float*         row_info;   // first GEMM only: [slots][kRowInfo] records, see below (null: not wanted)
    const float*   sorted_weights; // first GEMM only, for row_info
    int32_t        xs_stride;  // second GEMM only: floats between the scale rows of two slots
    int32_t        block_rows;   // sorted rows a workgroup's block covers: 32, or 16 when the arrays were sorted in blocks of 16
    int32_t        expert_shift; // such a block's entry in sorted_expert_ids is block >> expert_shift (sorting blocks of 64, 128)
    int32_t        pair_blocks;  // two consecutive blocks of one expert are multiplied together (many rows per expert)
    int32_t        fine_blocks;  // first GEMM, NT = 4: the blocks taken last that are cut into 16-column workgroups
    int64_t        lda;
};

// fragment of a pre-shuffled weight tile's K block: 2 KiB, lane (l16, kg) takes the 16 bytes at
// kg*512 + l16*16 and the 16 bytes 256 further on.  STREAM: the expert's weights are read by this
// block of rows only, so the loads are non-temporal (long-lived workgroups that stream with
// ordinary loads reach 5.7 TB/s here, with non-temporal ones 6.3-6.5 TB/s, whatever the order in
// which a workgroup walks its tiles); an expert with several blocks is read with ordinary loads,
// which let the later blocks find the weights in a cache.
template <bool STREAM>
__device__ __forceinline__ i32x8 load_w_fragment(const uint8_t* tile_kb, int l16, int kg)
{
    const i32x4* lo_at = (const i32x4*)(tile_kb + kg * 512 + l16 * 16);
    const i32x4* hi_at = (const i32x4*)(tile_kb + kg * 512 + 256 + l16 * 16);
    const i32x4  lo    = STREAM ? __builtin_nontemporal_load(lo_at) : *lo_at;
    const i32x4  hi    = STREAM ? __builtin_nontemporal_load(hi_at) : *hi_at;
    return i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}
// fragment of a row-major activation row's K block: 32 contiguous bytes at kg*32
__device__ __forceinline__ i32x8 load_x_fragment(const uint8_t* row_kb, int kg)
{
    const i32x4 lo = *(const i32x4*)(row_kb + kg * 32);
    const i32x4 hi = *(const i32x4*)(row_kb + kg * 32 + 16);
    return i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

__device__ __forceinline__ float activate(float g, int activation)
{
    if(activation == 0) // silu
        return g / (1.f + expf(-g));
    return 0.5f * g * (1.f + erff(g * 0.70710678118654752f)); // gelu (erf form)
}

// whether block `blk` is the only block of rows of its expert (its neighbours in the sorted order
// belong to other experts or lie past the valid rows): its weights are then read once
__device__ __forceinline__ bool only_block_of_its_expert(const MoeGemmParams& p, int blk, int expert)
{
    const bool prev = blk > 0 && p.sorted_expert_ids[(blk - 1) >> p.expert_shift] == expert;
    const bool next = (blk + 1) * p.block_rows < p.num_valid[0] && p.sorted_expert_ids[(blk + 1) >> p.expert_shift] == expert;
    return !prev && !next;
}

// Where block `blk` stands among the consecutive blocks of its expert in the sorted order: how many
// come before it, and whether one and two more follow.  Every lane of the calling wave gets the
// same answer from one request in the usual case (lanes 0 and 1 look at the next two blocks, lanes
// 2 .. 63 at the 62 blocks before; longer runs are followed 64 blocks at a time).
struct RunOfBlocks
{
    int  before;
    bool next, next2;
    // the only block of its expert: its weights are read once
    __device__ bool alone() const { return before == 0 && !next; }
};
// (blocks below `lo` do not count: they are multiplied on their own)
__device__ __forceinline__ RunOfBlocks run_of_blocks(const MoeGemmParams& p, int blk, int expert, int lo = 0)
{
    const int      lane  = threadIdx.x & 63, valid = p.num_valid[0];
    const int      b0    = lane < 2 ? blk + 1 + lane : blk + 1 - lane;
    const bool     in0   = lane < 2 ? b0 * p.block_rows < valid : b0 >= lo;
    const bool     same0 = in0 && p.sorted_expert_ids[(in0 ? b0 : blk) >> p.expert_shift] == expert;
    const uint64_t m0    = __ballot(same0);
    RunOfBlocks    r{0, (m0 & 1) != 0, (m0 & 3) == 3};
    const uint64_t back  = m0 >> 2 | (uint64_t)3 << 62;
    r.before             = back == ~(uint64_t)0 ? 62 : __builtin_ctzll(~back);
    bool more = r.before == 62;
    while(more)
    {
        const int      b    = blk - 1 - r.before - lane;
        const bool     same = b >= lo && p.sorted_expert_ids[(b >= lo ? b : lo) >> p.expert_shift] == expert;
        const uint64_t m    = __ballot(same);
        const int      run  = m == ~(uint64_t)0 ? 64 : __builtin_ctzll(~m);
        r.before += run;
        more = run == 64;
    }
    return r;
}

// Pairs of blocks (pair_blocks: set by the launcher where an expert has many rows).  Blocks 2i and
// 2i + 1 of an expert's run are multiplied together by the workgroups of both: each takes half of
// its columns, for the rows of both blocks, so that the expert's weights are read once per pair.
// For the block at `blk`: whether it has a partner, the pair's first block, which half this
// workgroup takes, and whether the pair is the expert's whole run (its weights are read once).
struct PairOfBlocks
{
    bool paired;
    int  first, half;
    bool once;
};
__device__ __forceinline__ PairOfBlocks pair_of_blocks(const MoeGemmParams& p, const RunOfBlocks& run, int blk)
{
    const bool odd = run.before & 1;
    PairOfBlocks q{p.pair_blocks && p.block_rows == 32 && (odd || run.next), blk - (odd ? 1 : 0), odd ? 1 : 0, false};
    q.once = odd ? run.before == 1 && !run.next : run.before == 0 && !run.next2;
    return q;
}

// First GEMM + activation.  Workgroup = (block of 32 sorted rows, NT x 16 inter columns): NT
// gate tiles and the NT matching up tiles; NT is picked at launch (wide units, which re-read the
// activations less often, where they cover the chip and their last round of workgroups is expected
// to be reasonably full; the narrowest otherwise, so that the last units to finish do not set the
// kernel's duration).  The waves take every eighth K
// block each and add their partial tiles through LDS in wave order.  One operand set per wave:
// several workgroups share a compute unit and cover each other's load latency.  A block whose
// second half is padding (the usual case when few tokens are routed) multiplies one 16-row tile
// only.  MFMA roles as in the dense kernels: weight rows are the "A" operand, activation rows
// the "B" operand, so a lane ends up with 4 consecutive columns of one row.
// waves per workgroup of the first GEMM: each keeps one K block of its tiles in flight, and a
// workgroup that has a compute unit to itself (the last units of a launch) should still stream at
// the unit's share of HBM
constexpr int kGateUpWaves = 8;
constexpr int kChipCus     = 256;

// The eight waves' sums of a block meet in LDS, all MT row tiles at once: red[row tile][wave][n tile][lane][c]
// (MT x NT x 16 KiB), and wave NT j + i adds up the pair (gate tile i, up tile NT + i) of row tile j in wave
// order (the sum does not depend on timing), applies the activation and stores the product.  One row tile
// after the other, with NT of the eight waves at work, a compute unit that holds a single workgroup requested
// nothing for as many rounds as there are row tiles.
constexpr size_t gate_up_red_bytes(int mt, int nt) { return (size_t)mt * kGateUpWaves * 2 * nt * 64 * 16; }
template <int MT, int NT>
__device__ __forceinline__ void gate_up_finish(const MoeGemmParams& p, float* red, const f32x4 (&acc)[MT][2 * NT], int blk, int grp)
{
    static_assert(MT * NT <= kGateUpWaves, "a wave per (row tile, column pair)");
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, l16 = lane & 15, kg = lane >> 4;
#pragma unroll
    for(int j = 0; j < MT; ++j)
#pragma unroll
        for(int q = 0; q < 2 * NT; ++q)
            *(f32x4*)(red + ((((size_t)j * kGateUpWaves + wave) * (2 * NT) + q) * 64 + lane) * 4) = acc[j][q];
    __syncthreads();
    const int j = wave / NT, i = wave % NT;
    if(j < MT)
    {
        f32x4 g = f32x4{0.f, 0.f, 0.f, 0.f}, u = g;
#pragma unroll
        for(int w = 0; w < kGateUpWaves; ++w)
        {
            g += *(const f32x4*)(red + ((((size_t)j * kGateUpWaves + w) * (2 * NT) + i) * 64 + lane) * 4);
            u += *(const f32x4*)(red + ((((size_t)j * kGateUpWaves + w) * (2 * NT) + NT + i) * 64 + lane) * 4);
        }
        float h[4];
#pragma unroll
        for(int c = 0; c < 4; ++c)
            h[c] = activate(g[c], p.activation) * u[c];
        const int slot = blk * p.block_rows + j * 16 + l16;
        const int col  = (grp * NT + i) * 16 + kg * 4;
        *(u32x2*)(p.out + (size_t)slot * p.inter + col) =
            u32x2{pack2<In16::bf16>(h[0], h[1]), pack2<In16::bf16>(h[2], h[3])};
    }
}

template <int MT, int NT, bool STREAM>
__device__ __forceinline__ void gate_up_body(const MoeGemmParams& p, float* red, int blk, int grp, int expert)
{
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, l16 = lane & 15, kg = lane >> 4;
    const uint8_t* xrow[MT];
    const float*   xsr[MT];
#pragma unroll
    for(int j = 0; j < MT; ++j)
    {
        const int id  = p.sorted_ids[blk * p.block_rows + j * 16 + l16] & 0xffffff;
        const int tok = id < p.M ? id : 0; // padding rows compute on token 0 and are never read
        xrow[j]       = p.xq + (size_t)tok * p.lda;
        xsr[j]        = p.xs + tok;
    }
    const size_t   tile_stride = (size_t)16 * (size_t)p.K;
    const size_t   wexp = (size_t)expert * (size_t)p.N * (size_t)p.K;
    const uint8_t* wg   = p.w + wexp + (size_t)(grp * NT) * tile_stride;
    const uint8_t* wu   = p.w + wexp + (size_t)((p.inter >> 4) + grp * NT) * tile_stride;
    const float*   ws_gate = p.wsc + ((size_t)expert * (p.N / 128) + (grp * NT * 16) / 128) * p.kblocks;
    const float*   ws_up   = p.wsc + ((size_t)expert * (p.N / 128) + (p.inter + grp * NT * 16) / 128) * p.kblocks;

    f32x4 acc[MT][2 * NT];
#pragma unroll
    for(int j = 0; j < MT; ++j)
#pragma unroll
        for(int i = 0; i < 2 * NT; ++i)
            acc[j][i] = f32x4{0.f, 0.f, 0.f, 0.f};

    for(int kb = wave; kb < p.kblocks; kb += kGateUpWaves)
    {
        i32x8 w[2 * NT], x[MT];
        float xs[MT];
#pragma unroll
        for(int i = 0; i < NT; ++i)
        {
            w[i]      = load_w_fragment<STREAM>(wg + i * tile_stride + (size_t)kb * 2048, l16, kg);
            w[NT + i] = load_w_fragment<STREAM>(wu + i * tile_stride + (size_t)kb * 2048, l16, kg);
        }
#pragma unroll
        for(int j = 0; j < MT; ++j)
        {
            x[j]  = load_x_fragment(xrow[j] + (size_t)kb * 128, kg);
            xs[j] = xsr[j][(size_t)kb * p.M];
        }
        const float sg = ws_gate[kb], su = ws_up[kb];
#pragma unroll
        for(int j = 0; j < MT; ++j)
#pragma unroll
            for(int i = 0; i < 2 * NT; ++i)
            {
                const f32x4 prod = mfma_16x16x128_fp8(w[i], x[j], f32x4{0.f, 0.f, 0.f, 0.f});
                const float sc   = xs[j] * (i < NT ? sg : su);
#pragma unroll
                for(int c = 0; c < 4; ++c)
                    acc[j][i][c] = __builtin_fmaf(prod[c], sc, acc[j][i][c]);
            }
    }

    gate_up_finish<MT, NT>(p, red, acc, blk, grp);
}

// The first GEMM for a pair of blocks (NT = 2: two gate tiles and their up tiles, MT = 3 or 4 row tiles), with
// the weights two K blocks ahead.
//
// In gate_up_body a wave asks for a K block, waits, multiplies, and has nothing in flight while it multiplies.
// With 16 MFMAs and 64 FMAs per 8 KiB of weights and eight waves per compute unit (the registers allow no more)
// that launch is bound by the latency of its loads: 4.9 TB/s at 1024 tokens where the narrower bodies, with
// twice the bytes per request, stream at 6.3.  Requesting the next K block into a second set of registers does
// not fit (256 registers and 407 spilled).  Here the weights travel through LDS instead: every wave owns two
// stages of 8 KiB that direct global->LDS loads fill (global_load_lds_dwordx4: no registers while in flight),
// so the weights of K blocks i + 1 and i + 2 are on their way while block i is multiplied; the token rows and
// their scales of block i + 1 are requested into a second set of registers.
//
// Loads return in order, so the order of issue decides what a wait can leave in flight:
//   ids W(0) W(1) X(0) | X(1) W(2) | X(2) W(3) | ...    (X: 3 MT register loads, W: 8 LDS-direct loads)
// Iteration i > 0 needs X(i) and W(i); the only younger loads are W(i + 1)'s eight: s_waitcnt vmcnt(8) (0 when
// there is no W(i + 1), and in iteration 0, whose X is the youngest).  It then copies W(i) from its stage into registers, which frees the stage for
// W(i + 2).  All of these loads are issued from asm, invisible to the compiler's wait counts; the compiler
// itself issues no vector memory loads inside the loop.  Products, scales and their order are those of
// gate_up_body: same bits.
// a pointer that is the same in every lane, said so to the compiler (asm operands that must be scalar registers)
template <typename T>
__device__ __forceinline__ const T* uniform_ptr(const T* ptr)
{
    const uint64_t v  = (uint64_t)(uintptr_t)ptr;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const T*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

constexpr int kRingStageBytes = 4 * 2048;                                  // four 16-row tiles of one K block
constexpr int kRingLdsBytes   = kGateUpWaves * 2 * kRingStageBytes;        // two stages per wave: 128 KiB

template <int MT, bool STREAM>
__device__ __forceinline__ void gate_up_ring_body(const MoeGemmParams& p, uint8_t* lds, int blk, int grp, int expert)
{
    constexpr int NT = 2;
    const int t = threadIdx.x, lane = t & 63, l16 = lane & 15, kg = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6); // scalar: K blocks, stages and scale addresses derive from it
    typedef uint8_t __attribute__((address_space(3)))*              lds_byte_ptr;
    typedef const volatile i32x4 __attribute__((address_space(3)))* lds_vec_ptr;
    const lds_byte_ptr lds3 = (lds_byte_ptr)lds;

    // The rows' token ids are asked for first (from asm as well: a load the compiler knows of would make it
    // wait for everything issued before its use), so that the first weights can be requested while they travel.
    int      row_id[MT];
    uint32_t xoff[MT], xsoff[MT]; // per-lane byte offsets of the token rows and of their scales, once the ids are here
    {
        const int32_t* ids = uniform_ptr(p.sorted_ids);
#pragma unroll
        for(int j = 0; j < MT; ++j)
        {
            const uint32_t at = (uint32_t)(blk * p.block_rows + j * 16 + l16) * 4u;
            asm volatile("global_load_dword %0, %1, %2" : "=v"(row_id[j]) : "v"(at), "s"(ids) : "memory");
        }
    }
    const size_t   tile_stride = (size_t)16 * (size_t)p.K;
    const size_t   wexp = (size_t)expert * (size_t)p.N * (size_t)p.K;
    const uint8_t* wt[2 * NT]; // uniform: the wave's four tiles (gate, gate, up, up)
#pragma unroll
    for(int i = 0; i < NT; ++i)
    {
        wt[i]      = p.w + wexp + (size_t)(grp * NT + i) * tile_stride;
        wt[NT + i] = p.w + wexp + (size_t)((p.inter >> 4) + grp * NT + i) * tile_stride;
    }
    // (read through the constant address space at scalar addresses, i.e. with scalar loads: a vector load here
    // would make the compiler wait for every load in flight)
    typedef const float __attribute__((address_space(4)))* const_f32_ptr;
    const const_f32_ptr ws_gate = (const_f32_ptr)(uintptr_t)uniform_ptr(p.wsc + ((size_t)expert * (p.N / 128) + (grp * NT * 16) / 128) * p.kblocks);
    const const_f32_ptr ws_up   = (const_f32_ptr)(uintptr_t)uniform_ptr(p.wsc + ((size_t)expert * (p.N / 128) + (p.inter + grp * NT * 16) / 128) * p.kblocks);

    const uint32_t stage0   = (uint32_t)(uintptr_t)(lds3 + wave * (2 * kRingStageBytes));
    const uint32_t lane16   = (uint32_t)lane * 16u, lane16b = lane16 + 1024u;
    const uint32_t frag_off = (uint32_t)kg * 512u + (uint32_t)l16 * 16u;

    // W(kb) -> stage: per tile two loads of 1 KiB (lane l's 16 bytes land at M0 + 16 l)
    auto issue_w = [&](int kb, int stage) {
#pragma unroll
        for(int i = 0; i < 2 * NT; ++i)
        {
            const uint8_t* base = uniform_ptr(wt[i] + (size_t)kb * 2048);
            const uint32_t dst  = __builtin_amdgcn_readfirstlane(stage0 + (uint32_t)stage * kRingStageBytes + (uint32_t)i * 2048u);
            if constexpr(STREAM)
            {
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(dst), "v"(lane16), "s"(base) : "memory");
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(dst + 1024u), "v"(lane16b), "s"(base) : "memory");
            }
            else
            {
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(lane16), "s"(base) : "memory");
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst + 1024u), "v"(lane16b), "s"(base) : "memory");
            }
        }
    };
    struct Rows
    {
        i32x4 lo[MT], hi[MT];
        float xs[MT];
    };
    // X(kb) -> registers (not valid before the wait that names them)
    auto issue_x = [&](int kb, Rows& r) {
        const uint8_t* xbase  = uniform_ptr(p.xq + (size_t)kb * 128);
        const float*   xsbase = uniform_ptr(p.xs + (size_t)kb * p.M);
#pragma unroll
        for(int j = 0; j < MT; ++j)
        {
            asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(r.lo[j]) : "v"(xoff[j]), "s"(xbase) : "memory");
            asm volatile("global_load_dwordx4 %0, %1, %2 offset:16" : "=v"(r.hi[j]) : "v"(xoff[j]), "s"(xbase) : "memory");
            asm volatile("global_load_dword %0, %1, %2" : "=v"(r.xs[j]) : "v"(xsoff[j]), "s"(xsbase) : "memory");
        }
    };
    // the wait of an iteration: everything but the eight youngest loads (W of the next K block) has arrived
    auto arrived = [&](Rows& r, bool next_w_in_flight) {
        if(next_w_in_flight)
            asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        for(int j = 0; j < MT; ++j)
            asm volatile("" : "+v"(r.lo[j]), "+v"(r.hi[j]), "+v"(r.xs[j]));
    };

    f32x4 acc[MT][2 * NT];
#pragma unroll
    for(int j = 0; j < MT; ++j)
#pragma unroll
        for(int i = 0; i < 2 * NT; ++i)
            acc[j][i] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int n = wave < p.kblocks ? (p.kblocks - wave + kGateUpWaves - 1) / kGateUpWaves : 0; // this wave's K blocks
    auto kb_of = [&](int i) { return wave + i * kGateUpWaves; };

    auto step = [&](int i, Rows& cur, Rows& nxt) {
        arrived(cur, i > 0 && i + 1 < n);
        i32x8 w[2 * NT];
#pragma unroll
        for(int q = 0; q < 2 * NT; ++q)
        {
            const uint32_t at = (uint32_t)(wave * (2 * kRingStageBytes) + (i & 1) * kRingStageBytes + q * 2048) + frag_off;
            const i32x4    lo = *(lds_vec_ptr)(lds3 + at);
            const i32x4    hi = *(lds_vec_ptr)(lds3 + at + 256);
            w[q]              = i32x8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
        // the fragments are in registers (the compiler waits for its LDS reads here): the stage is free
#pragma unroll
        for(int q = 0; q < 2 * NT; ++q)
            asm volatile("" : "+v"(w[q]));
        if(i + 1 < n)
            issue_x(kb_of(i + 1), nxt);
        if(i + 2 < n)
            issue_w(kb_of(i + 2), i & 1);
        const int   kb = kb_of(i);
        const float sg = ws_gate[kb], su = ws_up[kb];
#pragma unroll
        for(int j = 0; j < MT; ++j)
        {
            const i32x8 x = i32x8{cur.lo[j][0], cur.lo[j][1], cur.lo[j][2], cur.lo[j][3],
                                  cur.hi[j][0], cur.hi[j][1], cur.hi[j][2], cur.hi[j][3]};
#pragma unroll
            for(int q = 0; q < 2 * NT; ++q)
            {
                const f32x4 prod = mfma_16x16x128_fp8(w[q], x, f32x4{0.f, 0.f, 0.f, 0.f});
                const float sc   = cur.xs[j] * (q < NT ? sg : su);
#pragma unroll
                for(int c = 0; c < 4; ++c)
                    acc[j][q][c] = __builtin_fmaf(prod[c], sc, acc[j][q][c]);
            }
        }
    };

    // ids | W(0) W(1) | wait for the ids | X(0): the first iteration waits for everything
    Rows ra, rb;
    if(n > 0)
        issue_w(kb_of(0), 0);
    if(n > 1)
        issue_w(kb_of(1), 1);
    if(n > 1)
        asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    else if(n > 0)
        asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // the token rows: 32 bytes of every K block per lane
#pragma unroll
    for(int j = 0; j < MT; ++j)
    {
        asm volatile("" : "+v"(row_id[j]));
        const int id  = row_id[j] & 0xffffff;
        const int tok = id < p.M ? id : 0; // padding rows compute on token 0 and are never read
        xoff[j]       = (uint32_t)tok * (uint32_t)p.lda + (uint32_t)kg * 32u;
        xsoff[j]      = (uint32_t)tok * 4u;
    }
    if(n > 0)
        issue_x(kb_of(0), ra);
    for(int i = 0; i < n; i += 2)
    {
        step(i, ra, rb);
        if(i + 1 < n)
            step(i + 1, rb, ra);
    }
    // the sums meet where the stages were: every wave must be done with its stages first
    __syncthreads();
    gate_up_finish<MT, NT>(p, (float*)lds, acc, blk, grp);
}

// LDS of an instance: two row tiles of its own width, or (pairs) four of half the width, which is the ring's size
constexpr size_t gate_up_lds_bytes(int nt, bool pairs)
{
    return pairs ? (gate_up_red_bytes(4, 2) > (size_t)kRingLdsBytes ? gate_up_red_bytes(4, 2) : (size_t)kRingLdsBytes) : gate_up_red_bytes(2, nt);
}

// PAIRS: the instance that can multiply pairs of blocks, kept apart from the usual one (which needs
// fewer registers and only looks at a block's two neighbours)
template <int NT, bool PAIRS>
__global__ __launch_bounds__(64 * kGateUpWaves) void moe_gate_up_kernel(MoeGemmParams p)
{
    // dynamic LDS: the reduction buffer of the widest body of the instance (gate_up_lds_bytes), which in the
    // pairs instance is also the ring of gate_up_ring_body
    extern __shared__ __attribute__((aligned(1024))) uint8_t gate_up_lds[];
    float* const red_dyn = (float*)gate_up_lds;
    // Blocks are taken from the last valid one down: the experts with the highest ids come first.  A
    // shared expert, which every token is routed to and which conventionally has the last id, has the
    // most blocks, each of two full row tiles and read with ordinary loads: started first, they are not
    // what the launch ends on.
    // Wide units (NT = 4) occupy a compute unit each, so they run in rounds of kChipCus, and a last round
    // that is nearly empty still takes a unit's streaming time.  When the wide units of the valid blocks
    // leave such a remainder -- at most fine_blocks blocks' worth, a quarter of a round -- the blocks of
    // the remainder (the ones taken last) go out as narrow units of 16 columns instead, which the launch
    // reserves workgroups for behind the wide ones: the launch then ends on one short round.  Decided
    // here from the number of valid blocks, which the host does not know (DeepSeek-V3 layer, remainder
    // of 2-16 % of a round: 5-9 us of 240-270; a remainder of 60 % and more treated the same way costs 2-5).
    //
    //
    // Which block a workgroup takes.  Workgroups go round-robin over the 8 XCDs, each with an L2 of its own, and
    // the column groups of a block all gather the block's token rows: with consecutive workgroups on one block
    // every XCD fetches those rows for itself (1024 tokens: 1215 MB fetched for 943 MB of weights and 7 MB of
    // tokens).  In the instance for many rows per expert, workgroup w therefore takes block
    // 8 (w / 8 / n_groups) + w % 8 and column group (w / 8) % n_groups: a block's column groups all run on XCD
    // (block % 8) and its rows are fetched into one L2 (1024 tokens: 373.6 -> 369.0 us).  With fewer rows the
    // extra fetches are few and the plain order is as good or better (256 tokens: 245.2 us against 247.9).
    const int valid_blocks = (p.num_valid[0] + p.block_rows - 1) / p.block_rows;
    const int slot8 = (int)blockIdx.x >> 3;
    int       at  = PAIRS ? (slot8 / p.n_groups) * 8 + ((int)blockIdx.x & 7) : (int)blockIdx.x / p.n_groups;
    int       grp = PAIRS ? slot8 % p.n_groups : (int)blockIdx.x - at * p.n_groups;
    bool      fine = false;
    int       tail = 0; // blocks 0 .. tail - 1 are the remainder
    if constexpr(NT == 4)
    {
        const int left = (valid_blocks * p.n_groups) % kChipCus, left_blocks = (left + p.n_groups - 1) / p.n_groups;
        tail           = left_blocks <= p.fine_blocks && valid_blocks * p.n_groups > kChipCus ? left_blocks : 0;
        const int wide = ((p.max_blocks + 7) & ~7) * p.n_groups; // as the launch counts them
        if((int)blockIdx.x >= wide)
        {
            const int j = (int)blockIdx.x - wide, narrow_groups = 4 * p.n_groups;
            at          = valid_blocks - tail + j / narrow_groups;
            grp         = j % narrow_groups;
            fine        = true;
            if(j / narrow_groups >= tail)
                return;
        }
        else if(at >= valid_blocks - tail)
            return;
    }
    const int blk = valid_blocks - 1 - at;
    if(blk < 0)
        return;
    const int expert = p.sorted_expert_ids[blk >> p.expert_shift];
    if(expert < 0 || expert >= p.experts)
        return;
    if(grp == 0 && threadIdx.x < 64) // record which rows are real pairs, and where each pair sits, for the final sum
    {
        bool real = false;
        if((int)threadIdx.x < p.block_rows)
        {
            const int at = blk * p.block_rows + threadIdx.x;
            const int id = p.sorted_ids[at], token = id & 0xffffff, slot = (id >> 24) & 0xff;
            real         = token < p.M && slot < p.topk;
            if(real && p.where)
                p.where[(size_t)token * p.topk + slot] = at;
            if(p.row_info)
            {
                p.row_info[(size_t)at * kRowInfo + 4] = p.sorted_weights[at];
                p.row_info[(size_t)at * kRowInfo + 5] = __int_as_float(real ? token : p.M);
            }
        }
        const uint64_t rows = __ballot(real);
        if(threadIdx.x == 0 && p.block_mask)
            p.block_mask[blk] = (uint32_t)rows;
    }
    // rows of a block are real pairs first, padding after: the second 16 rows matter only if row 16 is real
    const bool second_half = p.block_rows == 32 && (p.sorted_ids[blk * 32 + 16] & 0xffffff) < p.M;
    bool once;
    if constexpr(PAIRS && NT == 4)
    {
        // (the blocks of the remainder stay out of the pairs: they are multiplied as narrow units)
        const RunOfBlocks  run = run_of_blocks(p, blk, expert, fine ? 0 : tail);
        const PairOfBlocks pr  = pair_of_blocks(p, run, blk);
        if(pr.paired && !fine)
        {
            // half as many columns (two gate tiles and their up tiles), the rows of both blocks; the second
            // block's second half only if it holds real rows (the first block of a pair is full)
            const int  group = pr.half * p.n_groups + grp;
            const bool full  = (p.sorted_ids[(pr.first + 1) * 32 + 16] & 0xffffff) < p.M;
            if(p.gate_ring)
            {
                if(full)
                    pr.once ? gate_up_ring_body<4, true>(p, gate_up_lds, pr.first, group, expert)
                            : gate_up_ring_body<4, false>(p, gate_up_lds, pr.first, group, expert);
                else
                    pr.once ? gate_up_ring_body<3, true>(p, gate_up_lds, pr.first, group, expert)
                            : gate_up_ring_body<3, false>(p, gate_up_lds, pr.first, group, expert);
                return;
            }
            if(full)
                pr.once ? gate_up_body<4, 2, true>(p, red_dyn, pr.first, group, expert)
                        : gate_up_body<4, 2, false>(p, red_dyn, pr.first, group, expert);
            else
                pr.once ? gate_up_body<3, 2, true>(p, red_dyn, pr.first, group, expert)
                        : gate_up_body<3, 2, false>(p, red_dyn, pr.first, group, expert);
            return;
        }
        once = run.alone();
    }
    else
        once = only_block_of_its_expert(p, blk, expert);
    if constexpr(NT == 4)
    {
        if(fine)
        {
            if(second_half)
                once ? gate_up_body<2, 1, true>(p, red_dyn, blk, grp, expert) : gate_up_body<2, 1, false>(p, red_dyn, blk, grp, expert);
            else
                once ? gate_up_body<1, 1, true>(p, red_dyn, blk, grp, expert) : gate_up_body<1, 1, false>(p, red_dyn, blk, grp, expert);
            return;
        }
    }
    if(second_half)
        once ? gate_up_body<2, NT, true>(p, red_dyn, blk, grp, expert) : gate_up_body<2, NT, false>(p, red_dyn, blk, grp, expert);
    else
        once ? gate_up_body<1, NT, true>(p, red_dyn, blk, grp, expert) : gate_up_body<1, NT, false>(p, red_dyn, blk, grp, expert);
}

// Second GEMM.  Workgroup = (block of 32 sorted rows, 512 output columns), wave = 128 columns =
// 8 weight tiles walked two at a time with the next two already requested; the block's
// activation rows (K = inter_dim, at most 4 K blocks on this path) stay in registers.
// `half` 0 / 1 with `halves` 2: a wave takes the first / second half of its columns only (pairs of blocks)
//
// The rows it writes.  A lane holds 4 consecutive columns of one row per tile, so stored from there one
// instruction writes 16 rows x 32 bytes: quarter lines, which the memory system pays for far beyond their
// bytes (the 59 / 117 MB of 16-bit rows at 512 / 1024 tokens cost 28 / 41 us of the layer that way).  With
// `out_staged` a wave parks two pairs of tiles (64 columns = one 128-byte line per row) in an LDS region of
// its own, rows 144 bytes apart, and stores them 8 rows x 128 bytes per instruction.
constexpr int kDownStagePitch = 144;
constexpr int down_stage_bytes(int waves, int mt) { return waves * mt * 16 * kDownStagePitch; }

template <int MT, int KB, bool STREAM>
__device__ __forceinline__ void down_body(const MoeGemmParams& p, uint8_t* stage_lds, int blk, int grp, int expert, int half = 0,
                                          int halves = 1)
{
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, l16 = lane & 15, kg = lane >> 4;
    const int n0 = (grp * p.waves + wave) * p.wave_cols + half * (p.wave_cols / halves);
    if(n0 >= p.N)
        return;
    const bool     staged = p.out_staged != 0; // uniform
    uint8_t* const stage  = stage_lds + wave * (MT * 16 * kDownStagePitch);
    // bit r: row r of the block (or pair of blocks) is a real row
    const uint64_t real_rows =
        __ballot(lane < MT * 16 && (p.sorted_ids[(size_t)blk * p.block_rows + (lane < MT * 16 ? lane : 0)] & 0xffffff) < p.M);
    i32x8 x[MT][KB];
    float xs[MT][KB];
    bool  real[MT]; // padding rows are multiplied along but not stored
#pragma unroll
    for(int j = 0; j < MT; ++j)
    {
        const size_t slot = (size_t)blk * p.block_rows + j * 16 + l16;
        real[j]           = (p.sorted_ids[slot] & 0xffffff) < p.M;
#pragma unroll
        for(int kb = 0; kb < KB; ++kb)
        {
            x[j][kb]  = load_x_fragment(p.xq + slot * p.lda + (size_t)kb * 128, kg);
            xs[j][kb] = p.xs[slot * p.xs_stride + kb];
        }
    }
    const size_t   tile_stride = (size_t)16 * (size_t)p.K;
    const uint8_t* wt  = p.w + (size_t)expert * (size_t)p.N * (size_t)p.K + (size_t)(n0 >> 4) * tile_stride;
    const float*   wsr = p.wsc + (size_t)expert * (p.N / 128) * KB;
    const int      want  = p.wave_cols / 32 / halves;
    const int      pairs = (p.N - n0) / 32 < want ? (p.N - n0) / 32 : want; // N is a multiple of 256

    auto fetch = [&](int pair, i32x8 (&w)[2][KB]) {
#pragma unroll
        for(int i = 0; i < 2; ++i)
#pragma unroll
            for(int kb = 0; kb < KB; ++kb)
                w[i][kb] = load_w_fragment<STREAM>(wt + (size_t)(pair * 2 + i) * tile_stride + (size_t)kb * 2048, l16, kg);
    };
    auto finish = [&](int pair, const i32x8 (&w)[2][KB]) {
#pragma unroll
        for(int i = 0; i < 2; ++i)
        {
            const int    n   = n0 + (pair * 2 + i) * 16;
            const float* wsn = wsr + (size_t)(n / 128) * KB;
#pragma unroll
            for(int j = 0; j < MT; ++j)
            {
                f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for(int kb = 0; kb < KB; ++kb)
                {
                    const f32x4 prod = mfma_16x16x128_fp8(w[i][kb], x[j][kb], f32x4{0.f, 0.f, 0.f, 0.f});
                    const float sc   = xs[j][kb] * wsn[kb];
#pragma unroll
                    for(int c = 0; c < 4; ++c)
                        acc[c] = __builtin_fmaf(prod[c], sc, acc[c]);
                }
                const size_t slot = (size_t)blk * p.block_rows + j * 16 + l16;
                const int    col  = n + kg * 4;
                if(staged)
                {
                    *(u32x2*)(stage + (j * 16 + l16) * kDownStagePitch + ((pair & 1) * 32 + i * 16 + kg * 4) * 2) =
                        u32x2{pack2<In16::bf16>(acc[0], acc[1]), pack2<In16::bf16>(acc[2], acc[3])};
                    continue;
                }
                if(!real[j])
                    continue;
                if(p.out_f32)
                    *(f32x4*)((float*)p.out + slot * p.N + col) = acc;
                else
                    *(u32x2*)(p.out + slot * p.N + col) =
                        u32x2{pack2<In16::bf16>(acc[0], acc[1]), pack2<In16::bf16>(acc[2], acc[3])};
            }
        }
        // every second pair (and the last one): the parked columns leave, a lane per 16 bytes, 8 rows per
        // instruction.  The wave's LDS operations complete in the order they were issued.
        if(staged && ((pair & 1) || pair + 1 == pairs))
        {
            const int first_col = n0 + (pair & ~1) * 32;
            const int chunks    = (pair & 1) ? 8 : 4; // 16-byte pieces per row that hold columns
            const int c         = lane & 7;
#pragma unroll
            for(int r0 = 0; r0 < MT * 16; r0 += 8)
            {
                const int   row = r0 + (lane >> 3);
                const u32x4 v   = *(const u32x4*)(stage + row * kDownStagePitch + c * 16);
                if(c < chunks && ((real_rows >> row) & 1))
                    *(u32x4*)(p.out + ((size_t)blk * p.block_rows + row) * p.N + first_col + c * 8) = v;
            }
        }
    };
    if constexpr(MT > 2)
    {
        // pairs of blocks: one pair of tiles at a time, nothing requested ahead (measured: 385 -> 380 us at
        // 1024 tokens; with one block per pass the requests ahead are worth 1.5 us at 512 tokens)
        i32x8 wa[2][KB];
        for(int pair = 0; pair < pairs; ++pair)
        {
            fetch(pair, wa);
            finish(pair, wa);
        }
        return;
    }
    i32x8 wa[2][KB], wb[2][KB];
    fetch(0, wa);
    for(int pair = 0; pair < pairs; pair += 2)
    {
        if(pair + 1 < pairs)
            fetch(pair + 1, wb);
        finish(pair, wa);
        if(pair + 1 >= pairs)
            break;
        if(pair + 2 < pairs)
            fetch(pair + 2, wa);
        finish(pair + 1, wb);
    }
}

// PAIRS: the instance that can multiply pairs of blocks (more registers: kept apart so that the usual
// instance keeps three workgroups of four waves per compute unit)
template <int KB, bool PAIRS>
__global__ __launch_bounds__(512) void moe_down_kernel(MoeGemmParams p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t down_stage[]; // down_stage_bytes(waves, 4 or 2) when rows are staged
    const int blk = blockIdx.x / p.n_groups, grp = blockIdx.x - blk * p.n_groups;
    if(blk * p.block_rows >= p.num_valid[0])
        return;
    const int expert = p.sorted_expert_ids[blk >> p.expert_shift];
    if(expert < 0 || expert >= p.experts)
        return;
    const bool second_half = p.block_rows == 32 && (p.sorted_ids[blk * 32 + 16] & 0xffffff) < p.M;
    bool once;
    if constexpr(PAIRS && KB <= 2) // the rows of two blocks stay in registers only for short K
    {
        const RunOfBlocks  run = run_of_blocks(p, blk, expert);
        const PairOfBlocks pr  = pair_of_blocks(p, run, blk);
        if(pr.paired)
        {
            const bool full = (p.sorted_ids[(pr.first + 1) * 32 + 16] & 0xffffff) < p.M;
            if(full)
                pr.once ? down_body<4, KB, true>(p, down_stage, pr.first, grp, expert, pr.half, 2)
                        : down_body<4, KB, false>(p, down_stage, pr.first, grp, expert, pr.half, 2);
            else
                pr.once ? down_body<3, KB, true>(p, down_stage, pr.first, grp, expert, pr.half, 2)
                        : down_body<3, KB, false>(p, down_stage, pr.first, grp, expert, pr.half, 2);
            return;
        }
        once = run.alone();
    }
    else
        once = only_block_of_its_expert(p, blk, expert);
    if(second_half)
        once ? down_body<2, KB, true>(p, down_stage, blk, grp, expert) : down_body<2, KB, false>(p, down_stage, blk, grp, expert);
    else
        once ? down_body<1, KB, true>(p, down_stage, blk, grp, expert) : down_body<1, KB, false>(p, down_stage, blk, grp, expert);
}

// The same for any K: workgroup = (block, 256 columns), wave = 64 columns, K blocks walked in turn.
template <bool STREAM>
__device__ __forceinline__ void down_long_k_body(const MoeGemmParams& p, int blk, int grp, int expert)
{
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, l16 = lane & 15, kg = lane >> 4;
    const int n0 = grp * 256 + wave * 64;
    if(n0 >= p.N)
        return;
    const uint8_t* xrow[2];
    const float*   xsr[2];
    bool           real[2];
#pragma unroll
    for(int j = 0; j < 2; ++j)
    {
        // a block of 16 rows has no second tile: it repeats the first and stores nothing
        const bool   have = j * 16 < p.block_rows;
        const size_t slot = (size_t)blk * p.block_rows + (have ? j * 16 : 0) + l16;
        xrow[j]           = p.xq + slot * p.lda;
        xsr[j]            = p.xs + slot * p.xs_stride;
        real[j]           = have && (p.sorted_ids[slot] & 0xffffff) < p.M;
    }
    const uint8_t* wt  = p.w + (size_t)expert * (size_t)p.N * (size_t)p.K + (size_t)(n0 >> 4) * 16 * (size_t)p.K;
    const float*   wsr = p.wsc + ((size_t)expert * (p.N / 128) + n0 / 128) * p.kblocks;

    f32x4 acc[2][4];
#pragma unroll
    for(int j = 0; j < 2; ++j)
#pragma unroll
        for(int i = 0; i < 4; ++i)
            acc[j][i] = f32x4{0.f, 0.f, 0.f, 0.f};
    for(int kb = 0; kb < p.kblocks; ++kb)
    {
        i32x8 w[4], x[2];
#pragma unroll
        for(int i = 0; i < 4; ++i)
            w[i] = load_w_fragment<STREAM>(wt + (size_t)i * 16 * (size_t)p.K + (size_t)kb * 2048, l16, kg);
        float       sc[2];
        const float wsv = wsr[kb];
#pragma unroll
        for(int j = 0; j < 2; ++j)
        {
            x[j]  = load_x_fragment(xrow[j] + (size_t)kb * 128, kg);
            sc[j] = xsr[j][kb] * wsv;
        }
#pragma unroll
        for(int j = 0; j < 2; ++j)
#pragma unroll
            for(int i = 0; i < 4; ++i)
            {
                const f32x4 prod = mfma_16x16x128_fp8(w[i], x[j], f32x4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
                for(int c = 0; c < 4; ++c)
                    acc[j][i][c] = __builtin_fmaf(prod[c], sc[j], acc[j][i][c]);
            }
    }
#pragma unroll
    for(int j = 0; j < 2; ++j)
#pragma unroll
        for(int i = 0; i < 4; ++i)
        {
            const size_t slot = (size_t)blk * p.block_rows + j * 16 + l16;
            const int    col  = n0 + i * 16 + kg * 4;
            if(!real[j])
                continue;
            if(p.out_f32)
                *(f32x4*)((float*)p.out + slot * p.N + col) = acc[j][i];
            else
                *(u32x2*)(p.out + slot * p.N + col) = u32x2{pack2<In16::bf16>(acc[j][i][0], acc[j][i][1]),
                                                            pack2<In16::bf16>(acc[j][i][2], acc[j][i][3])};
        }
}

__global__ __launch_bounds__(256) void moe_down_long_k_kernel(MoeGemmParams p)
{
    const int blk = blockIdx.x / p.n_groups, grp = blockIdx.x - blk * p.n_groups;
    if(blk * p.block_rows >= p.num_valid[0])
        return;
    const int expert = p.sorted_expert_ids[blk >> p.expert_shift];
    if(expert < 0 || expert >= p.experts)
        return;
    if(only_block_of_its_expert(p, blk, expert))
        down_long_k_body<true>(p, blk, grp, expert);
    else
        down_long_k_body<false>(p, blk, grp, expert);
}


// Second GEMM fused with the per-token sum, for decode-size batches.  Workgroup = two neighbouring
// 16-column weight tiles of every expert (8 KiB of an expert's weights are contiguous in memory and
// requested together, while four tiles leave too few workgroups for the compute units' ingest); wave =
// (walker, K block): it multiplies its K block of both tiles, so a unit's activation rows are
// fetched once for the two (a compute unit's intake counts them like the weights), and with two
// walkers per K block, each taking every other unit, a compute unit still has four waves at work.
// A wave walks its (block, 16-row half) units that hold real pairs, in sorted order, with the next
// kColsDepth units' operands already requested (a unit is 4 KiB of weights per wave: the depth is
// what keeps a wave's share of HBM in flight), and adds each weighted product row into its own
// [tokens][16] fp32 table per tile in LDS: one wave per table and a fixed walk, so the sum is
// deterministic.  The tables are added in K-block order, a K block's walkers in order, onto `out`.
// No rows are written to memory and no position table is needed.
struct DownColsParams
{
    const uint8_t*  xq;  // [slots][K] fp8 by sorted slot
    const float*    row_info; // [slots][kRowInfo]: scales, routing weight, token id of each sorted row
    const uint8_t*  w;   // [experts][N][K] fp8, pre-shuffled (16,16) per expert
    const float*    wsc; // [experts][N/128][K/128]
    const int32_t*  sorted_expert_ids;
    const int32_t*  num_valid;
    const uint32_t* block_mask; // [blocks], written by the first GEMM
    uint16_t*       out;        // [M][N], row stride out_stride
    int64_t         out_stride;
    int32_t         M, K, N, kblocks, max_blocks, experts;
    int32_t         block_rows, expert_shift; // as in MoeGemmParams
    int32_t         walkers; // waves per K block: each walks every walkers-th unit into tables of its own
};

// units a wave has requested ahead of the one it multiplies.  With the weights read non-temporally three is the
// measured optimum (DeepSeek-V3 layer, us at 1 / 32 / 128 / 256 tokens: depth 2 24.3 / 155.1 / 236.9 / 255.6, 3 24.3 /
// 151.9 / 233.0 / 255.9, 4 25.1 / 152.2 / 234.0 / 256.2, 7 25.9 / 154.1 / 236.4 / 258.9, 8 26.4 / 155.8 / 237.5 / 258.3):
// more requests in flight per compute unit only queue up
constexpr int kColsDepth     = 3;
constexpr int kColsTiles     = 2;    // 16-column tiles per workgroup, both multiplied by every wave
constexpr int kColsMaxBlocks = 1024; // blocks the unit scan takes (16 per lane)
constexpr size_t kColsTableBytes = (size_t)140 << 10; // LDS for the per-token tables; the unit list (16 KiB at most) comes on top

struct ColsStage
{
    i32x4    wlo[kColsTiles], whi[kColsTiles], xlo, xhi;
    float    xs, ws;
    u32x2    sw_tok; // routing weight (as bits) and token id
    uint32_t mask;
};

// The walk's loads are issued from asm and waited for by count: left to the compiler, every
// outstanding load is waited for at the head of the loop (one memory latency per kColsDepth units
// instead of a steady stream).  Not templates: asm operands in a kernel template have cost the
// kernel its host-side stub before.
__device__ __forceinline__ void cols_load16(i32x4& d, const void* p)
{
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(d) : "v"(p) : "memory");
}
// weights: read once, non-temporal (see load_w_fragment)
__device__ __forceinline__ void cols_load16_nt(i32x4& d, const void* p)
{
    asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(d) : "v"(p) : "memory");
}
__device__ __forceinline__ void cols_load16_at16(i32x4& d, const void* p)
{
    asm volatile("global_load_dwordx4 %0, %1, off offset:16" : "=v"(d) : "v"(p) : "memory");
}
__device__ __forceinline__ void cols_load16_at256(i32x4& d, const void* p)
{
    asm volatile("global_load_dwordx4 %0, %1, off offset:256 nt" : "=v"(d) : "v"(p) : "memory");
}
__device__ __forceinline__ void cols_load4(float& d, const void* p)
{
    asm volatile("global_load_dword %0, %1, off" : "=v"(d) : "v"(p) : "memory");
}
__device__ __forceinline__ void cols_load8_at16(u32x2& d, const void* p)
{
    asm volatile("global_load_dwordx2 %0, %1, off offset:16" : "=v"(d) : "v"(p) : "memory");
}
constexpr int kColsLoadsPerStage = 9; // loads the walk requests per unit, counted by cols_wait_oldest
// the stage requested kColsDepth - 1 stages ago has arrived once at most (kColsDepth - 1) *
// kColsLoadsPerStage = 18 younger loads are outstanding (loads return in order); the stage's
// registers are operands so that nothing that reads them is moved above the wait
__device__ __forceinline__ void cols_wait_oldest(ColsStage& s)
{
    asm volatile("s_waitcnt vmcnt(18)"
                 : "+v"(s.wlo[0]), "+v"(s.whi[0]), "+v"(s.wlo[1]), "+v"(s.whi[1]), "+v"(s.xlo), "+v"(s.xhi), "+v"(s.xs),
                   "+v"(s.ws), "+v"(s.sw_tok)
                 :
                 : "memory");
}
// waits for every outstanding load; the stage's registers are operands so that they count as
// occupied until then (a request past the last unit is still on its way into them after the walk)
__device__ __forceinline__ void cols_drain(ColsStage& s)
{
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(s.wlo[0]), "+v"(s.whi[0]), "+v"(s.wlo[1]), "+v"(s.whi[1]), "+v"(s.xlo), "+v"(s.xhi), "+v"(s.xs),
                   "+v"(s.ws), "+v"(s.sw_tok)
                 :
                 : "memory");
}
static_assert((kColsDepth - 1) * kColsLoadsPerStage == 18 && kColsTiles == 2, "cols_wait_oldest counts 18 younger loads");

template <In16 DT>
__global__ __launch_bounds__(256) void moe_down_cols_kernel(DownColsParams p)
{
    extern __shared__ __attribute__((aligned(16))) uint32_t cols_lds[];
    __shared__ int n_units_s;
    uint32_t*      unit_a = cols_lds;                    // block << 1 | half
    uint32_t*      unit_b = cols_lds + 2 * p.max_blocks; // expert << 16 | the half's row mask
    float*         acc    = (float*)(cols_lds + 4 * p.max_blocks); // [waves][M + 16][16], rows M.. are spares
    const int      t = threadIdx.x, lane = t & 63, wave = t >> 6, l16 = lane & 15, kg = lane >> 4;
    // wave = K block; it multiplies both of the workgroup's tiles, so a unit's activation rows are
    // fetched once for the two (a compute unit's intake counts them like the weights)
    const int      walker = wave / p.kblocks, kb = wave - walker * p.kblocks, tile = blockIdx.x * kColsTiles;

    if(wave == 0) // list the units in sorted order
    {
        const int nv    = p.num_valid[0];
        int       valid = (nv + p.block_rows - 1) / p.block_rows;
        valid           = valid < p.max_blocks ? valid : p.max_blocks;
        int      e[kColsMaxBlocks / 64];
        uint32_t m[kColsMaxBlocks / 64];
#pragma unroll
        for(int c = 0; c < kColsMaxBlocks / 64; ++c)
        {
            const int b = c * 64 + lane;
            e[c]        = b < valid ? p.sorted_expert_ids[b >> p.expert_shift] : -1;
            m[c]        = b < valid ? p.block_mask[b] : 0u;
        }
        int            base = 0;
        const uint64_t below = ((uint64_t)1 << lane) - 1;
#pragma unroll
        for(int c = 0; c < kColsMaxBlocks / 64; ++c)
        {
            const bool     ok = e[c] >= 0 && e[c] < p.experts;
            const bool     h0 = ok && (m[c] & 0xffffu) != 0, h1 = ok && (m[c] >> 16) != 0;
            const uint64_t b0 = __ballot(h0), b1 = __ballot(h1);
            int            at = base + __popcll(b0 & below) + __popcll(b1 & below);
            const uint32_t b  = (uint32_t)(c * 64 + lane);
            if(h0)
            {
                unit_a[at] = b << 1;
                unit_b[at] = (uint32_t)e[c] << 16 | (m[c] & 0xffffu);
                ++at;
            }
            if(h1)
            {
                unit_a[at] = b << 1 | 1u;
                unit_b[at] = (uint32_t)e[c] << 16 | (m[c] >> 16);
            }
            base += __popcll(b0) + __popcll(b1);
        }
        if(lane == 0)
            n_units_s = base;
    }
    for(int i = t; i < p.walkers * kColsTiles * p.kblocks * (p.M + 16) * 16; i += blockDim.x)
        acc[i] = 0.f;
    __syncthreads();
    // this wave's units: walker, walker + walkers, ... of the list
    const int units = (n_units_s - walker + p.walkers - 1) / p.walkers;

    const int      n0     = tile * 16;
    const size_t   wexp   = (size_t)p.N * (size_t)p.K;
    const uint8_t* wlane  = p.w + (size_t)tile * 16 * (size_t)p.K + (size_t)kb * 2048 + kg * 512 + l16 * 16;
    const float*   wslane = p.wsc + (size_t)(n0 / 128) * p.kblocks + kb; // (both tiles lie in one 128-column block)
    const size_t   wsexp  = (size_t)(p.N / 128) * p.kblocks;
    const size_t   wtile  = (size_t)16 * (size_t)p.K; // bytes between the two tiles
    // table of (walker, tile tw, K block kb): (walker * tiles + tw) * kblocks + kb
    float* const   mine   = acc + ((size_t)walker * kColsTiles * p.kblocks + kb) * (p.M + 16) * 16 + kg * 4;
    const size_t   table1 = (size_t)p.kblocks * (p.M + 16) * 16; // floats from tile 0's table to tile 1's

    // The walk is free of branches (the compiler then keeps the requested depth of loads in flight):
    // past the last unit the last unit is requested again and its product goes to spare rows.
    auto issue = [&](ColsStage& s, int u) {
        u = (u < units ? u : units - 1) * p.walkers + walker;
        const uint32_t a = __builtin_amdgcn_readfirstlane(unit_a[u]);
        const uint32_t b = __builtin_amdgcn_readfirstlane(unit_b[u]);
        const int      expert = (int)(b >> 16);
        s.mask                = b & 0xffffu;
        const uint8_t* wp     = wlane + (size_t)expert * wexp;
        cols_load16_nt(s.wlo[0], wp);
        cols_load16_at256(s.whi[0], wp);
        cols_load16_nt(s.wlo[1], wp + wtile);
        cols_load16_at256(s.whi[1], wp + wtile);
        cols_load4(s.ws, wslane + (size_t)expert * wsexp);
        // rows that are padding read the unit's first real row instead: same cache lines, no traffic
        const int    row  = (s.mask >> l16) & 1u ? l16 : __builtin_ctz(s.mask);
        const size_t slot = (size_t)(a >> 1) * p.block_rows + (a & 1u) * 16 + row;
        const uint8_t* xp = p.xq + slot * (size_t)p.K + (size_t)kb * 128 + kg * 32;
        cols_load16(s.xlo, xp);
        cols_load16_at16(s.xhi, xp);
        const float* info = p.row_info + slot * kRowInfo;
        cols_load4(s.xs, info + kb);
        cols_load8_at16(s.sw_tok, info);
    };
    auto consume = [&](ColsStage& s, bool live) {
        cols_wait_oldest(s);
        const i32x8 x = i32x8{s.xlo[0], s.xlo[1], s.xlo[2], s.xlo[3], s.xhi[0], s.xhi[1], s.xhi[2], s.xhi[3]};
        f32x4       prod[kColsTiles];
#pragma unroll
        for(int tw = 0; tw < kColsTiles; ++tw)
        {
            const i32x8 w = i32x8{s.wlo[tw][0], s.wlo[tw][1], s.wlo[tw][2], s.wlo[tw][3],
                                  s.whi[tw][0], s.whi[tw][1], s.whi[tw][2], s.whi[tw][3]};
            prod[tw]      = mfma_16x16x128_fp8(w, x, f32x4{0.f, 0.f, 0.f, 0.f});
        }
        // Padding rows go to a spare row per lane.  The table update is a plain read-add-write (LDS
        // float atomics cost 0.3 us per instruction here): right as long as the 16 rows of a unit are
        // 16 different tokens.  A routing that names an expert twice for a token puts the two pairs
        // next to each other in the sorted order; such a unit is added one row at a time.
        const bool  real = live && ((s.mask >> l16) & 1u);
        const int   key  = real ? (int)s.sw_tok[1] : -1 - l16;
        const int   prev = __builtin_amdgcn_update_dpp(-100, key, 0x111 /* row_shr:1 */, 0xf, 0xf, false);
        const int   row  = real ? key : p.M + l16;
        const float sc   = s.xs * s.ws;
        float*      dst  = mine + (size_t)row * 16;
        f32x4       add[kColsTiles];
#pragma unroll
        for(int tw = 0; tw < kColsTiles; ++tw)
#pragma unroll
            for(int c = 0; c < 4; ++c)
                add[tw][c] = prod[tw][c] * sc * __uint_as_float(s.sw_tok[0]);
        if(__builtin_expect(__ballot(real && prev == key) == 0, 1))
        {
            f32x4 cur0 = *(f32x4*)dst, cur1 = *(f32x4*)(dst + table1);
            cur0 += add[0];
            cur1 += add[1];
            *(f32x4*)dst            = cur0;
            *(f32x4*)(dst + table1) = cur1;
        }
        else
        {
            for(int r = 0; r < 16; ++r)
            {
                // rows of one token share `dst`: each row's read has to follow the previous row's
                // write, which a compiler that reasons per lane is free to undo without this
                asm volatile("" ::: "memory");
                if(l16 == r)
                {
#pragma unroll
                    for(int tw = 0; tw < kColsTiles; ++tw)
                    {
                        f32x4 cur = *(volatile f32x4*)(dst + tw * table1);
                        cur += add[tw];
                        *(volatile f32x4*)(dst + tw * table1) = cur;
                    }
                }
            }
        }
    };

    if(units > 0)
    {
        ColsStage st[kColsDepth];
#pragma unroll
        for(int d = 0; d < kColsDepth; ++d)
            issue(st[d], d);
        for(int u0 = 0; u0 < units; u0 += kColsDepth)
        {
#pragma unroll
            for(int d = 0; d < kColsDepth; ++d)
            {
                consume(st[d], u0 + d < units);
                issue(st[d], u0 + d + kColsDepth);
            }
        }
#pragma unroll
        for(int d = 0; d < kColsDepth; ++d)
            cols_drain(st[d]);
    }
    __syncthreads();

    // out[token][n0 .. n0+16) += the tables, K blocks in order
    for(int i = t; i < p.M * 4 * kColsTiles; i += blockDim.x)
    {
        const int tw = i / (p.M * 4), tok = (i - tw * p.M * 4) >> 2, q = i & 3;
        f32x4     sum = f32x4{0.f, 0.f, 0.f, 0.f};
        for(int k = 0; k < p.kblocks; ++k)
            for(int wk = 0; wk < p.walkers; ++wk)
                sum += *(const f32x4*)(acc + ((size_t)((wk * kColsTiles + tw) * p.kblocks + k) * (p.M + 16) + tok) * 16 + q * 4);
        uint16_t*   dst  = p.out + (size_t)tok * p.out_stride + (blockIdx.x * kColsTiles + tw) * 16 + q * 4;
        const u32x2 prev = *(const u32x2*)dst;
        float       o[4];
        if constexpr(DT == In16::bf16)
        {
            o[0] = __uint_as_float(prev[0] << 16);
            o[1] = __uint_as_float(prev[0] & 0xffff0000u);
            o[2] = __uint_as_float(prev[1] << 16);
            o[3] = __uint_as_float(prev[1] & 0xffff0000u);
        }
        else
        {
            o[0] = (float)__builtin_bit_cast(_Float16, (unsigned short)(prev[0] & 0xffffu));
            o[1] = (float)__builtin_bit_cast(_Float16, (unsigned short)(prev[0] >> 16));
            o[2] = (float)__builtin_bit_cast(_Float16, (unsigned short)(prev[1] & 0xffffu));
            o[3] = (float)__builtin_bit_cast(_Float16, (unsigned short)(prev[1] >> 16));
        }
        *(u32x2*)dst = u32x2{pack2<DT>(o[0] + sum[0], o[1] + sum[1]), pack2<DT>(o[2] + sum[2], o[3] + sum[3])};
    }
}

// out[token] += sum over the token's slots, in slot order, of weight * y[sorted position]
// The position table is never cleared: an entry counts only if the sorted array holds this very
// (token, slot) pair at that position, which a stale or uninitialised entry cannot fake (a pair
// occurs once in the sorted array, so an entry that passes is the pair's position).
template <In16 DT, bool Y32>
__global__ __launch_bounds__(256) void moe_combine_kernel(const void* __restrict__ y, const float* __restrict__ sorted_weights,
                                                          const int32_t* __restrict__ where,
                                                          const int32_t* __restrict__ sorted_ids,
                                                          const int32_t* __restrict__ num_valid, int32_t max_padded,
                                                          uint16_t* __restrict__ out, int32_t M, int32_t topk,
                                                          int32_t dim, int64_t out_stride)
{
    const int quads = dim / 4;
    const int token = blockIdx.x;
    const int q     = blockIdx.y * 256 + threadIdx.x;
    if(q >= quads)
        return;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for(int k = 0; k < topk; ++k)
    {
        const int32_t at    = where[(size_t)token * topk + k];
        const int32_t valid = num_valid[0] < max_padded ? num_valid[0] : max_padded;
        if(at < 0 || at >= valid || sorted_ids[at] != ((k << 24) | token))
            continue;
        const float w = sorted_weights[at];
        if constexpr(Y32)
        {
            const f32x4 v = *(const f32x4*)((const float*)y + (size_t)at * dim + (size_t)q * 4);
#pragma unroll
            for(int c = 0; c < 4; ++c)
                acc[c] = __builtin_fmaf(w, v[c], acc[c]);
        }
        else
        {
            const u32x2 v = *(const u32x2*)((const uint16_t*)y + (size_t)at * dim + (size_t)q * 4);
            acc[0] = __builtin_fmaf(w, __uint_as_float(v[0] << 16), acc[0]);
            acc[1] = __builtin_fmaf(w, __uint_as_float(v[0] & 0xffff0000u), acc[1]);
            acc[2] = __builtin_fmaf(w, __uint_as_float(v[1] << 16), acc[2]);
            acc[3] = __builtin_fmaf(w, __uint_as_float(v[1] & 0xffff0000u), acc[3]);
        }
    }
    uint16_t*   dst  = out + (size_t)token * out_stride + (size_t)q * 4;
    const u32x2 prev = *(const u32x2*)dst;
    float       o[4];
    if constexpr(DT == In16::bf16)
    {
        o[0] = __uint_as_float(prev[0] << 16);
        o[1] = __uint_as_float(prev[0] & 0xffff0000u);
        o[2] = __uint_as_float(prev[1] << 16);
        o[3] = __uint_as_float(prev[1] & 0xffff0000u);
    }
    else
    {
        o[0] = (float)__builtin_bit_cast(_Float16, (unsigned short)(prev[0] & 0xffffu));
        o[1] = (float)__builtin_bit_cast(_Float16, (unsigned short)(prev[0] >> 16));
        o[2] = (float)__builtin_bit_cast(_Float16, (unsigned short)(prev[1] & 0xffffu));
        o[3] = (float)__builtin_bit_cast(_Float16, (unsigned short)(prev[1] >> 16));
    }
    *(u32x2*)dst = u32x2{pack2<DT>(o[0] + acc[0], o[1] + acc[1]), pack2<DT>(o[2] + acc[2], o[3] + acc[3])};
}

// The same sum for rows kept in 16 bits, eight elements per lane: 16-byte loads, and a token's rows are all
// requested before the first is added (the additions stay in slot order: the same bits as above).
template <In16 DT>
__global__ __launch_bounds__(256) void moe_combine8_kernel(const uint16_t* __restrict__ y, const float* __restrict__ sorted_weights,
                                                           const int32_t* __restrict__ where,
                                                           const int32_t* __restrict__ sorted_ids,
                                                           const int32_t* __restrict__ num_valid, int32_t max_padded,
                                                           uint16_t* __restrict__ out, int32_t M, int32_t topk,
                                                           int32_t dim, int64_t out_stride)
{
    const int octs  = dim / 8;
    const int token = blockIdx.x;
    const int q     = blockIdx.y * 256 + threadIdx.x;
    if(q >= octs)
        return;
    const int32_t valid = num_valid[0] < max_padded ? num_valid[0] : max_padded;
    float         acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    constexpr int kChunk = 10; // top-8 and a shared expert in one pass
    for(int k0 = 0; k0 < topk; k0 += kChunk)
    {
        u32x4 v[kChunk];
        float w[kChunk];
        bool  ok[kChunk];
#pragma unroll
        for(int i = 0; i < kChunk; ++i)
        {
            const int     k  = k0 + i;
            const int32_t at = k < topk ? where[(size_t)token * topk + k] : -1;
            ok[i]            = at >= 0 && at < valid && sorted_ids[at] == ((k << 24) | token);
            const int32_t r  = ok[i] ? at : 0; // (row 0 exists; what is read there is not used)
            w[i]             = ok[i] ? sorted_weights[r] : 0.f;
            v[i]             = *(const u32x4*)(y + (size_t)r * dim + (size_t)q * 8);
        }
#pragma unroll
        for(int i = 0; i < kChunk; ++i)
            if(ok[i])
            {
#pragma unroll
                for(int c = 0; c < 4; ++c)
                {
                    acc[2 * c]     = __builtin_fmaf(w[i], __uint_as_float(v[i][c] << 16), acc[2 * c]);
                    acc[2 * c + 1] = __builtin_fmaf(w[i], __uint_as_float(v[i][c] & 0xffff0000u), acc[2 * c + 1]);
                }
            }
    }
    uint16_t*   dst  = out + (size_t)token * out_stride + (size_t)q * 8;
    const u32x4 prev = *(const u32x4*)dst;
    u32x4       res;
#pragma unroll
    for(int c = 0; c < 4; ++c)
    {
        float lo, hi;
        if constexpr(DT == In16::bf16)
        {
            lo = __uint_as_float(prev[c] << 16);
            hi = __uint_as_float(prev[c] & 0xffff0000u);
        }
        else
        {
            lo = (float)__builtin_bit_cast(_Float16, (unsigned short)(prev[c] & 0xffffu));
            hi = (float)__builtin_bit_cast(_Float16, (unsigned short)(prev[c] >> 16));
        }
        res[c] = pack2<DT>(lo + acc[2 * c], hi + acc[2 * c + 1]);
    }
    *(u32x4*)dst = res;
}

size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

// The second GEMM's rows wait in memory for the per-token sum: in fp32 while the real rows
// (tokens x topk) take at most 32 MiB -- the decode regime, where the bf16 rounding of rows that
// largely cancel in the sum is avoided at no measurable cost -- and in bf16 beyond, where writing
// them between the weight reads costs 5 % of the layer's time in fp32.
bool rows_in_f32(const MoeArgs& a) { return (size_t)a.M * a.topk * a.dim * 4 <= ((size_t)32 << 20); }

// Walkers per K block of moe_down_cols_kernel: two where their tables ([2 walkers][2 tiles][inter/128]
// [tokens + 16][16] fp32) and the unit list (16 bytes per block) fit the LDS the kernel may ask for and the
// workgroup stays within four waves, else one.
constexpr size_t kColsLdsBytes = kColsTableBytes + (size_t)kColsMaxBlocks * 16;
int cols_walkers(const MoeArgs& a)
{
    const int    kblocks = a.inter / 128;
    const size_t one     = (size_t)kColsTiles * kblocks * (a.M + 16) * 64;
    return (2 * one + (size_t)a.max_blocks * 16 <= kColsLdsBytes && 2 * kblocks <= 4) ? 2 : 1;
}

// Decode-size batches take the second GEMM that owns output columns and sums per token in LDS
// (moe_down_cols_kernel): its tables and its unit list have to fit the LDS.  Beyond, rows go through
// memory and moe_combine_kernel adds them.  down_mode 1 / 2 force the one / the other (2 only where it fits).
bool down_by_columns(const MoeArgs& a)
{
    const int  kblocks = a.inter / 128;
    const bool fits    = kblocks <= 4 && (size_t)kColsTiles * kblocks * (a.M + 16) * 64 <= kColsTableBytes &&
                      a.max_blocks <= kColsMaxBlocks && a.dim % (16 * kColsTiles) == 0;
    if(a.down_mode == 1 || !fits)
        return false;
    // measured on the DeepSeek-V3 layer against rows through memory: with two walkers 4 % faster at 1 token,
    // 6 % at 16-192, 8 % at 256 and 264 (275 against 297 us); with one walker (the tables of two no longer
    // fit) 2 % slower at 288-320 tokens
    return a.down_mode == 2 || cols_walkers(a) == 2;
}

} // namespace

hipError_t launch_topk_softmax(const TopkSoftmaxArgs& a, hipStream_t stream)
{
    if(a.tokens == 0)
        return hipSuccess;
    const dim3 grid((unsigned)((a.tokens + 3) / 4));
    switch(a.gating_dtype)
    {
    case 0:
        hipLaunchKernelGGL(topk_softmax_kernel<__bf16>, grid, dim3(256), 0, stream, (const __bf16*)a.gating, a.weights,
                           a.ids, a.src_rows, a.tokens, a.experts, a.topk, a.w_stride, a.id_stride, a.renorm ? 1 : 0);
        break;
    case 1:
        hipLaunchKernelGGL(topk_softmax_kernel<_Float16>, grid, dim3(256), 0, stream, (const _Float16*)a.gating,
                           a.weights, a.ids, a.src_rows, a.tokens, a.experts, a.topk, a.w_stride, a.id_stride,
                           a.renorm ? 1 : 0);
        break;
    default:
        hipLaunchKernelGGL(topk_softmax_kernel<float>, grid, dim3(256), 0, stream, (const float*)a.gating, a.weights,
                           a.ids, a.src_rows, a.tokens, a.experts, a.topk, a.w_stride, a.id_stride, a.renorm ? 1 : 0);
        break;
    }
    return hipGetLastError();
}

hipError_t launch_moe_sorting(const MoeSortArgs& a, hipStream_t stream, const char** why)
{
    SortParams p{};
    p.topk_ids          = a.topk_ids;
    p.topk_weights      = a.topk_weights;
    p.expert_mask       = a.expert_mask;
    p.num_local_tokens  = a.num_local_tokens;
    p.sorted_ids        = a.sorted_ids;
    p.sorted_weights    = a.sorted_weights;
    p.sorted_expert_ids = a.sorted_expert_ids;
    p.num_valid_ids     = a.num_valid_ids;
    p.M                 = a.M;
    p.w_rows            = a.w_rows;
    p.topk              = a.topk;
    p.experts           = a.experts;
    p.unit              = a.unit;
    p.max_padded        = a.max_padded;
    p.max_blocks        = a.max_blocks;
    p.id_stride         = a.id_stride;
    p.w_stride          = a.w_stride;
    const int64_t n     = (int64_t)a.M * a.topk;
    // a chunk is scattered by one wave, 64 pairs per step: short chunks while the scan (one pass over
    // the chunks per expert) stays short, long ones for very many pairs
    p.chunk_pairs       = n <= 65536 ? 256 : kSortChunkMulti;
    p.chunks            = (int32_t)((n + p.chunk_pairs - 1) / p.chunk_pairs);
    if(p.chunks < 1)
        p.chunks = 1;
    // histograms and expert offsets: a region of their own in the stream's arena (the expert layer
    // that follows on the same stream uses another)
    LaunchCtx ctx;
    ctx.device_id = a.device_id;
    ctx.stream    = stream;
    ctx.why       = why;
    WorkspaceLock lock;
    void*         block        = nullptr;
    const size_t  counts_bytes = align_up((size_t)p.chunks * a.experts * 4);
    hipError_t    e = workspace_acquire(ctx, lock, WsKind::moe_sort, counts_bytes + align_up(((size_t)a.experts + 1) * 4),
                                        false, &block);
    if(e != hipSuccess)
        return e;
    uint8_t* const scratch = (uint8_t*)block;
    p.counts       = (int32_t*)scratch;
    p.expert_begin = (int32_t*)(scratch + counts_bytes);

    // workgroups of 1024 threads that clear the output buffer, about 64 KiB each, riding in the first launch
    unsigned zero_groups = 0;
    if(a.moe_buf && a.moe_buf_bytes)
    {
        p.zero_dst  = (u32x4*)a.moe_buf;
        p.zero_vecs = a.moe_buf_bytes / 16;
        const size_t g = (p.zero_vecs + 4095) / 4096;
        zero_groups    = (unsigned)(g > 1024 ? 1024 : g);
    }
    if(n <= kSortChunk)
    {
        hipLaunchKernelGGL(moe_sort_single_kernel, dim3(1 + zero_groups), dim3(1024), 0, stream, p);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(moe_sort_count_kernel, dim3(p.chunks + zero_groups), dim3(1024), (size_t)a.experts * 4, stream, p);
    hipLaunchKernelGGL(moe_sort_scan_kernel, dim3(1), dim3(1024), 0, stream, p);
    hipLaunchKernelGGL(moe_sort_scatter_kernel, dim3(p.chunks), dim3(64), 0, stream, p);
    return hipGetLastError();
}

// floats per sorted row in the buffer the quantiser writes its scales to: a row record while the
// second GEMM's K has at most four scale blocks, the bare scales beyond
size_t scale_floats_per_slot(const MoeArgs& a) { return a.inter / 128 <= 4 ? (size_t)kRowInfo : (size_t)(a.inter / 128); }

size_t moe_workspace_bytes(const MoeArgs& a)
{
    const size_t slots = (size_t)a.max_padded;
    size_t       b     = 0;
    b += align_up(slots * a.inter * 2);          // activation product, bf16
    b += align_up(slots * a.inter);              // the same as fp8
    b += align_up(slots * scale_floats_per_slot(a) * 4); // its scales, or the row records that hold them
    b += align_up(slots * a.dim * (rows_in_f32(a) ? 4 : 2)); // second GEMM's rows
    b += align_up((size_t)a.M * a.topk * 4);     // sorted position of each (token, slot)
    b += align_up((size_t)a.max_blocks * 4);     // real rows of each block
    if(a.x16)
    {
        b += align_up((size_t)a.M * a.dim);             // quantised tokens
        b += align_up((size_t)a.M * (a.dim / 128) * 4); // their scales
    }
    return b;
}

hipError_t launch_fmoe_blockscale(const MoeArgs& a, hipStream_t stream, const char** why)
{
    if(a.M == 0 || a.max_padded == 0)
        return hipSuccess;
    LaunchCtx ctx;
    ctx.device_id = a.device_id;
    ctx.stream    = stream;
    ctx.why       = why;
    WorkspaceLock lock; // until the layer's last launch is enqueued
    void*         block = nullptr;
    hipError_t    e     = workspace_acquire(ctx, lock, WsKind::moe_layer, moe_workspace_bytes(a), false, &block);
    if(e != hipSuccess)
        return e;
    uint8_t* ws = (uint8_t*)block;
    const size_t slots = (size_t)a.max_padded;
    uint16_t*    h16   = (uint16_t*)ws;
    ws += align_up(slots * a.inter * 2);
    uint8_t* hq = ws;
    ws += align_up(slots * a.inter);
    float* hs = (float*)ws;
    ws += align_up(slots * scale_floats_per_slot(a) * 4);
    const bool y32 = rows_in_f32(a);
    uint16_t*  y   = (uint16_t*)ws;
    ws += align_up(slots * a.dim * (y32 ? 4 : 2));
    int32_t* where = (int32_t*)ws; // sorted position of each (token, slot) pair; stale where the pair is not routed here
    ws += align_up((size_t)a.M * a.topk * 4);
    uint32_t* block_mask = (uint32_t*)ws;
    ws += align_up((size_t)a.max_blocks * 4);
    const bool cols = down_by_columns(a);

    const uint8_t* xq = a.xq;
    const float*   xs = a.xs;
    if(a.x16) // 16-bit tokens: quantise them 1x128 first, scales transposed
    {
        uint8_t* q = ws;
        ws += align_up((size_t)a.M * a.dim);
        float* s = (float*)ws;
        QuantArgs qa{};
        qa.x               = a.x16;
        qa.y               = q;
        qa.scale           = s;
        qa.rows            = a.M;
        qa.groups_per_row  = a.dim / 128;
        qa.group           = 128;
        qa.transpose_scale = true;
        qa.num_rows        = nullptr;
        qa.num_rows_factor = 1;
        qa.dtype           = a.x16_dtype;
        e                  = launch_group_quant(qa, stream);
        if(e != hipSuccess)
            return e;
        xq = q;
        xs = s;
    }

    MoeGemmParams p{};
    p.xq                = xq;
    p.xs                = xs;
    p.w                 = a.w1;
    p.wsc               = a.w1_scale;
    p.sorted_ids        = a.sorted_ids;
    p.sorted_expert_ids = a.sorted_expert_ids;
    p.num_valid         = a.num_valid;
    p.out               = h16;
    p.M                 = a.M;
    p.K                 = a.dim;
    p.N                 = 2 * a.inter;
    p.inter             = a.inter;
    p.kblocks           = a.dim / 128;

    p.topk              = a.topk;
    p.where             = cols ? nullptr : where;
    p.block_mask        = block_mask;
    p.row_info          = a.inter / 128 <= 4 ? hs : nullptr;
    p.sorted_weights    = a.sorted_weights;
    p.max_blocks        = a.max_blocks;
    p.block_rows        = a.block_rows;
    p.expert_shift      = a.expert_shift;
    // pairs of blocks from 28 rows per expert on average (DeepSeek-V3 layer, us block by block / in pairs:
    // 704 tokens 304.7 / 311.1, 768: 317.8 / 319.4, 832: 330.4 / 325.4, 896: 363.7 / 345.4, 1024: 412.7 / 381.1;
    // at 256 and 512 tokens, where only the shared expert has runs of blocks, the gathered rows of a pair
    // cost more than its weights save)
    p.pair_blocks       = a.pair_blocks >= 0 ? a.pair_blocks : ((double)a.M * a.topk >= 28.0 * a.experts ? 1 : 0);
    p.experts           = a.experts;
    p.activation        = a.activation;
    p.lda               = a.x16 ? a.dim : a.lda;
    {
        // (expert, block) pairs to expect under a routing that spreads evenly: the experts hit at least once,
        // plus the full blocks.  A workgroup takes 64, 32 or 16 columns (one workgroup per compute unit at a
        // time).  The widest units that fill a single round of workgroups reasonably (at least two thirds of the
        // compute units, at most a tenth over); beyond a round, the wide units where their last round is three
        // quarters full or there are four rounds and more, else the narrowest, whose last round costs least.
        // DeepSeek-V3 layer, same routing, us with 16 / 32 / 64 columns: 2 tokens 35.3 / 33.5 / 41.2, 3 tokens
        // 38.6 / 36.2 / 42.8, 7 tokens 61.7 / 60.7 / 58.2, 12 tokens 83.9 / 85.1 / 92.1, 16 tokens 101.2 / 105.3 /
        // 100.9, 28 tokens 142.6 / 141.7 / 147.5, 48 tokens 184.7 / 187.2 / 191.8, 80 tokens 219.7 / 219.7 / 215.4.
        const double pairs  = (double)a.M * a.topk;
        const double blocks = (double)a.experts * (1.0 - exp(-pairs / (double)a.experts)) + pairs / 32.0;
        const double wide = blocks * (a.inter / 64), mid = blocks * (a.inter / 32), rounds = wide / 256.0;
        int          nt   = a.gate_tiles;
        if(nt != 1 && nt != 2 && nt != 4)
        {
            if(wide >= 170.0 && rounds <= 1.1)
                nt = 4;
            else if(mid >= 130.0 && mid <= 260.0)
                nt = 2;
            else if(wide >= 230.0 && (rounds - floor(rounds) >= 0.75 || rounds >= 4.0))
                nt = 4;
            else
                nt = 1;
        }
        p.n_groups = a.inter / (16 * nt);
        // wide units: workgroups for up to a quarter of a round of blocks cut into narrow units are launched
        // behind them (the kernel uses them when the valid blocks leave such a remainder)
        p.fine_blocks = (nt == 4 && a.fine_tail != 0) ? std::min(a.max_blocks, kChipCus / 4 / p.n_groups) : 0;
        // (blocks rounded up to a multiple of 8: the kernel deals them out to the 8 XCDs)
        const dim3 grid((unsigned)((size_t)((a.max_blocks + 7) & ~7) * p.n_groups + (size_t)p.fine_blocks * 4 * p.n_groups));
        // every instance keeps its LDS (reduction buffer; ring of the pairs instance) in the dynamic segment:
        // opt in to more than 64 KiB once per device and instance
        const bool paired = nt == 4 && p.pair_blocks;
        auto kernel = paired     ? moe_gate_up_kernel<4, true>
                      : nt == 4 ? moe_gate_up_kernel<4, false>
                      : nt == 2 ? moe_gate_up_kernel<2, false>
                                : moe_gate_up_kernel<1, false>;
        const size_t lds = gate_up_lds_bytes(nt, paired);
        static std::atomic<bool> raised[64][4];
        const int inst = paired ? 3 : nt == 4 ? 2 : nt == 2 ? 1 : 0;
        if(lds > 65536 && (a.device_id < 0 || a.device_id >= 64 || !raised[a.device_id][inst]))
        {
            e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if(e != hipSuccess)
                return e;
            if(a.device_id >= 0 && a.device_id < 64)
                raised[a.device_id][inst] = true;
        }
        // (32-bit byte offsets of the token rows in the ring body)
        p.gate_ring = (paired && a.gate_ring != 0 && (uint64_t)a.M * (uint64_t)a.lda < (1ull << 32) && (uint64_t)a.M * 4 < (1ull << 32)) ? 1 : 0;
        hipLaunchKernelGGL(kernel, grid, dim3(64 * kGateUpWaves), lds, stream, p);
    }

    QuantArgs qa{};
    qa.x               = h16;
    qa.y               = hq;
    qa.scale           = hs;
    qa.rows            = (int64_t)slots;
    qa.groups_per_row  = a.inter / 128;
    qa.group           = 128;
    qa.transpose_scale = false;
    qa.num_rows        = a.num_valid; // only the rows that exist
    qa.scale_row_stride = a.inter / 128 <= 4 ? kRowInfo : 0;
    qa.num_rows_factor = 1;
    qa.dtype           = In16::bf16;
    e                  = launch_group_quant(qa, stream);
    if(e != hipSuccess)
        return e;

    if(cols)
    {
        DownColsParams c{};
        c.xq                = hq;
        c.row_info          = hs;
        c.w                 = a.w2;
        c.wsc               = a.w2_scale;
        c.sorted_expert_ids = a.sorted_expert_ids;
        c.num_valid         = a.num_valid;
        c.block_mask        = block_mask;
        c.out               = (uint16_t*)a.out;
        c.out_stride        = a.out_stride;
        c.M                 = a.M;
        c.K                 = a.inter;
        c.N                 = a.dim;
        c.kblocks           = a.inter / 128;
        c.max_blocks        = a.max_blocks;
        c.block_rows        = a.block_rows;
        c.expert_shift      = a.expert_shift;
        c.experts           = a.experts;
        // two walkers per K block where their tables fit and the workgroup stays within four waves (DeepSeek-V3
        // layer, 16 / 64 / 256 tokens: 112 / 224 / 275 us with two, 118 / 240 / 299 with one, 114 / 226 / - with four)
        const size_t one    = (size_t)kColsTiles * c.kblocks * (a.M + 16) * 64;
        c.walkers           = cols_walkers(a);
        const size_t lds    = (size_t)a.max_blocks * 16 + (size_t)c.walkers * one;
        const dim3   grid((unsigned)(a.dim / (16 * kColsTiles))), block((unsigned)(64 * c.kblocks * c.walkers));
        auto kernel = a.out_dtype == In16::bf16 ? moe_down_cols_kernel<In16::bf16> : moe_down_cols_kernel<In16::fp16>;
        constexpr int            kMaxDevices = 64;
        static std::atomic<bool> raised[kMaxDevices][2]; // dynamic LDS above the default limit needs opting in, once
        const int                inst = a.out_dtype == In16::bf16 ? 0 : 1;
        if(a.device_id < 0 || a.device_id >= kMaxDevices)
            return hipErrorInvalidDevice;
        if(!raised[a.device_id][inst])
        {
            e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kColsLdsBytes);
            if(e != hipSuccess)
                return e;
            raised[a.device_id][inst] = true;
        }
        hipLaunchKernelGGL(kernel, grid, block, lds, stream, c);
        return hipGetLastError();
    }

    MoeGemmParams d = p;
    d.xq            = hq;
    d.xs            = hs;
    d.w             = a.w2;
    d.wsc           = a.w2_scale;
    d.out           = y;
    d.K             = a.inter;
    d.N             = a.dim;
    d.kblocks       = a.inter / 128;
    d.lda           = a.inter;
    d.xs_stride     = (int32_t)scale_floats_per_slot(a);
    d.out_f32       = y32 ? 1 : 0;
    if(d.kblocks <= 4)
    {
        d.waves         = (a.down_waves == 2 || a.down_waves == 4 || a.down_waves == 8) ? a.down_waves : 4;
        d.wave_cols     = a.down_wave_cols == 64 ? 64 : 128;
        d.n_groups      = (a.dim + d.wave_cols * d.waves - 1) / (d.wave_cols * d.waves);
        const dim3 grid((unsigned)((size_t)a.max_blocks * d.n_groups));
        // 16-bit rows leave through LDS as whole lines where a wave's pairs of tiles start on line boundaries
        // and the staging region of the widest body (four row tiles with pairs of blocks, else two) stays
        // within the LDS a launch gets without asking for more
        const bool   pairs_inst = d.pair_blocks && d.kblocks <= 2;
        const size_t stage      = (size_t)down_stage_bytes(d.waves, pairs_inst ? 4 : 2);
        d.out_staged = (!y32 && a.down_staged != 0 && (a.dim & 63) == 0 && ((uintptr_t)y & 127) == 0 && stage <= 65536) ? 1 : 0;
        const size_t lds = d.out_staged ? stage : 0;
        switch(d.kblocks)
        {
        case 1:
            if(d.pair_blocks)
                hipLaunchKernelGGL((moe_down_kernel<1, true>), grid, dim3(64 * d.waves), lds, stream, d);
            else
                hipLaunchKernelGGL((moe_down_kernel<1, false>), grid, dim3(64 * d.waves), lds, stream, d);
            break;
        case 2:
            if(d.pair_blocks)
                hipLaunchKernelGGL((moe_down_kernel<2, true>), grid, dim3(64 * d.waves), lds, stream, d);
            else
                hipLaunchKernelGGL((moe_down_kernel<2, false>), grid, dim3(64 * d.waves), lds, stream, d);
            break;
        case 3: hipLaunchKernelGGL((moe_down_kernel<3, false>), grid, dim3(64 * d.waves), lds, stream, d); break;
        default: hipLaunchKernelGGL((moe_down_kernel<4, false>), grid, dim3(64 * d.waves), lds, stream, d); break;
        }
    }
    else
    {
        d.n_groups = (a.dim + 255) / 256;
        hipLaunchKernelGGL(moe_down_long_k_kernel, dim3((unsigned)((size_t)a.max_blocks * d.n_groups)), dim3(256), 0,
                           stream, d);
    }

    if(!y32 && (a.dim & 7) == 0 && (a.out_stride & 7) == 0 && ((uintptr_t)a.out & 15) == 0 && ((uintptr_t)y & 15) == 0)
    {
        const dim3 grid8((unsigned)a.M, (unsigned)((a.dim / 8 + 255) / 256));
        auto combine8 = a.out_dtype == In16::bf16 ? moe_combine8_kernel<In16::bf16> : moe_combine8_kernel<In16::fp16>;
        hipLaunchKernelGGL(combine8, grid8, dim3(256), 0, stream, (const uint16_t*)y, a.sorted_weights, where, a.sorted_ids,
                           a.num_valid, a.max_padded, (uint16_t*)a.out, a.M, a.topk, a.dim, a.out_stride);
        return hipGetLastError();
    }
    const dim3 cgrid((unsigned)a.M, (unsigned)((a.dim / 4 + 255) / 256));
    auto combine = a.out_dtype == In16::bf16
                       ? (y32 ? moe_combine_kernel<In16::bf16, true> : moe_combine_kernel<In16::bf16, false>)
                       : (y32 ? moe_combine_kernel<In16::fp16, true> : moe_combine_kernel<In16::fp16, false>);
    hipLaunchKernelGGL(combine, cgrid, dim3(256), 0, stream, (const void*)y, a.sorted_weights, where, a.sorted_ids,
                       a.num_valid, a.max_padded, (uint16_t*)a.out, a.M, a.topk, a.dim, a.out_stride);
    return hipGetLastError();
}

} // namespace fp8bs
