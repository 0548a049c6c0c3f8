// moe_sorting for gfx950: stable token -> expert bucketing with padding to unit_size.
//
// Replaces ck_tile's MoeSortingKernel / MoeSortingMultiPhaseKernel_P0..P3
// (ops/fused_moe/kernel/moe_sorting_kernel.hpp:224-1152, :1576-3229) and produces exactly what
// ck_tile::reference_moe_sorting (host/reference/reference_moe_sorting.hpp:14-117) produces.
//
// Design (not ck_tile's mesh): the flat routing list ids[t*K+k] is cut into segments, one per
// wavefront.  Pass 1 counts experts per segment (wave ballot match + per-wave LDS histogram),
// pass 2 turns the [segment][expert] counts into output offsets (per-expert prefix over segments,
// padded prefix over experts), pass 3 walks every segment again and scatters: the rank of an
// entry inside its expert is segment offset + entries of that expert seen earlier in the wave
// walk + popcount of lower lanes holding the same expert.  The sort is stable by construction
// (no atomics decide an order), so the result is bit-exact with the host reference.  Small
// problems run all three passes in one workgroup; large ones in three launches.  Traffic is
// O(T*K) read twice plus O(segments*E) counters instead of ck_tile's O(E*T) mesh.
#include "common.hpp"
#include "device_utils.hpp"

#include <algorithm>
#include <mutex>

namespace mi355 {
namespace {

constexpr int kSeg               = 512;  // routing entries per wave segment (multi-launch path)
constexpr int kWalkBlock         = 256;  // 4 waves = 4 segments per workgroup
constexpr int kScanBlock         = 1024;
constexpr int kScanWaves         = kScanBlock / kWave;
constexpr int kMaxExperts        = 1024;
constexpr int kOneShotMaxEntries = 16384;
constexpr int kOneShotMaxExperts = 256;

// lanes of this wave whose expert id equals mine
__device__ inline uint64_t match_expert(int e, int nbits)
{
    uint64_t m = ~0ull;
    for(int b = 0; b < nbits; b++)
    {
        const bool bit     = (e >> b) & 1;
        const uint64_t bal = __ballot(bit);
        m &= bit ? bal : ~bal;
    }
    return m;
}

__device__ inline int real_tokens(const int* local_tokens, int tokens)
{
    if(local_tokens == nullptr)
        return tokens;
    int t = *local_tokens;
    return t < 0 ? 0 : (t > tokens ? tokens : t);
}

// One wave walks routing entries [begin, end) in order, 64 at a time.
// cnt[e] holds (COUNT) the number of entries of expert e seen so far, or (SCATTER) the output
// position of the next entry of expert e (negative: expert masked out, entries dropped).
// One 64-entry step of a wave's walk: lane handles routing entry i (expert e, weight w; e = -1 past
// the end).  cnt[e] holds (COUNT) the number of entries of expert e seen so far, or (SCATTER) the
// output position of the next entry of expert e (negative: expert masked out, entries dropped).
template <bool SCATTER>
__device__ inline void walk_step(int i, int e, float w, bool in_range, int K, int E, int nbits, int* cnt,
                                 int* __restrict__ out_ids, float* __restrict__ out_w, int* __restrict__ inv)
{
    const int lane   = threadIdx.x & (kWave - 1);
    const bool valid = e >= 0 && e < E;
    if(!valid)
        e = 0;
    const uint64_t same = match_expert(e, nbits) & __ballot(valid);
    const int before    = __popcll(same & ((1ull << lane) - 1ull));
    int base            = 0;
    if(valid)
        base = cnt[e];
    wave_sync(); // every lane has read cnt[] before a leader updates it
    if constexpr(SCATTER)
    {
        // inverse map for the grouped GEMMs' combine: where entry i went, -1 when it was dropped
        if(inv != nullptr && in_range)
            inv[i] = valid && base >= 0 ? base + before : -1;
    }
    if(valid)
    {
        if constexpr(SCATTER)
        {
            if(base >= 0)
            {
                const int t            = i / K;
                const int k            = i - t * K;
                out_ids[base + before] = mock_id(t, k);
                out_w[base + before]   = w;
            }
        }
        if(before == 0 && base >= 0)
            cnt[e] = base + __popcll(same);
    }
    wave_sync();
}

// One wave walks routing entries [begin, end) in order, 64 at a time.
template <bool SCATTER>
__device__ inline void walk_segment(const int* __restrict__ ids, const float* __restrict__ weights,
                                    int begin, int end, int K, int E, int nbits, int* cnt,
                                    int* __restrict__ out_ids, float* __restrict__ out_w,
                                    int* __restrict__ inv = nullptr)
{
    const int lane = threadIdx.x & (kWave - 1);
    // eight steps' entries are fetched together (a segment of the multi-phase passes is eight steps): one load
    // latency per segment instead of one per step
    constexpr int kAhead = 8;
    for(int i0 = begin; i0 < end; i0 += kAhead * kWave)
    {
        int ev[kAhead];
        float wv[kAhead];
#pragma unroll
        for(int u = 0; u < kAhead; u++)
        {
            const int i = i0 + u * kWave + lane;
            ev[u]       = i < end ? ids[i] : -1;
            wv[u]       = SCATTER && i < end ? weights[i] : 0.f;
        }
#pragma unroll
        for(int u = 0; u < kAhead; u++)
            if(i0 + u * kWave < end)
            {
                const int i = i0 + u * kWave + lane;
                walk_step<SCATTER>(i, ev[u], wv[u], i < end, K, E, nbits, cnt, out_ids, out_w, inv);
            }
    }
}

struct ScanShared
{
    int part[kScanBlock];  // [parts][Ep] partial sums over groups of segments
    int cnt[kMaxExperts];  // entries per expert
    int tiles[kMaxExperts];
    int tbase[kMaxExperts]; // first output tile of the expert
    int oeid[kMaxExperts];  // expert id written to sorted_expert_ids
    int wave[kScanWaves + 1];
    int wave3[3][kScanWaves + 1];
};

// Pass 2, run by one 1024-thread block.  counts is [nseg][E] (global or LDS): on entry the
// per-segment histogram, on exit the output position of each segment's first entry per expert
// (-1 for experts that produce no output).
__device__ inline void scan_phase(ScanShared& s, int* counts, int nseg, int E, int Ep, int U,
                                  const int* __restrict__ mask, int T, int K,
                                  int* __restrict__ sorted_ids, float* __restrict__ sorted_w,
                                  int* __restrict__ sorted_eid, int* __restrict__ total, const GemmPlan& plan,
                                  bool keep_empty)
{
    const int tid   = threadIdx.x;
    const int e     = tid & (Ep - 1);
    const int part  = tid / Ep;
    const int parts = kScanBlock / Ep;
    const int spp   = ceil_div(nseg, parts);
    const int s0    = part * spp;
    const int s1    = min(s0 + spp, nseg);

    // (both walks over the thread's segments fetch eight counters at a time: one workgroup runs this pass, and a chain
    // of dependent global loads, one per segment, would be most of its time)
    constexpr int kBatch = 8;
    int sum = 0;
    if(e < E)
    {
        int sg0 = s0;
        for(; sg0 + kBatch <= s1; sg0 += kBatch)
        {
            int c[kBatch];
#pragma unroll
            for(int u = 0; u < kBatch; u++)
                c[u] = counts[(sg0 + u) * E + e];
#pragma unroll
            for(int u = 0; u < kBatch; u++)
                sum += c[u];
        }
        for(; sg0 < s1; sg0++)
            sum += counts[sg0 * E + e];
    }
    s.part[part * Ep + e] = sum;
    __syncthreads();
    if(tid < Ep)
    {
        int run = 0;
        for(int p = 0; p < parts; p++)
        {
            const int v          = s.part[p * Ep + tid];
            s.part[p * Ep + tid] = run;
            run += v;
        }
        s.cnt[tid] = run;
    }
    if(tid >= Ep && tid < kMaxExperts)
        s.cnt[tid] = 0;
    __syncthreads();

    // an expert that is masked out is skipped without consuming an output expert id; an expert
    // with no token is skipped but does consume one (reference_moe_sorting.hpp:84-98), or, with
    // skip_experts_with_zero_token = false (keep_empty), owns one tile of padding like the reference's
    // expert_slices[e] = 1 (:43, :100-112)
    const bool on_rank = tid < E && (mask == nullptr || mask[tid] != 0);
    const int my_cnt   = tid < E ? s.cnt[tid] : 0;
    const int my_tiles = on_rank ? max(ceil_div(my_cnt, U), keep_empty ? 1 : 0) : 0;
    // one pass of block scans for the first output tile of each expert, the output expert ids and the number of
    // experts that have tokens
    const int scan_in[3] = {my_tiles, on_rank ? 1 : 0, on_rank && my_cnt > 0 ? 1 : 0};
    int scan_ex[3], scan_total[3];
    block_exclusive_scan_n<kScanWaves, 3>(scan_in, s.wave3, scan_ex, scan_total);
    const int tbase = scan_ex[0], oeid = scan_ex[1];
    const int total_tiles = scan_total[0], active = scan_total[2];
    if(tid < kMaxExperts)
    {
        s.tiles[tid] = my_tiles;
        s.tbase[tid] = tbase;
        s.oeid[tid]  = oeid;
    }
    __syncthreads();

    if(e < E)
    {
        int base = s.tiles[e] > 0 ? s.tbase[e] * U + s.part[part * Ep + e] : -1;
        int sg0 = s0;
        for(; sg0 + kBatch <= s1; sg0 += kBatch)
        {
            int c[kBatch];
#pragma unroll
            for(int u = 0; u < kBatch; u++)
                c[u] = counts[(sg0 + u) * E + e];
#pragma unroll
            for(int u = 0; u < kBatch; u++)
            {
                counts[(sg0 + u) * E + e] = base;
                if(base >= 0)
                    base += c[u];
            }
        }
        for(; sg0 < s1; sg0++)
        {
            const int c        = counts[sg0 * E + e];
            counts[sg0 * E + e] = base;
            if(base >= 0)
                base += c;
        }
    }

    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int pad  = mock_id(T, K);
    if((int64_t)E * U <= 65536)
    {
        // The usual sizes, flat over the whole block (this pass is one workgroup; a wave per expert walking its
        // tiles and pad cells in turn was a third of the one-workgroup sort's time at decode sizes).  An expert has
        // fewer than U pad cells: candidate (expert, o) is one of them when o < tiles * U - count.
        for(int idx = tid; idx < E * U; idx += kScanBlock)
        {
            const int ex = idx / U;
            const int o  = idx - ex * U;
            const int tl = s.tiles[ex];
            const int c  = s.cnt[ex];
            if(tl > 0 && o < tl * U - c)
            {
                const int pos   = s.tbase[ex] * U + c + o;
                sorted_ids[pos] = pad;
                sorted_w[pos]   = 0.f;
            }
        }
        // the expert of output tile t: the last one whose first tile is at or before t (experts without tiles share
        // their first-tile index with the next expert that has some, and come before it)
        for(int t = tid; t < total_tiles; t += kScanBlock)
        {
            int lo = 0, hi = E; // first expert with tbase > t
            while(lo < hi)
            {
                const int mid = (lo + hi) >> 1;
                if(s.tbase[mid] <= t)
                    lo = mid + 1;
                else
                    hi = mid;
            }
            sorted_eid[t] = s.oeid[lo - 1];
        }
    }
    else
    for(int ex = wave; ex < E; ex += kScanWaves)
    {
        const int tl = s.tiles[ex];
        if(tl == 0)
            continue;
        const int tb = s.tbase[ex];
        const int oe = s.oeid[ex];
        for(int j = lane; j < tl; j += kWave)
            sorted_eid[tb + j] = oe;
        for(int p = s.cnt[ex] + lane; p < tl * U; p += kWave)
        {
            sorted_ids[tb * U + p] = pad;
            sorted_w[tb * U + p]   = 0.f;
        }
    }
    if(tid == 0)
    {
        total[0] = total_tiles * U;
        total[1] = T;
    }

    // work list of the grouped GEMMs: the padded rows of an expert split evenly into tiles
    if(plan.tile_map != nullptr)
    {
        const int rows = tid < E ? s.tiles[tid] * U : 0;
        int rows_per_tile = plan.rows_per_tile;
        if(plan.alt_rows_per_tile > 0) // (uniform: every thread takes this branch or none)
        {
            if(active >= plan.alt_min_active && (int64_t)total_tiles * U >= (int64_t)plan.alt_min_rows * active)
                rows_per_tile = plan.alt_rows_per_tile;
            if(tid == 0)
                plan.tile_map[1] = rows_per_tile;
        }
        else if(tid == 0)
            plan.tile_map[1] = 0;
        const int nt   = ceil_div(rows, rows_per_tile);
        int n_tiles;
        const int tb = block_exclusive_scan<kScanWaves>(nt, s.wave, n_tiles);
        if(nt > 0)
        {
            const int per = round_up(ceil_div(rows, nt), 32);
            for(int j = 0; j < nt && tb + j < plan.max_tiles; j++)
            {
                int* ent = plan.tile_map + kMapHdr + (tb + j) * kMapEnt;
                ent[0]   = s.oeid[tid];
                ent[1]   = s.tbase[tid] * U + j * per;
                ent[2]   = min(per, rows - j * per);
                ent[3]   = tb;
                ent[4]   = nt;
                ent[5]   = s.tbase[tid] * U;
                ent[6]   = rows;
                ent[7]   = per;
            }
        }
        if(tid == 0)
            plan.tile_map[0] = min(n_tiles, plan.max_tiles);
    }
}

__device__ inline void zero_buffer(uint4* buf, int64_t nvec, int64_t first, int64_t stride)
{
    const uint4 z = {0u, 0u, 0u, 0u};
    for(int64_t i = first; i < nvec; i += stride)
        buf[i] = z;
}

struct SortParams
{
    const int* ids;
    const float* weights;
    const int* mask;
    const int* local_tokens;
    int* sorted_ids;
    float* sorted_w;
    int* sorted_eid;
    int* total;
    uint4* moe_buf;
    int64_t moe_row_vec16; // 16-byte vectors per token row of moe_buf
    int* counts;           // workspace [nseg][E]
    GemmPlan plan;         // tile_map == nullptr: nothing to prepare
    int tokens, K, E, Ep, nbits, U, nseg, work_blocks;
    int keep_empty; // experts without tokens own one tile of padding (SkipExpertsWithZeroTokens = false)
};

// ---- whole sort in one workgroup (block 0); the other blocks zero moe_buf.
// IN_REGS: the wave's entries fit kMaxSteps registers per lane and are read once; otherwise (a caller that forces the
// single kernel on a large problem) both walks stream them from memory.
template <bool IN_REGS>
__global__ __launch_bounds__(kScanBlock) void moe_sorting_oneshot_kernel(SortParams p)
{
    extern __shared__ int dyn_lds[]; // [kScanWaves][E]
    __shared__ ScanShared sh;
    const int T = real_tokens(p.local_tokens, p.tokens);
    if(blockIdx.x > 0)
    {
        zero_buffer(p.moe_buf, p.moe_row_vec16 * T,
                    (int64_t)(blockIdx.x - 1) * kScanBlock + threadIdx.x,
                    (int64_t)(gridDim.x - 1) * kScanBlock);
        return;
    }
    const int N      = T * p.K;
    const int lane   = threadIdx.x & (kWave - 1);
    const int wave   = threadIdx.x / kWave;
    const int seglen = round_up(ceil_div(N, kScanWaves), kWave);
    const int begin  = min(wave * seglen, N);
    const int end    = min(begin + seglen, N);
    int* cnt         = dyn_lds + wave * p.E;
    for(int e = lane; e < p.E; e += kWave)
        cnt[e] = 0;
    wave_sync();
    int* inv = p.plan.tile_map != nullptr ? p.plan.inv : nullptr;
    // The wave's entries are read once, all loads issued together, and stay in registers for both walks: fetched
    // step by step they would be a chain of dependent global loads in the one workgroup that does all the work.
    constexpr int kMaxSteps = IN_REGS ? kOneShotMaxEntries / kScanBlock : 1;
    int ev[kMaxSteps];
    float wv[kMaxSteps];
    if constexpr(IN_REGS)
    {
#pragma unroll
        for(int u = 0; u < kMaxSteps; u++)
        {
            const int i = begin + u * kWave + lane;
            ev[u]       = i < end ? p.ids[i] : -1;
            wv[u]       = i < end ? p.weights[i] : 0.f;
        }
#pragma unroll
        for(int u = 0; u < kMaxSteps; u++)
            if(begin + u * kWave < end)
            {
                const int i = begin + u * kWave + lane;
                walk_step<false>(i, ev[u], wv[u], i < end, p.K, p.E, p.nbits, cnt, nullptr, nullptr, nullptr);
            }
    }
    else
        walk_segment<false>(p.ids, p.weights, begin, end, p.K, p.E, p.nbits, cnt, nullptr, nullptr);
    __syncthreads();
    scan_phase(sh, dyn_lds, kScanWaves, p.E, p.Ep, p.U, p.mask, T, p.K, p.sorted_ids, p.sorted_w,
               p.sorted_eid, p.total, p.plan, p.keep_empty != 0);
    __syncthreads();
    if constexpr(IN_REGS)
    {
#pragma unroll
        for(int u = 0; u < kMaxSteps; u++)
            if(begin + u * kWave < end)
            {
                const int i = begin + u * kWave + lane;
                walk_step<true>(i, ev[u], wv[u], i < end, p.K, p.E, p.nbits, cnt, p.sorted_ids, p.sorted_w, inv);
            }
    }
    else
        walk_segment<true>(p.ids, p.weights, begin, end, p.K, p.E, p.nbits, cnt, p.sorted_ids, p.sorted_w, inv);
}

// ---- pass 1: per-segment expert histogram; trailing blocks zero moe_buf
__global__ __launch_bounds__(kWalkBlock) void moe_sorting_count_kernel(SortParams p)
{
    extern __shared__ int dyn_lds[]; // [4][E]
    const int T = real_tokens(p.local_tokens, p.tokens);
    if((int)blockIdx.x >= p.work_blocks)
    {
        zero_buffer(p.moe_buf, p.moe_row_vec16 * T,
                    (int64_t)(blockIdx.x - p.work_blocks) * kWalkBlock + threadIdx.x,
                    (int64_t)(gridDim.x - p.work_blocks) * kWalkBlock);
        return;
    }
    const int N    = T * p.K;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int seg  = blockIdx.x * (kWalkBlock / kWave) + wave;
    if(seg >= p.nseg)
        return;
    int* cnt = dyn_lds + wave * p.E;
    for(int e = lane; e < p.E; e += kWave)
        cnt[e] = 0;
    wave_sync();
    const int begin = min(seg * kSeg, N);
    const int end   = min(begin + kSeg, N);
    walk_segment<false>(p.ids, p.weights, begin, end, p.K, p.E, p.nbits, cnt, nullptr, nullptr);
    for(int e = lane; e < p.E; e += kWave)
        p.counts[seg * p.E + e] = cnt[e];
}

// ---- pass 2
__global__ __launch_bounds__(kScanBlock) void moe_sorting_scan_kernel(SortParams p)
{
    __shared__ ScanShared sh;
    const int T = real_tokens(p.local_tokens, p.tokens);
    scan_phase(sh, p.counts, p.nseg, p.E, p.Ep, p.U, p.mask, T, p.K, p.sorted_ids, p.sorted_w,
               p.sorted_eid, p.total, p.plan, p.keep_empty != 0);
}

// ---- pass 3
__global__ __launch_bounds__(kWalkBlock) void moe_sorting_scatter_kernel(SortParams p)
{
    extern __shared__ int dyn_lds[]; // [4][E]
    const int T    = real_tokens(p.local_tokens, p.tokens);
    const int N    = T * p.K;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int seg  = blockIdx.x * (kWalkBlock / kWave) + wave;
    if(seg >= p.nseg)
        return;
    int* cnt = dyn_lds + wave * p.E;
    for(int e = lane; e < p.E; e += kWave)
        cnt[e] = p.counts[seg * p.E + e];
    wave_sync();
    const int begin = min(seg * kSeg, N);
    const int end   = min(begin + kSeg, N);
    walk_segment<true>(p.ids, p.weights, begin, end, p.K, p.E, p.nbits, cnt, p.sorted_ids, p.sorted_w,
                       p.plan.tile_map != nullptr ? p.plan.inv : nullptr);
}

inline bool use_oneshot(int64_t entries, int experts)
{
    return entries <= kOneShotMaxEntries && experts <= kOneShotMaxExperts;
}

} // namespace

// dispatch_policy as in ck_tile's moe_sorting_get_workspace_size (moe_sorting_kernel.hpp:1407-1438): 0 = the library
// picks, 1 = always the single kernel (no workspace), 2 = always the multi-launch passes
size_t sorting_workspace_bytes(int32_t tokens, int32_t experts, int32_t topk, int32_t dispatch_policy)
{
    if(tokens < 0 || experts <= 0 || topk <= 0)
        return 0;
    const int64_t n = (int64_t)tokens * topk;
    if(dispatch_policy == 1 || (dispatch_policy != 2 && use_oneshot(n, experts)))
        return 0;
    return round_up<size_t>((size_t)std::max<int64_t>(ceil_div<int64_t>(n, kSeg), 1) * experts * sizeof(int), 256);
}

int launch_moe_sorting(const mi355_moe_sorting_args& a, hipStream_t stream, const GemmPlan* plan, bool keep_empty,
                       int dispatch_policy)
{
    if(dispatch_policy < 0 || dispatch_policy > 2)
        return fail(MI355_MOE_E_INVALID, "moe_sorting: dispatch_policy=%d outside [0, 2]", dispatch_policy);
    // (an empty batch writes nothing but the totals unless experts without tokens keep a unit: its arrays may be
    // empty, and an empty device array has no address)
    const bool writes_rows = a.tokens > 0 || keep_empty;
    if((a.tokens > 0 && (!a.p_topk_ids || !a.p_weights)) || !a.p_total_tokens_post_pad ||
       (writes_rows && (!a.p_sorted_token_ids || !a.p_sorted_weights || !a.p_sorted_expert_ids)))
        return fail(MI355_MOE_E_INVALID, "moe_sorting: null input or output pointer");
    if(a.tokens < 0 || a.tokens >= (1 << 24))
        return fail(MI355_MOE_E_INVALID, "moe_sorting: tokens=%d outside [0, 2^24)", a.tokens);
    if(a.topk < 1 || a.topk > 255)
        return fail(MI355_MOE_E_INVALID, "moe_sorting: topk=%d outside [1, 255]", a.topk);
    if(a.num_experts < 1 || a.num_experts > kMaxExperts)
        return fail(MI355_MOE_E_INVALID, "moe_sorting: num_experts=%d outside [1, %d]", a.num_experts,
                    kMaxExperts);
    if(a.unit_size < 1)
        return fail(MI355_MOE_E_INVALID, "moe_sorting: unit_size=%d", a.unit_size);
    const int64_t n = (int64_t)a.tokens * a.topk;
    if(n + (int64_t)a.num_experts * a.unit_size >= (1ll << 31))
        return fail(MI355_MOE_E_INVALID, "moe_sorting: tokens*topk too large for int32 positions");

    SortParams p{};
    p.ids          = static_cast<const int*>(a.p_topk_ids);
    p.weights      = static_cast<const float*>(a.p_weights);
    p.mask         = static_cast<const int*>(a.p_local_expert_mask);
    p.local_tokens = static_cast<const int*>(a.p_local_tokens);
    p.sorted_ids   = static_cast<int*>(a.p_sorted_token_ids);
    p.sorted_w     = static_cast<float*>(a.p_sorted_weights);
    p.sorted_eid   = static_cast<int*>(a.p_sorted_expert_ids);
    p.total        = static_cast<int*>(a.p_total_tokens_post_pad);
    if(plan != nullptr)
        p.plan = *plan;
    p.keep_empty   = keep_empty ? 1 : 0;
    p.tokens       = a.tokens;
    p.K            = a.topk;
    p.E            = a.num_experts;
    p.U            = a.unit_size;
    p.Ep           = 1;
    while(p.Ep < p.E)
        p.Ep <<= 1;
    p.nbits = 0;
    while((1 << p.nbits) < p.E)
        p.nbits++;

    int zero_blocks = 0;
    if(a.p_moe_buf != nullptr)
    {
        const int64_t row_bytes = (int64_t)a.moe_buf_interm_dim * a.moe_buf_elem_bytes;
        if(row_bytes <= 0 || row_bytes % 16 != 0)
            return fail(MI355_MOE_E_INVALID,
                        "moe_sorting: moe_buf row of %lld bytes is not a positive multiple of 16",
                        (long long)row_bytes);
        if(reinterpret_cast<uintptr_t>(a.p_moe_buf) % 16 != 0)
            return fail(MI355_MOE_E_INVALID, "moe_sorting: p_moe_buf is not 16-byte aligned");
        p.moe_buf       = static_cast<uint4*>(a.p_moe_buf);
        p.moe_row_vec16 = row_bytes / 16;
        const int64_t nvec = p.moe_row_vec16 * a.tokens;
        zero_blocks = (int)std::min<int64_t>(ceil_div<int64_t>(nvec, 4 * kScanBlock), (int64_t)device_info().num_cu * 4);
        if(nvec > 0 && zero_blocks < 1)
            zero_blocks = 1;
    }

    if(dispatch_policy == 1 || (dispatch_policy == 0 && use_oneshot(n, p.E)))
    {
        p.nseg = kScanWaves;
        KernelTimer timer(MI355_MOE_K_SORT_ONESHOT, stream);
        const size_t lds = kScanWaves * p.E * sizeof(int); // at most 64 KB beside the 30 KB of static LDS
        if(use_oneshot(n, p.E))
            hipLaunchKernelGGL(moe_sorting_oneshot_kernel<true>, dim3(1 + zero_blocks), dim3(kScanBlock), lds, stream, p);
        else
        {
            static std::once_flag once[64];
            int dev = 0;
            (void)hipGetDevice(&dev);
            hipError_t attr = hipSuccess;
            auto set_attr = [&] {
                attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_sorting_oneshot_kernel<false>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kScanWaves * kMaxExperts * (int)sizeof(int));
            };
            if(dev >= 0 && dev < 64)
                std::call_once(once[dev], set_attr);
            else
                set_attr();
            MI355_HIP_TRY(attr);
            hipLaunchKernelGGL(moe_sorting_oneshot_kernel<false>, dim3(1 + zero_blocks), dim3(kScanBlock), lds, stream, p);
        }
        MI355_HIP_TRY(hipGetLastError());
        return MI355_MOE_OK;
    }
    if(a.p_ws == nullptr)
        return fail(MI355_MOE_E_WORKSPACE, "moe_sorting: p_ws is null but %zu bytes are needed",
                    sorting_workspace_bytes(a.tokens, a.num_experts, a.topk, dispatch_policy));
    p.counts      = static_cast<int*>(a.p_ws);
    p.nseg        = (int)std::max<int64_t>(ceil_div<int64_t>(n, kSeg), 1);
    p.work_blocks = ceil_div(p.nseg, kWalkBlock / kWave);
    const size_t lds = (kWalkBlock / kWave) * p.E * sizeof(int);
    {
        KernelTimer timer(MI355_MOE_K_SORT_COUNT, stream);
        hipLaunchKernelGGL(moe_sorting_count_kernel, dim3(p.work_blocks + zero_blocks), dim3(kWalkBlock), lds,
                           stream, p);
    }
    MI355_HIP_TRY(hipGetLastError());
    {
        KernelTimer timer(MI355_MOE_K_SORT_SCAN, stream);
        hipLaunchKernelGGL(moe_sorting_scan_kernel, dim3(1), dim3(kScanBlock), 0, stream, p);
    }
    MI355_HIP_TRY(hipGetLastError());
    {
        KernelTimer timer(MI355_MOE_K_SORT_SCATTER, stream);
        hipLaunchKernelGGL(moe_sorting_scatter_kernel, dim3(p.work_blocks), dim3(kWalkBlock), lds, stream, p);
    }
    MI355_HIP_TRY(hipGetLastError());
    return MI355_MOE_OK;
}

} // namespace mi355
