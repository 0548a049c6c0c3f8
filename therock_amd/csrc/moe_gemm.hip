// Grouped GEMMs of the fused-MoE path for gfx950 (CDNA4, wave64, MFMA 32x32).
//
// Replaces ck_tile's FusedMoeGemmKernel + FusedMoeGemmPipeline_FlatmmUk
// (ops/fused_moe/kernel/fused_moegemm_kernel.hpp:238-259,
//  ops/fused_moe/pipeline/fused_moegemm_pipeline_flatmm_uk.hpp:169-416); numerics follow
// ck_tile::reference_fused_moe (host/reference/reference_fused_moe.hpp:42-204).
//
// Instead of ck_tile's single kernel (32 sorted rows x 512 intermediate columns per workgroup,
// bf16 atomics into the output) the path is three launches over a tile list built from the sort:
//   gemm0  Y[row, n]   = silu(x . Wgate[n]) * (x . Wup[n])      (gather rows by sorted token id)
//   gemm1  P[row, h]   = Y[row] . Wdown[h]                      (bf16 partial per sorted row)
//   combine O[t, h]    = sum_k w[t,k] * P[pos(t,k), h]  in slot order, fp32, one rounding to bf16
// A workgroup (4 waves) owns up to MBLK*32 sorted rows of ONE expert and 256 weight rows
// (gemm0: 128 gate + 128 up rows = 128 Y columns).  The MFMA's M side is the weight rows and its
// N side the tokens, so every lane ends up with 16 consecutive output channels of one token and
// the SiLU*up, the scales and the packing all happen in registers.  All four waves share the
// token tile and split the weight rows, which keeps the waves balanced for any number of rows.
// Operand tiles are staged through LDS (16-byte padded rows, conflict-free ds_read_b128) with the
// next K tile prefetched into registers while the current one feeds the MFMAs.
#include "moe_gemm_device.hpp"

#include <algorithm>

namespace mi355 {
using namespace gemm;
namespace {

// ---------------------------------------------------------------------------------------------
// GEMM0 : MODE in {kBf16, kFp8, kI8};  GEMM1 : MODE in {kBf16, kFp8, kBf16W8, kI8}
template <int MODE, bool GEMM0, int MBLK>
__global__ __launch_bounds__(kBlock, 2) void moe_gemm_kernel(const GemmParams p)
{
    using MT  = ModeTraits<MODE>;
    using Acc = typename MT::Acc;
    constexpr int kOpB     = MT::kOpB;
    constexpr int kWKB     = MT::kWKB;
    constexpr int kXKB     = MT::kXKB; // bytes of K per row of the token tile
    constexpr int kXStride = kXKB + kPadB;
    constexpr int kWStride = kWKB + kPadB;
    constexpr int kSteps   = kXKB / (2 * kOpB); // MFMAs along K per tile
    constexpr int kXChunks = kXKB / 16;
    constexpr int kXRowsPerPass = kBlock / kXChunks;
    constexpr int kXLoads  = MBLK * 32 / kXRowsPerPass;
    constexpr int kWChunks = kWKB / 16;            // 16-byte chunks per weight tile row
    constexpr int kWLoads  = kWRows * kWChunks / kBlock;
    constexpr int kWRowsPerPass = kBlock / kWChunks;
    constexpr bool kMx     = MODE == kFp8 && !GEMM0; // token operand carries e8m0 block scales

    extern __shared__ __align__(16) unsigned char lds[];
    unsigned char* lds_w = lds;
    unsigned char* lds_x = lds + kWRows * kWStride;

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int r32  = lane & 31;
    const int kg   = lane >> 5;

    // ---- work item: XCD x gets a contiguous range of the work list (workgroup ids are dealt
    // round-robin to the 8 XCDs), and inside an expert the M tiles of one weight tile are adjacent
    const TileRef tile = lookup_tile(p.tile_map, p.n_ntiles, p.max_tiles, blockIdx.x, p.tile_rows);
    if(!tile.ok)
        return;
    const int expert = tile.expert;
    const int row0   = tile.row0;
    const int nt     = tile.nt;
    const int nrows  = tile.nrows;
    const int nmb    = ceil_div(nrows, 32);

    // ---- global -> register staging assignments
    const int xchunk = tid % kXChunks;
    const int xrow   = tid / kXChunks; // + kXRowsPerPass*j
    const unsigned char* xptr[kXLoads];
    bool xvalid[kXLoads];
#pragma unroll
    for(int j = 0; j < kXLoads; j++)
    {
        const int r = xrow + kXRowsPerPass * j;
        if constexpr(GEMM0)
        {
            int sid = p.tokens;
            if(r < nrows)
                sid = p.sorted_ids[row0 + r];
            xvalid[j] = (sid & 0xffffff) < p.tokens;
            xptr[j]   = p.x + (int64_t)(xvalid[j] ? token_row(p, sid) : 0u) * p.x_row_bytes + xchunk * 16;
        }
        else
        {
            xvalid[j]   = r < nrows;
            int64_t src = row0 + (xvalid[j] ? r : 0);
            if(p.slot_rows > 0)
            {
                const int sid = p.sorted_ids[src];
                xvalid[j]     = xvalid[j] && (sid & 0xffffff) < p.tokens;
                src           = xvalid[j] ? slot_row(sid, p.slot_rows) : 0;
            }
            xptr[j] = p.x + src * p.x_row_bytes + xchunk * 16;
        }
    }

    // (row of the LDS weight tile, + kWRowsPerPass * j, and 16-byte chunk of the 128-byte K window) a thread fetches.
    // Row-major weights: 8 consecutive threads walk the 128 contiguous bytes of a row.  ck_tile's pre-shuffled layout
    // (1 KiB blocks of 16 rows x 64 bytes, pieces ordered by chunk, then row): 16 consecutive threads take the 16 rows
    // of a chunk, a wave one whole block - the rows whose channels, by chan_of_row(), are 16 (wave / 2) + tid % 16.
    static_assert(kWChunks == 8 && kWRowsPerPass == 32, "the pre-shuffled assignment below covers 32 rows x 8 chunks per pass");
    const bool wperm = p.w_permuted != 0;
    const int wchunk = wperm ? ((wave & 1) << 2) | ((tid >> 4) & 3) : tid % kWChunks;
    const int wrow   = wperm ? (((tid >> 3) & 1) << 4) | (((tid >> 2) & 1) << 3) | ((wave >> 1) << 2) | (tid & 3) : tid / kWChunks;
    const bool paired = GEMM0 && !p.gate_only; // gate rows paired with up rows (see run_epilogue)
    const int n_base  = nt * (paired ? 128 : 256);
    const unsigned char* wbase = p.w + (int64_t)expert * p.w_expert_bytes;
    const int w_kadv           = weight_k_advance(p, kWKB); // bytes between the K windows of two steps
    int64_t woff[kWLoads];
#pragma unroll
    for(int j = 0; j < kWLoads; j++)
    {
        const int lrow = wrow + kWRowsPerPass * j;
        const int blk  = lrow >> 5;
        const int c    = chan_of_row(lrow & 31);
        int grow;
        if(paired)
        {
            const int col = min(n_base + (blk >> 1) * 32 + c, p.n_out - 1);
            grow          = (blk & 1) * p.n_out + col;
        }
        else
        {
            grow = min(n_base + blk * 32 + c, p.n_total - 1);
        }
        // (row-major rows may lie 4 GiB or more into the expert: 64-bit there)
        woff[j] = wperm ? (int64_t)weight_offset(p, grow, wchunk) : (int64_t)grow * p.w_row_bytes + wchunk * 16;
    }

    uint4 xv[kXLoads];
    uint4 wv[kWLoads];
    uint32_t ys_next[MBLK], ys_cur[MBLK];
    const uint4 zero4 = {0u, 0u, 0u, 0u};

    auto load_tiles = [&](int kt) {
        const int kx = kt * kXKB + xchunk * 16;
#pragma unroll
        for(int j = 0; j < kXLoads; j++)
        {
            xv[j] = zero4;
            if(xvalid[j] && kx < p.k_bytes_x)
                xv[j] = *reinterpret_cast<const uint4*>(xptr[j] + kt * kXKB);
        }
        const int kw = kt * kWKB + wchunk * 16;
#pragma unroll
        for(int j = 0; j < kWLoads; j++)
        {
            wv[j] = zero4;
            if(kw < p.k_bytes_w)
            {
                // decode-sized tiles stream every weight exactly once: non-temporal loads reach a
                // markedly higher HBM rate than cached ones
                const uint4* src = reinterpret_cast<const uint4*>(wbase + woff[j] + kt * w_kadv);
                if constexpr(MBLK == 1)
                {
                    typedef __attribute__((ext_vector_type(4))) unsigned u32x4_t;
                    const u32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(src));
                    wv[j]           = make_uint4(t[0], t[1], t[2], t[3]);
                }
                else
                    wv[j] = *src;
            }
        }
        if constexpr(kMx)
        {
#pragma unroll
            for(int j = 0; j < MBLK; j++)
            {
                ys_next[j] = 0x7f7f7f7fu;
                const int r = j * 32 + r32;
                if(r < nrows)
                {
                    const unsigned char* sp = p.y_scale + (int64_t)(kt * 4) * p.ys_kb_stride + row0 + r;
                    ys_next[j] = sp[0] | (sp[p.ys_kb_stride] << 8) | (sp[2 * p.ys_kb_stride] << 16) |
                                 (static_cast<uint32_t>(sp[3 * p.ys_kb_stride]) << 24);
                }
            }
        }
    };

    Acc acc[MBLK][2];
#pragma unroll
    for(int j = 0; j < MBLK; j++)
#pragma unroll
        for(int b = 0; b < 2; b++)
#pragma unroll
            for(int v = 0; v < 16; v++)
                acc[j][b][v] = 0;

    const int kt_count = ceil_div(p.k_bytes_x, kXKB);
    load_tiles(0);
    for(int kt = 0; kt < kt_count; kt++)
    {
        // registers -> LDS
#pragma unroll
        for(int j = 0; j < kXLoads; j++)
            if(((xrow + kXRowsPerPass * j) >> 5) < nmb)
                *reinterpret_cast<uint4*>(lds_x + (xrow + kXRowsPerPass * j) * kXStride + xchunk * 16) = xv[j];
#pragma unroll
        for(int j = 0; j < kWLoads; j++)
            *reinterpret_cast<uint4*>(lds_w + (wrow + kWRowsPerPass * j) * kWStride + wchunk * 16) = wv[j];
        if constexpr(kMx)
        {
#pragma unroll
            for(int j = 0; j < MBLK; j++)
                ys_cur[j] = ys_next[j];
        }
        __syncthreads();
        if(kt + 1 < kt_count)
            load_tiles(kt + 1);

        // MFMAs from LDS
#pragma unroll
        for(int s = 0; s < kSteps; s++)
        {
            Frag wf[2];
#pragma unroll
            for(int b = 0; b < 2; b++)
            {
                const unsigned char* wp = lds_w + ((wave * 2 + b) * 32 + r32) * kWStride;
                if constexpr(MODE == kBf16W8)
                    wf[b].lo = int8x8_to_bf16x8(*reinterpret_cast<const uint2*>(wp + (2 * s + kg) * 8));
                else if constexpr(kOpB == 16)
                    wf[b].lo = *reinterpret_cast<const uint4*>(wp + (2 * s + kg) * 16);
                else
                {
                    // f8f6f4 operands: the low 16 bytes of lanes r and r+32 form one 32-element
                    // scale block, the high 16 bytes the next one
                    wf[b].lo = *reinterpret_cast<const uint4*>(wp + (4 * s + kg) * 16);
                    wf[b].hi = *reinterpret_cast<const uint4*>(wp + (4 * s + 2 + kg) * 16);
                }
            }
#pragma unroll
            for(int j = 0; j < MBLK; j++)
            {
                if(j < nmb)
                {
                    Frag xf;
                    const unsigned char* xp = lds_x + (j * 32 + r32) * kXStride;
                    uint32_t xs             = 127;
                    if constexpr(kOpB == 16)
                        xf.lo = *reinterpret_cast<const uint4*>(xp + (2 * s + kg) * 16);
                    else
                    {
                        xf.lo = *reinterpret_cast<const uint4*>(xp + (4 * s + kg) * 16);
                        xf.hi = *reinterpret_cast<const uint4*>(xp + (4 * s + 2 + kg) * 16);
                        // lane r carries the scale of block 2s, lane r+32 that of block 2s+1
                        if constexpr(kMx)
                            xs = (ys_cur[j] >> (8 * (2 * s + kg))) & 0xffu;
                    }
                    acc[j][0] = mfma<MODE>(wf[0], xf, xs, acc[j][0]);
                    acc[j][1] = mfma<MODE>(wf[1], xf, xs, acc[j][1]);
                }
            }
        }
        __syncthreads();
    }

    // ---- epilogue: lane owns token row (j*32 + r32) and 16 consecutive channels per block
    run_epilogue<MODE, GEMM0, MBLK, true>(p, acc, expert, row0, nrows, 0, 32, nmb, n_base, wave, r32, kg);
}

// ---------------------------------------------------------------------------------------------
// Tile list: one entry per (expert, group of <= rows_per_tile sorted rows), rows split evenly.
// Block 0 builds the list from sorted_expert_ids; every block helps reset the inverse map, which
// moe_inv_kernel then fills from the sorted ids (the sort does both itself in the fused entry point).
constexpr int kPrepBlock = 1024;
constexpr int kPrepWaves = kPrepBlock / kWave;

__global__ __launch_bounds__(kPrepBlock) void moe_prep_kernel(const int* __restrict__ sorted_eid,
                                                               const int* __restrict__ post_pad_ptr, int unit,
                                                               int experts, int rows_per_tile, int max_units,
                                                               int max_tiles, int* __restrict__ tile_map,
                                                               int* __restrict__ inv, int n_inv, int alt_rows_per_tile,
                                                               int alt_min_rows, int alt_min_active)
{
    for(int i = blockIdx.x * kPrepBlock + threadIdx.x; i < n_inv; i += gridDim.x * kPrepBlock)
        inv[i] = -1;
    if(blockIdx.x != 0)
        return;
    __shared__ int s_wave[kPrepWaves + 1];
    __shared__ int s_lo[kPrepBlock], s_hi[kPrepBlock]; // first and one-past-last sort unit of each expert
    const int post_pad = post_pad_ptr[0];
    int nunits         = post_pad / unit;
    nunits             = max(0, min(nunits, max_units));
    // sorted_expert_ids is non-decreasing: the units of an expert form one run, found by looking at each unit's
    // neighbours - independent loads, where a binary search per expert is a chain of a dozen dependent ones
    s_lo[threadIdx.x] = 0;
    s_hi[threadIdx.x] = 0;
    __syncthreads();
    for(int u = threadIdx.x; u < nunits; u += kPrepBlock)
    {
        const int e    = sorted_eid[u];
        const int prev = u > 0 ? sorted_eid[u - 1] : -1;
        const int next = u + 1 < nunits ? sorted_eid[u + 1] : -1;
        if(e >= 0 && e < experts)
        {
            if(prev != e)
                s_lo[e] = u;
            if(next != e)
                s_hi[e] = u + 1;
        }
    }
    __syncthreads();
    int total          = 0;
    for(int e0 = 0; e0 < experts; e0 += kPrepBlock) // experts <= 1024: one pass
    {
        const int e = e0 + threadIdx.x;
        int lo = 0, hi = 0;
        if(e < experts)
        {
            lo = s_lo[e];
            hi = max(s_hi[e], lo);
        }
        const int rows = (hi - lo) * unit;
        // the same choice between two tile heights as the sort makes in the fused entry point (see alt_mblk), from
        // the rows per active expert; 0 in the header: no choice, the kernels do not look
        if(alt_rows_per_tile > 0) // (uniform; experts <= 1024 = one pass of this loop)
        {
            int active;
            (void)block_exclusive_scan<kPrepWaves>(rows > 0 ? 1 : 0, s_wave, active);
            if(active >= alt_min_active && (int64_t)nunits * unit >= (int64_t)alt_min_rows * active)
                rows_per_tile = alt_rows_per_tile;
            if(threadIdx.x == 0)
                tile_map[1] = rows_per_tile;
        }
        else if(threadIdx.x == 0)
            tile_map[1] = 0;
        const int nt   = ceil_div(rows, rows_per_tile);
        int sum;
        const int tb   = total + block_exclusive_scan<kPrepWaves>(nt, s_wave, sum);
        total += sum;
        if(nt > 0)
        {
            const int per = round_up(ceil_div(rows, nt), 32);
            for(int j = 0; j < nt; j++)
            {
                if(tb + j >= max_tiles)
                    break;
                int* ent = tile_map + kMapHdr + (tb + j) * kMapEnt;
                ent[0]   = e;
                ent[1]   = lo * unit + j * per;
                ent[2]   = min(per, rows - j * per);
                ent[3]   = tb;
                ent[4]   = nt;
                ent[5]   = lo * unit;
                ent[6]   = rows;
                ent[7]   = per;
            }
        }
    }
    if(threadIdx.x == 0)
        tile_map[0] = min(total, max_tiles);
}

// inv[token * topk + slot] = sorted position, for every real entry of the sorted id list
__global__ __launch_bounds__(256) void moe_inv_kernel(const int* __restrict__ sorted_ids,
                                                       const int* __restrict__ post_pad_ptr, int max_pad, int tokens,
                                                       int topk, int* __restrict__ inv)
{
    const int post_pad = min(post_pad_ptr[0], max_pad);
    for(int pos = blockIdx.x * 256 + threadIdx.x; pos < post_pad; pos += gridDim.x * 256)
    {
        const int id   = sorted_ids[pos];
        const int tok  = id & 0xffffff;
        const int slot = static_cast<int>(static_cast<uint32_t>(id) >> 24);
        if(tok < tokens && slot < topk)
            inv[tok * topk + slot] = pos;
    }
}

// 16-byte fill (a kernel, not a memset node: the path may be captured in a graph)
__global__ __launch_bounds__(256) void fill_u32x4_kernel(uint4* __restrict__ dst, int64_t n, uint32_t v)
{
    for(int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
        dst[i] = make_uint4(v, v, v, v);
}

// O[t, h] = sum over slots (in slot order) of top-k weight * bf16 partial, fp32 accumulate, one rounding
__global__ __launch_bounds__(256) void moe_combine_kernel(const unsigned char* __restrict__ part,
                                                           const int* __restrict__ inv,
                                                           const float* __restrict__ sorted_w,
                                                           unsigned char* __restrict__ out, int topk, int hidden,
                                                           int64_t out_row_bytes, int accumulate,
                                                           const float* __restrict__ slot_scale,
                                                           const float* __restrict__ bias,
                                                           const int* __restrict__ sorted_eid, int unit, int f16,
                                                           const float* __restrict__ row_scale = nullptr)
{
    // f16: the partial rows and the output are fp16 instead of bf16 (a uniform branch)
    const int t  = blockIdx.x;
    const int h0 = (blockIdx.y * 256 + threadIdx.x) * 8;
    if(h0 >= hidden)
        return;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if(accumulate) // stand-alone down GEMM: add to what the output holds, as ck_tile's atomic epilogue does
    {
        const uint4 v = *reinterpret_cast<const uint4*>(out + (int64_t)t * out_row_bytes + (int64_t)h0 * 2);
        const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for(int i = 0; i < 4; i++)
        {
            acc[2 * i]     = f16 ? f16_bits_to_float(d[i] & 0xffffu) : __uint_as_float(d[i] << 16);
            acc[2 * i + 1] = f16 ? f16_bits_to_float(d[i] >> 16) : __uint_as_float(d[i] & 0xffff0000u);
        }
    }
    // four slots at a time (eight measured the same): their rows are fetched together (read once: non-temporal), then added in slot order
    constexpr int kSlotsPerPass = 4;
    using u32x4 = __attribute__((ext_vector_type(4))) uint32_t;
    for(int k0 = 0; k0 < topk; k0 += kSlotsPerPass)
    {
        int pos[kSlotsPerPass];
        float w[kSlotsPerPass];
        u32x4 v[kSlotsPerPass];
#pragma unroll
        for(int j = 0; j < kSlotsPerPass; j++)
            pos[j] = k0 + j < topk ? __builtin_amdgcn_readfirstlane(inv[t * topk + k0 + j]) : -1;
#pragma unroll
        for(int j = 0; j < kSlotsPerPass; j++)
        {
            w[j] = 0.f;
            v[j] = u32x4{0u, 0u, 0u, 0u};
            if(pos[j] >= 0)
            {
                w[j] = sorted_w[pos[j]];
                if(slot_scale) // per-row scale of the stand-alone down GEMM's quantised input, row = token * topk + slot
                    w[j] *= slot_scale[t * topk + k0 + j];
                if(row_scale) // per-row scale of re-quantised e4m3 intermediate activations, in sorted-row order
                    w[j] *= row_scale[pos[j]];
                v[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(part + ((int64_t)pos[j] * hidden + h0) * 2));
            }
        }
#pragma unroll
        for(int j = 0; j < kSlotsPerPass; j++)
        {
            if(pos[j] < 0)
                continue;
#pragma unroll
            for(int i = 0; i < 4; i++)
            {
                acc[2 * i] += w[j] * (f16 ? f16_bits_to_float(v[j][i] & 0xffffu) : __uint_as_float(v[j][i] << 16));
                acc[2 * i + 1] += w[j] * (f16 ? f16_bits_to_float(v[j][i] >> 16) : __uint_as_float(v[j][i] & 0xffff0000u));
            }
            if(bias != nullptr) // stand-alone down GEMM with an expert bias: (dot + bias) * top-k weight
            {
                const float wk  = sorted_w[pos[j]];
                const float* bp = bias + (int64_t)sorted_eid[pos[j] / unit] * hidden + h0;
#pragma unroll
                for(int i = 0; i < 8; i++)
                    acc[i] += wk * bp[i];
            }
        }
    }
    uint4 o;
    if(f16)
    {
        o.x = pack_f16x2(acc[0], acc[1]);
        o.y = pack_f16x2(acc[2], acc[3]);
        o.z = pack_f16x2(acc[4], acc[5]);
        o.w = pack_f16x2(acc[6], acc[7]);
    }
    else
    {
        o.x = pack_bf16x2(acc[0], acc[1]);
        o.y = pack_bf16x2(acc[2], acc[3]);
        o.z = pack_bf16x2(acc[4], acc[5]);
        o.w = pack_bf16x2(acc[6], acc[7]);
    }
    *reinterpret_cast<uint4*>(out + (int64_t)t * out_row_bytes + (int64_t)h0 * 2) = o;
}

// bytes per element of the intermediate activations the down GEMM reads: e4m3 on the fp8 path (per 32 columns from
// gemm0, or per row from the re-quantisation pass with fused_quant 1 / 2), int8 when the int8 path re-quantises them,
// bf16 otherwise
inline int y_bytes(const mi355_fused_moe_traits& t)
{
    return (t.prec_i == MI355_MOE_FP8 || (t.prec_i == MI355_MOE_INT8 && t.fused_quant != 0)) ? 1 : 2;
}

// the decode kernel's variant with two 32-row token blocks per tile exists for every operand type; for fp8 the
// other kernels are faster wherever it could run
inline bool two_block_decode_ok(const mi355_fused_moe_traits& t) { return t.prec_i != MI355_MOE_FP8; }

// the decode kernel takes tiles of this many 32-row blocks
inline bool decode_tile(const mi355_fused_moe_traits& t, int mblk)
{
    return mblk == 1 || (mblk == 2 && two_block_decode_ok(t));
}

// every operand of the problem can be addressed as a base plus a 32-bit byte offset (the large-tile and decode kernels)
inline bool offsets_fit(const mi355_fused_moe_traits& t, int64_t tokens, int topk, int experts, int hidden, int inter)
{
    const int eb  = (t.prec_i == MI355_MOE_BF16 || t.prec_i == MI355_MOE_FP16) ? 2 : 1;
    const int y_b = y_bytes(t);
    const int64_t lim     = (int64_t)1 << 32;
    const int64_t max_pad = topk * tokens + (int64_t)experts * t.block_m - topk;
    const int64_t x_rows  = t.fused_quant == 1 ? tokens * topk : tokens; // smooth-quant: a row per (slot, token)
    return (int64_t)2 * inter * hidden * eb < lim && max_pad * inter * y_b < lim && x_rows * hidden * eb < lim;
}

// the large-tile kernel can run this problem (its tiles start on whole 16-row slabs of Y: the sort unit must be a
// multiple of 16)
inline bool big_tile_ok(const mi355_fused_moe_traits& t, int64_t tokens, int topk, int experts, int hidden, int inter)
{
    const int eb  = (t.prec_i == MI355_MOE_BF16 || t.prec_i == MI355_MOE_FP16) ? 2 : 1;
    const int y_b = y_bytes(t);
    return t.block_m % 16 == 0 && offsets_fit(t, tokens, topk, experts, hidden, inter) &&
           big_tile_supported(t.prec_i, hidden * eb, inter * y_b, y_b == 1);
}

// 32-row blocks per M tile, from the expected rows per expert; big_tile_rows() / 32 selects the large-tile kernel
inline int pick_mblk(const mi355_fused_moe_traits& t, int64_t tokens, int topk, int experts, int hidden, int inter)
{
    const int64_t avg = tokens * topk / std::max(experts, 1);
    const bool fits   = offsets_fit(t, tokens, topk, experts, hidden, inter);
    // Measured crossovers (fp8, 256 experts; int8, 128 experts; bf16, 8 experts): the decode kernel with one
    // token block per tile wins up to about 24 rows per expert.  From about 28 on an expert often has more
    // than 32 rows and would stream its weights twice: with 16-bit and int8 operands the decode kernel with two
    // token blocks (64-row tiles) is the fastest up to about 56 rows per expert (5 to 25 % ahead of the
    // large-tile kernel, whose single workgroup per compute unit cannot hide a tile's prologue and epilogue
    // behind another tile's weight stream); with fp8 operands, and from there on for all types, the large-tile
    // kernel - it streams every weight tile once whatever the row count and fetches only the token slabs a
    // tile has - provided its tiles fill the chip.
    if(two_block_decode_ok(t) && fits && avg >= 28 && avg <= 56)
        return 2;
    const int64_t big_tiles = (int64_t)experts * std::max<int64_t>(1, ceil_div<int64_t>(avg, big_tile_rows())) * ceil_div(inter, 128);
    const bool big_ok = big_tile_ok(t, tokens, topk, experts, hidden, inter);
    if(big_ok && (avg >= 160 || (avg >= 28 && big_tiles >= device_info().num_cu)))
        return big_tile_rows() / 32;
    if(avg <= 32)
        return 1;
    if(avg <= 64)
        return 2;
    return 4;
}

// Skewed routing: the tile height above comes from the average rows per expert, tokens * topk / experts, but the
// experts that have tokens at all may hold several times that, and the decode tiles then stream a hot expert's
// weights once per 32 rows.  Where it pays (fp8: a Zipf-routed batch of 256 / 512 tokens of the 256-expert model runs
// 28 / 40 % faster on the large tiles; int8 and bf16 gain nothing up to the row counts where the average selects the
// large tiles anyway) the sort chooses between the two tile heights from the counts it holds, and both kernel
// families are launched: the workgroups of the one whose tile height was not chosen leave at once (two short empty
// launches per pass).  Returns the second tile height in 32-row blocks, 0: no choice.
inline int alt_mblk(const mi355_fused_moe_traits& t, int64_t tokens, int topk, int experts, int hidden, int inter)
{
    if(t.prec_i != MI355_MOE_FP8 || t.fused_quant != 0 || !big_tile_ok(t, tokens, topk, experts, hidden, inter))
        return 0;
    return pick_mblk(t, tokens, topk, experts, hidden, inter) <= 4 ? big_tile_rows() / 32 : 0;
}
constexpr int kAltMinRows = 48; // padded rows per active expert from which the large tiles are chosen

template <int MODE, bool GEMM0>
int launch_gemm(int mblk, const GemmParams& p, int max_tiles, hipStream_t stream)
{
    using MT = ModeTraits<MODE>;
    KernelTimer timer(GEMM0 ? MI355_MOE_K_GEMM0 : MI355_MOE_K_GEMM1, stream);
    const int grid = round_up(max_tiles * p.n_ntiles, 8);
    if(grid <= 0)
        return MI355_MOE_OK;
#define MI355_LAUNCH(MB)                                                                               \
    {                                                                                                  \
        const size_t lds = kWRows * (MT::kWKB + kPadB) + (MB)*32 * (MT::kXKB + kPadB);                 \
        hipLaunchKernelGGL((moe_gemm_kernel<MODE, GEMM0, MB>), dim3(grid), dim3(kBlock), lds, stream, p); \
    }
    if(mblk == 1)
        MI355_LAUNCH(1)
    else if(mblk == 2)
        MI355_LAUNCH(2)
    else
        MI355_LAUNCH(4)
#undef MI355_LAUNCH
    MI355_HIP_TRY(hipGetLastError());
    return MI355_MOE_OK;
}

// One grouped GEMM over the tile list: sets the column-tile count for the kernel family that runs this
// tile size and launches it.  use_decode: the caller found the decode kernel applicable (one or two 32-row blocks per
// tile, 32-bit offsets suffice).  The down GEMM of the int8 path multiplies bf16 Y by int8 weights, or, with
// y_i8, int8 Y (scaled per row) by int8 weights on the i8 MFMAs.
int launch_grouped_gemm(int prec, bool gemm0, int mblk, bool use_decode, GemmParams& p, int max_tiles, hipStream_t stream,
                        bool y_i8 = false)
{
    // (bf16 Y times int8 weights, the int8 path's down GEMM without re-quantisation: the decode kernel's variant with
    // two token blocks would stage twice the bytes per weight byte and spills; the 64-row small tiles run instead)
    if(mblk == 2 && prec == MI355_MOE_INT8 && !gemm0 && !y_i8)
        use_decode = false;
    // output columns per tile: the tile's weight rows, halved where gate and up rows share them
    const int pair = gemm0 && !p.gate_only ? 2 : 1;
    p.max_tiles    = max_tiles;
    p.n_ntiles     = ceil_div(p.n_out, (use_decode ? decode_tile_cols(false) : 256) / pair);
    if(use_decode)
        return launch_gemm_decode(prec, gemm0, mblk, p, max_tiles, stream, y_i8);
    if(mblk > 4)
        return launch_gemm_big(prec, gemm0, p, max_tiles, stream, y_i8);
    if(prec == MI355_MOE_BF16)
        return gemm0 ? launch_gemm<kBf16, true>(mblk, p, max_tiles, stream) : launch_gemm<kBf16, false>(mblk, p, max_tiles, stream);
    if(prec == MI355_MOE_FP16)
        return gemm0 ? launch_gemm<kF16, true>(mblk, p, max_tiles, stream) : launch_gemm<kF16, false>(mblk, p, max_tiles, stream);
    if(prec == MI355_MOE_FP8)
        return gemm0 ? launch_gemm<kFp8, true>(mblk, p, max_tiles, stream) : launch_gemm<kFp8, false>(mblk, p, max_tiles, stream);
    if(gemm0)
        return launch_gemm<kI8, true>(mblk, p, max_tiles, stream);
    return y_i8 ? launch_gemm<kI8, false>(mblk, p, max_tiles, stream) : launch_gemm<kBf16W8, false>(mblk, p, max_tiles, stream);
}

// the narrow decode tiles re-read the input rows once per 64 output columns: for the down GEMM they pay off
// only where the 256-column tiles would leave most compute units without a workgroup
bool down_gemm_wants_decode(int experts, int64_t entries, int hidden)
{
    return std::min<int64_t>(experts, entries) * ceil_div(hidden, 256) < device_info().num_cu;
}

} // namespace

int check_traits(const mi355_fused_moe_traits& t)
{
    // output: bf16, or fp16 with fp16 operands (ck_tile's two instances, fused_moegemm_pipeline_flatmm_policy.hpp:790-807)
    const bool prec_ok = (t.prec_i == MI355_MOE_BF16 || t.prec_i == MI355_MOE_FP8 || t.prec_i == MI355_MOE_INT8 ||
                          t.prec_i == MI355_MOE_FP16) &&
                         t.prec_w == t.prec_i && t.prec_o == (t.prec_i == MI355_MOE_FP16 ? MI355_MOE_FP16 : MI355_MOE_BF16);
    if(!prec_ok)
        return fail(MI355_MOE_E_UNSUPPORTED, "fused_moe: unsupported precision (i=%d w=%d o=%d)", t.prec_i, t.prec_w,
                    t.prec_o);
    if(t.prec_st != MI355_MOE_FP32 || t.prec_sw != MI355_MOE_FP32 || t.prec_kw != MI355_MOE_FP32)
        return fail(MI355_MOE_E_UNSUPPORTED, "fused_moe: scales and top-k weights must be fp32");
    if(t.activation != 0 && t.activation != 1)
        return fail(MI355_MOE_E_UNSUPPORTED, "fused_moe: activation=%d (0 = gelu, 1 = silu)", t.activation);
    if(t.gate_only != 0 && t.gate_only != 1)
        return fail(MI355_MOE_E_UNSUPPORTED, "fused_moe: gate_only=%d (0 or 1)", t.gate_only);
    if(t.fused_quant < 0 || t.fused_quant > 2 ||
       (t.fused_quant != 0 && t.prec_i != MI355_MOE_INT8 && t.prec_i != MI355_MOE_FP8))
        return fail(MI355_MOE_E_UNSUPPORTED, "fused_moe: fused_quant=%d with precision %d (1 = smooth-dynamic-quant and "
                                             "2 = dynamic-quant of the intermediate activations exist for int8 and fp8)",
                    t.fused_quant, t.prec_i);
    if(t.block_m < 1 || t.block_m > 1024)
        return fail(MI355_MOE_E_UNSUPPORTED, "fused_moe: block_m=%d", t.block_m);
    if(t.weight_permute != 0 && t.weight_permute != 1)
        return fail(MI355_MOE_E_UNSUPPORTED, "fused_moe: weight_permute=%d (0 = no_permute, 1 = b_nr_kr_kw_nw_kv)",
                    t.weight_permute);
    return MI355_MOE_OK;
}

int gemm_tile_rows(const mi355_fused_moe_traits& t, int32_t tokens, int32_t experts, int32_t topk, int32_t hidden,
                   int32_t inter)
{
    return pick_mblk(t, tokens, topk, experts, hidden, inter) * 32;
}

int gemm_alt_tile_rows(const mi355_fused_moe_traits& t, int32_t tokens, int32_t experts, int32_t topk, int32_t hidden,
                       int32_t inter)
{
    return alt_mblk(t, tokens, topk, experts, hidden, inter) * 32;
}

WorkspaceLayout workspace_layout(const mi355_fused_moe_traits& t, int32_t tokens, int32_t experts, int32_t topk,
                                 int32_t hidden, int32_t inter)
{
    WorkspaceLayout w{};
    auto bump = [&](size_t bytes) {
        const size_t off = w.total;
        w.total += round_up<size_t>(bytes, 256);
        return off;
    };
    const int mblk   = pick_mblk(t, tokens, topk, experts, hidden, inter);
    w.max_pad        = (int64_t)topk * tokens + (int64_t)experts * t.block_m - topk;
    w.max_tiles      = (int32_t)(experts + w.max_pad / (mblk * 32) + 1);
    // gemm0 writes e4m3 on the fp8 path (bf16 with fused_quant) and bf16 otherwise; with fused_quant the int8 and fp8
    // paths re-quantise that bf16 Y, one scale per row, into a second buffer the down GEMM reads
    const bool requant = (t.prec_i == MI355_MOE_INT8 || t.prec_i == MI355_MOE_FP8) && t.fused_quant != 0;
    const int y_b      = (t.prec_i == MI355_MOE_FP8 && !requant) ? 1 : 2;
    w.sort_off       = bump(sorting_workspace_bytes(tokens, experts, topk));
    w.map_off        = bump(sizeof(int) * (kMapHdr + (size_t)kMapEnt * w.max_tiles));
    w.inv_off        = bump(sizeof(int) * (size_t)tokens * topk);
    w.y_off          = bump((size_t)round_up<int64_t>(w.max_pad, 16) * inter * y_b); // whole 16-row slabs
    w.ys_kb_stride   = round_up<int64_t>(w.max_pad, 256) + 512;
    w.ys_off         = bump(t.prec_i == MI355_MOE_FP8 ? (size_t)w.ys_kb_stride * (inter / 32) : 0);
    w.yq_off         = bump(requant ? (size_t)round_up<int64_t>(w.max_pad, 16) * inter : 0);
    w.yrs_off        = bump(requant ? (size_t)w.max_pad * sizeof(float) : 0);
    w.p_off          = bump((size_t)w.max_pad * hidden * 2);
    return w;
}

GemmPlan make_gemm_plan(const mi355_fused_moe_traits& t, void* ws_ptr, int32_t tokens, int32_t experts, int32_t topk,
                        int32_t hidden, int32_t inter)
{
    const WorkspaceLayout ws = workspace_layout(t, tokens, experts, topk, hidden, inter);
    unsigned char* wsb       = static_cast<unsigned char*>(ws_ptr);
    GemmPlan g{};
    g.tile_map      = reinterpret_cast<int*>(wsb + ws.map_off);
    g.rows_per_tile = pick_mblk(t, tokens, topk, experts, hidden, inter) * 32;
    g.max_tiles     = ws.max_tiles;
    g.inv           = reinterpret_cast<int*>(wsb + ws.inv_off);
    // the second candidate needs enough active experts for its gate+up tiles (256 weight rows each) to fill the chip
    g.alt_rows_per_tile = alt_mblk(t, tokens, topk, experts, hidden, inter) * 32;
    g.alt_min_rows      = kAltMinRows;
    g.alt_min_active    = ceil_div(device_info().num_cu, ceil_div((t.gate_only ? 1 : 2) * inter, 256));
    return g;
}

bool sizes_in_range(int32_t tokens, int32_t experts, int32_t topk, int32_t hidden, int32_t inter)
{
    // (sorted ids hold the token in 24 bits; row indices of the padded routing list are 32-bit integers)
    return tokens >= 0 && tokens <= 0xffffff && experts > 0 && experts <= 1024 && topk > 0 && topk <= 255 && hidden > 0 &&
           inter > 0 && (int64_t)tokens * topk + (int64_t)experts * 1024 < INT32_MAX;
}

// Everything that can be checked on the host before anything is launched: the fused entry point calls it ahead
// of the sort, so that a rejected call leaves the caller's sort outputs and workspace untouched.
int validate_fused_moegemm(const mi355_fused_moe_traits& t, const mi355_fused_moegemm_args& a, const void* ws_ptr,
                           size_t ws_bytes)
{
    int rc = check_traits(t);
    if(rc != MI355_MOE_OK)
        return rc;
    const int H = a.hidden_size, I = a.intermediate_size, T = a.num_tokens, E = a.num_experts, K = a.topk;
    if(!sizes_in_range(T, E, K, H, I) || a.stride_token < H)
        return fail(MI355_MOE_E_INVALID, "fused_moegemm: bad sizes (H=%d I=%d T=%d E=%d K=%d stride=%d)", H, I, T, E,
                    K, a.stride_token);
    const WorkspaceLayout ws = workspace_layout(t, T, E, K, H, I);
    if(ws_ptr == nullptr || ws_bytes < ws.total)
        return fail(MI355_MOE_E_WORKSPACE, "fused_moegemm: workspace of %zu bytes needed, %zu given", ws.total,
                    ws_ptr ? ws_bytes : (size_t)0);
    if(reinterpret_cast<uintptr_t>(ws_ptr) % 256 != 0)
        return fail(MI355_MOE_E_INVALID, "fused_moegemm: workspace must be 256-byte aligned");
    if(T == 0)
        return MI355_MOE_OK; // an empty batch: nothing to compute, and its tensors may have no storage
    if(!a.a_ptr || !a.g_ptr || !a.d_ptr || !a.o_ptr || !a.sorted_token_ids_ptr || !a.sorted_weight_ptr ||
       !a.sorted_expert_ids_ptr || !a.num_sorted_tiles_ptr)
        return fail(MI355_MOE_E_INVALID, "fused_moegemm: null tensor pointer");
    if((t.fused_quant == 1) != (a.y_smooth_scale_ptr != nullptr))
        return fail(MI355_MOE_E_INVALID, "fused_moegemm: y_smooth_scale goes with fused_quant 1 and only with it "
                                         "(fused_quant=%d)", t.fused_quant);
    if(t.fused_quant == 1 && (reinterpret_cast<uintptr_t>(a.y_smooth_scale_ptr) % 16 != 0 || I % 8 != 0))
        return fail(MI355_MOE_E_INVALID, "fused_moegemm: y_smooth_scale must be 16-byte aligned");
    const bool quant = t.prec_i != MI355_MOE_BF16 && t.prec_i != MI355_MOE_FP16;
    if(quant && (!a.a_scale_ptr || !a.g_scale_ptr || !a.d_scale_ptr))
        return fail(MI355_MOE_E_INVALID, "fused_moegemm: quantised dtypes need a_scale, g_scale and d_scale");
    const int eb = quant ? 1 : 2; // bytes per activation / weight element
    if(H % 32 != 0 || I % 32 != 0 || (t.prec_i == MI355_MOE_FP8 && I % 128 != 0) ||
       ((int64_t)a.stride_token * eb) % 16 != 0 || ((int64_t)a.stride_token * 2) % 16 != 0)
        return fail(MI355_MOE_E_UNSUPPORTED,
                    "fused_moegemm: hidden and intermediate must be multiples of 32 (128 for fp8 intermediate) and "
                    "token rows 16-byte aligned (H=%d I=%d stride=%d)", H, I, a.stride_token);
    for(const void* ptr : {a.a_ptr, a.g_ptr, a.d_ptr, static_cast<const void*>(a.o_ptr)})
        if(reinterpret_cast<uintptr_t>(ptr) % 16 != 0)
            return fail(MI355_MOE_E_INVALID, "fused_moegemm: a, g, d and o must be 16-byte aligned");
    // pre-shuffled weights: blocks of 16 rows x 64 bytes of K, addressed with 32-bit offsets inside an expert
    if(t.weight_permute != 0 && (((int64_t)H * eb) % 64 != 0 || ((int64_t)I * eb) % 64 != 0 ||
                                 (int64_t)2 * I * H * eb >= ((int64_t)1 << 32)))
        return fail(MI355_MOE_E_UNSUPPORTED, "fused_moegemm: pre-shuffled weights need rows of whole 64-byte blocks and "
                                             "experts below 4 GiB (H=%d I=%d)", H, I);
    const int mblk = pick_mblk(t, T, K, E, H, I);
    // (smooth-quant activations hold a row per (slot, token))
    if(mblk > 4 && (int64_t)T * (t.fused_quant == 1 ? K : 1) * a.stride_token * eb >= ((int64_t)1 << 32))
        return fail(MI355_MOE_E_UNSUPPORTED, "fused_moegemm: a token buffer of 4 GiB or more (stride_token=%d) is not "
                                             "supported at this problem size", a.stride_token);
    return MI355_MOE_OK;
}

int launch_fused_moegemm(const mi355_fused_moe_traits& t, const mi355_fused_moegemm_args& a, void* ws_ptr,
                         size_t ws_bytes, hipStream_t stream, bool prep_done)
{
    int rc = validate_fused_moegemm(t, a, ws_ptr, ws_bytes);
    if(rc != MI355_MOE_OK)
        return rc;
    if(a.num_tokens == 0)
        return MI355_MOE_OK;
    const bool quant = t.prec_i != MI355_MOE_BF16 && t.prec_i != MI355_MOE_FP16;
    const int H = a.hidden_size, I = a.intermediate_size, T = a.num_tokens, E = a.num_experts, K = a.topk;
    const int eb = quant ? 1 : 2;
    const WorkspaceLayout ws = workspace_layout(t, T, E, K, H, I);
    unsigned char* wsb = static_cast<unsigned char*>(ws_ptr);
    int* tile_map      = reinterpret_cast<int*>(wsb + ws.map_off);
    int* inv           = reinterpret_cast<int*>(wsb + ws.inv_off);
    const int mblk     = pick_mblk(t, T, K, E, H, I);
    const int max_units = (int)ceil_div<int64_t>(ws.max_pad, t.block_m);
    // the sort chose between two tile heights (see alt_mblk): both kernel families are launched for each GEMM
    const int alt           = alt_mblk(t, T, K, E, H, I);
    const int alt_max_tiles = alt ? (int)std::min<int64_t>(ws.max_tiles, E + ws.max_pad / (alt * 32) + 1) : 0;

    const int n_inv      = T * K;
    const int prep_grid  = 1 + std::min(ceil_div(n_inv, kPrepBlock * 4), 64);
    if(!prep_done)
    {
        KernelTimer timer(MI355_MOE_K_PREP, stream);
        hipLaunchKernelGGL(moe_prep_kernel, dim3(prep_grid), dim3(kPrepBlock), 0, stream,
                           static_cast<const int*>(a.sorted_expert_ids_ptr),
                           static_cast<const int*>(a.num_sorted_tiles_ptr), t.block_m, E, mblk * 32, max_units,
                           ws.max_tiles, tile_map, inv, n_inv, alt * 32, kAltMinRows,
                           ceil_div(device_info().num_cu, ceil_div((t.gate_only ? 1 : 2) * I, 256)));
        hipLaunchKernelGGL(moe_inv_kernel, dim3(std::min<int>(ceil_div<int64_t>(ws.max_pad, 256), 1024)), dim3(256), 0,
                           stream, static_cast<const int*>(a.sorted_token_ids_ptr),
                           static_cast<const int*>(a.num_sorted_tiles_ptr), (int)ws.max_pad, T, K, inv);
    }
    MI355_HIP_TRY(hipGetLastError());

    GemmParams p{};
    p.sorted_ids = static_cast<const int*>(a.sorted_token_ids_ptr);
    p.tile_map   = tile_map;
    p.tokens     = T;
    p.y_scale    = wsb + ws.ys_off;
    p.ys_kb_stride = ws.ys_kb_stride;
    p.tile_rows  = alt ? mblk * 32 : 0;
    p.w_permuted = t.weight_permute;

    // ---- gemm0: gate+up, SiLU*up
    const bool requant  = quant && t.fused_quant != 0;
    const bool requant8 = requant && t.prec_i == MI355_MOE_FP8; // e4m3 rows with one scale each instead of one per 32 columns
    const int y_b       = (t.prec_i == MI355_MOE_FP8 && !requant) ? 1 : 2; // bytes per element of what gemm0 writes
    p.y_bf16            = requant8 ? 1 : 0;
    p.x_slot_major     = t.fused_quant == 1 ? 1 : 0;
    p.x               = static_cast<const unsigned char*>(a.a_ptr);
    p.x_row_bytes     = (int64_t)a.stride_token * eb;
    p.x_scale         = quant ? static_cast<const float*>(a.a_scale_ptr) : nullptr;
    p.w               = static_cast<const unsigned char*>(a.g_ptr);
    p.w_row_bytes     = (int64_t)H * eb;
    const int g_rows  = t.gate_only ? I : 2 * I; // weight rows per expert of the first GEMM
    p.gate_only       = t.gate_only;
    p.act             = t.activation;
    p.w_expert_bytes  = (int64_t)g_rows * H * eb;
    p.w_scale         = quant ? static_cast<const float*>(a.g_scale_ptr) : nullptr;
    p.out             = wsb + ws.y_off;
    p.out_row_bytes   = (int64_t)I * y_b;
    p.k_bytes_x       = H * eb;
    p.k_bytes_w       = H * eb;
    p.n_out           = I;
    p.n_total         = g_rows;
    // decode-sized problems (one or two 32-row blocks per tile) have their own kernel
    const bool decode = decode_tile(t, mblk) && decode_supported((int64_t)T * (p.x_slot_major ? K : 1) * a.stride_token * eb,
                                                      ws.max_pad * (int64_t)I * y_b, (int64_t)2 * I * H * eb);
    // the two large-tile GEMMs hand Y over in the slab-major layout (the re-quantisation pass writes it when there
    // is one; gemm0 then stores plain rows)
    const int yq_b   = requant ? 1 : y_b; // bytes per element of what the down GEMM reads
    const int y_slab = (mblk > 4 && ((int64_t)I * yq_b) % 64 == 0) ? (int)((int64_t)I * yq_b / 64) : 0;
    p.y_slab         = requant ? 0 : y_slab;
    const int alt_y_slab = (alt && ((int64_t)I * y_b) % 64 == 0) ? (int)((int64_t)I * y_b / 64) : 0;
    {
        KernelTimerGroup both(MI355_MOE_K_GEMM0, stream, alt != 0);
        rc = launch_grouped_gemm(t.prec_i, true, mblk, decode, p, ws.max_tiles, stream);
        if(rc != MI355_MOE_OK)
            return rc;
        if(alt)
        {
            GemmParams pa = p;
            pa.tile_rows  = alt * 32;
            pa.y_slab     = alt_y_slab;
            rc            = launch_grouped_gemm(t.prec_i, true, alt, false, pa, alt_max_tiles, stream);
            if(rc != MI355_MOE_OK)
                return rc;
        }
    }
    p.x_slot_major = 0;
    p.y_bf16       = 0;
    if(requant)
    {
        rc = launch_requant_y(wsb + ws.y_off, I, static_cast<const float*>(a.y_smooth_scale_ptr), p.sorted_ids,
                              static_cast<const int*>(a.sorted_expert_ids_ptr),
                              static_cast<const int*>(a.num_sorted_tiles_ptr), t.block_m, T, y_slab, ws.max_pad,
                              wsb + ws.yq_off, reinterpret_cast<float*>(wsb + ws.yrs_off), stream, requant8);
        if(rc != MI355_MOE_OK)
            return rc;
        if(requant8)
        {
            // the down GEMM runs the block-scaled MFMA: every block scale is 2^0, the row scales go into the combine
            const int64_t n16 = (ws.ys_kb_stride * (I / 32) + 15) / 16; // the buffer is a multiple of 256 bytes
            hipLaunchKernelGGL(fill_u32x4_kernel, dim3((unsigned)std::min<int64_t>(ceil_div<int64_t>(n16, 256), 4096)),
                               dim3(256), 0, stream, reinterpret_cast<uint4*>(wsb + ws.ys_off), n16, 0x7f7f7f7fu);
        }
    }

    // ---- gemm1: down, * top-k weight, bf16 partial per (token, slot)
    p.y_slab         = y_slab;
    p.x              = requant ? wsb + ws.yq_off : wsb + ws.y_off;
    p.x_row_bytes    = (int64_t)I * yq_b;
    p.x_scale        = requant && !requant8 ? reinterpret_cast<const float*>(wsb + ws.yrs_off) : nullptr;
    p.gate_only      = 0;
    p.w              = static_cast<const unsigned char*>(a.d_ptr);
    p.w_row_bytes    = (int64_t)I * eb;
    p.w_expert_bytes = (int64_t)H * I * eb;
    p.w_scale        = quant ? static_cast<const float*>(a.d_scale_ptr) : nullptr;
    p.out            = wsb + ws.p_off;
    p.out_row_bytes  = (int64_t)H * 2;
    p.k_bytes_x      = I * yq_b;
    p.k_bytes_w      = I * eb;
    p.n_out          = H;
    p.n_total        = H;
    {
        KernelTimerGroup both(MI355_MOE_K_GEMM1, stream, alt != 0);
        rc = launch_grouped_gemm(t.prec_i, false, mblk, decode && down_gemm_wants_decode(E, (int64_t)T * K, H), p,
                                 ws.max_tiles, stream, requant && !requant8);
        if(rc != MI355_MOE_OK)
            return rc;
        if(alt)
        {
            GemmParams pa = p;
            pa.tile_rows  = alt * 32;
            pa.y_slab     = alt_y_slab;
            rc            = launch_grouped_gemm(t.prec_i, false, alt, false, pa, alt_max_tiles, stream);
            if(rc != MI355_MOE_OK)
                return rc;
        }
    }

    // ---- combine
    {
    KernelTimer timer(MI355_MOE_K_COMBINE, stream);
    hipLaunchKernelGGL(moe_combine_kernel, dim3(T, ceil_div(H, 256 * 8)), dim3(256), 0, stream, wsb + ws.p_off, inv,
                       static_cast<const float*>(a.sorted_weight_ptr), static_cast<unsigned char*>(a.o_ptr), K, H,
                       (int64_t)a.stride_token * 2, 0, static_cast<const float*>(nullptr), static_cast<const float*>(nullptr),
                       static_cast<const int*>(nullptr), 1, t.prec_i == MI355_MOE_FP16 ? 1 : 0,
                       requant8 ? reinterpret_cast<const float*>(wsb + ws.yrs_off) : static_cast<const float*>(nullptr));
    }
    MI355_HIP_TRY(hipGetLastError());
    return MI355_MOE_OK;
}

// ---------------------------------------------------------------------------------------------
// Stand-alone grouped GEMMs behind ck_tile's MoeFlatmmHostArgs: the same kernels as the fused path,
// with the intermediate in ck_tile's [tokens * topk, .] layout instead of sorted-row order.
namespace {
struct FlatmmLayout
{
    size_t map_off, inv_off, p_off, ys_off, total;
    int64_t max_pad, ys_kb_stride;
    int32_t max_tiles;
    int mblk, hidden, inter;
    int alt; // second tile height (32-row blocks) the tile-list pass may choose from the routing, 0: none (see alt_mblk)
    mi355_fused_moe_traits traits;
};

int flatmm_layout(int kind, const mi355_moe_flatmm_args& a, FlatmmLayout& L)
{
    if(kind != MI355_MOE_GEMM1_GATE_ONLY && kind != MI355_MOE_GEMM1_GATE_UP && kind != MI355_MOE_GEMM2)
        return fail(MI355_MOE_E_UNSUPPORTED, "moe_flatmm: kind %d (0 = gate only, 1 = gate+up, 2 = down)", kind);
    const bool g1     = kind != MI355_MOE_GEMM2;
    const bool go     = kind == MI355_MOE_GEMM1_GATE_ONLY;
    const bool w8     = a.prec_b == MI355_MOE_INT8;
    const bool f8     = a.prec_b == MI355_MOE_FP8;
    const bool f16    = a.prec_b == MI355_MOE_FP16;
    const bool ok_typ = (a.prec_b == MI355_MOE_BF16 && a.prec_a == MI355_MOE_BF16) || (f16 && a.prec_a == MI355_MOE_FP16) ||
                        (f8 && a.prec_a == MI355_MOE_FP8) || (w8 && a.prec_a == (g1 ? MI355_MOE_INT8 : MI355_MOE_BF16));
    if(!ok_typ)
        return fail(MI355_MOE_E_UNSUPPORTED, "moe_flatmm: operand types a=%d b=%d (bf16 x bf16, fp16 x fp16, fp8 x fp8, "
                                             "int8 x int8 for the gate+up GEMM, bf16 x int8 for the down GEMM)", a.prec_a,
                    a.prec_b);
    if(!sizes_in_range(a.NumTokens, a.NumExperts, a.TopK, a.N, a.K) ||
       a.block_m < 1 || a.block_m > 1024 || a.k_batch > 1 || (g1 && !go && a.N % 2 != 0))
        return fail(MI355_MOE_E_INVALID, "moe_flatmm: bad sizes (tokens=%d experts=%d topk=%d N=%d K=%d block_m=%d k_batch=%d)",
                    a.NumTokens, a.NumExperts, a.TopK, a.N, a.K, a.block_m, a.k_batch);
    if(a.n_padded_zeros < 0 || a.n_padded_zeros >= a.N || a.k_padded_zeros < 0 || a.k_padded_zeros >= a.K)
        return fail(MI355_MOE_E_INVALID, "moe_flatmm: padded zeros (n=%d of N=%d, k=%d of K=%d)", a.n_padded_zeros, a.N,
                    a.k_padded_zeros, a.K);
    if(a.activation != MI355_MOE_ACT_SILU && a.activation != MI355_MOE_ACT_SWIGLU)
        return fail(MI355_MOE_E_UNSUPPORTED, "moe_flatmm: activation %d (0 = MoeSilu, 1 = Swiglu)", a.activation);
    {
        const int64_t b_b = (a.prec_b == MI355_MOE_BF16 || a.prec_b == MI355_MOE_FP16) ? 2 : 1;
        if(a.b_shuffle != 0 && (a.b_shuffle != 1 || (a.K * b_b) % 64 != 0 || a.N % 16 != 0 || a.k_padded_zeros != 0 ||
                                (int64_t)a.N * a.K * b_b >= ((int64_t)1 << 32)))
            return fail(MI355_MOE_E_UNSUPPORTED, "moe_flatmm: b_shuffle=%d needs K rows of whole 64-byte blocks, N a "
                                                 "multiple of 16, no k_padded_zeros and experts below 4 GiB (N=%d K=%d)",
                        a.b_shuffle, a.N, a.K);
    }
    L.hidden = g1 ? a.K : a.N;
    L.inter  = g1 ? (go ? a.N : a.N / 2) : a.K;
    if(L.hidden % 32 != 0 || L.inter % 32 != 0 || (f8 && !g1 && L.inter % 128 != 0))
        return fail(MI355_MOE_E_UNSUPPORTED, "moe_flatmm: N and K must give hidden and intermediate sizes that are "
                                             "multiples of 32, K of the fp8 down GEMM of 128 (hidden=%d inter=%d)", L.hidden,
                    L.inter);
    const int prec = w8 ? MI355_MOE_INT8 : f8 ? MI355_MOE_FP8 : f16 ? MI355_MOE_FP16 : MI355_MOE_BF16;
    L.traits       = mi355_fused_moe_traits{prec, prec, f16 ? MI355_MOE_FP16 : MI355_MOE_BF16, MI355_MOE_FP32, MI355_MOE_FP32, MI355_MOE_FP32,
                                            MI355_MOE_FP32, a.block_m, 1, 0, 0, 0};
    L.mblk         = pick_mblk(L.traits, a.NumTokens, a.TopK, a.NumExperts, L.hidden, L.inter);
    if(a.k_padded_zeros > 0)
    {
        // the K loops of the small-tile and decode kernels stop at any multiple of 16 bytes; the large-tile kernel
        // wants whole 128-byte lines
        const int a_b = (a.prec_a == MI355_MOE_BF16 || a.prec_a == MI355_MOE_FP16) ? 2 : 1;
        const int b_b = (a.prec_b == MI355_MOE_BF16 || a.prec_b == MI355_MOE_FP16) ? 2 : 1;
        const int k_eff = a.K - a.k_padded_zeros;
        if((k_eff * a_b) % 16 != 0 || (k_eff * b_b) % 16 != 0 || (f8 && k_eff % 32 != 0))
            return fail(MI355_MOE_E_UNSUPPORTED, "moe_flatmm: K - k_padded_zeros = %d must cover whole 16-byte pieces of A "
                                                 "and B (32 elements for fp8)", k_eff);
        L.mblk = std::min(L.mblk, 4);
    }
    // skewed decode-sized batches: the same choice between two tile heights as the fused entry points make
    L.alt          = a.k_padded_zeros == 0 ? alt_mblk(L.traits, a.NumTokens, a.TopK, a.NumExperts, L.hidden, L.inter) : 0;
    L.max_pad      = (int64_t)a.TopK * a.NumTokens + (int64_t)a.NumExperts * a.block_m - a.TopK;
    L.max_tiles    = (int32_t)(a.NumExperts + L.max_pad / (L.mblk * 32) + 1);
    L.total        = 0;
    auto bump      = [&](size_t bytes) {
        const size_t off = L.total;
        L.total += round_up<size_t>(bytes, 256);
        return off;
    };
    L.map_off = bump(sizeof(int) * (kMapHdr + (size_t)kMapEnt * L.max_tiles));
    L.inv_off = bump(sizeof(int) * (size_t)a.NumTokens * a.TopK);
    L.p_off   = bump(g1 ? 0 : (size_t)L.max_pad * L.hidden * 2);
    // the fp8 down GEMM runs the block-scaled MFMA: its input carries one scale per row, so every block scale is 2^0
    L.ys_kb_stride = round_up<int64_t>(L.max_pad, 256) + 512;
    L.ys_off       = bump(f8 && !g1 ? (size_t)L.ys_kb_stride * (L.inter / 32) : 0);
    return MI355_MOE_OK;
}
} // namespace

size_t moe_flatmm_workspace_bytes(int kind, const mi355_moe_flatmm_args& a)
{
    FlatmmLayout L{};
    return flatmm_layout(kind, a, L) == MI355_MOE_OK ? L.total : 0;
}

int launch_moe_flatmm(int kind, const mi355_moe_flatmm_args& a, void* ws_ptr, size_t ws_bytes, hipStream_t stream)
{
    FlatmmLayout L{};
    int rc = flatmm_layout(kind, a, L);
    if(rc != MI355_MOE_OK)
        return rc;
    const bool g1 = kind != MI355_MOE_GEMM2;
    const bool go = kind == MI355_MOE_GEMM1_GATE_ONLY;
    const bool w8 = a.prec_b == MI355_MOE_INT8;
    const bool f8 = a.prec_b == MI355_MOE_FP8;
    if(a.NumTokens == 0)
        return MI355_MOE_OK; // an empty batch: nothing to compute, and its tensors may have no storage
    if(!a.p_sorted_token_ids || !a.p_sorted_expert_ids || !a.p_max_token_id || !a.a_ptr || !a.b_ptr || !a.c_ptr ||
       (!g1 && !a.p_sorted_expert_weights))
        return fail(MI355_MOE_E_INVALID, "moe_flatmm: null pointer");
    if(a.exp_bias != nullptr && reinterpret_cast<uintptr_t>(a.exp_bias) % 16 != 0)
        return fail(MI355_MOE_E_INVALID, "moe_flatmm: exp_bias must be 16-byte aligned");
    if((w8 || f8) && (!a.scale_n || ((g1 || f8) && !a.scale_m)))
        return fail(MI355_MOE_E_INVALID, "moe_flatmm: quantised weights need scale_n, quantised activations scale_m");
    const int T = a.NumTokens, E = a.NumExperts, K = a.TopK, H = L.hidden, I = L.inter;
    const int a_b = (a.prec_a == MI355_MOE_BF16 || a.prec_a == MI355_MOE_FP16) ? 2 : 1, b_b = (w8 || f8) ? 1 : 2;
    if(a.stride_A < a.K || a.stride_B != a.K || a.stride_C < (g1 ? I : H) || ((int64_t)a.stride_A * a_b) % 16 != 0 ||
       ((int64_t)a.stride_C * 2) % 16 != 0)
        return fail(MI355_MOE_E_INVALID, "moe_flatmm: strides (A=%d B=%d C=%d): B must be [experts, N, K] with K "
                                         "contiguous, rows of A and C 16-byte aligned", a.stride_A, a.stride_B, a.stride_C);
    for(const void* ptr : {a.a_ptr, a.b_ptr, static_cast<const void*>(a.c_ptr)})
        if(reinterpret_cast<uintptr_t>(ptr) % 16 != 0)
            return fail(MI355_MOE_E_INVALID, "moe_flatmm: a, b and c must be 16-byte aligned");
    if(T == 0)
        return MI355_MOE_OK;
    if(ws_ptr == nullptr || ws_bytes < L.total)
        return fail(MI355_MOE_E_WORKSPACE, "moe_flatmm: workspace of %zu bytes needed, %zu given", L.total,
                    ws_ptr ? ws_bytes : (size_t)0);
    if(reinterpret_cast<uintptr_t>(ws_ptr) % 256 != 0)
        return fail(MI355_MOE_E_INVALID, "moe_flatmm: workspace must be 256-byte aligned");
    unsigned char* wsb = static_cast<unsigned char*>(ws_ptr);
    int* tile_map      = reinterpret_cast<int*>(wsb + L.map_off);
    int* inv           = reinterpret_cast<int*>(wsb + L.inv_off);
    const int mblk     = L.mblk;
    const int prec     = L.traits.prec_i;
    if((g1 ? T : (int64_t)T * K) * a.stride_A * a_b >= ((int64_t)1 << 32) && (mblk > 4 || L.alt != 0))
        return fail(MI355_MOE_E_UNSUPPORTED, "moe_flatmm: A of 4 GiB or more is not supported at this problem size");
    const int alt           = L.alt;
    const int alt_max_tiles = alt ? (int)std::min<int64_t>(L.max_tiles, E + L.max_pad / (alt * 32) + 1) : 0;
    {
        KernelTimer timer(MI355_MOE_K_PREP, stream);
        const int n_inv     = T * K;
        const int prep_grid = 1 + std::min(ceil_div(n_inv, kPrepBlock * 4), 64);
        hipLaunchKernelGGL(moe_prep_kernel, dim3(prep_grid), dim3(kPrepBlock), 0, stream,
                           static_cast<const int*>(a.p_sorted_expert_ids), static_cast<const int*>(a.p_max_token_id),
                           a.block_m, E, mblk * 32, (int)ceil_div<int64_t>(L.max_pad, a.block_m), L.max_tiles, tile_map,
                           inv, n_inv, alt * 32, kAltMinRows,
                           ceil_div(device_info().num_cu, ceil_div(a.N, 256))); // enough tiles of this GEMM to fill the chip
        if(!g1)
            hipLaunchKernelGGL(moe_inv_kernel, dim3(std::min<int>(ceil_div<int64_t>(L.max_pad, 256), 1024)), dim3(256), 0,
                               stream, static_cast<const int*>(a.p_sorted_token_ids),
                               static_cast<const int*>(a.p_max_token_id), (int)L.max_pad, T, K, inv);
    }
    MI355_HIP_TRY(hipGetLastError());

    GemmParams p{};
    p.sorted_ids     = static_cast<const int*>(a.p_sorted_token_ids);
    p.tile_map       = tile_map;
    p.tokens         = T;
    p.slot_rows      = K;
    p.tile_rows      = alt ? mblk * 32 : 0;
    p.act            = a.activation == MI355_MOE_ACT_SWIGLU ? 2 : 1; // MoeSilu (ck_tile's default FusedActivation) or Swiglu
    p.swiglu_alpha   = a.swiglu_alpha;
    p.swiglu_limit   = a.swiglu_limit;
    p.n_padded       = a.n_padded_zeros;
    p.bias           = g1 ? static_cast<const float*>(a.exp_bias) : nullptr; // (the down GEMM's bias is added by the combine)
    p.x              = static_cast<const unsigned char*>(a.a_ptr);
    p.x_row_bytes    = (int64_t)a.stride_A * a_b;
    p.w              = static_cast<const unsigned char*>(a.b_ptr);
    p.w_row_bytes    = (int64_t)a.K * b_b;
    p.w_expert_bytes = (int64_t)a.N * a.K * b_b;
    p.w_permuted     = a.b_shuffle;
    p.w_scale        = (w8 || f8) ? static_cast<const float*>(a.scale_n) : nullptr;
    p.k_bytes_x      = (a.K - a.k_padded_zeros) * a_b;
    p.k_bytes_w      = (a.K - a.k_padded_zeros) * b_b;
    const int64_t a_rows = g1 ? T : (int64_t)T * K;
    const bool decode = decode_tile(L.traits, mblk) && decode_supported(a_rows * p.x_row_bytes, a_rows * p.x_row_bytes, p.w_expert_bytes);
    if(g1)
    {
        p.x_scale       = (w8 || f8) ? static_cast<const float*>(a.scale_m) : nullptr;
        p.y_bf16        = 1; // C is a 16-bit float whatever the operand type (fp16 with fp16 operands, else bf16)
        p.out           = static_cast<unsigned char*>(a.c_ptr);
        p.out_row_bytes = (int64_t)a.stride_C * 2;
        p.gate_only     = go;
        p.n_out         = I;
        p.n_total       = a.N;
        KernelTimerGroup both(MI355_MOE_K_GEMM0, stream, alt != 0);
        rc = launch_grouped_gemm(prec, true, mblk, decode, p, L.max_tiles, stream);
        if(rc == MI355_MOE_OK && alt)
        {
            GemmParams pa = p;
            pa.tile_rows  = alt * 32;
            rc            = launch_grouped_gemm(prec, true, alt, false, pa, alt_max_tiles, stream);
        }
        return rc;
    }
    p.out           = wsb + L.p_off;
    p.out_row_bytes = (int64_t)H * 2;
    p.n_out         = H;
    p.n_total       = H;
    if(f8)
    {
        p.y_scale      = wsb + L.ys_off;
        p.ys_kb_stride = L.ys_kb_stride;
        const int64_t n16 = (L.ys_kb_stride * (I / 32) + 15) / 16; // the buffer is a multiple of 256 bytes
        hipLaunchKernelGGL(fill_u32x4_kernel, dim3((unsigned)std::min<int64_t>(ceil_div<int64_t>(n16, 256), 4096)), dim3(256), 0,
                           stream, reinterpret_cast<uint4*>(p.y_scale), n16, 0x7f7f7f7fu);
    }
    {
        KernelTimerGroup both(MI355_MOE_K_GEMM1, stream, alt != 0);
        rc = launch_grouped_gemm(prec, false, mblk, decode && down_gemm_wants_decode(E, (int64_t)T * K, H), p, L.max_tiles, stream);
        if(rc == MI355_MOE_OK && alt)
        {
            GemmParams pa = p;
            pa.tile_rows  = alt * 32;
            rc            = launch_grouped_gemm(prec, false, alt, false, pa, alt_max_tiles, stream);
        }
    }
    if(rc != MI355_MOE_OK)
        return rc;
    {
        KernelTimer timer(MI355_MOE_K_COMBINE, stream);
        hipLaunchKernelGGL(moe_combine_kernel, dim3(T, ceil_div(H, 256 * 8)), dim3(256), 0, stream, wsb + L.p_off, inv,
                           static_cast<const float*>(a.p_sorted_expert_weights), static_cast<unsigned char*>(a.c_ptr), K, H,
                           (int64_t)a.stride_C * 2, 1, f8 ? static_cast<const float*>(a.scale_m) : nullptr,
                           static_cast<const float*>(a.exp_bias), static_cast<const int*>(a.p_sorted_expert_ids), a.block_m,
                           prec == MI355_MOE_FP16 ? 1 : 0);
    }
    MI355_HIP_TRY(hipGetLastError());
    return MI355_MOE_OK;
}

} // namespace mi355
