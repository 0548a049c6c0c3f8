// Grouped GEMM for decode-sized expert batches (one or two 32-row blocks per expert tile; gfx950).
//
// With a handful of tokens per expert the two GEMMs are pure weight streaming, and what decides
// the rate is the shape of the HBM requests: 128-byte pieces of 256 different rows (the tile shape
// of moe_gemm_kernel) reach about 5.3 TB/s on rows of 4 KB, 512 contiguous bytes per row about
// 6.9 TB/s.  So here a workgroup owns only 64 weight rows (gate+up GEMM: 32 gate + 32 up rows = 32 Y
// columns) and walks K in steps of 512 bytes per row.  The four waves split each step along K: wave
// w multiplies bytes [128 w, 128 w + 128) of every row with the matching token columns, and the four
// partial accumulators are added through LDS at the end (in wave order, so the result is
// deterministic).  Same MFMA orientation (weight rows on the M side), operand layouts and epilogues
// as moe_gemm_kernel; operand tiles are staged through LDS with the next step prefetched into
// registers, weights with non-temporal loads.  NXB = 2 multiplies every weight tile with two token
// blocks (tiles of up to 64 sorted rows), so that experts with 33 .. 64 rows still stream their
// weights once.
#include "moe_gemm_device.hpp"

#include <algorithm>
#include <type_traits>

namespace mi355 {
using namespace gemm;
namespace {

constexpr int kDecWRows = 64;  // weight rows per workgroup
constexpr int kDecWKB   = 512; // weight bytes per row and step

template <int MODE, bool GEMM0, int NXB, bool WPERM>
__global__ __launch_bounds__(kBlock, (NXB > 1 || MODE == kBf16W8 || MODE == kFp8) ? 2 : 3) void moe_gemm_decode_kernel(const GemmParams p)
{
    using MT  = ModeTraits<MODE>;
    using Acc = typename MT::Acc;
    constexpr int kOpB     = MT::kOpB;
    constexpr int kXMul    = MT::kXKB / MT::kWKB;     // token bytes per weight byte (2 for bf16 x int8)
    constexpr int kXKB     = kDecWKB * kXMul;         // token bytes per row and step
    constexpr int kWStride = kDecWKB + kPadB;
    constexpr int kXStride = kXKB + kPadB;
    constexpr int kWaveWB  = kDecWKB / 4;             // weight bytes of a row one wave multiplies per step
    constexpr int kSteps   = kWaveWB * kXMul / (2 * kOpB); // MFMAs along K per wave and step
    constexpr int kWLoads  = kDecWRows * (kDecWKB / 16) / kBlock; // 8
    constexpr int kXLoads  = NXB * 32 * (kXKB / 16) / kBlock;     // 4 or 8 per token block
    constexpr int kWRowsPerPass = kBlock / (kDecWKB / 16);        // 8
    constexpr int kXRowsPerPass = kBlock / (kXKB / 16);
    constexpr bool kMx     = MODE == kFp8 && !GEMM0;

    extern __shared__ __align__(16) unsigned char lds[];
    unsigned char* lds_w = lds;
    unsigned char* lds_x = lds + kDecWRows * kWStride;

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int r32  = lane & 31;
    const int kg   = lane >> 5;

    // ---- work item (same XCD-aware order as moe_gemm_kernel)
    const TileRef tile = lookup_tile(p.tile_map, p.n_ntiles, p.max_tiles, blockIdx.x, p.tile_rows);
    if(!tile.ok)
        return;
    const int expert = tile.expert;
    const int row0   = tile.row0;
    const int nt     = tile.nt;
    const int nrows  = min(tile.nrows, 32 * NXB);
    // a tile of at most 32 rows leaves the second token block out: no LDS traffic and no MFMAs for it (its loads are
    // masked row by row anyway)
    const bool two   = NXB > 1 && nrows > 32;
    const bool paired = GEMM0 && !p.gate_only; // gate rows paired with up rows (see run_epilogue)
    const int n_base  = nt * (paired ? 32 : 64);

    // ---- global -> register staging assignments: 32 consecutive lanes fetch 512 contiguous bytes
    const int xchunk = tid % (kXKB / 16);
    const int xrow   = tid / (kXKB / 16);
    // addresses are a uniform base plus a 32-bit byte offset (the launcher checks that this suffices)
    uint32_t xoff[kXLoads];
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
            xoff[j]   = (xvalid[j] ? token_row(p, sid) : 0u) * (uint32_t)p.x_row_bytes + xchunk * 16;
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
            xoff[j] = (uint32_t)src * (uint32_t)p.x_row_bytes + xchunk * 16;
        }
    }
    // Which 16 bytes of the 64 x 512-byte weight tile thread `tid` fetches with load j, as (tile row, 16-byte chunk) =
    // (w_row0 + w_row_add(j), w_chunk0 + w_chunk_add(j)).  Row-major weights: 32 consecutive threads walk the 512
    // contiguous bytes of a row.  ck_tile's pre-shuffled layout (16 rows x 64 bytes per 1 KiB block, the 16-byte
    // pieces of a block ordered by chunk, then row): 16 consecutive threads take the 16 rows of one chunk, 64 a
    // whole block, the four waves four consecutive blocks - a wave's load is 1 KiB of contiguous memory there too.
    // (Bits of the row: 0-1 = tid bits 0-1, 2 = j bit 1, 3-4 = tid bits 2-3, 5 = j bit 2, so that the channels
    // chan_of_row() gives the rows are 16 (j bit 1) + tid % 16; chunk: 0-3 = tid bits 4-7, 4 = j bit 0.)
    // (a template argument: chosen at run time the per-load offsets stop being constants, which costs the registers
    // that three workgroups per compute unit leave no room for)
    constexpr bool wperm = WPERM;
    const int w_chunk0 = wperm ? ((tid >> 6) << 2) | ((tid >> 4) & 3) : tid % (kDecWKB / 16);
    const int w_row0   = wperm ? (((tid >> 3) & 1) << 4) | (((tid >> 2) & 1) << 3) | (tid & 3) : tid / (kDecWKB / 16);
    auto w_row_add     = [&](int j) { return wperm ? ((j >> 2) << 5) | (((j >> 1) & 1) << 2) : kWRowsPerPass * j; };
    auto w_chunk_add   = [&](int j) { return wperm ? (j & 1) << 4 : 0; };
    static_assert(kWLoads == 8 && kWRowsPerPass == 8, "the assignments above cover 64 rows x 32 chunks with 8 loads of 256 threads");
    const unsigned char* wbase = p.w + (int64_t)expert * p.w_expert_bytes;
    uint32_t woff[kWLoads];
#pragma unroll
    for(int j = 0; j < kWLoads; j++)
    {
        const int lrow = w_row0 + w_row_add(j);
        const int blk  = lrow >> 5;
        const int c    = chan_of_row(lrow & 31);
        int grow;
        if(paired)
            grow = blk * p.n_out + min(n_base + c, p.n_out - 1);
        else
            grow = min(n_base + blk * 32 + c, p.n_total - 1);
        woff[j] = weight_offset(p, grow, w_chunk0 + w_chunk_add(j));
    }

    const int w_kadv = weight_k_advance(p, kDecWKB); // bytes between the K windows of two steps
    // two steps are kept in flight per workgroup: with three workgroups on a compute unit that is what it
    // takes to have enough bytes outstanding to cover the HBM latency
    uint4 xv_[2][kXLoads];
    uint4 wv_[2][kWLoads];
    uint32_t ys_next_[2][NXB], ys_cur[NXB];
#pragma unroll
    for(int i = 0; i < NXB; i++)
        ys_next_[0][i] = ys_next_[1][i] = ys_cur[i] = 0x7f7f7f7fu;
    const uint4 zero4 = {0u, 0u, 0u, 0u};

    auto load_tiles = [&](int kt, auto buf_tag) __attribute__((always_inline)) {
        constexpr int B   = decltype(buf_tag)::value;
        auto& xv          = xv_[B];
        auto& wv          = wv_[B];
        auto& ys_next     = ys_next_[B];
        const int kx = kt * kXKB + xchunk * 16;
#pragma unroll
        for(int j = 0; j < kXLoads; j++)
        {
            xv[j] = zero4;
            if(xvalid[j] && kx < p.k_bytes_x)
                xv[j] = *reinterpret_cast<const uint4*>(p.x + (xoff[j] + (uint32_t)(kt * kXKB)));
        }
        const int kw = kt * kDecWKB + w_chunk0 * 16;
#pragma unroll
        for(int j = 0; j < kWLoads; j++)
        {
            wv[j] = zero4;
            if(kw + w_chunk_add(j) * 16 < p.k_bytes_w)
            {
                typedef __attribute__((ext_vector_type(4))) unsigned u32x4_t;
                const u32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(wbase + (woff[j] + (uint32_t)(kt * w_kadv))));
                wv[j]           = make_uint4(t[0], t[1], t[2], t[3]);
            }
        }
        if constexpr(kMx)
        {
            // the four e8m0 scales of this wave's 128 columns of the step, per token block
            const int kb = kt * (kDecWKB / 32) + wave * 4;
#pragma unroll
            for(int i = 0; i < NXB; i++)
            {
                ys_next[i] = 0x7f7f7f7fu;
                if(r32 + 32 * i < nrows && kb * 32 < p.k_bytes_x)
                {
                    const unsigned char* sp = p.y_scale + (int64_t)kb * p.ys_kb_stride + row0 + r32 + 32 * i;
                    ys_next[i] = sp[0] | (sp[p.ys_kb_stride] << 8) | (sp[2 * p.ys_kb_stride] << 16) |
                                 (static_cast<uint32_t>(sp[3 * p.ys_kb_stride]) << 24);
                }
            }
        }
    };

    Acc acc[NXB][2];
#pragma unroll
    for(int i = 0; i < NXB; i++)
#pragma unroll
        for(int b = 0; b < 2; b++)
#pragma unroll
            for(int v = 0; v < 16; v++)
                acc[i][b][v] = 0;

    const int kt_count = ceil_div(p.k_bytes_w, kDecWKB);
    auto k_step = [&](int kt, auto buf_tag) __attribute__((always_inline)) {
        constexpr int B = decltype(buf_tag)::value;
        auto& xv        = xv_[B];
        auto& wv        = wv_[B];
#pragma unroll
        for(int j = 0; j < kXLoads; j++)
            if(j < kXLoads / NXB || two)
                *reinterpret_cast<uint4*>(lds_x + (xrow + kXRowsPerPass * j) * kXStride + xchunk * 16) = xv[j];
#pragma unroll
        for(int j = 0; j < kWLoads; j++)
            *reinterpret_cast<uint4*>(lds_w + (w_row0 + w_row_add(j)) * kWStride + (w_chunk0 + w_chunk_add(j)) * 16) = wv[j];
#pragma unroll
        for(int i = 0; i < NXB; i++)
            ys_cur[i] = ys_next_[B][i];
        __syncthreads();
        if(kt + 2 < kt_count)
            load_tiles(kt + 2, buf_tag);
        const unsigned char* xp = lds_x + r32 * kXStride + wave * kWaveWB * kXMul;
#pragma unroll
        for(int s = 0; s < kSteps; s++)
        {
            Frag wf[2];
#pragma unroll
            for(int b = 0; b < 2; b++)
            {
                const unsigned char* wp = lds_w + (b * 32 + r32) * kWStride + wave * kWaveWB;
                if constexpr(MODE == kBf16W8)
                    wf[b].lo = int8x8_to_bf16x8(*reinterpret_cast<const uint2*>(wp + (2 * s + kg) * 8));
                else if constexpr(kOpB == 16)
                    wf[b].lo = *reinterpret_cast<const uint4*>(wp + (2 * s + kg) * 16);
                else
                {
                    wf[b].lo = *reinterpret_cast<const uint4*>(wp + (4 * s + kg) * 16);
                    wf[b].hi = *reinterpret_cast<const uint4*>(wp + (4 * s + 2 + kg) * 16);
                }
            }
#pragma unroll
            for(int i = 0; i < NXB; i++)
            {
                if(i > 0 && !two)
                    continue;
                Frag xf;
                uint32_t xs              = 127;
                const unsigned char* xpi = xp + i * 32 * kXStride;
                if constexpr(kOpB == 16)
                    xf.lo = *reinterpret_cast<const uint4*>(xpi + (2 * s + kg) * 16);
                else
                {
                    xf.lo = *reinterpret_cast<const uint4*>(xpi + (4 * s + kg) * 16);
                    xf.hi = *reinterpret_cast<const uint4*>(xpi + (4 * s + 2 + kg) * 16);
                    if constexpr(kMx)
                        xs = (ys_cur[i] >> (8 * (2 * s + kg))) & 0xffu;
                }
                acc[i][0] = mfma<MODE>(wf[0], xf, xs, acc[i][0]);
                acc[i][1] = mfma<MODE>(wf[1], xf, xs, acc[i][1]);
            }
        }
        __syncthreads();
    };
    using B0 = std::integral_constant<int, 0>;
    using B1 = std::integral_constant<int, 1>;
    load_tiles(0, B0{});
    if(1 < kt_count)
        load_tiles(1, B1{});
    for(int kt = 0; kt < kt_count; kt += 2)
    {
        k_step(kt, B0{});
        if(kt + 1 < kt_count)
            k_step(kt + 1, B1{});
    }

    // ---- add the four K slices: waves 1..3 park their accumulators in LDS, wave 0 sums in wave order
    using AccElem   = decltype(acc[0][0][0] + acc[0][0][0]);
    AccElem* red    = reinterpret_cast<AccElem*>(lds); // [3][NXB][2][16][64]
    if(wave > 0)
    {
#pragma unroll
        for(int i = 0; i < NXB; i++)
        {
            if(i > 0 && !two)
                continue;
#pragma unroll
            for(int b = 0; b < 2; b++)
#pragma unroll
                for(int v = 0; v < 16; v++)
                    red[((((wave - 1) * NXB + i) * 2 + b) * 16 + v) * 64 + lane] = acc[i][b][v];
        }
    }
    __syncthreads();
    if(wave > 0)
        return;
    // one wave's 32 values at a time: fetching all 96 at once does not fit the register budget of three
    // workgroups per compute unit
#pragma nounroll
    for(int w = 0; w < 3; w++)
#pragma unroll
        for(int i = 0; i < NXB; i++)
        {
            if(i > 0 && !two)
                continue;
#pragma unroll
            for(int b = 0; b < 2; b++)
#pragma unroll
                for(int v = 0; v < 16; v++)
                    acc[i][b][v] += red[(((w * NXB + i) * 2 + b) * 16 + v) * 64 + lane];
        }

    run_epilogue<MODE, GEMM0, NXB, true>(p, acc, expert, row0, nrows, 0, 32, ceil_div(nrows, 32), n_base, 0, r32, kg);
}

template <int MODE, bool GEMM0, int NXB, bool WPERM>
int launch_decode_w(const GemmParams& p, int max_tiles, hipStream_t stream)
{
    using MT            = ModeTraits<MODE>;
    constexpr int kXMul = MT::kXKB / MT::kWKB;
    constexpr size_t lds = kDecWRows * (kDecWKB + kPadB) + NXB * 32 * (kDecWKB * kXMul + kPadB);
    static_assert(3 * NXB * 2 * 16 * 64 * 4 <= lds, "the reduction buffer fits in the operand tiles");
    const int grid = round_up(max_tiles * p.n_ntiles, 8);
    if(grid <= 0)
        return MI355_MOE_OK;
    KernelTimer timer(GEMM0 ? MI355_MOE_K_GEMM0 : MI355_MOE_K_GEMM1, stream);
    if constexpr(lds > 64 * 1024)
    {
        // the dynamic LDS limit is an attribute of the function on one device: set once per device
        static bool attr_ok[64] = {};
        int dev = 0;
        (void)hipGetDevice(&dev);
        if(dev < 0 || dev >= 64 || !attr_ok[dev])
        {
            MI355_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_gemm_decode_kernel<MODE, GEMM0, NXB, WPERM>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            if(dev >= 0 && dev < 64)
                attr_ok[dev] = true;
        }
    }
    hipLaunchKernelGGL((moe_gemm_decode_kernel<MODE, GEMM0, NXB, WPERM>), dim3(grid), dim3(kBlock), lds, stream, p);
    MI355_HIP_TRY(hipGetLastError());
    return MI355_MOE_OK;
}

template <int MODE, bool GEMM0, int NXB>
int launch_decode_n(const GemmParams& p, int max_tiles, hipStream_t stream)
{
    return p.w_permuted ? launch_decode_w<MODE, GEMM0, NXB, true>(p, max_tiles, stream)
                        : launch_decode_w<MODE, GEMM0, NXB, false>(p, max_tiles, stream);
}

// blocks: 32-row token blocks per tile (1 or 2)
template <int MODE, bool GEMM0>
int launch_decode_t(int blocks, const GemmParams& p, int max_tiles, hipStream_t stream)
{
    return blocks == 1 ? launch_decode_n<MODE, GEMM0, 1>(p, max_tiles, stream) : launch_decode_n<MODE, GEMM0, 2>(p, max_tiles, stream);
}

} // namespace

int decode_tile_cols(bool gemm0) { return gemm0 ? 32 : 64; }

// byte offsets inside the token buffer, Y and one expert's weights must fit 32 bits
bool decode_supported(int64_t x_bytes, int64_t y_bytes, int64_t w_expert_bytes)
{
    const int64_t lim = (int64_t)1 << 32;
    return x_bytes < lim && y_bytes < lim && w_expert_bytes < lim;
}

int launch_gemm_decode(int prec, bool gemm0, int blocks, const GemmParams& p, int max_tiles, hipStream_t stream, bool y_i8)
{
    if(blocks != 1 && blocks != 2)
        return fail(MI355_MOE_E_UNSUPPORTED, "decode kernel: %d token blocks per tile", blocks);
    const int b = blocks;
    if(prec == MI355_MOE_INT8 && !gemm0 && y_i8)
        return launch_decode_t<kI8, false>(b, p, max_tiles, stream);
    if(prec == MI355_MOE_BF16)
        return gemm0 ? launch_decode_t<kBf16, true>(b, p, max_tiles, stream) : launch_decode_t<kBf16, false>(b, p, max_tiles, stream);
    if(prec == MI355_MOE_FP16)
        return gemm0 ? launch_decode_t<kF16, true>(b, p, max_tiles, stream) : launch_decode_t<kF16, false>(b, p, max_tiles, stream);
    if(prec == MI355_MOE_FP8 && b == 1) // (with two token blocks the fp8 kernels spill and the other families are faster)
        return gemm0 ? launch_decode_n<kFp8, true, 1>(p, max_tiles, stream) : launch_decode_n<kFp8, false, 1>(p, max_tiles, stream);
    if(prec == MI355_MOE_INT8 && gemm0)
        return launch_decode_t<kI8, true>(b, p, max_tiles, stream);
    if(prec == MI355_MOE_INT8 && b == 1) // (two token blocks of bf16 Y per int8 weight tile do not fit the register budget)
        return launch_decode_n<kBf16W8, false, 1>(p, max_tiles, stream);
    return fail(MI355_MOE_E_UNSUPPORTED, "no decode kernel for precision %d with %d token blocks per tile", prec, b);
}

} // namespace mi355
