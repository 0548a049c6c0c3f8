// Large-tile grouped GEMM for prefill-sized expert batches (gfx950).
//
// Same math and epilogues as moe_gemm_kernel, different machinery:
//   * 512 threads = 8 waves as 2 (token halves) x 4 (weight-row quarters); the workgroup owns up to
//     320 sorted rows of one expert (ten 32-row blocks, interleaved between the two token halves)
//     and 256 weight rows.  320 rather than 256 so that an expert of the DeepSeek-V3-shaped
//     workload (about 270 rows) is one tile and its weights are fetched once.
//   * Both operands go global -> LDS with global_load_lds_dwordx4 (no staging registers) through a
//     ring of four 64-byte-deep K stages, three of them in flight.  The loads are issued from
//     inline assembly so that their completion is tracked by hand: s_waitcnt vmcnt(n) with n = the
//     DMA instructions this wave issued after the stage about to be consumed, then one workgroup
//     barrier per stage, which also frees the buffer the next stage is written into.
//   * An LDS row is 64 bytes (four 16-byte chunks); chunk c of row r sits at chunk position
//     c ^ ((r >> 2) & 3), which makes both the linear DMA writes and the ds_read_b128 operand
//     fetches conflict-free on the 64-bank LDS.  Rows that must read as zero (padding ids, rows
//     past the tile) are fetched from a zero page, so the number of DMA instructions per wave and
//     stage, and with it every wait count, is a compile-time constant.
//   * The K loop is specialised on the number of token blocks a wave owns, so the MFMA region is
//     straight-line code.
#include "moe_gemm_device.hpp"

#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace mi355 {
using namespace gemm;
namespace {

constexpr int kBigThreads   = 512;
constexpr int kStageKB      = 64; // bytes of K per stage and row
constexpr int kStages       = 4;
constexpr int kChunks       = kStageKB / 16;
constexpr int kRowsPerDma   = 64 / kChunks; // rows one 64-lane DMA instruction fills (16)
constexpr int kBigWRows     = 256;
constexpr int kBigXRows     = 320;
constexpr int kMaxNB        = kBigXRows / 64; // token blocks per wave (5)
constexpr int kWRegion      = kBigWRows * kStageKB;
constexpr int kXRegion      = kBigXRows * kStageKB;
constexpr int kStageBytes   = kWRegion + kXRegion;
constexpr int kYsRows       = 512;                       // padded rows per K block of the scale stage
constexpr int kYsStageBytes = (kStageKB / 32) * kYsRows; // fp8 gemm1: e8m0 scales of 2 K blocks
constexpr int kDmaMax       = 5;                         // DMA instructions per wave and stage (4 or 5)

typedef __attribute__((address_space(3))) unsigned char lds_byte_t;

__device__ inline uint32_t lds_offset(const void* p)
{
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const lds_byte_t*)p));
}

// lane i of the wave copies 16 (4) bytes from its global address to LDS byte m0 + 16*i (4*i)
__device__ inline void dma16(const void* gptr, uint32_t m0_uniform)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(m0_uniform), "v"(gptr) : "memory");
}
__device__ inline void dma4(const void* gptr, uint32_t m0_uniform)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(m0_uniform), "v"(gptr) : "memory");
}

template <int N>
__device__ inline void wait_vmcnt()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int MODE, bool GEMM0>
__global__ __launch_bounds__(kBigThreads) void moe_gemm_big_kernel(const GemmParams p)
{
    using MT  = ModeTraits<MODE>;
    using Acc = typename MT::Acc;
    constexpr int kOpB   = MT::kOpB;
    constexpr int kSteps = kStageKB / (2 * kOpB); // MFMAs along K per stage: 1 (fp8) or 2 (bf16, i8)
    constexpr bool kMx   = MODE == kFp8 && !GEMM0;
    static_assert(MODE == kBf16 || MODE == kFp8 || MODE == kI8, "no large-tile kernel for this mode");

    extern __shared__ __align__(16) unsigned char lds[];

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r32  = lane & 31;
    const int kg   = lane >> 5;
    // waves w and w+4 share a SIMD: give them the two token halves of the same weight quarter, so
    // that every SIMD carries the same number of token blocks
    const int wt   = wave >> 2; // token half: blocks wt, wt+2, ...
    const int ww   = wave & 3;  // weight-row quarter

    // ---- work item (same XCD-aware order as moe_gemm_kernel)
    const int live_tiles = p.tile_map[0];
    const int total      = live_tiles * p.n_ntiles;
    const int per_xcd    = ceil_div(total, 8);
    const int slot       = blockIdx.x >> 3;
    const int work       = (blockIdx.x & 7) * per_xcd + slot;
    if(slot >= per_xcd || work >= total)
        return;
    int mt, nt;
    {
        const int t0     = work / p.n_ntiles;
        const int* ent0  = p.tile_map + kMapHdr + t0 * kMapEnt;
        const int first  = ent0[3];
        const int ntiles = ent0[4];
        const int rel    = work - first * p.n_ntiles;
        nt               = rel / ntiles;
        mt               = first + (rel - nt * ntiles);
    }
    const int* ent   = p.tile_map + kMapHdr + mt * kMapEnt;
    const int expert = ent[0];
    const int row0   = ent[1];
    const int nrows  = ent[2];
    const int nmb    = ceil_div(nrows, 32);
    const int n_base = nt * (GEMM0 ? 128 : 256);

    // ---- DMA assignments.  A stage is 16 weight slabs then 20 token slabs of 1 KB (16 rows x 64 B).
    // Wave w fills weight slabs w, w+8 and token slabs w, w+8; waves 0..3 also token slab 16+w.
    // On the fp8 down-GEMM waves 4..7 fetch the e8m0 scales instead, so every wave issues five.
    const int lrow16 = lane >> 2;
    const int cchunk = (lane & 3) ^ ((lane >> 4) & 3); // logical chunk this lane fetches
    const int n_dma  = (kMx || wave < 4) ? 5 : 4;
    const unsigned char* gptr[kDmaMax];
    int ginc[kDmaMax];
#pragma unroll
    for(int j = 0; j < kDmaMax; j++)
    {
        gptr[j] = p.zero_page;
        ginc[j] = 0;
        if(j < 2)
        {
            const int lrow = (wave + 8 * j) * kRowsPerDma + lrow16;
            const int blk  = lrow >> 5;
            const int c    = chan_of_row(lrow & 31);
            int grow;
            if constexpr(GEMM0)
                grow = (blk & 1) * p.n_out + min(n_base + (blk >> 1) * 32 + c, p.n_out - 1);
            else
                grow = min(n_base + blk * 32 + c, p.n_total - 1);
            gptr[j] = p.w + (int64_t)expert * p.w_expert_bytes + (int64_t)grow * p.w_row_bytes + cchunk * 16;
            ginc[j] = kStageKB;
        }
        else if(j < 4 || wave < 4)
        {
            const int xslab = j < 4 ? wave + 8 * (j - 2) : 16 + wave;
            const int lrow  = xslab * kRowsPerDma + lrow16;
            bool ok         = lrow < nrows;
            int64_t src     = row0 + lrow;
            if constexpr(GEMM0)
            {
                int tok = p.tokens;
                if(ok)
                    tok = p.sorted_ids[row0 + lrow] & 0xffffff;
                ok  = tok < p.tokens;
                src = tok;
            }
            gptr[j] = ok ? p.x + src * p.x_row_bytes + cchunk * 16 : p.zero_page + cchunk * 16;
            ginc[j] = ok ? kStageKB : 0;
        }
        else if constexpr(kMx)
        {
            // wave 4+q: K block (q >> 1) of the stage, rows (q & 1) * 256 .. + 255
            const int q = wave - 4;
            gptr[j]     = p.y_scale + (int64_t)(q >> 1) * p.ys_kb_stride + row0 + (q & 1) * 256 + lane * 4;
        }
    }
    const int64_t ys_step = (kStageKB / 32) * p.ys_kb_stride;

    const uint32_t lds_base = lds_offset(lds);
    const uint32_t ys_base  = lds_base + kStages * kStageBytes;

    auto issue = [&](int k) {
        const uint32_t sbase = lds_base + (k & (kStages - 1)) * kStageBytes;
#pragma unroll
        for(int j = 0; j < 4; j++)
        {
            const int slab_off = (j < 2 ? 0 : kWRegion) + (wave + 8 * (j & 1)) * 1024;
            dma16(gptr[j], __builtin_amdgcn_readfirstlane(sbase + slab_off));
            gptr[j] += ginc[j];
        }
        if(wave < 4)
        {
            dma16(gptr[4], __builtin_amdgcn_readfirstlane(sbase + kWRegion + (16 + wave) * 1024));
            gptr[4] += ginc[4];
        }
        else if constexpr(kMx)
        {
            const int q = wave - 4;
            dma4(gptr[4], __builtin_amdgcn_readfirstlane(ys_base + (k & (kStages - 1)) * kYsStageBytes +
                                                        (q >> 1) * kYsRows + (q & 1) * 256));
            gptr[4] += ys_step;
        }
    };

    Acc acc[kMaxNB][2];
#pragma unroll
    for(int i = 0; i < kMaxNB; i++)
#pragma unroll
        for(int b = 0; b < 2; b++)
#pragma unroll
            for(int v = 0; v < 16; v++)
                acc[i][b][v] = 0;

    const int kt_count = p.k_bytes_x / kStageKB;
    for(int k = 0; k < kStages - 1 && k < kt_count; k++)
        issue(k);

    // per-lane LDS read offsets inside a stage (swizzled chunk positions are per-lane constants)
    const int sw    = (r32 >> 2) & 3;
    const int w_off = (ww * 64 + r32) * kStageKB;
    const int x_off = kWRegion + (wt * 32 + r32) * kStageKB;

    auto k_loop = [&](auto nb_tag) {
        constexpr int NB = decltype(nb_tag)::value;
        constexpr int NF = NB > 0 ? NB : 1;
        for(int k = 0; k < kt_count; k++)
        {
            // stage k has landed once at most the DMA instructions of the later stages are pending
            const int later = min(kt_count - 1 - k, kStages - 2);
            if(later >= 2)
            {
                if(n_dma == 5)
                    wait_vmcnt<10>();
                else
                    wait_vmcnt<8>();
            }
            else if(later == 1)
            {
                if(n_dma == 5)
                    wait_vmcnt<5>();
                else
                    wait_vmcnt<4>();
            }
            else
                wait_vmcnt<0>();
            // stage k visible to all waves; everyone is done reading stage k-1 (a bare barrier: the
            // DMA completion was awaited above and LDS reads are consumed by MFMAs before a wave
            // gets here)
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if(k + kStages - 1 < kt_count && !(p.debug & 1))
                issue(k + kStages - 1);
            if(p.debug & 2)
                continue;

            const unsigned char* st = lds + (k & (kStages - 1)) * kStageBytes;
            [[maybe_unused]] const unsigned char* ysl =
                lds + kStages * kStageBytes + (k & (kStages - 1)) * kYsStageBytes + kg * kYsRows + wt * 32 + r32;
#pragma unroll
            for(int s = 0; s < kSteps; s++)
            {
                Frag wf[2];
                Frag xf[NF];
                uint32_t xs[NF];
                const int c_lo = kOpB == 16 ? ((2 * s + kg) ^ sw) * 16 : (kg ^ sw) * 16;
                const int c_hi = ((2 + kg) ^ sw) * 16;
#pragma unroll
                for(int b = 0; b < 2; b++)
                {
                    const unsigned char* wp = st + w_off + b * 32 * kStageKB;
                    wf[b].lo                = *reinterpret_cast<const uint4*>(wp + c_lo);
                    if constexpr(kOpB == 32)
                        wf[b].hi = *reinterpret_cast<const uint4*>(wp + c_hi);
                }
#pragma unroll
                for(int i = 0; i < NB; i++)
                {
                    const unsigned char* xp = st + x_off + i * 64 * kStageKB;
                    xf[i].lo                = *reinterpret_cast<const uint4*>(xp + c_lo);
                    if constexpr(kOpB == 32)
                        xf[i].hi = *reinterpret_cast<const uint4*>(xp + c_hi);
                    xs[i] = 127;
                    if constexpr(kMx)
                        xs[i] = ysl[i * 64];
                }
#pragma unroll
                for(int i = 0; i < NB; i++)
                {
                    if constexpr(MODE == kFp8 && GEMM0)
                    {
                        acc[i][0] = mfma_fp8_unscaled(wf[0], xf[i], acc[i][0]);
                        acc[i][1] = mfma_fp8_unscaled(wf[1], xf[i], acc[i][1]);
                    }
                    else
                    {
                        acc[i][0] = mfma<MODE>(wf[0], xf[i], xs[i], acc[i][0]);
                        acc[i][1] = mfma<MODE>(wf[1], xf[i], xs[i], acc[i][1]);
                    }
                }
            }
        }
    };
    const int nb_w = max(0, min(kMaxNB, (nmb - wt + 1) / 2));
    switch(nb_w)
    {
    case 5: k_loop(std::integral_constant<int, 5>{}); break;
    case 4: k_loop(std::integral_constant<int, 4>{}); break;
    case 3: k_loop(std::integral_constant<int, 3>{}); break;
    case 2: k_loop(std::integral_constant<int, 2>{}); break;
    case 1: k_loop(std::integral_constant<int, 1>{}); break;
    default: k_loop(std::integral_constant<int, 0>{}); break;
    }

    // ---- epilogue
    run_epilogue<MODE, GEMM0, kMaxNB>(p, acc, expert, row0, nrows, wt * 32, 64, nb_w, n_base, ww, nt == 0, r32, kg);
}

template <int MODE, bool GEMM0>
int launch_big_t(const GemmParams& p, int max_tiles, hipStream_t stream)
{
    constexpr bool kMx  = MODE == kFp8 && !GEMM0;
    const size_t lds    = kStages * kStageBytes + (kMx ? kStages * kYsStageBytes : 0);
    static bool attr_ok = false; // the limit is a per-function attribute; setting it again is harmless
    if(!attr_ok)
    {
        MI355_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_gemm_big_kernel<MODE, GEMM0>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_ok = true;
    }
    const int grid = round_up(max_tiles * p.n_ntiles, 8);
    if(grid <= 0)
        return MI355_MOE_OK;
    GemmParams q = p;
    if(const char* dbg = getenv("MI355_MOE_DEBUG"))
        q.debug = atoi(dbg);
    KernelTimer timer(GEMM0 ? MI355_MOE_K_GEMM0 : MI355_MOE_K_GEMM1, stream);
    hipLaunchKernelGGL((moe_gemm_big_kernel<MODE, GEMM0>), dim3(grid), dim3(kBigThreads), lds, stream, q);
    MI355_HIP_TRY(hipGetLastError());
    return MI355_MOE_OK;
}

} // namespace

int big_tile_rows() { return kBigXRows; }

bool big_tile_supported(int prec, int k_bytes0, int k_bytes1)
{
    return (prec == MI355_MOE_BF16 || prec == MI355_MOE_FP8) && k_bytes0 % kStageKB == 0 && k_bytes1 % kStageKB == 0;
}

int launch_gemm_big(int prec, bool gemm0, const GemmParams& p, int max_tiles, hipStream_t stream)
{
    if(prec == MI355_MOE_BF16)
        return gemm0 ? launch_big_t<kBf16, true>(p, max_tiles, stream) : launch_big_t<kBf16, false>(p, max_tiles, stream);
    if(prec == MI355_MOE_FP8)
        return gemm0 ? launch_big_t<kFp8, true>(p, max_tiles, stream) : launch_big_t<kFp8, false>(p, max_tiles, stream);
    return fail(MI355_MOE_E_UNSUPPORTED, "no large-tile kernel for precision %d", prec);
}

} // namespace mi355
