// Large-tile grouped GEMM for prefill-sized expert batches (gfx950).
//
// Same math and epilogues as moe_gemm_kernel, different machinery:
//   * 512 threads = 8 waves as 2 (token halves) x 4 (weight-row quarters); the workgroup owns up to
//     320 sorted rows of one expert (ten 32-row blocks, interleaved between the two token halves)
//     and 256 weight rows.  320 rather than 256 so that an expert of the DeepSeek-V3-shaped
//     workload (about 270 rows) is one tile and its weights are fetched once.
//   * Both operands go global -> LDS with global_load_lds_dwordx4 (no staging registers).  The K loop
//     advances in 64-byte steps.  Tokens (re-read from L2 by every column tile) arrive one 64-byte
//     step at a time through a ring of three stages.  Weights are streamed from HBM exactly once, as
//     full 128-byte lines, half of the tile's rows per unit (unit u = rows (u&1)*128.., K bytes
//     [128*(u>>1), +128)), through a ring of six units issued four steps ahead.
//   * The loads are issued from inline assembly so that their completion is tracked by hand:
//     s_waitcnt vmcnt(n) with n = the DMA instructions this wave issued after the data about to be
//     consumed, then one workgroup barrier per step, which also frees the buffers the next issues
//     write into.  Loads of one wave return in order, so the two streams are issued by different
//     waves (0..3 weights, 4..7 tokens): mixed in one wave, the L2-hit token loads would queue
//     behind the HBM-miss weight loads.
//   * What bounds the kernel is the compute unit's vector memory path: L2 hits queued behind HBM misses do
//     not overtake them, so the token stream costs its stand-alone time on top of the weight stream (about
//     19 bytes per clock together; a step of this tile needs up to 36.9 KB for 1400 clocks of MFMA work).
//   * LDS rows are swizzled: 64-byte token rows keep chunk c of row r at c ^ ((r >> 2) & 3), 128-byte
//     token rows at c ^ ((r >> 1) & 7), 128-byte weight rows at c ^ weight_row_swizzle(r); both the linear DMA
//     writes and the ds_read_b128 operand fetches are then conflict-free on the 64-bank LDS.  Weight rows sit in
//     LDS in channel order (row r of a 32-row block = channel r; the lane whose MFMA row is m reads row
//     chan_of_row(m)), so that the eight rows of a DMA instruction are eight consecutive channels: eight full
//     128-byte lines in the row-major layout and in ck_tile's pre-shuffled one alike.  Token rows past the tile's last row inside a
//     fetched 64-row group (and padding ids) fetch some real row instead - their MFMA columns are never
//     stored; whole groups the tile does not have are not fetched.
//   * The K loop is specialised on the number of token blocks a wave owns, on the number of 64-row token
//     groups the tile has and on whether the weight DMA is non-temporal, so that the MFMA region is
//     straight-line code and every wait count a compile-time constant: scalar branches in the issue path
//     cost 5 % of the kernel's time when tried.
//   * The int8 path runs here too: i8 MFMAs for the gate+up GEMM; for the down GEMM bf16 tokens against
//     int8 weights that are converted after the LDS read, one 128-byte weight line lasting four K steps.
//   * Work items go to the XCDs in chunks of 32 (see lookup_tile).
#include "moe_gemm_device.hpp"

#include <algorithm>
#include <mutex>
#include <type_traits>

namespace mi355 {
using namespace gemm;
namespace {

constexpr int kBigThreads   = 512;
constexpr int kStepKB       = 64;  // bytes of K per compute step and row
constexpr int kBigWRows     = 256;
constexpr int kBigXRows     = 320;
constexpr int kMaxNB        = kBigXRows / 64; // token blocks per wave (5)
constexpr int kWHalfRows    = kBigWRows / 2;
constexpr int kWUnitBytes   = kWHalfRows * 2 * kStepKB; // 128 rows x 128 B
constexpr int kWSlots       = 6;
constexpr int kXStageBytes  = kBigXRows * kStepKB;
constexpr int kXStages      = 3;
constexpr int kYsRows       = 512;                      // padded rows per K block of a scale stage
constexpr int kYsStageBytes = (kStepKB / 32) * kYsRows; // fp8 gemm1: e8m0 scales of 2 K blocks
constexpr int kXOffset      = kWSlots * kWUnitBytes;
constexpr int kYsOffset     = kXOffset + kXStages * kXStageBytes;
constexpr int kLdsBytes     = kYsOffset + kXStages * kYsStageBytes;
static_assert(kLdsBytes <= 160 * 1024, "LDS budget of a gfx950 compute unit");
// Gate+up GEMM (token rows gathered by id): a token stage holds 128 bytes of K per row, two compute steps, so that a
// token DMA instruction fetches eight whole 128-byte lines instead of sixteen half lines (a compute unit's address
// path moves 100 GB/s in whole lines and 58 GB/s in halves).  Two such stages and a weight ring of five slots.
constexpr int kXPairBytes   = kBigXRows * 2 * kStepKB;
constexpr int kWSlotsPair   = 5;
constexpr int kXOffsetPair  = kWSlotsPair * kWUnitBytes;
constexpr int kLdsBytesPair = kXOffsetPair + 2 * kXPairBytes;
static_assert(kLdsBytesPair <= 160 * 1024, "LDS budget of a gfx950 compute unit");

typedef __attribute__((address_space(3))) unsigned char lds_byte_t;

// Chunk swizzle of the 128-byte weight rows in LDS.  The 16 lanes that a ds_read_b128 serves together read the rows
// chan_of_row(16 i .. 16 i + 15) = {0..3, 16..19, 4..7, 20..23} (+ 8 for i = 1): among the rows of equal parity (two
// rows span the 64 banks) bits 1, 2 and 4 of the row number take all eight values.
__device__ __host__ constexpr int weight_row_swizzle(int r) { return ((r >> 1) & 3) | (((r >> 4) & 1) << 2); }


__device__ inline uint32_t lds_offset(const void* p)
{
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const lds_byte_t*)p));
}

__device__ inline const unsigned char* uniform_ptr(const unsigned char* p)
{
    const uint64_t v  = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    return reinterpret_cast<const unsigned char*>((static_cast<uint64_t>(hi) << 32) | lo);
}

// lane i of the wave copies 16 (4) bytes from base + off (a wave-uniform base, a per-lane 32-bit offset)
// to LDS byte m0 + 16*i (4*i)
__device__ inline void dma16(const unsigned char* base_uniform, uint32_t off, uint32_t m0_uniform)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0_uniform), "v"(off), "s"(uniform_ptr(base_uniform))
                 : "memory");
}
__device__ inline void dma16nt(const unsigned char* base_uniform, uint32_t off, uint32_t m0_uniform)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(m0_uniform), "v"(off), "s"(uniform_ptr(base_uniform))
                 : "memory");
}
__device__ inline void dma4(const unsigned char* base_uniform, uint32_t off, uint32_t m0_uniform)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(m0_uniform), "v"(off), "s"(uniform_ptr(base_uniform))
                 : "memory");
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): indices that are constants before any loop pass runs
template <int N, typename F>
__device__ __attribute__((always_inline)) inline void static_for(F&& f)
{
    if constexpr(N > 0)
    {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

template <int N>
__device__ inline void wait_vmcnt()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// WPERM: the weights are in ck_tile's pre-shuffled layout, where 128 contiguous bytes are one 16-byte chunk of eight
// consecutive rows.  The eight rows x eight chunks of a weight DMA instruction then sit in LDS chunk-major - lane
// 8 c' + r fetches chunk c' ^ s of row r, s = bit 1 of the instruction's number, and lands at byte 128 c' + 16 r of
// the instruction's 1 KiB - so that eight consecutive lanes fetch one whole line, as they do for row-major weights
// in the row-major LDS layout (eight chunks of one row).  The operand fetches of sixteen lanes (rows 0..7 of one
// instruction, rows 16..23 of the one two further on, same chunk) cover 256 contiguous bytes modulo the bank span
// thanks to s.
template <int MODE, bool GEMM0, bool WPERM>
__global__ __launch_bounds__(kBigThreads) void moe_gemm_big_kernel(const GemmParams p)
{
    using MT  = ModeTraits<MODE>;
    using Acc = typename MT::Acc;
    constexpr int kOpB   = MT::kOpB;
    constexpr int kSteps = kStepKB / (2 * kOpB); // MFMAs along K per compute step: 1 (fp8) or 2 (bf16, i8)
    // int8 weights against bf16 tokens (down GEMM of the int8 path): a 64-byte token step is 32 elements = 32
    // weight bytes, so the 128-byte lines of a weight unit last four steps instead of two
    constexpr bool kW8 = MODE == kBf16W8;
    constexpr bool kMx   = MODE == kFp8 && !GEMM0;
    static_assert(MODE == kBf16 || MODE == kF16 || MODE == kFp8 || MODE == kI8 || (MODE == kBf16W8 && !GEMM0),
                  "no large-tile kernel for this mode");
    // Software-pipelined K loop (kPipe): the operands of step k+1 are fetched from LDS into registers during step
    // k, each fragment right behind the last MFMA that reads its register, so that after a barrier the MFMAs start
    // at once instead of waiting for operand fetches that all eight waves issue at the same moment.  The barrier of
    // step k then has to guarantee the data of step k+1: every transfer runs one step further ahead.
    constexpr bool kPipe  = !kW8 && !kMx;
    constexpr bool kXPair = kPipe && GEMM0; // 128-byte token stages
    constexpr int kWS     = kXPair ? kWSlotsPair : kWSlots;
    constexpr int kXO     = kXPair ? kXOffsetPair : kXOffset;

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
    const TileRef tile = lookup_tile<true>(p.tile_map, p.n_ntiles, p.max_tiles, blockIdx.x, p.tile_rows);
    if(!tile.ok)
        return;
    const int expert = tile.expert;
    const int row0   = tile.row0;
    const int nt     = tile.nt;
    const int nrows  = tile.nrows;
    const int nmb    = ceil_div(nrows, 32);
    const bool paired = GEMM0 && !p.gate_only; // gate rows paired with up rows (see run_epilogue)
    const int n_base  = nt * (paired ? 128 : 256);

    // ---- DMA assignments.
    // Loads of one wave return in order, so a wave that mixed the two streams would see its L2-hit
    // token loads queue behind HBM-miss weight loads.  The streams are therefore issued by different
    // waves: waves 0..3 the weights, waves 4..7 the tokens (and, on the fp8 down-GEMM, the e8m0 scales).
    // Weights: unit u = rows (u & 1) * 128 .. + 127 of the tile, K bytes [128 * (u >> 1), + 128).  One unit
    // is 16 instructions of 8 rows x 128 B (full cache lines); wave w issues instructions w, w+4, w+8, w+12.
    // Tokens: step x = the tile's rows, K bytes [64 x, + 64), up to 20 slabs of 16 rows x 64 B; wave 4+q fills
    // slabs q, q+4, .. as far as the tile has rows (one instruction per 64 rows of the tile) and fetches 256
    // scale bytes.  The count is a template argument of the K loop: selecting the instructions and the
    // matching wait with scalar branches inside the loop cost 5 % of the kernel's time.
    // Every source address is a wave-uniform base (operand base + K offset of the unit, kept in
    // scalar registers) plus a per-lane 32-bit row offset doff[] that never changes: weights
    // doff[4 * half + j]; tokens doff[0..4], scales doff[5].  Token rows that do not exist (padding
    // ids, rows past the tile) read row 0 instead: their MFMA columns are never stored.
    const bool w_role = wave < 4;
    const int q4      = wave & 3;
    uint32_t doff[kXPair ? 10 : 8];
    const unsigned char* dbase;
    if(w_role)
    {
        dbase = uniform_ptr(p.w + (int64_t)expert * p.w_expert_bytes);
#pragma unroll
        for(int h = 0; h < 2; h++)
#pragma unroll
            for(int j = 0; j < 4; j++)
            {
                const int inst   = q4 + 4 * j;                      // instruction of the unit: LDS rows 8 inst .. + 7
                const int rih    = inst * 8 + (WPERM ? lane & 7 : lane >> 3); // LDS row inside the half
                const int trow   = h * kWHalfRows + rih;
                const int blk    = trow >> 5;
                const int c      = trow & 31; // LDS row r of a 32-row block holds weight channel r (see weight_row_swizzle)
                const int cchunk = WPERM ? (lane >> 3) ^ ((inst >> 1) & 1) : (lane & 7) ^ weight_row_swizzle(rih);
                int grow;
                if(paired)
                    grow = (blk & 1) * p.n_out + min(n_base + (blk >> 1) * 32 + c, p.n_out - 1);
                else
                    grow = min(n_base + blk * 32 + c, p.n_total - 1);
                doff[h * 4 + j] = weight_offset(p, grow, cchunk);
            }
    }
    else
    {
        dbase = uniform_ptr(p.x);
        if constexpr(kXPair)
        {
            // instruction j of wave 4 + q: rows (q + 4 j) * 8 .. + 7 of the tile, 128 bytes each, chunks swizzled
            // like the weight rows
#pragma unroll
            for(int j = 0; j < 10; j++)
            {
                const int lrow = (q4 + 4 * j) * 8 + (lane >> 3);
                int sid        = p.tokens;
                if(lrow < nrows)
                    sid = p.sorted_ids[row0 + lrow];
                const uint32_t src = (sid & 0xffffff) < p.tokens ? token_row(p, sid) : 0u;
                doff[j]            = src * (uint32_t)p.x_row_bytes + ((lane & 7) ^ ((lrow >> 1) & 7)) * 16;
            }
        }
        else
        {
            const int lrow16 = lane >> 2;
            const int cchunk = (lane & 3) ^ ((lane >> 4) & 3);
#pragma unroll
            for(int j = 0; j < 5; j++)
            {
                const int lrow = (q4 + 4 * j) * 16 + lrow16;
                uint32_t src   = lrow < nrows ? row0 + lrow : row0;
                if(GEMM0 || p.slot_rows > 0)
                {
                    int sid = p.tokens;
                    if(lrow < nrows)
                        sid = p.sorted_ids[row0 + lrow];
                    const bool ok = (sid & 0xffffff) < p.tokens;
                    src           = !ok ? 0u : GEMM0 ? token_row(p, sid) : (uint32_t)slot_row(sid, p.slot_rows);
                }
                doff[j] = src * (uint32_t)p.x_row_bytes + cchunk * 16;
                if(!GEMM0 && p.y_slab > 0) // slab-major Y: whole slabs; slabs past the tile's rows read its first
                    doff[j] = (uint32_t)(((row0 >> 4) + ((q4 + 4 * j) * 16 < nrows ? q4 + 4 * j : 0)) * p.y_slab) * 1024u +
                              lrow16 * 64 + cchunk * 16;
            }
            // scales: K block (q >> 1) of the step, rows (q & 1) * 256 .. + 255 (the rows are padded)
            doff[5] = (uint32_t)((q4 >> 1) * p.ys_kb_stride + row0 + (q4 & 1) * 256 + lane * 4);
            doff[6] = doff[7] = 0;
        }
    }
    const int64_t ys_step = (kStepKB / 32) * p.ys_kb_stride;
    const int x_step      = (!GEMM0 && p.y_slab > 0) ? 1024 : kStepKB; // bytes between token steps

    const uint32_t lds_base = lds_offset(lds);
    const int kt_count      = p.k_bytes_x / kStepKB; // compute steps (even; a multiple of four with int8 weights)
    const int n_wunits      = kW8 ? kt_count / 2 : kt_count; // two units (row halves) per 128 bytes of weight K

    // weight role: unit u (half u & 1) -> ring slot u % 6
    // Weights no other row tile re-reads (the expert has a single one) are fetched non-temporal: measured
    // -8 % on the gate+up GEMM at 32 rows per expert, -2 % at 256; with several row tiles per expert the
    // re-reads should hit L2, and non-temporal fetches cost 3 % there.  NT is a template argument like the
    // slab-group count, for the same reason.
    const bool w_nt = tile.expert_tiles == 1;
    const int w_kadv = weight_k_advance(p, 2 * kStepKB); // bytes between the 128-byte K windows of two weight units
    auto issue_w = [&](int u, auto half_tag, auto nt_tag) __attribute__((always_inline)) {
        constexpr int H = decltype(half_tag)::value;
        constexpr bool NT = decltype(nt_tag)::value;
        if(u >= n_wunits)
            return;
        const uint32_t sbase     = lds_base + (u % kWS) * kWUnitBytes + q4 * 1024;
        const unsigned char* src = dbase + (u >> 1) * w_kadv;
#pragma unroll
        for(int j = 0; j < 4; j++)
        {
            // H < 0: the row half is not known at compile time (int8 weights: one unit every other step); the
            // choice is spelled as arithmetic, a select between two elements of doff[] turns the array into an
            // indexed one in scratch memory
            const uint32_t off = H >= 0 ? doff[(H >= 0 ? H : 0) * 4 + j]
                                        : doff[j] ^ ((doff[j] ^ doff[4 + j]) & (0u - (uint32_t)(u & 1)));
            if constexpr(NT)
                dma16nt(src, off, __builtin_amdgcn_readfirstlane(sbase + j * 4096));
            else
                dma16(src, off, __builtin_amdgcn_readfirstlane(sbase + j * 4096));
        }
    };
    // token role: step x -> ring stage x % 3
    auto issue_x = [&](int x, int groups) __attribute__((always_inline)) {
        if(x >= kt_count)
            return;
        const uint32_t sbase     = lds_base + kXOffset + (x % kXStages) * kXStageBytes + q4 * 1024;
        const unsigned char* src = dbase + x * x_step;
#pragma unroll
        for(int j = 0; j < 5; j++)
            if(j < groups)
                dma16(src, doff[j], __builtin_amdgcn_readfirstlane(sbase + j * 4096));
        if constexpr(kMx)
            dma4(p.y_scale + x * ys_step, doff[5],
                 __builtin_amdgcn_readfirstlane(lds_base + kYsOffset + (x % kXStages) * kYsStageBytes +
                                                (q4 >> 1) * kYsRows + (q4 & 1) * 256));
    };

    // 128-byte token stages: pair m = steps 2 m and 2 m + 1 -> stage m & 1; two instructions per 64 rows of the tile
    auto issue_x_pair = [&](int m, int groups) __attribute__((always_inline)) {
        if constexpr(kXPair)
        {
            if(2 * m >= kt_count)
                return;
            const uint32_t sbase     = lds_base + kXO + (m & 1) * kXPairBytes + q4 * 1024;
            const unsigned char* src = dbase + m * (2 * kStepKB);
#pragma unroll
            for(int j = 0; j < 10; j++)
                if(j < 2 * groups)
                    dma16(src, doff[j], __builtin_amdgcn_readfirstlane(sbase + j * 4096));
        }
    };

    // token blocks of this wave (blocks wt, wt + 2, ..) and 64-row slab groups that hold rows of the tile
    const int nb_w     = __builtin_amdgcn_readfirstlane(max(0, min(kMaxNB, (nmb - wt + 1) / 2)));
    const int x_groups = __builtin_amdgcn_readfirstlane(max(1, (nmb + 1) / 2));

    Acc acc[kMaxNB][2];
#pragma unroll
    for(int i = 0; i < kMaxNB; i++)
#pragma unroll
        for(int b = 0; b < 2; b++)
#pragma unroll
            for(int v = 0; v < 16; v++)
                acc[i][b][v] = 0;

    // prologue: weight units 0..3 (0..4 when pipelined with six slots), token steps 0 and 1 (and 2; or pairs 0 and 1)
    using H0 = std::integral_constant<int, 0>;
    using H1 = std::integral_constant<int, 1>;
    if(w_role)
    {
        if(w_nt)
        {
            issue_w(0, H0{}, std::true_type{});
            issue_w(1, H1{}, std::true_type{});
            issue_w(2, H0{}, std::true_type{});
            issue_w(3, H1{}, std::true_type{});
            if constexpr(kPipe && !kXPair)
                issue_w(4, H0{}, std::true_type{});
        }
        else
        {
            issue_w(0, H0{}, std::false_type{});
            issue_w(1, H1{}, std::false_type{});
            issue_w(2, H0{}, std::false_type{});
            issue_w(3, H1{}, std::false_type{});
            if constexpr(kPipe && !kXPair)
                issue_w(4, H0{}, std::false_type{});
        }
    }
    else if constexpr(kXPair)
    {
        issue_x_pair(0, x_groups);
        issue_x_pair(1, x_groups);
    }
    else
    {
        issue_x(0, x_groups);
        issue_x(1, x_groups);
        if constexpr(kPipe)
            issue_x(2, x_groups);
    }

    // per-lane LDS read offsets (swizzled chunk positions are per-lane constants)
    const int sw_w  = (r32 >> 1) & 7; // 128-byte token rows of the gate+up GEMM
    const int w_row = chan_of_row(r32); // LDS row that holds the channel of this lane's MFMA row
    const int sw_wr = WPERM ? (w_row >> 4) & 1 : weight_row_swizzle(w_row);
    constexpr int kWChunkB = WPERM ? 128 : 16; // LDS bytes between two chunks of a weight row
    const int sw_x  = (r32 >> 2) & 3; // 64-byte token rows
    const int w_off = WPERM ? ((ww & 1) * 8 + (w_row >> 3)) * 1024 + (w_row & 7) * 16 : ((ww & 1) * 64 + w_row) * (2 * kStepKB);
    const int w_h   = ww >> 1;
    const int x_off = kXOffset + (wt * 32 + r32) * kStepKB;

    // NB: token blocks of this wave; XG: slab groups a token-role wave issues per step (0 in a weight-role wave)
    auto k_loop = [&](auto nb_tag, auto xg_tag, auto nt_tag) __attribute__((always_inline)) {
        constexpr int NB = decltype(nb_tag)::value;
        constexpr int XG = decltype(xg_tag)::value;
        constexpr int NF = NB > 0 ? NB : 1;
        if constexpr(kPipe)
        {
            // operand registers of the step about to run
            Frag wf[kSteps][2];
            Frag xf[kSteps][NF];
            uint32_t xs[kSteps][NF];
            // weight fragment b of sub-step s of step kk (parity P), token fragment i of sub-step s of step kk
            auto load_wf = [&](int kk, auto p_tag, int s, int b) __attribute__((always_inline)) {
                constexpr int P          = decltype(p_tag)::value;
                constexpr int kh         = P * 4; // first chunk of the step inside the 128-byte weight row
                const unsigned char* wp  = lds + (((kk & ~1) + w_h) % kWS) * kWUnitBytes + w_off + b * 32 * (2 * kStepKB);
                const int cw_lo          = kOpB == 16 ? ((kh + 2 * s + kg) ^ sw_wr) * kWChunkB : ((kh + kg) ^ sw_wr) * kWChunkB;
                const int cw_hi          = ((kh + 2 + kg) ^ sw_wr) * kWChunkB;
                Frag f;
                f.lo = *reinterpret_cast<const uint4*>(wp + cw_lo);
                if constexpr(kOpB == 32)
                    f.hi = *reinterpret_cast<const uint4*>(wp + cw_hi);
                return f;
            };
            auto load_xf = [&](int kk, int s, int i, uint32_t& scale) __attribute__((always_inline)) {
                Frag f;
                scale = 127;
                if constexpr(kXPair)
                {
                    const unsigned char* xp = lds + kXO + ((kk >> 1) & 1) * kXPairBytes + (wt * 32 + r32 + i * 64) * (2 * kStepKB);
                    const int kh            = (kk & 1) * 4;
                    const int cx_lo         = kOpB == 16 ? ((kh + 2 * s + kg) ^ sw_w) * 16 : ((kh + kg) ^ sw_w) * 16;
                    const int cx_hi         = ((kh + 2 + kg) ^ sw_w) * 16;
                    f.lo                    = *reinterpret_cast<const uint4*>(xp + cx_lo);
                    if constexpr(kOpB == 32)
                        f.hi = *reinterpret_cast<const uint4*>(xp + cx_hi);
                }
                else
                {
                    const unsigned char* xp = lds + x_off + (kk % kXStages) * kXStageBytes + i * 64 * kStepKB;
                    const int cx_lo         = kOpB == 16 ? ((2 * s + kg) ^ sw_x) * 16 : (kg ^ sw_x) * 16;
                    const int cx_hi         = ((2 + kg) ^ sw_x) * 16;
                    f.lo                    = *reinterpret_cast<const uint4*>(xp + cx_lo);
                    if constexpr(kOpB == 32)
                        f.hi = *reinterpret_cast<const uint4*>(xp + cx_hi);
                    if constexpr(kMx)
                        scale = lds[kYsOffset + (kk % kXStages) * kYsStageBytes + kg * kYsRows + wt * 32 + r32 + i * 64];
                }
                return f;
            };
            // own transfers of the data named `need` have landed (the instructions issued after them may be
            // pending), everyone's are visible after the barrier, and nobody reads the buffers of the step before
            auto sync = [&](bool counted, auto w_tag, auto x_tag) __attribute__((always_inline)) {
                if(counted)
                {
                    if(w_role)
                        wait_vmcnt<decltype(w_tag)::value>();
                    else
                        wait_vmcnt<decltype(x_tag)::value>();
                }
                else
                    wait_vmcnt<0>();
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // own operand fetches are complete
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            };
            constexpr int kXI = XG + (kMx ? 1 : 0); // token-role instructions of one step
            // step 0's data: weight units 0 and 1 (2, 3, 4 may be pending), token step 0 (1 and 2 pending); with
            // 128-byte token stages weight units 2 and 3 and token pair 1 may be pending
            if constexpr(kXPair)
                sync(kt_count >= 6, std::integral_constant<int, 8>{}, std::integral_constant<int, 2 * XG>{});
            else
                sync(kt_count >= 6, std::integral_constant<int, 12>{}, std::integral_constant<int, 2 * kXI>{});
            static_for<kSteps>([&](auto s_tag) __attribute__((always_inline)) {
                constexpr int s = decltype(s_tag)::value;
                wf[s][0]        = load_wf(0, H0{}, s, 0);
                wf[s][1]        = load_wf(0, H0{}, s, 1);
                static_for<NB>([&](auto i_tag) __attribute__((always_inline)) {
                    constexpr int i = decltype(i_tag)::value;
                    xf[s][i]        = load_xf(0, s, i, xs[s][i]);
                });
            });
            auto step = [&](int k, auto par_tag) __attribute__((always_inline)) {
                constexpr int PAR = decltype(par_tag)::value;
                using NPAR        = std::integral_constant<int, 1 - PAR>;
                // The barrier of step k guarantees step k+1: token step k+1 (k+2 may be pending) and the weight pair
                // of step k+1, that is units up to k+1 for even k (k+2 .. k+4 pending) or up to k+2 for odd k.
                // 128-byte token stages: a weight unit less is in flight (unit k+3 may be pending at odd k), and the
                // token pair of steps k+1 and k+2 is due at odd k, where it is the wave's only transfer.
                // Steps 2 m and 2 m + 1 read the same weight pair and the same token stage, so only the barrier of
                // the odd step has anything to guarantee, and what the even step overwrites (the slot of weight unit
                // k - 1) was last read before the barrier of step k - 1: the even step has no barrier.
                // Measured: without it the bf16 and int8 GEMMs (two MFMA sub-steps per step) run 2 % faster, the fp8
                // GEMM (one) 5 % slower, so that one keeps it.
                if constexpr(kXPair)
                {
                    if constexpr(PAR == 1 || kSteps == 1)
                        sync(k + 4 < kt_count, std::integral_constant<int, (PAR ? 4 : 8)>{},
                             std::integral_constant<int, (PAR ? 0 : 2 * XG)>{});
                }
                else
                    sync(k + 4 < kt_count, std::integral_constant<int, (PAR ? 8 : 12)>{}, std::integral_constant<int, kXI>{});
                // the transfers of the step go out behind the MFMAs of the second token block (measured: 1 to 2 %
                // faster than right after the barrier, where all eight waves queue up at the address unit while the
                // MFMA pipe has nothing to do; one instruction behind every block is 5 % slower)
                auto issue_next = [&]() __attribute__((always_inline)) {
                    if constexpr(kXPair)
                    {
                        // slot (k + 4) % 5 held unit k - 1, stage ((k + 3) / 2) & 1 held the pair of steps k - 1 and
                        // k - 2: both were last read during step k - 1, into registers, before this step's barrier
                        if(w_role)
                            issue_w(k + 4, par_tag, nt_tag);
                        else if constexpr(PAR == 1)
                            issue_x_pair((k + 3) >> 1, XG);
                    }
                    else if(w_role)
                        issue_w(k + 5, NPAR{}, nt_tag);
                    else
                        issue_x(k + 3, XG);
                };
                constexpr int kIssueAfter = 1;
                if constexpr(NB <= kIssueAfter)
                    issue_next();
                static_for<kSteps>([&](auto s_tag) __attribute__((always_inline)) {
                    constexpr int s = decltype(s_tag)::value;
                    static_for<NB>([&](auto i_tag) __attribute__((always_inline)) {
                        constexpr int i = decltype(i_tag)::value;
                        if constexpr(MODE == kFp8 && GEMM0)
                        {
                            acc[i][0] = mfma_fp8_unscaled(wf[s][0], xf[s][i], acc[i][0]);
                            acc[i][1] = mfma_fp8_unscaled(wf[s][1], xf[s][i], acc[i][1]);
                        }
                        else
                        {
                            acc[i][0] = mfma<MODE>(wf[s][0], xf[s][i], xs[s][i], acc[i][0]);
                            acc[i][1] = mfma<MODE>(wf[s][1], xf[s][i], xs[s][i], acc[i][1]);
                        }
                        // the fragment's registers are free: fetch its successor (stale data after the last step)
                        __builtin_amdgcn_sched_barrier(0);
                        xf[s][i] = load_xf(k + 1, s, i, xs[s][i]);
                        if constexpr(NB > kIssueAfter && s == 0 && i == kIssueAfter)
                            issue_next();
                        __builtin_amdgcn_sched_barrier(0);
                    });
                    wf[s][0] = load_wf(k + 1, NPAR{}, s, 0);
                    wf[s][1] = load_wf(k + 1, NPAR{}, s, 1);
                    __builtin_amdgcn_sched_barrier(0);
                });
            };
            for(int k = 0; k < kt_count; k += 2)
            {
                step(k, H0{});
                step(k + 1, H1{});
            }
            return;
        }
        // one compute step; PAR = k & 1
        auto step = [&](int k, auto par_tag) __attribute__((always_inline)) {
            constexpr int PAR = decltype(par_tag)::value;
            // Needed now: token step k and the weight units of pair k >> 1.  Issued after them and allowed
            // to stay pending: token step k+1; weight units k+2, k+3 (even k) or k+1 .. k+3 (odd k).
            if(k + 3 < kt_count)
            {
                if(w_role)
                    wait_vmcnt<PAR ? 12 : 8>();
                else
                    wait_vmcnt<XG + (kMx ? 1 : 0)>(); // token-role instructions of one step
            }
            else
                wait_vmcnt<0>();
            // data of step k visible to all waves; everyone is done reading step k-1 (a bare barrier:
            // the DMA completion was awaited above and LDS reads are consumed by MFMAs before a
            // wave gets here)
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            auto issue_next = [&]() __attribute__((always_inline)) {
                if(w_role)
                {
                    if constexpr(!kW8)
                        issue_w(k + 4, par_tag, nt_tag);
                    else if constexpr(PAR == 0)
                        issue_w((k >> 1) + 4, std::integral_constant<int, -1>{}, nt_tag);
                }
                else
                    issue_x(k + 2, XG);
            };
            // Where in the step the transfers go out: right here, or after the MFMAs of token block kIssueAfter.  The
            // buffers they write are free from the barrier on either way, but issued here the handful of scalar and
            // DMA instructions sits between the barrier and the first operand fetch, on every wave's critical path;
            // issued behind the first MFMAs it runs while the matrix pipe is busy (measured -2 % fp8, -4 % bf16 on the
            // gate+up GEMM).  After all MFMAs is too late (the transfers then start up to a step later), and the fp8
            // down GEMM has no register to spare for the scheduling fence this needs.
            constexpr int kIssueAfter = kMx ? -1 : 1;
            if constexpr(kIssueAfter < 0 || NB <= kIssueAfter)
                issue_next();

            // first unit of the pair that holds this step's weight bytes
            const int pair0          = kW8 ? (k >> 2) << 1 : (k & ~1);
            const unsigned char* wst = lds + ((pair0 + w_h) % kWSlots) * kWUnitBytes + w_off;
            const unsigned char* xst = lds + x_off + (k % kXStages) * kXStageBytes;
            [[maybe_unused]] const unsigned char* ysl =
                lds + kYsOffset + (k % kXStages) * kYsStageBytes + kg * kYsRows + wt * 32 + r32;
            constexpr int kh = PAR * 4; // first chunk of this step inside the 128-byte weight row
#pragma unroll
            for(int s = 0; s < kSteps; s++)
            {
                Frag wf[2];
                Frag xf[NF];
                uint32_t xs[NF];
                const int cx_lo = kOpB == 16 ? ((2 * s + kg) ^ sw_x) * 16 : (kg ^ sw_x) * 16;
                const int cx_hi = ((2 + kg) ^ sw_x) * 16;
                const int cw_lo = kOpB == 16 ? ((kh + 2 * s + kg) ^ sw_wr) * kWChunkB : ((kh + kg) ^ sw_wr) * kWChunkB;
                const int cw_hi = ((kh + 2 + kg) ^ sw_wr) * kWChunkB;
#pragma unroll
                for(int b = 0; b < 2; b++)
                {
                    const unsigned char* wp = wst + b * 32 * (2 * kStepKB);
                    if constexpr(kW8)
                    {
                        // 8 int8 of this lane's K group: 16-byte chunk (k & 3) * 2 + s of the row, half kg
                        const int c8 = ((((k & 3) << 1) + s) ^ sw_wr) * kWChunkB + kg * 8;
                        wf[b].lo     = int8x8_to_bf16x8(*reinterpret_cast<const uint2*>(wp + c8));
                    }
                    else
                    {
                        wf[b].lo = *reinterpret_cast<const uint4*>(wp + cw_lo);
                        if constexpr(kOpB == 32)
                            wf[b].hi = *reinterpret_cast<const uint4*>(wp + cw_hi);
                    }
                }
#pragma unroll
                for(int i = 0; i < NB; i++)
                {
                    const unsigned char* xp = xst + i * 64 * kStepKB;
                    xf[i].lo                = *reinterpret_cast<const uint4*>(xp + cx_lo);
                    if constexpr(kOpB == 32)
                        xf[i].hi = *reinterpret_cast<const uint4*>(xp + cx_hi);
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
                    if(kIssueAfter >= 0 && NB > kIssueAfter && s == 0 && i == kIssueAfter)
                    {
                        __builtin_amdgcn_sched_barrier(0);
                        issue_next();
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        };
        for(int k = 0; k < kt_count; k += 2)
        {
            step(k, H0{});
            step(k + 1, H1{});
        }
    };
    // weight-role waves own blocks 0, 2, .. (ceil(nmb / 2) of them), token-role waves blocks 1, 3, ..
    // (floor(nmb / 2)) and issue ceil(nmb / 2) slab groups: the same count, or one more when nmb is odd
    using I0 = std::integral_constant<int, 0>;
    auto run = [&](auto nb_tag) {
        constexpr int NB = decltype(nb_tag)::value;
        if(w_role && w_nt)
            k_loop(nb_tag, I0{}, std::true_type{});
        else if(w_role)
            k_loop(nb_tag, I0{}, std::false_type{});
        else if(x_groups == NB)
            k_loop(nb_tag, std::integral_constant<int, (NB > 0 ? NB : 1)>{}, std::false_type{});
        else
            k_loop(nb_tag, std::integral_constant<int, (NB < kMaxNB ? NB + 1 : kMaxNB)>{}, std::false_type{});
    };
    switch(nb_w)
    {
    case 5: run(std::integral_constant<int, 5>{}); break;
    case 4: run(std::integral_constant<int, 4>{}); break;
    case 3: run(std::integral_constant<int, 3>{}); break;
    case 2: run(std::integral_constant<int, 2>{}); break;
    case 1: run(std::integral_constant<int, 1>{}); break;
    default: run(std::integral_constant<int, 0>{}); break;
    }

    // ---- epilogue
    run_epilogue<MODE, GEMM0, kMaxNB, false>(p, acc, expert, row0, nrows, wt * 32, 64, nb_w, n_base, ww, r32, kg);
}

template <int MODE, bool GEMM0, bool WPERM>
int launch_big_w(const GemmParams& p, int max_tiles, hipStream_t stream)
{
    constexpr bool kMx  = MODE == kFp8 && !GEMM0;
    const size_t lds    = (GEMM0 && MODE != kBf16W8) ? kLdsBytesPair : kMx ? kLdsBytes : kYsOffset;
    // the dynamic LDS limit is an attribute of the function on one device: set once per device, whichever host
    // thread gets there first (the others wait for it)
    static std::once_flag attr_once[64];
    int dev = 0;
    (void)hipGetDevice(&dev);
    hipError_t attr = hipSuccess;
    auto set_attr   = [&] {
        attr = hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_gemm_big_kernel<MODE, GEMM0, WPERM>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    };
    if(dev >= 0 && dev < 64)
        std::call_once(attr_once[dev], set_attr);
    else
        set_attr();
    MI355_HIP_TRY(attr);
    const int grid = round_up(max_tiles * p.n_ntiles, 256); // whole rounds of 32-item chunks over the 8 XCDs
    if(grid <= 0)
        return MI355_MOE_OK;
    KernelTimer timer(GEMM0 ? MI355_MOE_K_GEMM0 : MI355_MOE_K_GEMM1, stream);
    hipLaunchKernelGGL((moe_gemm_big_kernel<MODE, GEMM0, WPERM>), dim3(grid), dim3(kBigThreads), lds, stream, p);
    MI355_HIP_TRY(hipGetLastError());
    return MI355_MOE_OK;
}

template <int MODE, bool GEMM0>
int launch_big_t(const GemmParams& p, int max_tiles, hipStream_t stream)
{
    return p.w_permuted ? launch_big_w<MODE, GEMM0, true>(p, max_tiles, stream) : launch_big_w<MODE, GEMM0, false>(p, max_tiles, stream);
}

} // namespace

int big_tile_rows() { return kBigXRows; }

bool big_tile_supported(int prec, int k_bytes0, int k_bytes1, bool y_i8)
{
    // K in whole pairs of 64-byte steps; the int8 path's down GEMM with bf16 Y against int8 weights in fours
    if(prec == MI355_MOE_INT8)
        return k_bytes0 % (2 * kStepKB) == 0 && k_bytes1 % ((y_i8 ? 2 : 4) * kStepKB) == 0;
    return (prec == MI355_MOE_BF16 || prec == MI355_MOE_FP16 || prec == MI355_MOE_FP8) && k_bytes0 % (2 * kStepKB) == 0 &&
           k_bytes1 % (2 * kStepKB) == 0;
}

int launch_gemm_big(int prec, bool gemm0, const GemmParams& p, int max_tiles, hipStream_t stream, bool y_i8)
{
    if(prec == MI355_MOE_INT8 && !gemm0 && y_i8)
        return launch_big_t<kI8, false>(p, max_tiles, stream);
    if(prec == MI355_MOE_BF16)
        return gemm0 ? launch_big_t<kBf16, true>(p, max_tiles, stream) : launch_big_t<kBf16, false>(p, max_tiles, stream);
    if(prec == MI355_MOE_FP16)
        return gemm0 ? launch_big_t<kF16, true>(p, max_tiles, stream) : launch_big_t<kF16, false>(p, max_tiles, stream);
    if(prec == MI355_MOE_FP8)
        return gemm0 ? launch_big_t<kFp8, true>(p, max_tiles, stream) : launch_big_t<kFp8, false>(p, max_tiles, stream);
    if(prec == MI355_MOE_INT8)
        return gemm0 ? launch_big_t<kI8, true>(p, max_tiles, stream) : launch_big_t<kBf16W8, false>(p, max_tiles, stream);
    return fail(MI355_MOE_E_UNSUPPORTED, "no large-tile kernel for precision %d", prec);
}

} // namespace mi355
