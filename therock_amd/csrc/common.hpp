// Shared host/device helpers of libmi355_moe.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/mi355_moe.h"

namespace mi355 {

constexpr int kWave = 64;

// thread-local error text behind mi355_moe_last_error()
char* error_buffer();
int fail(int code, const char* fmt, ...);

#define MI355_HIP_TRY(expr)                                                                   \
    do                                                                                        \
    {                                                                                         \
        hipError_t e_ = (expr);                                                               \
        if(e_ != hipSuccess)                                                                  \
            return ::mi355::fail(MI355_MOE_E_HIP, "%s failed: %s", #expr, hipGetErrorString(e_)); \
    } while(0)

template <typename T>
__host__ __device__ constexpr T ceil_div(T a, T b)
{
    return (a + b - 1) / b;
}

template <typename T>
__host__ __device__ constexpr T round_up(T a, T b)
{
    return ceil_div(a, b) * b;
}

// token | slot << 24, the id format of ck_tile's moe_sorting (moe_sorting_kernel.hpp:78-80)
__host__ __device__ inline int32_t mock_id(int32_t token, int32_t slot)
{
    return static_cast<int32_t>((static_cast<uint32_t>(token) & 0x00ffffffu) |
                                ((static_cast<uint32_t>(slot) & 0xffu) << 24));
}

struct DeviceInfo
{
    int num_cu;
    int max_lds;
};
// cached per device (ck_tile queries hipGetDeviceProperties on every call)
const DeviceInfo& device_info();

// ---- optional per-kernel event timing (mi355_moe_profile_start / _stop)
bool profiling_enabled(int kind);
void profile_mark(int kind, hipStream_t stream, bool begin);

// brackets one kernel launch with events while profiling is on
struct KernelTimer
{
    int kind;
    hipStream_t stream;
    bool on;
    KernelTimer(int k, hipStream_t s) : kind(k), stream(s), on(profiling_enabled(k))
    {
        if(on)
            profile_mark(kind, stream, true);
    }
    ~KernelTimer()
    {
        if(on)
            profile_mark(kind, stream, false);
    }
};

// One event pair around several launches that count as one kernel of kind `k` (two candidate kernels of which one
// finds nothing to do): the launches' own timers stay off meanwhile.
void profile_hold(int kind, bool on);
struct KernelTimerGroup
{
    int kind;
    hipStream_t stream;
    bool on;
    KernelTimerGroup(int k, hipStream_t s, bool wanted) : kind(k), stream(s), on(wanted && profiling_enabled(k))
    {
        if(on)
        {
            profile_mark(kind, stream, true);
            profile_hold(kind, true);
        }
    }
    ~KernelTimerGroup()
    {
        if(on)
        {
            profile_hold(kind, false);
            profile_mark(kind, stream, false);
        }
    }
};

// ---- work list of the grouped GEMMs: int32 [kMapHdr + kMapEnt * max_tiles]; [0] = live tiles, [1] = the tile
// height (rows) the list was built for when the sort chose between two (else 0), then per
// tile (local expert id, first sorted row, rows, first tile of the expert, tiles of the expert, first sorted
// row of the expert, rows of the expert, rows per tile of the expert): any tile of an expert can be worked
// out from the entry of any other.  Entries are 32-byte aligned.
constexpr int kMapHdr = 8;
constexpr int kMapEnt = 8;

// Order of an expert's work items in the large-tile kernel: blocks of kTileRowBlock row tiles; inside a block column
// tile by column tile, the block's row tiles adjacent; the expert's last rows % kTileRowBlock row tiles form a
// narrower block of their own.  rel = item number inside the expert (0 .. rows * cols - 1) -> column tile, row tile.
constexpr int kTileRowBlock = 4;
__host__ __device__ inline void blocked_tile_of(int rel, int rows, int cols, int& col, int& row)
{
    const int full    = rows / kTileRowBlock * kTileRowBlock; // row tiles in whole blocks
    const int in_full = full * cols;
    if(rel < in_full)
    {
        const int blk = rel / (kTileRowBlock * cols);
        const int r2  = rel - blk * (kTileRowBlock * cols);
        col           = r2 / kTileRowBlock;
        row           = blk * kTileRowBlock + (r2 - col * kTileRowBlock);
    }
    else
    {
        const int rest = rows - full; // 1 .. kTileRowBlock - 1 row tiles, or the expert's only ones
        const int r2   = rel - in_full;
        col            = r2 / (rest > 0 ? rest : 1);
        row            = full + (r2 - col * rest);
    }
}

// what the sort can prepare for the GEMMs while it has the per-expert counts at hand
struct GemmPlan
{
    int* tile_map;     // work list, see above
    int rows_per_tile; // sorted rows per GEMM tile (multiple of 32)
    int max_tiles;     // capacity of tile_map
    int* inv;          // [tokens * topk]: sorted position of every (token, slot), -1 when dropped
    // A second tile height the sort may choose instead, from what only the device knows: with skewed routing the
    // experts that have tokens at all hold many more rows than tokens * topk / experts suggests.  Chosen when at least
    // alt_min_active experts are active and their padded rows average alt_min_rows or more; 0 rows: no choice.
    int alt_rows_per_tile;
    int alt_min_rows;
    int alt_min_active;
};

// ---- sorting launcher shared by the stand-alone and the fused entry points
// keep_empty: experts without tokens own one tile of padding (ck_tile's SkipExpertsWithZeroTokens = false);
// dispatch_policy: 0 = the library picks, 1 = single kernel, 2 = multi-launch passes
int launch_moe_sorting(const mi355_moe_sorting_args& a, hipStream_t stream, const GemmPlan* plan = nullptr,
                       bool keep_empty = false, int dispatch_policy = 0);

int launch_topk_softmax(const mi355_topk_softmax_traits& t, const mi355_topk_softmax_args& a, hipStream_t stream);

// matrix-core rate sustained on register operands (mfma_ceiling.hip)
int mfma_sustained(int prec, int milliseconds, int zeros, double* tflops, hipStream_t stream);

size_t sorting_workspace_bytes(int32_t tokens, int32_t experts, int32_t topk, int32_t dispatch_policy = 0);

} // namespace mi355
