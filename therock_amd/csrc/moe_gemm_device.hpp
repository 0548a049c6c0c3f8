// Device code shared by the grouped-GEMM kernels: operand types, MFMA wrappers, the per-lane
// epilogues (scales, SiLU*up, packing) and the kernel parameter block.
#pragma once

#include "moe_gemm.hpp"
#include "device_utils.hpp"

namespace mi355 {
namespace gemm {
// Every device function below is forced inline: with several instantiations of a kernel in one translation unit
// the inliner leaves the larger ones out of line, and their array arguments (accumulators, GemmParams) then live
// in scratch memory.

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(16))) int i32x16_t;
typedef __attribute__((ext_vector_type(4))) int i32x4_t;
typedef __attribute__((ext_vector_type(8))) int i32x8_t;

enum Mode
{
    kBf16   = 0, // x bf16, w bf16, bf16 MFMA
    kFp8    = 1, // x e4m3, w e4m3, block-scaled f8f6f4 MFMA
    kI8     = 2, // x int8, w int8, i8 MFMA (gemm1: int8 Y with a per-row scale, the fused_quant variants)
    kBf16W8 = 3, // x bf16, w int8 converted to bf16 after the LDS read (gemm1 of the int8 path)
    kF16    = 4  // x fp16, w fp16, f16 MFMA; Y, the partial rows and the output are fp16 (ck_tile's other instance)
};

constexpr int kBlock   = 256;
constexpr int kWRows   = 256; // weight rows per workgroup tile
constexpr int kPadB    = 16;

struct GemmParams
{
    const unsigned char* x;  // gemm0: activations [tokens, x_row_bytes]; gemm1: Y [rows, x_row_bytes]
    const unsigned char* w;  // [experts, n_total, k] K contiguous
    const float* x_scale;    // gemm0: per-token scale or null
    const float* w_scale;    // [experts, n_total] or null
    const int* sorted_ids;
    const int* tile_map;
    unsigned char* out;      // gemm0: Y; gemm1: P (both in sorted-row order)
    unsigned char* y_scale;  // e8m0 block scales of Y (fp8 path): written by gemm0, read by gemm1
    int64_t x_row_bytes;
    int64_t w_row_bytes;
    // weight layout: 0 = rows of K bytes ([experts, n, k], FusedMoeGemmWeightPermuteEnum::no_permute); 1 = ck_tile's
    // pre-shuffled b_nr_kr_kw_nw_kv (fused_moegemm_traits.hpp:10-17): blocks of 16 rows x 64 bytes of K, 1 KiB each,
    // ordered [n / 16][k bytes / 64]; inside a block the 16-byte piece c of row r sits at 256 c + 16 r
    int w_permuted;
    int64_t w_expert_bytes;
    int64_t out_row_bytes;
    int64_t ys_kb_stride;    // bytes between consecutive 32-column blocks of y_scale ([inter/32][rows])
    int k_bytes_x;           // bytes of K in a row of x
    int k_bytes_w;           // bytes of K in a row of w
    int n_out;               // gemm0: inter; gemm1: hidden
    int n_total;             // weight rows per expert (gemm0: 2*inter, gemm1: hidden)
    int n_ntiles;            // tiles along n
    int tokens;
    // Row addressing of the stand-alone GEMM entry point (0 in the fused path, where Y and P are in
    // sorted-row order): slot_rows = top-k count when gemm0's output rows, respectively gemm1's input
    // rows, are token * topk + slot (ck_tile's MoeFlatmm convention, moe_flatmm_kernel.hpp:790-801)
    int slot_rows;
    // Y layout between the two large-tile GEMMs: 0 = row-major; otherwise the number of 64-byte K
    // segments of a row, and Y is stored slab-major: [row / 16][segment][row % 16][64 B], so that the
    // 16 rows x 64 B one token DMA instruction of the down GEMM fetches are 1 KiB of consecutive memory
    // (8 whole cache lines instead of 16 half lines)
    int y_slab;
    // gemm0 variants of ck_tile's fused_moe_traits: gate_only = the weights hold gate rows only ([experts,
    // n_out, k]; a tile then covers twice the Y columns and y = act(gate)); act: 0 = gelu (erf form), 1 = silu
    int gate_only;
    int act;
    // fp8 gate+up GEMM of the stand-alone entry point: write bf16 instead of e4m3 with block scales
    int y_bf16;
    int tile_rows; // != 0: run only if the tile list was built for this tile height (see lookup_tile)
    int max_tiles; // entries the tile list has room for (upper bound of live tiles)
    // stand-alone GEMMs (ck_tile's MoeFlatmmHostArgs, moe_flatmm_kernel.hpp:17-31): expert bias [experts, n_total] added
    // to the scaled dot products (null: none); the last n_padded weight rows of every expert are padding and
    // count as zeros; act 2 = moe::Swiglu{swiglu_alpha, swiglu_limit}
    const float* bias;
    int n_padded;
    float swiglu_alpha;
    float swiglu_limit;
    // gemm0 of the smooth-quant path (fused_quant 1): the activations are one quantised row per (slot, token),
    // x [topk, tokens, .] with scales [topk, tokens] (ck_tile's MoeSmoothquant output, moe_sorting_kernel.hpp:82-83);
    // x_slot_major = 1 selects that addressing, 0 the usual row per token
    int x_slot_major;
};

// row of the gate+up GEMM's activations (and index of its per-row scale) a sorted id refers to
__device__ __attribute__((always_inline)) inline uint32_t token_row(const GemmParams& p, int sid)
{
    const uint32_t tok = static_cast<uint32_t>(sid) & 0xffffffu;
    return p.x_slot_major ? (static_cast<uint32_t>(sid) >> 24) * static_cast<uint32_t>(p.tokens) + tok : tok;
}

// byte offset of K byte kb of row `row` in the slab-major Y layout
__device__ __attribute__((always_inline)) inline int64_t y_slab_offset(int64_t row, int kb, int segs)
{
    return (((row >> 4) * segs + (kb >> 6)) << 10) + ((row & 15) << 6) + (kb & 63);
}

// row of a [tokens * topk, .] buffer a sorted id refers to
__device__ __attribute__((always_inline)) inline int64_t slot_row(int sid, int topk)
{
    return (int64_t)(sid & 0xffffff) * topk + static_cast<int>(static_cast<uint32_t>(sid) >> 24);
}

// Byte offset, inside one expert's weight matrix, of the 16 bytes of row `row` that start `chunk16` 16-byte pieces
// into a window of K that begins on a multiple of 64 bytes; and what moving that window by `bytes` (a multiple of
// 64) adds to it.  Row-major: row * row_bytes + 16 * chunk16, + bytes.  Pre-shuffled: the row's block row, the block
// (chunk16 / 4) of the window, the piece inside the block; a window 64 bytes further on is the next 1 KiB block.
__device__ __attribute__((always_inline)) inline uint32_t weight_offset(const GemmParams& p, int row, int chunk16)
{
    if(p.w_permuted == 0)
        return (uint32_t)row * (uint32_t)p.w_row_bytes + chunk16 * 16;
    return (uint32_t)(row >> 4) * (uint32_t)(p.w_row_bytes * 16) + (chunk16 >> 2) * 1024 + (chunk16 & 3) * 256 + (row & 15) * 16;
}
__device__ __attribute__((always_inline)) inline int weight_k_advance(const GemmParams& p, int bytes) { return p.w_permuted == 0 ? bytes : bytes * 16; }

// Work item -> tile.  Workgroup ids are dealt round-robin to the 8 XCDs; inside an expert the row tiles of one
// weight tile are adjacent.  One entry of the list describes the whole expert, so a single load resolves any of
// its tiles.  Two orders: XCD x takes a contiguous eighth of the work list (the weight-streaming kernels: every
// XCD walks its own region of the weights), or chunks of 32 consecutive work items go round-robin to the XCDs (the
// large-tile kernel: tiles of hot and cold experts cost very different amounts, and chunks spread them - 5 % on
// the Zipf-routed workload; the position then does not depend on the live tile count, so that count and the
// tile's entry are fetched together instead of one after the other).
struct TileRef
{
    int expert, row0, nrows, nt; // nt: column tile
    int expert_tiles;            // row tiles of this expert (each of them re-reads the same weight tiles)
    bool ok;
};
// tile_rows != 0: the launch is one of two candidates and runs only if the sort built the list for its tile height
// (tile_map[1]); the other candidate's workgroups all leave at once.
template <bool CHUNKED = false>
__device__ __attribute__((always_inline)) inline TileRef lookup_tile(const int* __restrict__ tile_map, int n_ntiles, int max_tiles, int block,
                                      int tile_rows = 0)
{
    TileRef t;
    if(tile_rows != 0 && tile_map[1] != tile_rows)
    {
        t.expert = t.row0 = t.nrows = t.nt = t.expert_tiles = 0;
        t.ok = false;
        return t;
    }
    const int slot = block >> 3;
    int work, total;
    if constexpr(CHUNKED)
    {
        work  = ((((slot >> 5) << 3) + (block & 7)) << 5) + (slot & 31);
        t.ok  = true;
    }
    else
    {
        total             = tile_map[0] * n_ntiles;
        const int per_xcd = ceil_div(total, 8);
        work              = (block & 7) * per_xcd + slot;
        t.ok              = slot < per_xcd && work < total;
    }
    // (chunked: the entry is fetched before the item is known to be live, so the index is kept inside the list)
    const int t0  = CHUNKED ? min(work / n_ntiles, max_tiles - 1) : (t.ok ? work / n_ntiles : 0);
    const int4* e = reinterpret_cast<const int4*>(tile_map + kMapHdr + t0 * kMapEnt);
    if constexpr(CHUNKED)
        total = tile_map[0] * n_ntiles;
    const int4 a  = e[0]; // expert, row0, nrows, first tile of the expert
    const int4 b  = e[1]; // tiles of the expert, its first row, its rows, rows per tile
    if constexpr(CHUNKED)
        t.ok = work < total;
    const int rel     = work - a.w * n_ntiles;
    int j;
    if constexpr(CHUNKED)
    {
        // An expert's items in blocks of four row tiles (blocked_tile_of): inside a block column tile by column tile,
        // the block's row tiles adjacent.  The 32 consecutive items that run together on one XCD are then 4 row tiles
        // x 8 column tiles: every K slice of their tokens is fetched into that L2 once for 8 column tiles and every
        // weight slice once for 4 row tiles.  With all row tiles of a column tile adjacent (the order of the other
        // kernels) an expert of 100 row tiles re-read its tokens from beyond L2 for every column tile: 9.2 GB of
        // fetches against 0.9 GB of operands on the Zipf-routed workload.
        blocked_tile_of(rel, max(b.x, 1), n_ntiles, t.nt, j);
    }
    else
    {
        t.nt = rel / max(b.x, 1);
        j    = rel - t.nt * b.x;
    }
    t.expert          = a.x;
    t.expert_tiles    = b.x;
    t.row0            = b.y + j * b.w;
    t.nrows           = min(b.w, b.z - j * b.w);
    return t;
}

template <int MODE>
struct ModeTraits;
template <>
struct ModeTraits<kBf16>
{
    using Acc                  = f32x16_t;
    static constexpr int kOpB  = 16; // operand bytes per lane per MFMA
    static constexpr int kWKB  = 128;
    static constexpr int kXKB  = 128;
};
template <>
struct ModeTraits<kF16> : ModeTraits<kBf16>
{
};
template <>
struct ModeTraits<kFp8>
{
    using Acc                  = f32x16_t;
    static constexpr int kOpB  = 32;
    static constexpr int kWKB  = 128;
    static constexpr int kXKB  = 128;
};
template <>
struct ModeTraits<kI8>
{
    using Acc                  = i32x16_t;
    static constexpr int kOpB  = 16;
    static constexpr int kWKB  = 128;
    static constexpr int kXKB  = 128;
};
template <>
struct ModeTraits<kBf16W8>
{
    using Acc                  = f32x16_t;
    static constexpr int kOpB  = 16;
    static constexpr int kWKB  = 128; // int8 weights: 128 K elements per tile row ...
    static constexpr int kXKB  = 256; // ... against 128 bf16 activations
};

// MFMA row m of a 32-row weight block holds weight channel chan_of_row(m); with the 32x32
// accumulator layout (register v = 4j+i of lane l is row 8j + 4(l/32) + i) lane l then owns the 16
// consecutive channels 16*(l/32) .. +15 of its token in registers 0..15.
__device__ __host__ constexpr int chan_of_row(int m) { return 16 * ((m >> 2) & 1) + 4 * (m >> 3) + (m & 3); }

__device__ __attribute__((always_inline)) inline float silu(float x) { return x * __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }
// Gelu in the erf form of ck_tile::element_wise::Gelu (unary_element_wise_operation.hpp:975-986):
// x * Phi(x) with erfc(z) = poly(t) * exp(-z^2), t = 1 / (1 + 0.3275911 z) (Abramowitz & Stegun 7.1.26,
// absolute error of erf <= 1.5e-7), branch-free and free of cancellation in the negative tail
__device__ __attribute__((always_inline)) inline float gelu(float x)
{
    const float z = fabsf(x) * 0.70710678118f;
    const float t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * z);
    const float q = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f)))) *
                    __expf(-z * z); // erfc(z)
    return x >= 0.f ? x * (1.0f - 0.5f * q) : 0.5f * x * q;
}

// 8 int8 (two dwords) -> 8 bf16 (exact: |v| <= 128 fits bf16's 8 significant bits)
__device__ __attribute__((always_inline)) inline uint4 int8x8_to_bf16x8(uint2 v)
{
    uint4 r;
    uint32_t d[2] = {v.x, v.y};
    uint32_t o[4];
#pragma unroll
    for(int h = 0; h < 2; h++)
    {
        const int s = static_cast<int>(d[h]);
        const uint32_t f0 = __float_as_uint(static_cast<float>((s << 24) >> 24));
        const uint32_t f1 = __float_as_uint(static_cast<float>((s << 16) >> 24));
        const uint32_t f2 = __float_as_uint(static_cast<float>((s << 8) >> 24));
        const uint32_t f3 = __float_as_uint(static_cast<float>(s >> 24));
        o[2 * h]     = (f1 & 0xffff0000u) | (f0 >> 16);
        o[2 * h + 1] = (f3 & 0xffff0000u) | (f2 >> 16);
    }
    r.x = o[0];
    r.y = o[1];
    r.z = o[2];
    r.w = o[3];
    return r;
}

template <typename To, typename From>
__device__ __attribute__((always_inline)) inline To bit_cast_dev(const From& f)
{
    static_assert(sizeof(To) == sizeof(From), "size mismatch");
    To t;
    __builtin_memcpy(&t, &f, sizeof(To));
    return t;
}

struct Frag
{
    uint4 lo, hi; // hi only used by 32-byte operands
};

template <int MODE>
__device__ __attribute__((always_inline)) inline typename ModeTraits<MODE>::Acc mfma(const Frag& w, const Frag& x, uint32_t x_scale,
                                                      typename ModeTraits<MODE>::Acc c)
{
    if constexpr(MODE == kBf16 || MODE == kBf16W8)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(bit_cast_dev<bf16x8_t>(w.lo), bit_cast_dev<bf16x8_t>(x.lo), c,
                                                       0, 0, 0);
    }
    else if constexpr(MODE == kF16)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(bit_cast_dev<f16x8_t>(w.lo), bit_cast_dev<f16x8_t>(x.lo), c, 0, 0, 0);
    }
    else if constexpr(MODE == kI8)
    {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(bit_cast_dev<i32x4_t>(w.lo), bit_cast_dev<i32x4_t>(x.lo), c, 0,
                                                     0, 0);
    }
    else
    {
        i32x8_t a, b;
        a[0] = w.lo.x; a[1] = w.lo.y; a[2] = w.lo.z; a[3] = w.lo.w;
        a[4] = w.hi.x; a[5] = w.hi.y; a[6] = w.hi.z; a[7] = w.hi.w;
        b[0] = x.lo.x; b[1] = x.lo.y; b[2] = x.lo.z; b[3] = x.lo.w;
        b[4] = x.hi.x; b[5] = x.hi.y; b[6] = x.hi.z; b[7] = x.hi.w;
        // cbsz = blgp = 0: both operands e4m3; weights carry the unit block scale 2^0 (e8m0 127),
        // the token operand its per-32 block scale in byte 0 (op_sel 0)
        return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 127, 0, static_cast<int>(x_scale));
    }
}


// e4m3 x e4m3 without block scales (both scale operands literal 0 select the unscaled encoding,
// which issues faster than the scaled one)
__device__ __attribute__((always_inline)) inline f32x16_t mfma_fp8_unscaled(const Frag& w, const Frag& x, f32x16_t c)
{
    i32x8_t a, b;
    a[0] = w.lo.x; a[1] = w.lo.y; a[2] = w.lo.z; a[3] = w.lo.w;
    a[4] = w.hi.x; a[5] = w.hi.y; a[6] = w.hi.z; a[7] = w.hi.w;
    b[0] = x.lo.x; b[1] = x.lo.y; b[2] = x.lo.z; b[3] = x.lo.w;
    b[4] = x.hi.x; b[5] = x.hi.y; b[6] = x.hi.z; b[7] = x.hi.w;
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

// two results -> the 16-bit type the mode stores (fp16 for kF16, bf16 otherwise), both round to nearest even
template <int MODE>
__device__ __attribute__((always_inline)) inline uint32_t pack_out2(float lo, float hi)
{
    if constexpr(MODE == kF16)
        return pack_f16x2(lo, hi);
    else
        return pack_bf16x2(lo, hi);
}

// ---------------------------------------------------------------------------------------------
// Epilogues.  With the weight rows on the MFMA's M side and chan_of_row(), a lane holds, for the
// token in column (lane % 32), the 16 consecutive output channels col0 .. col0+15 in acc[0..15].

// The operands of the epilogues (sorted ids, top-k weights, scales) are loaded by the callers in
// one batch right after the K loop, so that their latencies overlap instead of adding up.

// per-channel scales of the 16 channels a lane owns (1.0 when the path is unscaled)
__device__ __attribute__((always_inline)) inline void load_channel_scales(const float* scale, float (&out)[16])
{
    if(scale != nullptr)
    {
        const float4* s4 = reinterpret_cast<const float4*>(scale);
#pragma unroll
        for(int q = 0; q < 4; q++)
        {
            const float4 t = s4[q];
            out[4 * q] = t.x; out[4 * q + 1] = t.y; out[4 * q + 2] = t.z; out[4 * q + 3] = t.w;
        }
    }
    else
    {
#pragma unroll
        for(int v = 0; v < 16; v++)
            out[v] = 1.0f;
    }
}

// ck_tile::moe::Swiglu (moe_flatmm_kernel.hpp:149-183, device branch): gate' = min(gate, limit),
// linear' = clamp(linear, -limit, limit), gate' * rcp(1 + exp(-alpha * gate')) * (linear' + 1)
__device__ __attribute__((always_inline)) inline float swiglu(float gate, float linear, float alpha, float limit)
{
    gate   = fminf(gate, limit);
    linear = fminf(fmaxf(linear, -limit), limit);
    return gate * __builtin_amdgcn_rcpf(1.0f + __expf(-alpha * gate)) * (linear + 1.0f);
}

// Bias and padding of the stand-alone GEMMs for the 16 channels chan0 .. chan0 + 15 of one expert (row index
// inside the expert's weight): v = dot * scale, then the padded channels lose their dot product and every
// channel gains its bias.  Rare (a uniform branch at the call sites), so the bias is fetched here rather than
// carried in registers beside the scales.
__device__ __attribute__((always_inline)) inline void bias_and_padding(const GemmParams& p, float (&v)[16], int expert, int chan0)
{
    if(p.n_padded > 0)
    {
#pragma unroll
        for(int i = 0; i < 16; i++)
            v[i] = chan0 + i < p.n_total - p.n_padded ? v[i] : 0.0f;
    }
    if(p.bias != nullptr)
    {
        const float4* b4 = reinterpret_cast<const float4*>(p.bias + (int64_t)expert * p.n_total + chan0);
#pragma unroll
        for(int q = 0; q < 4; q++)
        {
            const float4 t = b4[q];
            v[4 * q] += t.x; v[4 * q + 1] += t.y; v[4 * q + 2] += t.z; v[4 * q + 3] += t.w;
        }
    }
}

// gemm0: y = act(gate) * up (silu, gelu) or swiglu(gate, up), with the per-token scale sa and the per-channel
// scales folded in; stored as bf16 or (fp8 path) as e4m3 with one power-of-two scale per 32 columns.  Every lane of
// the wave must call it (the fp8 path exchanges the block maximum with lane ^ 32); `store` masks
// the writes.  single: gate-only weights, y = act(gate) (swiglu: act(gate, 1)) and the up operands are ignored.
// col0: first of the lane's 16 output columns = first gate channel; the up channels are n_out + col0 ...
template <int MODE>
__device__ __attribute__((always_inline)) inline void epilogue_gemm0(const GemmParams& p, const typename ModeTraits<MODE>::Acc& acc_gate,
                                      const typename ModeTraits<MODE>::Acc& acc_up, const float (&gs)[16],
                                      const float (&us)[16], float sa, int64_t grow, bool store, int col0, int kg,
                                      bool single = false, int expert = 0)
{
    float y[16];
    const bool extras = p.bias != nullptr || p.n_padded > 0 || p.act == 2; // uniform
    if(extras)
    {
        // stand-alone GEMMs with an expert bias, padded weight rows or the clamped SwiGLU
        float g[16], u[16];
#pragma unroll
        for(int v = 0; v < 16; v++)
        {
            g[v] = static_cast<float>(acc_gate[v]) * (sa * gs[v]);
            u[v] = single ? 1.0f : static_cast<float>(acc_up[v]) * (sa * us[v]);
        }
        bias_and_padding(p, g, expert, col0);
        if(!single)
            bias_and_padding(p, u, expert, p.n_out + col0);
#pragma unroll
        for(int v = 0; v < 16; v++)
        {
            if(p.act == 2)
                y[v] = swiglu(g[v], u[v], p.swiglu_alpha, p.swiglu_limit);
            else
                y[v] = (p.act == 0 ? gelu(g[v]) : silu(g[v])) * u[v];
        }
    }
    else
    {
        // p.act is uniform: one scalar branch
        if(p.act == 0)
        {
#pragma unroll
            for(int v = 0; v < 16; v++)
                y[v] = gelu(static_cast<float>(acc_gate[v]) * (sa * gs[v]));
        }
        else
        {
#pragma unroll
            for(int v = 0; v < 16; v++)
                y[v] = silu(static_cast<float>(acc_gate[v]) * (sa * gs[v]));
        }
        if(!single)
        {
#pragma unroll
            for(int v = 0; v < 16; v++)
                y[v] *= static_cast<float>(acc_up[v]) * (sa * us[v]);
        }
    }
    const bool as_fp8  = MODE == kFp8 && !p.y_bf16;
    const int y_b      = as_fp8 ? 1 : 2;
    unsigned char* dst = p.y_slab > 0 ? p.out + y_slab_offset(grow, col0 * y_b, p.y_slab)
                                      : p.out + grow * p.out_row_bytes + (int64_t)col0 * y_b;
    if(as_fp8)
    {
        float amax = 0.f;
#pragma unroll
        for(int v = 0; v < 16; v++)
            amax = fmaxf(amax, fabsf(y[v]));
        amax = fmaxf(amax, __shfl_xor(amax, 32));
        // scale 2^s with amax / 2^s <= 448 = 1.75 * 2^8; stored as e8m0 (s + 127)
        const uint32_t ab = __float_as_uint(amax);
        int sb            = static_cast<int>(ab >> 23) - 8 + ((ab & 0x7fffffu) > 0x600000u ? 1 : 0);
        sb                = amax == 0.f ? 0 : max(0, min(254, sb));
        const float inv   = __uint_as_float(static_cast<uint32_t>(254 - sb) << 23);
        uint32_t q[4];
#pragma unroll
        for(int v = 0; v < 4; v++)
        {
            const float a0 = fminf(fmaxf(y[4 * v] * inv, -448.f), 448.f);
            const float a1 = fminf(fmaxf(y[4 * v + 1] * inv, -448.f), 448.f);
            const float a2 = fminf(fmaxf(y[4 * v + 2] * inv, -448.f), 448.f);
            const float a3 = fminf(fmaxf(y[4 * v + 3] * inv, -448.f), 448.f);
            int pk         = __builtin_amdgcn_cvt_pk_fp8_f32(a0, a1, 0, false);
            pk             = __builtin_amdgcn_cvt_pk_fp8_f32(a2, a3, pk, true);
            q[v]           = static_cast<uint32_t>(pk);
        }
        if(store)
        {
            *reinterpret_cast<uint4*>(dst) = make_uint4(q[0], q[1], q[2], q[3]);
            if(kg == 0)
                p.y_scale[(int64_t)(col0 >> 5) * p.ys_kb_stride + grow] = static_cast<unsigned char>(sb);
        }
    }
    else if(store)
    {
        uint4 o0, o1;
        o0.x = pack_out2<MODE>(y[0], y[1]);   o0.y = pack_out2<MODE>(y[2], y[3]);
        o0.z = pack_out2<MODE>(y[4], y[5]);   o0.w = pack_out2<MODE>(y[6], y[7]);
        o1.x = pack_out2<MODE>(y[8], y[9]);   o1.y = pack_out2<MODE>(y[10], y[11]);
        o1.z = pack_out2<MODE>(y[12], y[13]); o1.w = pack_out2<MODE>(y[14], y[15]);
        uint4* d4 = reinterpret_cast<uint4*>(dst);
        d4[0]     = o0;
        d4[1]     = o1;
    }
}

// gemm1: * per-channel scale (+ expert bias), bf16 partial row in sorted-row order (the combine applies the top-k weight)
// (sa: per-row scale of a quantised Y, 1 otherwise)
template <int MODE>
__device__ __attribute__((always_inline)) inline void epilogue_gemm1(const GemmParams& p, const typename ModeTraits<MODE>::Acc& acc,
                                      const float (&ds)[16], float sa, int64_t prow, bool store, int col0, int expert = 0)
{
    float y[16];
#pragma unroll
    for(int v = 0; v < 16; v++)
        y[v] = static_cast<float>(acc[v]) * (sa * ds[v]);
    if(p.bias != nullptr || p.n_padded > 0) // uniform: stand-alone down GEMM with a bias or padded rows
        bias_and_padding(p, y, expert, col0);
    uint4 o0, o1;
    o0.x = pack_out2<MODE>(y[0], y[1]);   o0.y = pack_out2<MODE>(y[2], y[3]);
    o0.z = pack_out2<MODE>(y[4], y[5]);   o0.w = pack_out2<MODE>(y[6], y[7]);
    o1.x = pack_out2<MODE>(y[8], y[9]);   o1.y = pack_out2<MODE>(y[10], y[11]);
    o1.z = pack_out2<MODE>(y[12], y[13]); o1.w = pack_out2<MODE>(y[14], y[15]);
    if(store)
    {
        uint4* d4 = reinterpret_cast<uint4*>(p.out + prow * p.out_row_bytes + (int64_t)col0 * 2);
        d4[0]     = o0;
        d4[1]     = o1;
    }
}

// Shared tail of both GEMM kernels, in three parts so that a kernel that walks several tiles can fetch the
// operands early (load), make sure they have arrived at a point of its choosing (pin) and do the arithmetic and
// the stores later (apply).  NBLK token blocks per wave: block i covers sorted rows
// row0 + first_row + i * row_step + r32; wblk is the wave's first 32-row weight block of the tile.
// SKIP_PAD (gemm1): look the sorted id up and do not store partial rows of padding ids - worth the
// load where padding dominates (decode: a handful of real rows per 32-row unit).
template <int NBLK>
struct EpilogueRows
{
    float sa[NBLK];  // per-row scale
    bool real[NBLK]; // the row holds a token (not a padding id)
    int orow[NBLK];  // output row (the launchers keep tokens * topk below 2^31)
};
struct EpilogueColumns
{
    int col_a, col_b; // first output column of the wave's two accumulator groups for this lane
    bool a_ok, b_ok, paired;
};
template <int NBLK>
struct EpilogueOperands
{
    float sc0[16], sc1[16]; // per-channel scales of the wave's two accumulator groups
    EpilogueRows<NBLK> rows;
    EpilogueColumns cols;
};

template <bool GEMM0>
__device__ __attribute__((always_inline)) inline EpilogueColumns epilogue_columns(const GemmParams& p, int n_base, int wblk, int kg)
{
    // gate+up tiles pair weight block 2w (gate) with 2w+1 (up) on the same 32 columns; every other kind of
    // tile (down, gate-only) maps its blocks 2w and 2w+1 to consecutive groups of 32 columns
    EpilogueColumns c;
    c.paired = GEMM0 && !p.gate_only;
    c.col_a  = c.paired ? n_base + wblk * 32 + 16 * kg : n_base + (wblk * 2) * 32 + 16 * kg;
    c.col_b  = c.paired ? c.col_a : c.col_a + 32;
    c.a_ok   = (c.paired ? n_base + wblk * 32 : n_base + wblk * 64) < p.n_out;
    c.b_ok   = c.paired ? c.a_ok : (n_base + wblk * 64 + 32) < p.n_out;
    return c;
}

template <int MODE, bool GEMM0, int NBLK, bool SKIP_PAD>
__device__ __attribute__((always_inline)) inline void load_epilogue_rows(const GemmParams& p, EpilogueRows<NBLK>& o, int row0, int nrows, int first_row,
                                          int row_step, int r32)
{
#pragma unroll
    for(int i = 0; i < NBLK; i++)
    {
        o.sa[i]   = 1.0f;
        o.real[i] = true;
        o.orow[i] = row0 + first_row + i * row_step + r32;
        if((GEMM0 && (p.x_scale != nullptr || p.slot_rows > 0)) || (!GEMM0 && SKIP_PAD))
        {
            const int r   = min(first_row + i * row_step + r32, nrows - 1); // clamped: always a valid cell
            const int sid = p.sorted_ids[row0 + r];
            const int tok = sid & 0xffffff;
            o.real[i]     = tok < p.tokens;
            if constexpr(GEMM0)
            {
                if(p.x_scale != nullptr)
                    o.sa[i] = o.real[i] ? p.x_scale[token_row(p, sid)] : 0.0f;
                if(p.slot_rows > 0)
                    o.orow[i] = o.real[i] ? (int)slot_row(sid, p.slot_rows) : 0;
            }
        }
        if constexpr(!GEMM0 && MODE == kI8)
        {
            // per-row scale of the int8 intermediate activations, in sorted-row order like Y itself
            const int r = min(first_row + i * row_step + r32, nrows - 1);
            o.sa[i]     = p.x_scale[row0 + r];
        }
    }
}

template <int NBLK>
__device__ __attribute__((always_inline)) inline void pin_epilogue_rows(EpilogueRows<NBLK>& o)
{
#pragma unroll
    for(int i = 0; i < NBLK; i++)
    {
        int real = o.real[i];
        asm volatile("" : "+v"(o.sa[i]), "+v"(o.orow[i]), "+v"(real));
        o.real[i] = real != 0;
    }
}

template <int MODE, bool GEMM0, int NBLK, bool SKIP_PAD>
__device__ __attribute__((always_inline)) inline void load_epilogue(const GemmParams& p, EpilogueOperands<NBLK>& o, int expert, int row0, int nrows,
                                     int first_row, int row_step, int n_base, int wblk, int r32, int kg)
{
    o.cols             = epilogue_columns<GEMM0>(p, n_base, wblk, kg);
    const float* sbase = p.w_scale ? p.w_scale + (int64_t)expert * p.n_total : nullptr;
    load_channel_scales(sbase && o.cols.a_ok ? sbase + o.cols.col_a : nullptr, o.sc0);
    load_channel_scales(sbase && o.cols.b_ok ? sbase + (o.cols.paired ? p.n_out + o.cols.col_a : o.cols.col_b) : nullptr,
                        o.sc1);
    load_epilogue_rows<MODE, GEMM0, NBLK, SKIP_PAD>(p, o.rows, row0, nrows, first_row, row_step, r32);
}

// Every load of load_epilogue completes here, on every path: a load left pending on a path that does not use
// its result would make the compiler guard later register reuse with a wait for all vector memory
// operations - inside the caller's K loop when the caller walks several tiles.
template <int NBLK>
__device__ __attribute__((always_inline)) inline void pin_epilogue(EpilogueOperands<NBLK>& o)
{
#pragma unroll
    for(int v = 0; v < 16; v++)
        asm volatile("" : "+v"(o.sc0[v]), "+v"(o.sc1[v]));
    pin_epilogue_rows(o.rows);
}

// one token block of a wave: scales, activation, packing, stores
template <int MODE, bool GEMM0, int NBLK>
__device__ __attribute__((always_inline)) inline void apply_epilogue_block(const GemmParams& p, typename ModeTraits<MODE>::Acc (&acc)[2],
                                            const float (&sc0)[16], const float (&sc1)[16], const EpilogueRows<NBLK>& rows,
                                            const EpilogueColumns& c, int i, int row0, int nrows, int first_row,
                                            int row_step, int r32, int kg, int expert)
{
    const int r = first_row + i * row_step + r32;
    if constexpr(GEMM0)
    {
        const bool st = r < nrows && (p.slot_rows == 0 || rows.real[i]);
        if(c.a_ok)
            epilogue_gemm0<MODE>(p, acc[0], acc[1], sc0, sc1, rows.sa[i], rows.orow[i], st, c.col_a, kg, !c.paired, expert);
        if(!c.paired && c.b_ok) // gate-only tile: the second accumulator holds the next 32 gate columns
            epilogue_gemm0<MODE>(p, acc[1], acc[1], sc1, sc1, rows.sa[i], rows.orow[i], st, c.col_b, kg, true, expert);
    }
    else
    {
        const bool in_tile = r < nrows;
        if(c.a_ok)
            epilogue_gemm1<MODE>(p, acc[0], sc0, rows.sa[i], row0 + r, in_tile && rows.real[i], c.col_a, expert);
        if(c.b_ok)
            epilogue_gemm1<MODE>(p, acc[1], sc1, rows.sa[i], row0 + r, in_tile && rows.real[i], c.col_b, expert);
    }
}

template <int MODE, bool GEMM0, int NBLK>
__device__ __attribute__((always_inline)) inline void apply_epilogue(const GemmParams& p, typename ModeTraits<MODE>::Acc (&acc)[NBLK][2],
                                      const EpilogueOperands<NBLK>& o, int row0, int nrows, int first_row, int row_step,
                                      int nblk_live, int r32, int kg, int expert)
{
    // block by block, so that a block's accumulators are dead before the next block's temporaries
    // are needed (the large-tile kernel has no registers to spare)
#pragma unroll
    for(int i = 0; i < NBLK; i++)
    {
        if(i >= nblk_live)
            continue;
        apply_epilogue_block<MODE, GEMM0, NBLK>(p, acc[i], o.sc0, o.sc1, o.rows, o.cols, i, row0, nrows, first_row, row_step,
                                                r32, kg, expert);
    }
}

template <int MODE, bool GEMM0, int NBLK, bool SKIP_PAD>
__device__ __attribute__((always_inline)) inline void run_epilogue(const GemmParams& p, typename ModeTraits<MODE>::Acc (&acc)[NBLK][2], int expert,
                                    int row0, int nrows, int first_row, int row_step, int nblk_live, int n_base,
                                    int wblk, int r32, int kg)
{
    EpilogueOperands<NBLK> o;
    load_epilogue<MODE, GEMM0, NBLK, SKIP_PAD>(p, o, expert, row0, nrows, first_row, row_step, n_base, wblk, r32, kg);
    pin_epilogue(o);
    apply_epilogue<MODE, GEMM0, NBLK>(p, acc, o, row0, nrows, first_row, row_step, nblk_live, r32, kg, expert);
}

} // namespace gemm
} // namespace mi355
