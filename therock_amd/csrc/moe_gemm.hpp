// Host-side declarations of the grouped-GEMM half of libmi355_moe.so.
#pragma once

#include "common.hpp"

namespace mi355 {

// Carving of the caller's workspace (all offsets 256-byte aligned).
struct WorkspaceLayout
{
    size_t sort_off;   // moe_sorting segment counters
    size_t map_off;    // int32 [4 + 8 * max_tiles]: live tile count, then one entry per M tile
    size_t inv_off;    // int32 [tokens * topk]: sorted position of the (token, slot) entry, -1 when dropped
    size_t y_off;      // intermediate activations Y [max_pad, inter] (bf16 or e4m3)
    size_t ys_off;     // e8m0 block scales of Y [inter / 32][ys_kb_stride] (fp8 path only)
    int64_t ys_kb_stride;
    size_t yq_off;     // int8 (e4m3) copy of Y [max_pad, inter] and ...
    size_t yrs_off;    // ... its fp32 per-row scales [max_pad] (int8 and fp8 paths with fused_quant 1 / 2 only)
    size_t p_off;      // partial outputs per sorted row [max_pad, hidden] bf16
    size_t total;
    int64_t max_pad;
    int32_t max_tiles; // upper bound of M tiles
};

int check_traits(const mi355_fused_moe_traits& t);

WorkspaceLayout workspace_layout(const mi355_fused_moe_traits& t, int32_t tokens, int32_t experts,
                                 int32_t topk, int32_t hidden, int32_t inter);

// sorted rows per GEMM workgroup at this problem size
// the second tile height the sort may choose on the device for this problem (0: none)
int gemm_alt_tile_rows(const mi355_fused_moe_traits& t, int32_t tokens, int32_t experts, int32_t topk, int32_t hidden,
                       int32_t inter);
int gemm_tile_rows(const mi355_fused_moe_traits& t, int32_t tokens, int32_t experts, int32_t topk, int32_t hidden,
                   int32_t inter);

// true when the sizes are ones the path can index (24-bit token ids, 8-bit slots, at most 1024 experts)
bool sizes_in_range(int32_t tokens, int32_t experts, int32_t topk, int32_t hidden, int32_t inter);

// host-side checks of launch_fused_moegemm, launching nothing
int validate_fused_moegemm(const mi355_fused_moe_traits& t, const mi355_fused_moegemm_args& a, const void* ws_ptr,
                           size_t ws_bytes);

// prep_done: the tile list and the inverse map were already written by the sort (GemmPlan)
int launch_fused_moegemm(const mi355_fused_moe_traits& t, const mi355_fused_moegemm_args& a, void* ws_ptr,
                         size_t ws_bytes, hipStream_t stream, bool prep_done = false);

// the plan the sort has to fill for launch_fused_moegemm(..., prep_done = true)
GemmPlan make_gemm_plan(const mi355_fused_moe_traits& t, void* ws_ptr, int32_t tokens, int32_t experts,
                        int32_t topk, int32_t hidden, int32_t inter);

namespace gemm {
struct GemmParams;
}
// large-tile kernel (moe_gemm_big.hip)
int big_tile_rows();
// (y_i8: the down GEMM of the int8 path reads int8 Y with per-row scales instead of bf16 Y)
bool big_tile_supported(int prec, int k_bytes0, int k_bytes1, bool y_i8 = false);
int launch_gemm_big(int prec, bool gemm0, const gemm::GemmParams& p, int max_tiles, hipStream_t stream, bool y_i8 = false);

// decode kernel (moe_gemm_decode.hip): tiles of `blocks` (1 or 2) 32-row blocks x decode_tile_cols() output columns
int decode_tile_cols(bool gemm0);
bool decode_supported(int64_t x_bytes, int64_t y_bytes, int64_t w_expert_bytes);
int launch_gemm_decode(int prec, bool gemm0, int blocks, const gemm::GemmParams& p, int max_tiles, hipStream_t stream,
                       bool y_i8 = false);

size_t moe_flatmm_workspace_bytes(int kind, const mi355_moe_flatmm_args& a);
int launch_moe_flatmm(int kind, const mi355_moe_flatmm_args& a, void* ws_ptr, size_t ws_bytes, hipStream_t stream);

int launch_permute_weights(const void* src, void* dst, int32_t experts, int32_t n, int32_t k, int32_t elem_bytes,
                           int32_t nw, int32_t kw, int32_t kv, int32_t inverse, hipStream_t stream);

int launch_moe_smoothquant(const mi355_moe_smoothquant_args& a, int32_t q_dtype, hipStream_t stream);

// int8 re-quantisation of the sorted rows of Y between the two GEMMs (smooth: [experts, inter] or null;
// total[0] = rows of the sorted prefix; segs > 0: slab-major output)
int launch_requant_y(const void* y, int32_t inter, const float* smooth, const int* sorted_ids, const int* sorted_expert_ids,
                     const int* total, int32_t unit, int32_t tokens, int32_t segs, int64_t max_rows, void* yq, float* yscale,
                     hipStream_t stream, bool fp8 = false);

int launch_rowwise_quant(const void* x, int64_t rows, int32_t cols, int64_t stride_x, int32_t q_dtype,
                         void* q, void* scale, hipStream_t stream);

} // namespace mi355
