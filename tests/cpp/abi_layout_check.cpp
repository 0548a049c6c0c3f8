// Compile-time check that the C ABI's argument blocks are the ck_tile host argument blocks: same size, same
// field offsets, so a pointer to one can be handed over as the other.  Compiled (never run) by
// tests/test_capi.py with hipcc's host pass; where the ck_tile headers are not installed the check is empty.
#include <cstring> // ck_tile's headers use std::memcpy without including it
#include <cstddef>

#include "../../include/mi355_moe.h"

#if __has_include(<ck_tile/ops/fused_moe/kernel/fused_moegemm_kernel.hpp>) && \
    __has_include(<ck_tile/ops/fused_moe/kernel/moe_sorting_kernel.hpp>)
#include <ck_tile/core.hpp>
#include <ck_tile/ops/fused_moe/kernel/fused_moegemm_kernel.hpp>
#include <ck_tile/ops/fused_moe/kernel/moe_sorting_kernel.hpp>
#define MI355_HAVE_CK_TILE 1

#define SAME_FIELD(mine, theirs, field)                                                             \
    static_assert(offsetof(mine, field) == offsetof(theirs, field), #mine "." #field ": offset differs"); \
    static_assert(sizeof(((mine*)nullptr)->field) == sizeof(((theirs*)nullptr)->field), #mine "." #field ": size differs")

// ---- FusedMoeGemmHostArgs (ops/fused_moe/kernel/fused_moegemm_kernel.hpp:97-120)
static_assert(sizeof(mi355_fused_moegemm_args) == sizeof(ck_tile::FusedMoeGemmHostArgs), "FusedMoeGemmHostArgs: size");
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, a_ptr);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, a_scale_ptr);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, g_ptr);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, d_ptr);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, g_scale_ptr);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, d_scale_ptr);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, y_smooth_scale_ptr);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, o_ptr);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, sorted_token_ids_ptr);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, sorted_weight_ptr);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, sorted_expert_ids_ptr);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, num_sorted_tiles_ptr);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, hidden_size);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, intermediate_size);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, num_tokens);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, num_experts);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, topk);
SAME_FIELD(mi355_fused_moegemm_args, ck_tile::FusedMoeGemmHostArgs, stride_token);

// ---- MoeSortingHostArgs (ops/fused_moe/kernel/moe_sorting_kernel.hpp:188-222)
static_assert(sizeof(mi355_moe_sorting_args) == sizeof(ck_tile::MoeSortingHostArgs), "MoeSortingHostArgs: size");
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, p_topk_ids);
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, p_weights);
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, p_local_expert_mask);
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, p_local_tokens);
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, p_sorted_token_ids);
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, p_sorted_weights);
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, p_sorted_expert_ids);
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, p_total_tokens_post_pad);
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, p_moe_buf);
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, p_ws);
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, tokens);
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, unit_size);
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, num_experts);
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, topk);
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, moe_buf_interm_dim);
SAME_FIELD(mi355_moe_sorting_args, ck_tile::MoeSortingHostArgs, moe_buf_elem_bytes);
#else
#define MI355_HAVE_CK_TILE 0
#endif

// read by the test that compiles this file: 1 = the assertions above were compiled
extern "C" const int mi355_abi_layout_checked = MI355_HAVE_CK_TILE;
