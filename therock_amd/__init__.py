"""MI355X-native fused-MoE inference path (moe_sorting + gate/up GEMM with SiLU*up + down GEMM with
top-k combine), a drop-in for Composable Kernel's ck_tile fused_moe host API.  The compute lives in
libmi355_moe.so (hand-written HIP for gfx950, C ABI in include/mi355_moe.h); this package is the
host-side mirror of the CK example API plus the synthetic-input harness."""
from .moe import (ACT_SILU, ACT_SWIGLU, GEMM1_GATE_ONLY, GEMM1_GATE_UP, GEMM2, MoeBuffers, fused_moe, fused_moe_args, fused_moe_get_workspace_size, fused_moe_static_ws, fused_moe_static_ws_capacity, fused_moe_chosen_tile_rows, fused_moe_tile_rows, fused_moe_traits,  # noqa: F401
                  fused_moegemm, make_args, moe_max_num_tokens_padded, moe_sorting, moe_sorting_args,
                  moe_flatmm, moe_flatmm_get_workspace_size, moe_smoothquant, moe_sorting_get_workspace_size, moe_sorting_trait, permute_weights, rowwise_quant,
                  topk_softmax)
