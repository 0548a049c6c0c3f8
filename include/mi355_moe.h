/*
 * mi355_moe.h - C ABI of the MI355X-native fused-MoE path (libmi355_moe.so).
 *
 * Every entry point takes plain pointers and sizes; all data pointers are DEVICE pointers owned by
 * the caller, launches are asynchronous on the given HIP stream (passed as void*, NULL = default
 * stream) and nothing is allocated behind the caller's back.  The structs mirror the host argument
 * blocks of Composable Kernel's ck_tile fused-MoE (ck_tile 1.2.0, paths relative to
 * /opt/rocm/include/ck_tile):
 *
 *   mi355_moe_sorting_args   == MoeSortingHostArgs    ops/fused_moe/kernel/moe_sorting_kernel.hpp:188-222
 *   mi355_fused_moegemm_args == FusedMoeGemmHostArgs  ops/fused_moe/kernel/fused_moegemm_kernel.hpp:97-120
 *   mi355_fused_moe_args     <- fused_moe_args  of CK's example/ck_tile/15_fused_moe/fused_moe.hpp
 *   mi355_fused_moe_traits   <- fused_moe_traits of the same example, with enums for its strings
 *
 * The first two have the same fields at the same offsets as the ck_tile structs (a pointer to one can
 * be cast to the other; tests/cpp/abi_layout_check.cpp asserts it against the ck_tile headers).  What
 * this library needs beyond them - device memory for the intermediate activations - travels beside the
 * argument block as a mi355_moe_workspace.
 *
 * Return value of every int function: 0 on success, negative on failure (MI355_MOE_E_*);
 * mi355_moe_last_error() returns a human-readable description for the calling thread.
 */
#ifndef MI355_MOE_H
#define MI355_MOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 210: mi355_fused_moe_traits gained weight_permute and mi355_moe_flatmm_args gained b_shuffle (both appended; a
 * caller built against 200 must be rebuilt), mi355_fused_moe_chosen_tile_rows added */
#define MI355_MOE_VERSION 220

enum mi355_moe_status
{
    MI355_MOE_OK            = 0,
    MI355_MOE_E_UNSUPPORTED = -1, /* no kernel for these traits (ck_tile's fused_moe() returns -1 too) */
    MI355_MOE_E_INVALID     = -2, /* null pointer, size out of range, misaligned stride ... */
    MI355_MOE_E_HIP         = -3, /* a HIP runtime call failed */
    MI355_MOE_E_WORKSPACE   = -4  /* workspace missing or too small */
};

/* element types; the strings are the spellings of ck_tile's traits ("bf16", "fp8", "int8", ...) */
enum mi355_moe_dtype
{
    MI355_MOE_BF16 = 0,
    MI355_MOE_FP8  = 1, /* OCP e4m3 */
    MI355_MOE_INT8 = 2,
    MI355_MOE_FP32 = 3,
    MI355_MOE_INT32 = 4,
    MI355_MOE_FP16 = 5
};

/* Device memory the GEMM entry points use for their intermediates (tile list, the activations between
 * the two GEMMs, per-slot partial outputs).  ck_tile's fused kernel needs none, so it is not part of
 * the argument blocks: it is passed beside them.  ptr: 256-byte aligned device memory of at least the
 * size the matching *_workspace_size() function returns; it need not be cleared, and holds nothing
 * between calls.  Calls that share a workspace must not overlap. */
typedef struct mi355_moe_workspace
{
    void* ptr;
    size_t bytes;
} mi355_moe_workspace;

/* ------------------------------------------------------------------------------ moe_sorting
 * Replaces ck_tile::MoeSortingKernel / MoeSortingMultiPhaseKernel_* behind MoeSortingHostArgs
 * (moe_sorting_kernel.hpp:188-222) and the example's moe_sorting(trait, args, stream).
 * Output contract = ck_tile::reference_moe_sorting (host/reference/reference_moe_sorting.hpp:14-117)
 * with skip_experts_with_zero_token = true: cells past the written prefix are left untouched. */
typedef struct mi355_moe_sorting_args
{
    const void* p_topk_ids;          /* [tokens, topk] int32, distinct experts per token */
    const void* p_weights;           /* [tokens, topk] fp32 */
    const void* p_local_expert_mask; /* [num_experts] int32 or NULL; 0 = expert not on this rank */
    const void* p_local_tokens;      /* [1] int32 or NULL; if set, the token count is read on device */
    void* p_sorted_token_ids;        /* [max_num_tokens_padded] int32: token | topk_slot << 24 */
    void* p_sorted_weights;          /* [max_num_tokens_padded] fp32 */
    void* p_sorted_expert_ids;       /* [ceil(max_num_tokens_padded / unit_size)] int32 */
    void* p_total_tokens_post_pad;   /* [2] int32: [0] tokens after padding, [1] actual tokens */
    void* p_moe_buf;                 /* buffer to zero alongside the sort, or NULL */
    void* p_ws;                      /* mi355_moe_sorting_workspace_size() bytes (may be NULL if 0);
                                        unlike ck_tile it need not be cleared */
    int32_t tokens;                  /* token count, or its upper bound when p_local_tokens is set */
    int32_t unit_size;               /* block_m of the GEMM that consumes the result */
    int32_t num_experts;
    int32_t topk;
    int32_t moe_buf_interm_dim;      /* p_moe_buf is [tokens, moe_buf_interm_dim] elements ... */
    int32_t moe_buf_elem_bytes;      /* ... of this many bytes; a row must be a multiple of 16 B */
} mi355_moe_sorting_args;

/* max_num_tokens_padded = topk*tokens + num_experts*unit_size - topk (moe_sorting_kernel.hpp:64) */
int64_t mi355_moe_max_num_tokens_padded(int32_t tokens, int32_t num_experts, int32_t topk, int32_t unit_size);

/* replaces moe_sorting_get_workspace_size() (moe_sorting_kernel.hpp:1394-1438) */
size_t mi355_moe_sorting_workspace_size(int32_t tokens, int32_t num_experts, int32_t topk);

/* the same with ck_tile's fourth argument (moe_sorting_kernel.hpp:1407-1438): dispatch_policy 0 = the library picks
 * the kernel (what the three-argument form returns), 1 = always the single kernel (0 bytes), 2 = always the
 * multi-launch passes; other values return 0 */
size_t mi355_moe_sorting_workspace_size2(int32_t tokens, int32_t num_experts, int32_t topk, int32_t dispatch_policy);

/* replaces moe_sorting(moe_sorting_trait, moe_sorting_args, stream_config) of CK's
 * example/ck_tile/13_moe_sorting; index type int32 and weight type fp32 are the only ones CK has */
int mi355_moe_sorting(const mi355_moe_sorting_args* args, void* stream);

/* moe_sorting_trait of CK's example/ck_tile/13_moe_sorting (enums for its strings) plus the one switch of
 * MoeSortingProblemEx / MoeSortingProblemMp that changes the output (moe_sorting_problem.hpp:35,60). */
typedef struct mi355_moe_sorting_traits
{
    int32_t index_type;                 /* mi355_moe_dtype: INT32 */
    int32_t weight_type;                /* FP32 */
    int32_t local_expert_masking;       /* 0: p_local_expert_mask is ignored */
    int32_t clear_workspace_inside_api; /* accepted; the workspace never needs clearing here */
    int32_t dispatch_policy;            /* 0 | 1 | 2 as for mi355_moe_sorting_workspace_size2; with 1 p_ws may be NULL
                                           whatever the size (one workgroup then walks the whole routing list) */
    int32_t skip_experts_with_zero_tokens; /* 1 = ck_tile's default.  0: an expert of this rank that no token chose
                                           still owns one unit of padding ids and its expert id in the outputs
                                           (reference_moe_sorting's skip_experts_with_zero_token = false); the
                                           output arrays then need topk*tokens + num_experts*unit_size cells */
} mi355_moe_sorting_traits;

/* mi355_moe_sorting with traits; returns MI355_MOE_E_UNSUPPORTED for index / weight types ck_tile has no kernel for */
int mi355_moe_sorting2(const mi355_moe_sorting_traits* traits, const mi355_moe_sorting_args* args, void* stream);

/* ----------------------------------------------------------------------------- topk_softmax
 * Router front-end.  Replaces ck_tile::TopkSoftmaxKernel behind TopkSoftmaxHostArgs
 * (ops/topk_softmax/kernel/topk_softmax_kernel.hpp:15-25): softmax (or sigmoid) over the expert
 * logits of every row, then the topk largest values in descending order with their expert ids.
 * Output contract = ck_tile::reference_softmax + reference_topk (host/reference/reference_softmax.hpp:12-78,
 * host/reference/reference_topk.hpp:30-103), fp32; equal values are ordered by expert id. */
typedef struct mi355_topk_softmax_args
{
    const void* p_input;   /* [num_rows, stride_input] logits */
    void* p_output;        /* [num_rows, stride_output] fp32 weights of the chosen experts */
    void* p_indices;       /* [num_rows, stride_output] int32 expert ids */
    int32_t num_rows;
    int32_t num_experts;   /* at most 1024 */
    int32_t topk;          /* at most 64 */
    int32_t stride_input;  /* row stride of p_input in elements, at least num_experts */
    int32_t stride_output; /* row stride of p_output / p_indices in elements, at least topk */
} mi355_topk_softmax_args;

/* topk_softmax_trait of CK's example/ck_tile/09_topk_softmax, enums for its strings */
typedef struct mi355_topk_softmax_traits
{
    int32_t input_type;  /* mi355_moe_dtype: FP32 | BF16 | FP16 (ck_tile's kernel is generic over InputType,
                            topk_softmax_kernel.hpp:33); the arithmetic is fp32 for all three */
    int32_t weight_type; /* FP32 */
    int32_t experts;     /* CK selects an instance by this upper bound; here informational */
    int32_t activation;  /* 0 = softmax, 1 = sigmoid (TopkSoftmaxWarpPerRowProblem::ActivationIsSoftmax) */
    int32_t renormalize; /* extension, 0 in CK: 1 = divide the chosen weights by their sum */
} mi355_topk_softmax_traits;

int mi355_topk_softmax(const mi355_topk_softmax_traits* traits, const mi355_topk_softmax_args* args, void* stream);

/* ------------------------------------------------------------------------------- fused MoE */
typedef struct mi355_fused_moe_traits
{
    int32_t prec_i;  /* activation dtype  (mi355_moe_dtype): BF16 | FP16 | FP8 | INT8 */
    int32_t prec_w;  /* weight dtype: same as prec_i */
    int32_t prec_o;  /* output dtype: BF16; FP16 with FP16 operands (ck_tile's two instances,
                        fused_moegemm_pipeline_flatmm_policy.hpp:790-807) */
    int32_t prec_st; /* per-token activation scale dtype: FP32 */
    int32_t prec_sw; /* per-channel weight scale dtype: FP32 */
    int32_t prec_sq; /* smooth-quant scale dtype: FP32 (unused) */
    int32_t prec_kw; /* top-k weight dtype: FP32 */
    int32_t block_m; /* rows per sorted tile = unit_size of the sort: 16, 32, 64 or 128 */
    int32_t activation;  /* 0 = gelu (erf form, ck_tile::element_wise::Gelu), 1 = silu */
    int32_t gate_only;   /* 0 = gate and up (g [e, 2*inter, hidden]), 1 = gate only (g [e, inter, hidden], y = act(gate)) */
    int32_t fused_quant; /* 0 = none (quantised dtypes always take a_scale/g_scale/d_scale; the int8 path keeps the
                            intermediate activations in bf16, the fp8 path rounds them to e4m3 with a power-of-two
                            scale per 32 columns inside the gate+up GEMM).  INT8 and FP8: 2 = dynamic-quant, the
                            intermediate activations are re-quantised to int8 (e4m3) with one fp32 scale per row in a
                            pass between the GEMMs and the down GEMM runs on int8 (fp8) MFMAs; 1 =
                            smooth-dynamic-quant, the same after a multiplication by y_smooth_scale[expert], and the
                            activations arrive as MoeSmoothquant leaves them: one quantised row per (slot, token),
                            a [topk, tokens, stride_token], a_scale [topk, tokens]
                            (UseSmoothQuant of fused_moegemm_traits.hpp:19-35; layouts moe_sorting_kernel.hpp:82-83) */
    int32_t local_expert_masking; /* 1 = apply local_expert_mask_ptr in the sort */
    int32_t weight_permute; /* layout of g and d, FusedMoeGemmWeightPermuteEnum (fused_moegemm_traits.hpp:10-17; a
                               template argument of ck_tile's kernel, not a field of its example's traits): 0 =
                               no_permute, rows of K elements as ck_tile's host reference takes them; 1 =
                               b_nr_kr_kw_nw_kv, what ck_tile's device kernel takes and its example produces before
                               the call: [e, n/16, k/(4 kv), 4, 16, kv] with kv = 16 bytes of elements (8 for bf16 and
                               fp16, 16 for fp8 and int8); needs K rows that are multiples of 64 bytes.  The kernels
                               read either layout in place (mi355_moe_permute_weights converts between them) */
} mi355_fused_moe_traits;

/* FusedMoeGemmHostArgs (fused_moegemm_kernel.hpp:97-120), field for field.  g and d in the layout that
 * mi355_fused_moe_traits.weight_permute names: rows of K elements (what ck_tile's host reference takes) or
 * ck_tile's pre-shuffled b_nr_kr_kw_nw_kv (what its device kernel takes; fused_moegemm_traits.hpp:10-17). */
typedef struct mi355_fused_moegemm_args
{
    const void* a_ptr;              /* [tokens, stride_token] activations ([topk, tokens, stride_token] with fused_quant 1) */
    const void* a_scale_ptr;        /* [tokens] fp32 per-token scale (quantised dtypes; [topk, tokens] with fused_quant 1) or NULL */
    const void* g_ptr;              /* [experts, 2*inter, hidden] gate rows then up rows; gate_only: [experts, inter, hidden] */
    const void* d_ptr;              /* [experts, hidden, inter] */
    const void* g_scale_ptr;        /* [experts, 2*inter] ([experts, inter] when gate_only) fp32 or NULL */
    const void* d_scale_ptr;        /* [experts, hidden] fp32 or NULL */
    const void* y_smooth_scale_ptr; /* [experts, inter] fp32, 16-byte aligned: with fused_quant 1 and only then, else NULL */
    void* o_ptr;                    /* [tokens, stride_token] output, written (not accumulated) */
    const void* sorted_token_ids_ptr;  /* as written by mi355_moe_sorting */
    const void* sorted_weight_ptr;
    const void* sorted_expert_ids_ptr;
    const void* num_sorted_tiles_ptr;  /* [>=1] int32: [0] holds tokens_post_pad (:243-246) */
    int32_t hidden_size;
    int32_t intermediate_size;
    int32_t num_tokens;
    int32_t num_experts;
    int32_t topk;
    int32_t stride_token;           /* elements between rows of a and of o (>= hidden_size) */
} mi355_fused_moegemm_args;

/* fused_moe_args of CK's example (example/ck_tile/15_fused_moe/fused_moe.hpp): the GEMM arguments plus
 * routing inputs, sort outputs and the sort's workspace, in the example's order */
typedef struct mi355_fused_moe_args
{
    const void* a_ptr;
    const void* a_scale_ptr;
    const void* g_ptr;
    const void* d_ptr;
    const void* g_scale_ptr;
    const void* d_scale_ptr;
    const void* y_smooth_scale_ptr;
    const void* local_expert_mask_ptr; /* [experts] int32, used when traits.local_expert_masking */
    void* o_ptr;
    void* ws_ptr;                      /* the example's sort workspace: accepted and never touched (it comes without
                                          a size; the sort's counters live in the mi355_moe_workspace); may be NULL */
    const void* topk_ids_ptr;          /* [tokens, topk] int32 */
    const void* topk_weight_ptr;       /* [tokens, topk] fp32 */
    void* sorted_token_ids_ptr;        /* outputs of the sort, sized as for mi355_moe_sorting */
    void* sorted_weight_ptr;
    void* sorted_expert_ids_ptr;
    void* num_sorted_tiles_ptr;        /* [2] int32 */
    int32_t block_m;
    int32_t hidden_size;
    int32_t intermediate_size;
    int32_t num_tokens;
    int32_t num_experts;
    int32_t topk;
    int32_t stride_token;
} mi355_fused_moe_args;

/* 1 if a kernel exists for these traits, else 0 (ck_tile's dispatcher returns -1 from fused_moe) */
int mi355_fused_moe_supported(const mi355_fused_moe_traits* traits);

/* bytes of the mi355_moe_workspace for mi355_fused_moe / mi355_fused_moegemm (includes the sort's own
 * workspace); 0 for unsupported traits or sizes out of range */
size_t mi355_fused_moe_workspace_size(const mi355_fused_moe_traits* traits, int32_t tokens,
                                      int32_t num_experts, int32_t topk, int32_t hidden_size,
                                      int32_t intermediate_size);

/* sorted rows one GEMM workgroup owns at this problem size: 32, 64 or 128 (moe_gemm_kernel) or 320
 * (moe_gemm_big_kernel); 0 for unsupported traits.  The counterpart of Block_M0 of the instance
 * ck_tile's dispatcher selects (fused_moegemm_shape.hpp:43-64); here it is chosen per problem size. */
int32_t mi355_fused_moe_tile_rows(const mi355_fused_moe_traits* traits, int32_t tokens, int32_t num_experts,
                                  int32_t topk, int32_t hidden_size, int32_t intermediate_size);

/* For harnesses and tests: the tile height the last mi355_fused_moe or mi355_fused_moegemm call on `ws` ran with.  Where
 * the routing decides (fp8 operands below about 28 rows per expert on average: a skewed batch whose active experts hold
 * 48 padded rows or more each runs on the 320-row tiles, chosen on the device by the pass that builds the work list: the
 * sort, or the GEMM entry point's own pass over sorted_expert_ids) the value is read back from the work list
 * in `ws`, after synchronising `stream`; everywhere else it is mi355_fused_moe_tile_rows().  No counterpart in ck_tile. */
int32_t mi355_fused_moe_chosen_tile_rows(const mi355_fused_moe_traits* traits, int32_t tokens, int32_t num_experts,
                                         int32_t topk, int32_t hidden_size, int32_t intermediate_size,
                                         const mi355_moe_workspace* ws, void* stream);

/* replaces fused_moegemm(traits, args, stream): FusedMoeGemmKernel (fused_moegemm_kernel.hpp:238-259).
 * Gate+up GEMM with SiLU*up, down GEMM, top-k weighted combine into o. */
int mi355_fused_moegemm(const mi355_fused_moe_traits* traits, const mi355_fused_moegemm_args* args,
                        const mi355_moe_workspace* ws, void* stream);

/* replaces fused_moe(traits, args, stream) of CK's example: mi355_moe_sorting then
 * mi355_fused_moegemm on one stream */
int mi355_fused_moe(const mi355_fused_moe_traits* traits, const mi355_fused_moe_args* args,
                    const mi355_moe_workspace* ws, void* stream);

/* The same pass with no workspace argument, for callers that cannot allocate device memory (code under HIP graph
 * capture, serving loops, harnesses that forbid hipMalloc) and have no workspace to pass.  It has no counterpart
 * in ck_tile, whose fused kernel needs no workspace.  The intermediates live in a buffer of
 * mi355_fused_moe_static_ws_capacity() bytes (96 MiB, enough for the decode regime: 256 tokens of a 128-expert
 * top-8 layer with hidden 4096 and intermediate 1536) that is part of the library's device image: every GPU the
 * library runs on holds it from the first use of the library until the process ends.  Nothing is allocated or
 * freed by the call.  A problem whose mi355_fused_moe_workspace_size() exceeds the capacity is rejected with
 * MI355_MOE_E_WORKSPACE.  All calls on one GPU share the buffer: calls that overlap on one GPU (two streams, two
 * threads) race; calls on one stream are ordered and safe.  The buffer's device address is looked up on the first
 * call on each device (not a stream operation; make that first call outside a capture). */
size_t mi355_fused_moe_static_ws_capacity(void);
int mi355_fused_moe_static_ws(const mi355_fused_moe_traits* traits, const mi355_fused_moe_args* args, void* stream);

/* per-row dynamic quantisation of bf16 activations, the step in front of the quantised path:
 * scale[m] = amax(row)/qmax, q = convert(saturate(x/scale)) (host/reference/reference_rowwise_quantization2d.hpp:12-31);
 * as in ck_tile the int8 conversion truncates toward zero (core/numeric/int8.hpp:101), e4m3 rounds to nearest even;
 * a row of zeros gets scale 1 and codes 0.
 * x [rows, stride_x] bf16 -> q [rows, cols] (FP8 or INT8), scale [rows] fp32. */
int mi355_moe_rowwise_quant(const void* x, int64_t rows, int32_t cols, int64_t stride_x, int32_t q_dtype,
                            void* q, void* scale, void* stream);

/* MoE smooth-quant in front of the int8 / fp8 path.  Replaces ck_tile::MoeSmoothquant behind
 * MoeSmoothquantHostArgs (ops/smoothquant/kernel/moe_smoothquant_kernel.hpp:12-27): for slot k of token t
 * routed to expert e = topk_ids[t, k]: y = x[t, :] * smscale[e, :] (fp32), yscale[k * tokens + t] =
 * amax|y| / qmax, qy[k * tokens + t, :] = convert(saturate(y / yscale))
 * (ops/smoothquant/pipeline/smoothquant_pipeline_one_pass.hpp:73-118).  A row of zeros gets yscale 0 and codes 0
 * (ck_tile converts 0 / 0 there, which is undefined). */
typedef struct mi355_moe_smoothquant_args
{
    const void* p_x;        /* [tokens, x_stride] bf16 */
    const void* p_smscale;  /* [experts, hidden_size] fp32 column-wise smooth scale */
    const void* p_topk_ids; /* [tokens, topk] int32 */
    void* p_yscale;         /* [topk * tokens] fp32 row-wise quantisation scale */
    void* p_qy;             /* [topk * tokens, y_stride] int8 or e4m3 */
    int32_t tokens;
    int32_t hidden_size;
    int32_t experts;
    int32_t topk;
    int32_t x_stride; /* row stride of x in elements */
    int32_t y_stride; /* row stride of qy in elements */
} mi355_moe_smoothquant_args;

int mi355_moe_smoothquant(const mi355_moe_smoothquant_args* args, int32_t q_dtype, void* stream);

/* Load-time layout tool for checkpoints that were pre-shuffled for ck_tile's device kernel
 * (FusedMoeGemmWeightPermuteEnum::b_nr_kr_kw_nw_kv, ops/fused_moe/pipeline/fused_moegemm_traits.hpp:10-17):
 * the row-major weight [experts, n, k] viewed as [experts, n/nw, nw, k/(kw*kv), kw, kv] and permuted with
 * (0, 1, 3, 4, 2, 5) (host/reference/reference_permute.hpp:20-57).  inverse = 0 produces that layout from
 * row-major, inverse = 1 turns it back into the row-major layout this library's GEMMs take.  CK's example
 * uses nw = 16, kw = 4 with kv = 8 for 16-bit and kv = 16 for 8-bit weights.  src and dst must not overlap. */
int mi355_moe_permute_weights(const void* src, void* dst, int32_t experts, int32_t n, int32_t k, int32_t elem_bytes,
                              int32_t nw, int32_t kw, int32_t kv, int32_t inverse, void* stream);

/* ------------------------------------------------------------------- stand-alone grouped GEMMs
 * The two GEMMs as separate launches, for callers that keep sort / gemm1 / gemm2 apart.  Replaces
 * ck_tile::MoeFlatmmKernel behind MoeFlatmmHostArgs (ops/flatmm/kernel/moe_flatmm_kernel.hpp:17-127, kinds
 * :130-135); semantics as in host/reference/reference_moe_gemm.hpp:18-241:
 *   gate+up: C[token * TopK + slot, n] = act(A[token] . B[e, n] + bias[e, n], A[token] . B[e, N/2 + n] + bias[e, N/2 + n]),  n < N/2
 *   gate only: C[token * TopK + slot, n] = act(A[token] . B[e, n] + bias[e, n])
 *   down   : C[token, n] += sum over the token's slots of w * (A[token * TopK + slot] . B[e, n] + bias[e, n])
 * with the per-row scale scale_m and the per-channel scale scale_n folded into the dot products.  act is the
 * FusedActivation of the ck_tile kernel (moe_flatmm_kernel.hpp:139-183): MoeSilu, silu(gate) * linear, or
 * moe::Swiglu{alpha, limit}, gate' * sigmoid(alpha * gate') * (linear' + 1) with gate' = min(gate, limit) and
 * linear' = clamp(linear, -limit, limit) (gate only: linear = 1 for MoeSilu).  Unlike ck_tile's atomic bf16
 * epilogue the down GEMM sums a token's slots in fp32, in slot order, and rounds once. */
enum mi355_moe_flatmm_kind
{
    MI355_MOE_GEMM1_GATE_ONLY = 0, /* C = act(A x B^T), B [experts, N, K] */
    MI355_MOE_GEMM1_GATE_UP   = 1,
    MI355_MOE_GEMM2           = 2
};

enum mi355_moe_flatmm_activation
{
    MI355_MOE_ACT_SILU   = 0, /* ck_tile::moe::MoeSilu, the default FusedActivation */
    MI355_MOE_ACT_SWIGLU = 1  /* ck_tile::moe::Swiglu{swiglu_alpha, swiglu_limit} */
};

/* the arguments of MoeFlatmmHostArgs' constructor (moe_flatmm_kernel.hpp:79-127) in its order, then what the
 * ck_tile kernel takes as template arguments (operand types, activation) */
typedef struct mi355_moe_flatmm_args
{
    const void* p_sorted_token_ids;      /* as written by mi355_moe_sorting: token | slot << 24 */
    const void* p_sorted_expert_weights; /* fp32 per sorted row (down GEMM) */
    const void* p_sorted_expert_ids;
    const void* p_max_token_id;          /* [1] int32: rows after padding (p_total_tokens_post_pad) */
    const void* a_ptr;    /* gate+up: [NumTokens, stride_A]; down: [NumTokens * TopK, stride_A] */
    const void* b_ptr;    /* [NumExperts, N, K], K contiguous (stride_B = K), or pre-shuffled (b_shuffle) */
    void* c_ptr;          /* bf16 (fp16 with fp16 operands); gate+up: [NumTokens * TopK, stride_C] (N/2 columns); down: [NumTokens, stride_C] */
    int32_t NumTokens;
    int32_t NumExperts;
    int32_t TopK;
    int32_t k_batch;      /* 0 or 1 */
    int32_t M;            /* length of the sorted id list (informational) */
    int32_t N;
    int32_t K;
    int32_t stride_A;
    int32_t stride_B;
    int32_t stride_C;
    int32_t n_padded_zeros; /* the last n_padded_zeros rows of every expert's B are padding: read as zero */
    int32_t k_padded_zeros; /* the last k_padded_zeros columns of A and B are padding: read as zero */
    const void* scale_m;  /* fp32 per row of A, or NULL (ScaleM) */
    const void* scale_n;  /* fp32 [NumExperts, N], or NULL (ScaleN) */
    const void* exp_bias; /* fp32 [NumExperts, N] added to the scaled dot products, or NULL (ExpertBias) */
    int32_t prec_a;       /* mi355_moe_dtype of A: BF16, FP16 (with FP16 weights), FP8 (with FP8 weights), or INT8 for the gate+up GEMM with int8 weights */
    int32_t prec_b;       /* mi355_moe_dtype of B: BF16 | FP16 | FP8 | INT8 */
    int32_t block_m;      /* unit_size the sort was run with */
    int32_t activation;   /* mi355_moe_flatmm_activation (gate GEMMs) */
    float swiglu_alpha;   /* 1.702 in ck_tile's default */
    float swiglu_limit;   /* 7.0 in ck_tile's default */
    int32_t b_shuffle;    /* layout of B: 0 = rows of K elements; 1 = what ck_tile::shuffle_b gives a flatmm kernel with
                             N_Warp_Tile = 16 and 64 bytes of K per warp tile (host/tensor_shuffle_utils.hpp:26-68:
                             [n/16][k bytes/64][4][16][16 bytes], the b_nr_kr_kw_nw_kv of the fused kernel), read in
                             place; needs K rows of whole 64-byte blocks, N a multiple of 16 and no k_padded_zeros.
                             Other warp tiles: convert once with mi355_moe_permute_weights */
} mi355_moe_flatmm_args;

/* bytes of the mi355_moe_workspace for this call; 0 when the arguments have no kernel */
size_t mi355_moe_flatmm_workspace_size(int32_t kind, const mi355_moe_flatmm_args* args);
int mi355_moe_flatmm(int32_t kind, const mi355_moe_flatmm_args* args, const mi355_moe_workspace* ws, void* stream);

/* ------------------------------------------------------------------------------ kernel timing
 * Counterpart of ck_tile::stream_config::time_kernel_ (host/stream_config.hpp:29-39,
 * host/kernel_launch.hpp:106-143): between _start and _stop every kernel the library launches is
 * bracketed by HIP events on its own stream.  _stop waits for the events, adds the elapsed
 * milliseconds and launch counts per kernel kind into ms[] / launches[] (MI355_MOE_NUM_KERNELS
 * entries each) and switches timing off.  Process-wide, not re-entrant; for benchmarks only. */
enum mi355_moe_kernel_kind
{
    MI355_MOE_K_SORT_ONESHOT = 0,
    MI355_MOE_K_SORT_COUNT   = 1,
    MI355_MOE_K_SORT_SCAN    = 2,
    MI355_MOE_K_SORT_SCATTER = 3,
    MI355_MOE_K_PREP         = 4,
    MI355_MOE_K_GEMM0        = 5,
    MI355_MOE_K_GEMM1        = 6,
    MI355_MOE_K_COMBINE      = 7,
    MI355_MOE_K_QUANT        = 8,
    MI355_MOE_K_ROUTER       = 9,
    MI355_MOE_NUM_KERNELS    = 10
};
int mi355_moe_profile_start(void);
/* same, timing only the kernel kinds whose bit (1 << kind) is set: every pair of event records sits between
 * two launches and costs a few microseconds of the stream's time, which matters for the decode regime */
int mi355_moe_profile_start_kinds(uint32_t kind_mask);
int mi355_moe_profile_stop(double* ms, int32_t* launches);
const char* mi355_moe_kernel_name(int32_t kind);

/* ------------------------------------------------------------------- sustained matrix-core rate
 * No counterpart in ck_tile: a measurement aid for benchmarks.  Runs, for about `milliseconds` on `stream`, a loop of
 * independent MFMAs of the instruction the grouped GEMMs use for `prec` (mi355_moe_dtype: FP8, BF16, FP16, INT8) on
 * register operands, without any memory traffic, and returns the rate in TFLOP/s (TOP/s for INT8) averaged over the
 * second half of that time.  zero_operands = 0: operands with random signs, mantissas and exponents (what real
 * tensors look like to the multipliers); 1: all zeros.  The two differ widely on a power-limited part: the published
 * peak is reached on zeros only.  Blocks the calling thread until done; allocates nothing. */
int mi355_moe_mfma_sustained(int32_t prec, int32_t milliseconds, int32_t zero_operands, double* tflops, void* stream);

const char* mi355_moe_last_error(void);
int mi355_moe_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MI355_MOE_H */
