// mi355_fused_moe.hpp - C++ host API of the MI355X-native fused-MoE path.
//
// Same names, fields and conventions as Composable Kernel's example-level API
// (example/ck_tile/15_fused_moe/fused_moe.hpp, fused_moesorting.hpp, fused_moegemm.hpp and
// example/ck_tile/13_moe_sorting/moe_sorting_api.hpp), so that code written against
//     float fused_moe(fused_moe_traits, fused_moe_args, const ck_tile::stream_config&)
//     float moe_sorting(moe_sorting_trait, moe_sorting_args, ck_tile::stream_config)
// switches by changing the namespace.  Everything here is a thin inline layer over the C ABI of
// libmi355_moe.so (mi355_moe.h): strings become enums, a non-zero status becomes -1 (no kernel for
// the traits) or a std::runtime_error (HIP / argument errors, as ck_tile's HIP_CHECK_ERROR does,
// host/hip_check_error.hpp:22-33), and timing follows ck_tile::launch_kernel
// (host/kernel_launch.hpp:106-143, 173-193): 0 when not timing, else mean milliseconds.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <map>
#include <mutex>
#include <stdexcept>
#include <string>
#include <utility>

#include "mi355_moe.h"

namespace mi355 {

using index_t = int32_t;

// ck_tile::stream_config (host/stream_config.hpp:29-39)
struct stream_config
{
    hipStream_t stream_id_ = nullptr;
    bool time_kernel_      = false;
    int log_level_         = 0;
    int cold_niters_       = 3;
    int nrepeat_           = 10;
    bool is_gpu_timer_     = true;
};

// ---------------------------------------------------------------------------------- moe_sorting
struct moe_sorting_trait
{
    std::string index_type  = "int32";
    std::string weight_type = "fp32";
    bool local_expert_masking = false;
    bool clear_workspace_inside_api = false; // accepted: the workspace never needs clearing
    int dispatch_policy             = 0;     // 0 the library picks, 1 single kernel, 2 multi-launch passes
    // MoeSortingProblemEx::SkipExpertsWithZeroTokens (ops/fused_moe/kernel/moe_sorting_problem.hpp:35), a template
    // argument of ck_tile's kernel: false gives every expert of this rank that no token chose one unit of padding
    bool skip_experts_with_zero_tokens = true;
};

// ck_tile::MoeSortingHostArgs (ops/fused_moe/kernel/moe_sorting_kernel.hpp:188-222)
struct moe_sorting_args : public mi355_moe_sorting_args
{
};

inline int moe_sorting_get_workspace_size(int tokens, int num_experts, int topk, int dispatch_policy = 0)
{
    return static_cast<int>(mi355_moe_sorting_workspace_size2(tokens, num_experts, topk, dispatch_policy));
}

namespace detail {

inline void throw_on_error(int rc, const char* what)
{
    if(rc != MI355_MOE_OK && rc != MI355_MOE_E_UNSUPPORTED)
        throw std::runtime_error(std::string(what) + ": " + mi355_moe_last_error());
}

inline int dtype_of(const std::string& s)
{
    if(s == "bf16") return MI355_MOE_BF16;
    if(s == "fp8") return MI355_MOE_FP8;
    if(s == "int8") return MI355_MOE_INT8;
    if(s == "fp32") return MI355_MOE_FP32;
    if(s == "int32") return MI355_MOE_INT32;
    if(s == "fp16") return MI355_MOE_FP16;
    return -1;
}

inline void hip_check(hipError_t e, const char* what)
{
    if(e != hipSuccess)
        throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

// runs `launch` once, or cold_niters_ + nrepeat_ times between two events when timing
template <typename F>
inline float run_timed(const stream_config& s, F&& launch)
{
    if(!s.time_kernel_)
    {
        const int rc = launch();
        return rc == MI355_MOE_E_UNSUPPORTED ? -1.f : 0.f;
    }
    for(int i = 0; i < s.cold_niters_; i++)
        if(launch() == MI355_MOE_E_UNSUPPORTED)
            return -1.f;
    hipEvent_t e0, e1;
    hip_check(hipEventCreate(&e0), "hipEventCreate");
    hip_check(hipEventCreate(&e1), "hipEventCreate");
    hip_check(hipEventRecord(e0, s.stream_id_), "hipEventRecord");
    for(int i = 0; i < s.nrepeat_; i++)
        launch();
    hip_check(hipEventRecord(e1, s.stream_id_), "hipEventRecord");
    hip_check(hipEventSynchronize(e1), "hipEventSynchronize");
    float ms = 0.f;
    hip_check(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return ms / (s.nrepeat_ > 0 ? s.nrepeat_ : 1);
}

// Workspace for callers that pass none (CK's fused_moe needs none, so CK-style call sites have none to pass).
// One block per (device, stream): calls on different streams never share intermediates.  A block that was
// handed out is never freed or moved - work already enqueued, or a captured graph, may still refer to it - so
// growth allocates a new block and keeps the old one until the process ends.  Growth needs hipMalloc, which a
// capturing stream does not allow: such callers pass their own workspace (or call once before capturing).
// Calls that overlap on ONE stream's block from several host threads are the caller's to serialise.
inline mi355_moe_workspace cached_workspace(size_t bytes, hipStream_t stream)
{
    struct Block
    {
        void* ptr    = nullptr;
        size_t bytes = 0;
    };
    static std::mutex mu;
    static std::map<std::pair<int, hipStream_t>, Block> blocks;
    int dev = 0;
    hip_check(hipGetDevice(&dev), "hipGetDevice");
    std::lock_guard<std::mutex> lock(mu);
    Block& b = blocks[std::make_pair(dev, stream)];
    if(b.bytes < bytes)
    {
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        if(hipStreamIsCapturing(stream, &st) == hipSuccess && st != hipStreamCaptureStatusNone)
            throw std::runtime_error("mi355: the stream is capturing and the cached workspace would have to grow; "
                                     "pass a workspace of fused_moe_get_workspace_size() bytes instead");
        void* p = nullptr;
        hip_check(hipMalloc(&p, bytes), "hipMalloc(workspace)");
        b.ptr   = p; // the previous block, if any, stays allocated
        b.bytes = bytes;
    }
    return mi355_moe_workspace{b.ptr, b.bytes};
}

} // namespace detail

inline float moe_sorting(moe_sorting_trait t, moe_sorting_args a, stream_config s = {})
{
    if(t.index_type != "int32" || t.weight_type != "fp32")
        return -1.f;
    const mi355_moe_sorting_traits ct{MI355_MOE_INT32, MI355_MOE_FP32, t.local_expert_masking ? 1 : 0,
                                      t.clear_workspace_inside_api ? 1 : 0, t.dispatch_policy,
                                      t.skip_experts_with_zero_tokens ? 1 : 0};
    return detail::run_timed(s, [&] {
        const int rc = mi355_moe_sorting2(&ct, &a, s.stream_id_);
        detail::throw_on_error(rc, "moe_sorting");
        return rc;
    });
}

// --------------------------------------------------------------------------------- topk_softmax
// topk_softmax_trait / topk_softmax_kargs of CK's example/ck_tile/09_topk_softmax
struct topk_softmax_trait
{
    std::string input_type  = "fp32"; // fp32 | bf16
    std::string weight_type = "fp32";
    int experts             = 0;
    std::string activation  = "softmax"; // softmax | sigmoid
    bool renormalize        = false;     // extension: divide the chosen weights by their sum
};

// ck_tile::TopkSoftmaxHostArgs (ops/topk_softmax/kernel/topk_softmax_kernel.hpp:15-25)
struct topk_softmax_kargs : public mi355_topk_softmax_args
{
};

inline float topk_softmax(topk_softmax_trait t, topk_softmax_kargs a, stream_config s = {})
{
    if((t.activation != "softmax" && t.activation != "sigmoid") || t.weight_type != "fp32" ||
       (t.input_type != "fp32" && t.input_type != "bf16"))
        return -1.f;
    const mi355_topk_softmax_traits p{detail::dtype_of(t.input_type), detail::dtype_of(t.weight_type), t.experts,
                                      t.activation == "sigmoid" ? 1 : 0, t.renormalize ? 1 : 0};
    return detail::run_timed(s, [&] {
        const int rc = mi355_topk_softmax(&p, &a, s.stream_id_);
        detail::throw_on_error(rc, "topk_softmax");
        return rc;
    });
}

// ----------------------------------------------------------------------------------- moe_flatmm
// ck_tile::MoeFlatmmHostArgs (ops/flatmm/kernel/moe_flatmm_kernel.hpp:17-127) and MoeFlatmmKind (:130-135)
enum class MoeFlatmmKind
{
    kFFN_gemm1_gate_only = MI355_MOE_GEMM1_GATE_ONLY,
    kFFN_gemm1_gate_up   = MI355_MOE_GEMM1_GATE_UP,
    kFFN_gemm2           = MI355_MOE_GEMM2,
};

struct moe_flatmm_args : public mi355_moe_flatmm_args
{
};

// ws: caller-owned workspace of mi355_moe_flatmm_workspace_size() bytes; when its ptr is null a cached block of
// this (device, stream) is used.  Returns -1 when no kernel matches.
inline float moe_flatmm(MoeFlatmmKind kind, moe_flatmm_args a, stream_config s = {}, mi355_moe_workspace ws = {})
{
    const int k = static_cast<int>(kind);
    if(ws.ptr == nullptr)
    {
        const size_t bytes = mi355_moe_flatmm_workspace_size(k, &a);
        if(bytes == 0)
            return -1.f;
        ws = detail::cached_workspace(bytes, s.stream_id_);
    }
    bool unsupported = false;
    const float ms   = detail::run_timed(s, [&] {
        const int rc = mi355_moe_flatmm(k, &a, &ws, s.stream_id_);
        if(rc == MI355_MOE_E_UNSUPPORTED)
        {
            unsupported = true;
            return 0;
        }
        detail::throw_on_error(rc, "moe_flatmm");
        return rc;
    });
    return unsupported ? -1.f : ms;
}

// ------------------------------------------------------------------------------ moe_smoothquant
// moe_smoothquant_traits / moe_smoothquant_args of CK's example/ck_tile/14_moe_smoothquant
struct moe_smoothquant_traits
{
    std::string in_type  = "bf16"; // input type
    std::string out_type = "int8"; // int8 | fp8
};

// ck_tile::MoeSmoothquantHostArgs (ops/smoothquant/kernel/moe_smoothquant_kernel.hpp:12-27)
struct moe_smoothquant_args : public mi355_moe_smoothquant_args
{
};

inline float moe_smoothquant(moe_smoothquant_traits t, moe_smoothquant_args a, stream_config s = {})
{
    if(t.in_type != "bf16" || (t.out_type != "int8" && t.out_type != "fp8"))
        return -1.f;
    const int32_t q = detail::dtype_of(t.out_type);
    return detail::run_timed(s, [&] {
        const int rc = mi355_moe_smoothquant(&a, q, s.stream_id_);
        detail::throw_on_error(rc, "moe_smoothquant");
        return rc;
    });
}

// ------------------------------------------------------------------------------------ fused_moe
struct fused_moe_traits
{
    std::string prec_i  = "bf16"; // input precision
    std::string prec_w  = "bf16"; // weight precision
    std::string prec_o  = "bf16"; // output precision
    std::string prec_st = "fp32"; // token scale data type
    std::string prec_sw = "fp32"; // weight scale data type
    std::string prec_sq = "fp32"; // smooth quant scale
    std::string prec_kw = "fp32"; // topk-weight data type
    int block_m         = 32;
    int activation      = 1; // 0: gelu, 1: silu
    int gate_only       = 0;
    int fused_quant     = 0; // 0: no-sweep, 1: smooth-dynamic-quant, 2: dynamic-quant
    bool local_expert_masking = false;
    // FusedMoeGemmWeightPermuteEnum of the ck_tile kernel (a template argument there): 1 = g and d arrive in
    // b_nr_kr_kw_nw_kv, as CK's example pre-shuffles them
    int weight_permute = 0;

    mi355_fused_moe_traits pod() const
    {
        using detail::dtype_of;
        return mi355_fused_moe_traits{dtype_of(prec_i),  dtype_of(prec_w),  dtype_of(prec_o), dtype_of(prec_st),
                                      dtype_of(prec_sw), dtype_of(prec_sq), dtype_of(prec_kw), block_m,
                                      activation,        gate_only,         fused_quant,       local_expert_masking ? 1 : 0,
                                      weight_permute};
    }
};

// fused_moe_args of CK's example (ws_ptr is the example's sort workspace and may stay null)
struct fused_moe_args : public mi355_fused_moe_args
{
};

// ck_tile::FusedMoeGemmHostArgs (ops/fused_moe/kernel/fused_moegemm_kernel.hpp:97-120), same layout
struct fused_moegemm_args : public mi355_fused_moegemm_args
{
};

inline size_t fused_moe_get_workspace_size(const fused_moe_traits& t, int tokens, int num_experts, int topk,
                                           int hidden_size, int intermediate_size)
{
    const mi355_fused_moe_traits p = t.pod();
    return mi355_fused_moe_workspace_size(&p, tokens, num_experts, topk, hidden_size, intermediate_size);
}

namespace detail {
inline bool pick_workspace(const mi355_fused_moe_traits& p, int tokens, int experts, int topk, int hidden, int inter,
                           hipStream_t stream, mi355_moe_workspace& ws)
{
    if(ws.ptr != nullptr)
        return true;
    const size_t bytes = mi355_fused_moe_workspace_size(&p, tokens, experts, topk, hidden, inter);
    if(bytes == 0)
        return false; // sizes the library cannot index: let the entry point describe the error
    ws = cached_workspace(bytes, stream);
    return true;
}
} // namespace detail

// CK's signature plus an optional caller-owned workspace (fused_moe_get_workspace_size() bytes, 256-byte aligned);
// without one a cached block of this (device, stream) is used
inline float fused_moe(fused_moe_traits t, fused_moe_args a, const stream_config& s = {}, mi355_moe_workspace ws = {})
{
    const mi355_fused_moe_traits p = t.pod();
    if(!mi355_fused_moe_supported(&p))
        return -1.f;
    detail::pick_workspace(p, a.num_tokens, a.num_experts, a.topk, a.hidden_size, a.intermediate_size, s.stream_id_, ws);
    return detail::run_timed(s, [&] {
        const int rc = mi355_fused_moe(&p, &a, &ws, s.stream_id_);
        detail::throw_on_error(rc, "fused_moe");
        return rc;
    });
}

inline float fused_moegemm(fused_moe_traits t, fused_moegemm_args a, const stream_config& s = {},
                           mi355_moe_workspace ws = {})
{
    const mi355_fused_moe_traits p = t.pod();
    if(!mi355_fused_moe_supported(&p))
        return -1.f;
    detail::pick_workspace(p, a.num_tokens, a.num_experts, a.topk, a.hidden_size, a.intermediate_size, s.stream_id_, ws);
    return detail::run_timed(s, [&] {
        const int rc = mi355_fused_moegemm(&p, &a, &ws, s.stream_id_);
        detail::throw_on_error(rc, "fused_moegemm");
        return rc;
    });
}

} // namespace mi355
