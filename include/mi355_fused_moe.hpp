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
};

// ck_tile::MoeSortingHostArgs (ops/fused_moe/kernel/moe_sorting_kernel.hpp:188-222)
struct moe_sorting_args : public mi355_moe_sorting_args
{
};

inline int moe_sorting_get_workspace_size(int tokens, int num_experts, int topk, int /*dispatch_policy*/ = 0)
{
    return static_cast<int>(mi355_moe_sorting_workspace_size(tokens, num_experts, topk));
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

// grow-only per-device scratch for callers that pass no workspace (CK's fused_moe needs none)
inline void* cached_workspace(size_t bytes)
{
    struct Slot
    {
        void* ptr    = nullptr;
        size_t bytes = 0;
    };
    static std::mutex mu;
    static std::map<int, Slot> slots;
    int dev = 0;
    hip_check(hipGetDevice(&dev), "hipGetDevice");
    std::lock_guard<std::mutex> lock(mu);
    Slot& s = slots[dev];
    if(s.bytes < bytes)
    {
        if(s.ptr != nullptr)
        {
            hip_check(hipDeviceSynchronize(), "hipDeviceSynchronize");
            hip_check(hipFree(s.ptr), "hipFree");
        }
        hip_check(hipMalloc(&s.ptr, bytes), "hipMalloc(workspace)");
        s.bytes = bytes;
    }
    return s.ptr;
}

} // namespace detail

inline float moe_sorting(moe_sorting_trait t, moe_sorting_args a, stream_config s = {})
{
    if(t.index_type != "int32" || t.weight_type != "fp32")
        return -1.f;
    if(!t.local_expert_masking)
        a.p_local_expert_mask = nullptr;
    return detail::run_timed(s, [&] {
        const int rc = mi355_moe_sorting(&a, s.stream_id_);
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

// ws_ptr may be left null: a cached per-device workspace is used.  Returns -1 when no kernel matches.
inline float moe_flatmm(MoeFlatmmKind kind, moe_flatmm_args a, stream_config s = {})
{
    const int k = static_cast<int>(kind);
    if(a.ws_ptr == nullptr)
    {
        a.ws_bytes = mi355_moe_flatmm_workspace_size(k, &a);
        if(a.ws_bytes == 0)
            return -1.f;
        a.ws_ptr = detail::cached_workspace(a.ws_bytes);
    }
    bool unsupported = false;
    const float ms   = detail::run_timed(s, [&] {
        const int rc = mi355_moe_flatmm(k, &a, s.stream_id_);
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

    mi355_fused_moe_traits pod() const
    {
        using detail::dtype_of;
        return mi355_fused_moe_traits{dtype_of(prec_i),  dtype_of(prec_w),  dtype_of(prec_o), dtype_of(prec_st),
                                      dtype_of(prec_sw), dtype_of(prec_sq), dtype_of(prec_kw), block_m,
                                      activation,        gate_only,         fused_quant,       local_expert_masking ? 1 : 0};
    }
};

// fused_moe_args of CK's example.  ws_ptr may be left null: a cached per-device workspace is used.
struct fused_moe_args : public mi355_fused_moe_args
{
};

struct fused_moegemm_args : public mi355_fused_moegemm_args
{
};

inline size_t fused_moe_get_workspace_size(const fused_moe_traits& t, int tokens, int num_experts, int topk,
                                           int hidden_size, int intermediate_size)
{
    const mi355_fused_moe_traits p = t.pod();
    return mi355_fused_moe_workspace_size(&p, tokens, num_experts, topk, hidden_size, intermediate_size);
}

inline float fused_moe(fused_moe_traits t, fused_moe_args a, const stream_config& s = {})
{
    const mi355_fused_moe_traits p = t.pod();
    if(!mi355_fused_moe_supported(&p))
        return -1.f;
    if(a.ws_ptr == nullptr)
    {
        a.ws_bytes = mi355_fused_moe_workspace_size(&p, a.num_tokens, a.num_experts, a.topk, a.hidden_size,
                                                    a.intermediate_size);
        a.ws_ptr   = detail::cached_workspace(a.ws_bytes);
    }
    return detail::run_timed(s, [&] {
        const int rc = mi355_fused_moe(&p, &a, s.stream_id_);
        detail::throw_on_error(rc, "fused_moe");
        return rc;
    });
}

inline float fused_moegemm(fused_moe_traits t, fused_moegemm_args a, const stream_config& s = {})
{
    const mi355_fused_moe_traits p = t.pod();
    if(!mi355_fused_moe_supported(&p))
        return -1.f;
    if(a.ws_ptr == nullptr)
    {
        a.ws_bytes = mi355_fused_moe_workspace_size(&p, a.num_tokens, a.num_experts, a.topk, a.hidden_size,
                                                    a.intermediate_size);
        a.ws_ptr   = detail::cached_workspace(a.ws_bytes);
    }
    return detail::run_timed(s, [&] {
        const int rc = mi355_fused_moegemm(&p, &a, s.stream_id_);
        detail::throw_on_error(rc, "fused_moegemm");
        return rc;
    });
}

} // namespace mi355
