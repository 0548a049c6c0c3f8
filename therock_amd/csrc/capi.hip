// extern "C" surface of libmi355_moe.so: argument checking, workspace carving, launches.
#include "common.hpp"
#include "moe_gemm.hpp"

#include <cstring>
#include <mutex>
#include <vector>

namespace mi355 {

char* error_buffer()
{
    static thread_local char buf[512] = {0};
    return buf;
}

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

const DeviceInfo& device_info()
{
    constexpr int kMaxDev = 64;
    static DeviceInfo info[kMaxDev];
    static std::once_flag once[kMaxDev];
    int dev = 0;
    (void)hipGetDevice(&dev);
    if(dev < 0 || dev >= kMaxDev)
        dev = 0;
    std::call_once(once[dev], [dev] {
        int v = 0;
        info[dev].num_cu = hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0 ? v : 256;
        info[dev].max_lds = hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) == hipSuccess && v > 0 ? v : 65536;
    });
    return info[dev];
}

namespace {
struct ProfileState
{
    bool enabled  = false;
    uint32_t mask = 0xffffffffu; // kernel kinds that are timed
    uint32_t held = 0;           // kinds whose launches are inside an enclosing event pair (KernelTimerGroup)
    std::vector<hipEvent_t> pool; // events created so far
    size_t used = 0;
    struct Rec
    {
        int kind;
        hipEvent_t e0, e1;
    };
    std::vector<Rec> recs;
    hipEvent_t pending[MI355_MOE_NUM_KERNELS] = {};
    hipEvent_t get()
    {
        if(used == pool.size())
        {
            hipEvent_t e = nullptr;
            if(hipEventCreate(&e) != hipSuccess)
                return nullptr;
            pool.push_back(e);
        }
        return pool[used++];
    }
};
ProfileState g_prof;
} // namespace

bool profiling_enabled(int kind)
{
    return g_prof.enabled && ((g_prof.mask >> kind) & 1u) != 0 && ((g_prof.held >> kind) & 1u) == 0;
}

void profile_hold(int kind, bool on)
{
    if(kind >= 0 && kind < 32)
        g_prof.held = on ? (g_prof.held | (1u << kind)) : (g_prof.held & ~(1u << kind));
}

void profile_mark(int kind, hipStream_t stream, bool begin)
{
    if(kind < 0 || kind >= MI355_MOE_NUM_KERNELS)
        return;
    hipEvent_t e = g_prof.get();
    if(e == nullptr)
        return;
    (void)hipEventRecord(e, stream);
    if(begin)
        g_prof.pending[kind] = e;
    else if(g_prof.pending[kind] != nullptr)
    {
        g_prof.recs.push_back({kind, g_prof.pending[kind], e});
        g_prof.pending[kind] = nullptr;
    }
}

} // namespace mi355

using namespace mi355;

// ---- library-owned workspace of mi355_fused_moe_static_ws(): device memory that exists from the moment the code
// object is loaded, so that the entry point never allocates.  In host code `scratch` is only a handle for
// hipGetSymbolAddress: the address kernels and copies use is the one that call returns, and every device has its own
// copy of the array at its own address.
constexpr size_t kStaticWsBytes = (size_t)96 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticWsBytes];

namespace {
// device address of `scratch` on the current device, resolved once per device; nullptr (and the error text) on failure
void* static_workspace()
{
    constexpr int kMaxDev = 64;
    static void* ptr[kMaxDev] = {};
    static std::mutex mu;
    int dev = 0;
    if(hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev)
    {
        fail(MI355_MOE_E_HIP, "fused_moe_static_ws: no current device (or a device index above %d)", kMaxDev - 1);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(mu);
    if(ptr[dev] == nullptr)
    {
        void* p            = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if(e != hipSuccess || p == nullptr)
        {
            fail(MI355_MOE_E_HIP, "hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        ptr[dev] = p;
    }
    return ptr[dev];
}
} // namespace

extern "C" {

__attribute__((visibility("default"))) const char* mi355_moe_last_error(void) { return error_buffer(); }

__attribute__((visibility("default"))) int mi355_moe_version(void) { return MI355_MOE_VERSION; }

__attribute__((visibility("default"))) const char* mi355_moe_kernel_name(int32_t kind)
{
    static const char* names[MI355_MOE_NUM_KERNELS] = {
        "moe_sorting_oneshot", "moe_sorting_count", "moe_sorting_scan", "moe_sorting_scatter", "moe_prep",
        "moe_gemm0_gate_up_silu", "moe_gemm1_down", "moe_combine", "rowwise_quant", "topk_softmax"};
    return kind >= 0 && kind < MI355_MOE_NUM_KERNELS ? names[kind] : "?";
}

__attribute__((visibility("default"))) int mi355_moe_profile_start_kinds(uint32_t kind_mask);

__attribute__((visibility("default"))) int mi355_moe_profile_start(void)
{
    return mi355_moe_profile_start_kinds(0xffffffffu);
}

__attribute__((visibility("default"))) int mi355_moe_profile_start_kinds(uint32_t kind_mask)
{
    g_prof.mask = kind_mask;
    g_prof.held = 0;
    g_prof.used = 0;
    g_prof.recs.clear();
    for(auto& p : g_prof.pending)
        p = nullptr;
    g_prof.enabled = true;
    return MI355_MOE_OK;
}

__attribute__((visibility("default"))) int mi355_moe_profile_stop(double* ms, int32_t* launches)
{
    g_prof.enabled = false;
    if(ms == nullptr || launches == nullptr)
        return fail(MI355_MOE_E_INVALID, "profile_stop: null output");
    for(int k = 0; k < MI355_MOE_NUM_KERNELS; k++)
    {
        ms[k]       = 0.0;
        launches[k] = 0;
    }
    for(const auto& r : g_prof.recs)
    {
        MI355_HIP_TRY(hipEventSynchronize(r.e1));
        float t = 0.f;
        MI355_HIP_TRY(hipEventElapsedTime(&t, r.e0, r.e1));
        ms[r.kind] += t;
        launches[r.kind] += 1;
    }
    g_prof.recs.clear();
    g_prof.used = 0;
    return MI355_MOE_OK;
}

__attribute__((visibility("default"))) int
mi355_moe_mfma_sustained(int32_t prec, int32_t milliseconds, int32_t zero_operands, double* tflops, void* stream)
{
    return mfma_sustained(prec, milliseconds, zero_operands, tflops, static_cast<hipStream_t>(stream));
}

__attribute__((visibility("default"))) int64_t
mi355_moe_max_num_tokens_padded(int32_t tokens, int32_t num_experts, int32_t topk, int32_t unit_size)
{
    return (int64_t)topk * tokens + (int64_t)num_experts * unit_size - topk;
}

__attribute__((visibility("default"))) size_t
mi355_moe_sorting_workspace_size(int32_t tokens, int32_t num_experts, int32_t topk)
{
    return sorting_workspace_bytes(tokens, num_experts, topk);
}

__attribute__((visibility("default"))) size_t
mi355_moe_sorting_workspace_size2(int32_t tokens, int32_t num_experts, int32_t topk, int32_t dispatch_policy)
{
    if(dispatch_policy < 0 || dispatch_policy > 2)
        return 0;
    return sorting_workspace_bytes(tokens, num_experts, topk, dispatch_policy);
}

__attribute__((visibility("default"))) int mi355_moe_sorting(const mi355_moe_sorting_args* args, void* stream)
{
    if(args == nullptr)
        return fail(MI355_MOE_E_INVALID, "moe_sorting: args is null");
    return launch_moe_sorting(*args, static_cast<hipStream_t>(stream));
}

__attribute__((visibility("default"))) int
mi355_moe_sorting2(const mi355_moe_sorting_traits* traits, const mi355_moe_sorting_args* args, void* stream)
{
    if(traits == nullptr || args == nullptr)
        return fail(MI355_MOE_E_INVALID, "moe_sorting: traits or args is null");
    if(traits->index_type != MI355_MOE_INT32 || traits->weight_type != MI355_MOE_FP32)
        return fail(MI355_MOE_E_UNSUPPORTED, "moe_sorting: index type %d / weight type %d (int32 / fp32 only)",
                    traits->index_type, traits->weight_type);
    mi355_moe_sorting_args a = *args;
    if(!traits->local_expert_masking)
        a.p_local_expert_mask = nullptr;
    return launch_moe_sorting(a, static_cast<hipStream_t>(stream), nullptr, traits->skip_experts_with_zero_tokens == 0,
                              traits->dispatch_policy);
}

__attribute__((visibility("default"))) int
mi355_topk_softmax(const mi355_topk_softmax_traits* traits, const mi355_topk_softmax_args* args, void* stream)
{
    if(traits == nullptr || args == nullptr)
        return fail(MI355_MOE_E_INVALID, "topk_softmax: traits or args is null");
    return launch_topk_softmax(*traits, *args, static_cast<hipStream_t>(stream));
}

__attribute__((visibility("default"))) int mi355_fused_moe_supported(const mi355_fused_moe_traits* t)
{
    return t != nullptr && check_traits(*t) == MI355_MOE_OK ? 1 : 0;
}

__attribute__((visibility("default"))) size_t
mi355_fused_moe_workspace_size(const mi355_fused_moe_traits* traits, int32_t tokens, int32_t num_experts,
                               int32_t topk, int32_t hidden_size, int32_t intermediate_size)
{
    if(traits == nullptr || check_traits(*traits) != MI355_MOE_OK ||
       !sizes_in_range(tokens, num_experts, topk, hidden_size, intermediate_size))
        return 0;
    return workspace_layout(*traits, tokens, num_experts, topk, hidden_size, intermediate_size).total;
}

__attribute__((visibility("default"))) int32_t
mi355_fused_moe_tile_rows(const mi355_fused_moe_traits* traits, int32_t tokens, int32_t num_experts, int32_t topk,
                          int32_t hidden_size, int32_t intermediate_size)
{
    if(traits == nullptr || check_traits(*traits) != MI355_MOE_OK ||
       !sizes_in_range(tokens, num_experts, topk, hidden_size, intermediate_size))
        return 0;
    return gemm_tile_rows(*traits, tokens, num_experts, topk, hidden_size, intermediate_size);
}

__attribute__((visibility("default"))) int32_t
mi355_fused_moe_chosen_tile_rows(const mi355_fused_moe_traits* traits, int32_t tokens, int32_t num_experts, int32_t topk,
                                 int32_t hidden_size, int32_t intermediate_size, const mi355_moe_workspace* ws, void* stream)
{
    if(traits == nullptr || check_traits(*traits) != MI355_MOE_OK ||
       !sizes_in_range(tokens, num_experts, topk, hidden_size, intermediate_size))
        return 0;
    const int host_rows = gemm_tile_rows(*traits, tokens, num_experts, topk, hidden_size, intermediate_size);
    if(gemm_alt_tile_rows(*traits, tokens, num_experts, topk, hidden_size, intermediate_size) == 0)
        return host_rows;
    const WorkspaceLayout L = workspace_layout(*traits, tokens, num_experts, topk, hidden_size, intermediate_size);
    if(ws == nullptr || ws->ptr == nullptr || ws->bytes < L.total)
    {
        fail(MI355_MOE_E_WORKSPACE, "fused_moe_chosen_tile_rows: the workspace of the call is needed");
        return 0;
    }
    int32_t rows = 0;
    const hipStream_t s = static_cast<hipStream_t>(stream);
    if(hipMemcpyAsync(&rows, static_cast<const unsigned char*>(ws->ptr) + L.map_off + sizeof(int32_t), sizeof(int32_t),
                      hipMemcpyDeviceToHost, s) != hipSuccess ||
       hipStreamSynchronize(s) != hipSuccess)
    {
        fail(MI355_MOE_E_HIP, "fused_moe_chosen_tile_rows: reading the work list failed");
        return 0;
    }
    return rows;
}

__attribute__((visibility("default"))) int
mi355_fused_moegemm(const mi355_fused_moe_traits* traits, const mi355_fused_moegemm_args* args,
                    const mi355_moe_workspace* ws, void* stream)
{
    if(traits == nullptr || args == nullptr)
        return fail(MI355_MOE_E_INVALID, "fused_moegemm: traits or args is null");
    return launch_fused_moegemm(*traits, *args, ws ? ws->ptr : nullptr, ws ? ws->bytes : 0,
                                static_cast<hipStream_t>(stream));
}

} // extern "C"

namespace {
// sort + grouped GEMMs + combine on one stream, everything the kernels need beyond the caller's tensors in ws_ptr
int run_fused_moe(const mi355_fused_moe_traits* traits, const mi355_fused_moe_args* a, void* ws_ptr, size_t ws_bytes,
                  void* stream)
{
    int rc = check_traits(*traits);
    if(rc != MI355_MOE_OK)
        return rc;
    if(a->block_m != traits->block_m)
        return fail(MI355_MOE_E_INVALID, "fused_moe: args.block_m=%d differs from traits.block_m=%d",
                    a->block_m, traits->block_m);
    if(traits->local_expert_masking && a->local_expert_mask_ptr == nullptr)
        return fail(MI355_MOE_E_INVALID, "fused_moe: local_expert_masking set but mask pointer is null");

    mi355_fused_moegemm_args g{};
    g.a_ptr                 = a->a_ptr;
    g.a_scale_ptr           = a->a_scale_ptr;
    g.g_ptr                 = a->g_ptr;
    g.d_ptr                 = a->d_ptr;
    g.g_scale_ptr           = a->g_scale_ptr;
    g.d_scale_ptr           = a->d_scale_ptr;
    g.y_smooth_scale_ptr    = a->y_smooth_scale_ptr;
    g.o_ptr                 = a->o_ptr;
    g.sorted_token_ids_ptr  = a->sorted_token_ids_ptr;
    g.sorted_weight_ptr     = a->sorted_weight_ptr;
    g.sorted_expert_ids_ptr = a->sorted_expert_ids_ptr;
    g.num_sorted_tiles_ptr  = a->num_sorted_tiles_ptr;
    g.hidden_size           = a->hidden_size;
    g.intermediate_size     = a->intermediate_size;
    g.num_tokens            = a->num_tokens;
    g.num_experts           = a->num_experts;
    g.topk                  = a->topk;
    g.stride_token          = a->stride_token;
    // every host-side check of both halves comes before the first launch: a rejected call has written nothing
    rc = validate_fused_moegemm(*traits, g, ws_ptr, ws_bytes);
    if(rc != MI355_MOE_OK)
        return rc;
    if(a->num_tokens > 0 && (a->topk_ids_ptr == nullptr || a->topk_weight_ptr == nullptr))
        return fail(MI355_MOE_E_INVALID, "fused_moe: topk_ids or topk_weight is null");
    const WorkspaceLayout wl = workspace_layout(*traits, a->num_tokens, a->num_experts, a->topk,
                                                a->hidden_size, a->intermediate_size);

    // the combine writes every element of o, so the sort does not need to zero it
    mi355_moe_sorting_args s{};
    s.p_topk_ids              = a->topk_ids_ptr;
    s.p_weights               = a->topk_weight_ptr;
    s.p_local_expert_mask     = traits->local_expert_masking ? a->local_expert_mask_ptr : nullptr;
    s.p_local_tokens          = nullptr;
    s.p_sorted_token_ids      = a->sorted_token_ids_ptr;
    s.p_sorted_weights        = a->sorted_weight_ptr;
    s.p_sorted_expert_ids     = a->sorted_expert_ids_ptr;
    s.p_total_tokens_post_pad = a->num_sorted_tiles_ptr;
    s.p_moe_buf               = nullptr;
    // Always the slice of the library workspace: args->ws_ptr (the example's own sort workspace) comes without a
    // size, and one sized by another formula than mi355_moe_sorting_workspace_size() would be overrun.  It is
    // accepted and not touched.
    s.p_ws                    = static_cast<char*>(ws_ptr) + wl.sort_off;
    s.tokens                  = a->num_tokens;
    s.unit_size               = a->block_m;
    s.num_experts             = a->num_experts;
    s.topk                    = a->topk;
    const GemmPlan plan = make_gemm_plan(*traits, ws_ptr, a->num_tokens, a->num_experts, a->topk, a->hidden_size,
                                         a->intermediate_size);
    rc = launch_moe_sorting(s, static_cast<hipStream_t>(stream), &plan);
    if(rc != MI355_MOE_OK)
        return rc;
    return launch_fused_moegemm(*traits, g, ws_ptr, ws_bytes, static_cast<hipStream_t>(stream), /*prep_done=*/true);
}
} // namespace

extern "C" {

__attribute__((visibility("default"))) int
mi355_fused_moe(const mi355_fused_moe_traits* traits, const mi355_fused_moe_args* a, const mi355_moe_workspace* ws,
                void* stream)
{
    if(traits == nullptr || a == nullptr)
        return fail(MI355_MOE_E_INVALID, "fused_moe: traits or args is null");
    return run_fused_moe(traits, a, ws ? ws->ptr : nullptr, ws ? ws->bytes : 0, stream);
}

__attribute__((visibility("default"))) size_t mi355_fused_moe_static_ws_capacity(void) { return kStaticWsBytes; }

__attribute__((visibility("default"))) int
mi355_fused_moe_static_ws(const mi355_fused_moe_traits* traits, const mi355_fused_moe_args* a, void* stream)
{
    if(traits == nullptr || a == nullptr)
        return fail(MI355_MOE_E_INVALID, "fused_moe_static_ws: traits or args is null");
    int rc = check_traits(*traits);
    if(rc != MI355_MOE_OK)
        return rc;
    if(!sizes_in_range(a->num_tokens, a->num_experts, a->topk, a->hidden_size, a->intermediate_size))
        return fail(MI355_MOE_E_INVALID, "fused_moe_static_ws: bad sizes (H=%d I=%d T=%d E=%d K=%d)", a->hidden_size,
                    a->intermediate_size, a->num_tokens, a->num_experts, a->topk);
    const size_t need = workspace_layout(*traits, a->num_tokens, a->num_experts, a->topk, a->hidden_size,
                                         a->intermediate_size).total;
    if(need > kStaticWsBytes)
        return fail(MI355_MOE_E_WORKSPACE,
                    "fused_moe_static_ws: this problem needs a workspace of %zu bytes, the library-owned one holds %zu; "
                    "call mi355_fused_moe with a workspace of your own", need, kStaticWsBytes);
    void* ws_ptr = static_workspace();
    if(ws_ptr == nullptr)
        return MI355_MOE_E_HIP;
    return run_fused_moe(traits, a, ws_ptr, kStaticWsBytes, stream);
}

__attribute__((visibility("default"))) size_t
mi355_moe_flatmm_workspace_size(int32_t kind, const mi355_moe_flatmm_args* args)
{
    return args != nullptr ? moe_flatmm_workspace_bytes(kind, *args) : 0;
}

__attribute__((visibility("default"))) int
mi355_moe_flatmm(int32_t kind, const mi355_moe_flatmm_args* args, const mi355_moe_workspace* ws, void* stream)
{
    if(args == nullptr)
        return fail(MI355_MOE_E_INVALID, "moe_flatmm: args is null");
    return launch_moe_flatmm(kind, *args, ws ? ws->ptr : nullptr, ws ? ws->bytes : 0, static_cast<hipStream_t>(stream));
}

__attribute__((visibility("default"))) int
mi355_moe_permute_weights(const void* src, void* dst, int32_t experts, int32_t n, int32_t k, int32_t elem_bytes,
                          int32_t nw, int32_t kw, int32_t kv, int32_t inverse, void* stream)
{
    return launch_permute_weights(src, dst, experts, n, k, elem_bytes, nw, kw, kv, inverse, static_cast<hipStream_t>(stream));
}

__attribute__((visibility("default"))) int
mi355_moe_smoothquant(const mi355_moe_smoothquant_args* args, int32_t q_dtype, void* stream)
{
    if(args == nullptr)
        return fail(MI355_MOE_E_INVALID, "moe_smoothquant: args is null");
    return launch_moe_smoothquant(*args, q_dtype, static_cast<hipStream_t>(stream));
}

__attribute__((visibility("default"))) int
mi355_moe_rowwise_quant(const void* x, int64_t rows, int32_t cols, int64_t stride_x, int32_t q_dtype, void* q,
                        void* scale, void* stream)
{
    return launch_rowwise_quant(x, rows, cols, stride_x, q_dtype, q, scale, static_cast<hipStream_t>(stream));
}
}
