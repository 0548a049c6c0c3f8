// Drives the C++ host API (include/mi355_fused_moe.hpp) the way CK's example main does:
// seeded inputs, DeviceMem-style buffers, fused_moe(traits, args, stream_config), copy back, compare
// with the host oracle (oracle/libmoe_oracle.so).  Exit code 0 = parity within tolerance.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/mi355_fused_moe.hpp"

extern "C" {
int moe_oracle_sorting(const int32_t*, const float*, const int32_t*, int32_t, int32_t, int32_t, int32_t, int32_t,
                       int32_t*, float*, int32_t*, int32_t*);
int moe_oracle_fused_moe(const void*, int, const float*, const void*, int, const float*, const void*, int,
                         const float*, void*, int, const int32_t*, const float*, const int32_t*, int32_t, int32_t,
                         int32_t, int32_t, int32_t, int32_t, int32_t, int32_t, int32_t, float*, int32_t);
uint16_t moe_oracle_f32_to_bf16(float);
float moe_oracle_bf16_to_f32(uint16_t);
}

#define HIP_OK(x)                                                                   \
    do                                                                              \
    {                                                                               \
        hipError_t e_ = (x);                                                        \
        if(e_ != hipSuccess)                                                        \
        {                                                                           \
            std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));            \
            return 2;                                                               \
        }                                                                           \
    } while(0)

static uint32_t g_state = 12345u;
static float uniform() { g_state = g_state * 1664525u + 1013904223u; return ((g_state >> 8) + 0.5f) / 16777216.0f; }
static float normal() { return std::sqrt(-2.0f * std::log(uniform())) * std::cos(6.2831853f * uniform()); }

template <typename T>
static T* to_device(const std::vector<T>& v)
{
    T* p = nullptr;
    if(hipMalloc(&p, v.size() * sizeof(T) + 16) != hipSuccess) return nullptr;
    if(hipMemcpy(p, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
    return p;
}

// the host-side weight pre-shuffle of CK's fused-MoE example for 2-byte elements: the row-major [e, n, k] weight viewed
// as [e, n/16, 16, k/32, 4, 8] and permuted to [e, n/16, k/32, 4, 16, 8] (b_nr_kr_kw_nw_kv)
static std::vector<uint16_t> preshuffle(const std::vector<uint16_t>& w, int e, int n, int k)
{
    std::vector<uint16_t> out(w.size());
    size_t o = 0;
    for(int x = 0; x < e; x++)
        for(int nr = 0; nr < n / 16; nr++)
            for(int kr = 0; kr < k / 32; kr++)
                for(int kw = 0; kw < 4; kw++)
                    for(int nw = 0; nw < 16; nw++)
                        for(int kv = 0; kv < 8; kv++)
                            out[o++] = w[((size_t)x * n + nr * 16 + nw) * k + kr * 32 + kw * 8 + kv];
    return out;
}

int main()
{
    const int T = 70, H = 256, I = 192, E = 6, K = 2, U = 32;
    std::vector<uint16_t> a(T * H), g(E * 2 * I * H), d(E * H * I);
    for(auto& v : a) v = moe_oracle_f32_to_bf16(normal());
    for(auto& v : g) v = moe_oracle_f32_to_bf16(0.02f * normal());
    for(auto& v : d) v = moe_oracle_f32_to_bf16(0.02f * normal());
    std::vector<int32_t> ids(T * K);
    std::vector<float> w(T * K);
    for(int t = 0; t < T; t++)
    {
        ids[t * K]     = static_cast<int>(uniform() * E) % E;
        ids[t * K + 1] = (ids[t * K] + 1 + static_cast<int>(uniform() * (E - 1)) % (E - 1)) % E;
        w[t * K]       = 0.25f + 0.5f * uniform();
        w[t * K + 1]   = 1.0f - w[t * K];
    }
    const int max_pad = static_cast<int>(mi355_moe_max_num_tokens_padded(T, E, K, U));
    const int tiles   = (max_pad + U - 1) / U;

    // oracle
    std::vector<int32_t> s_ids(max_pad, -1), s_eid(tiles, -1);
    std::vector<float> s_w(max_pad, -1.f);
    int32_t post_pad = 0;
    moe_oracle_sorting(ids.data(), w.data(), nullptr, T, K, E, U, 1, s_ids.data(), s_w.data(), s_eid.data(), &post_pad);
    std::vector<uint16_t> o_ref(T * H);
    moe_oracle_fused_moe(a.data(), 1, nullptr, g.data(), 1, nullptr, d.data(), 1, nullptr, o_ref.data(), 1, s_ids.data(),
                         s_w.data(), s_eid.data(), post_pad, U, T, E, H, I, K, 0, 0, nullptr, /*activation: silu*/ 1);

    // device path through the C++ API
    mi355::fused_moe_traits traits; // bf16, silu, block_m 32
    mi355::fused_moe_args args{};
    std::vector<int32_t> z_ids(max_pad, -1), z_eid(tiles, -1), z_tot(2, 0);
    std::vector<float> z_w(max_pad, -1.f);
    std::vector<uint16_t> z_o(T * H, 0);
    args.a_ptr = to_device(a);
    args.g_ptr = to_device(g);
    args.d_ptr = to_device(d);
    args.topk_ids_ptr = to_device(ids);
    args.topk_weight_ptr = to_device(w);
    args.sorted_token_ids_ptr = to_device(z_ids);
    args.sorted_weight_ptr = to_device(z_w);
    args.sorted_expert_ids_ptr = to_device(z_eid);
    args.num_sorted_tiles_ptr = to_device(z_tot);
    args.o_ptr = to_device(z_o);
    args.block_m = U; args.hidden_size = H; args.intermediate_size = I; args.num_tokens = T; args.num_experts = E;
    args.topk = K; args.stride_token = H;
    const float rc = mi355::fused_moe(traits, args, mi355::stream_config{});
    if(rc != 0.f) { std::fprintf(stderr, "fused_moe returned %f\n", rc); return 3; }
    HIP_OK(hipDeviceSynchronize());
    std::vector<uint16_t> o(T * H);
    std::vector<int32_t> d_ids(max_pad);
    HIP_OK(hipMemcpy(o.data(), args.o_ptr, o.size() * 2, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(d_ids.data(), args.sorted_token_ids_ptr, d_ids.size() * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(z_tot.data(), args.num_sorted_tiles_ptr, 8, hipMemcpyDeviceToHost));
    if(z_tot[0] != post_pad || std::memcmp(d_ids.data(), s_ids.data(), sizeof(int32_t) * post_pad) != 0)
    { std::fprintf(stderr, "sorted ids differ from the oracle\n"); return 4; }
    double num = 0, den = 0;
    for(size_t i = 0; i < o.size(); i++)
    {
        const double x = moe_oracle_bf16_to_f32(o[i]), r = moe_oracle_bf16_to_f32(o_ref[i]);
        num += (x - r) * (x - r);
        den += r * r;
    }
    const double err = std::sqrt(num / den);
    // the same call with g and d pre-shuffled on the host the way CK's example does it before calling its kernel
    mi355::fused_moe_traits shuffled = traits;
    shuffled.weight_permute = 1;
    mi355::fused_moe_args args2 = args;
    args2.g_ptr = to_device(preshuffle(g, E, 2 * I, H));
    args2.d_ptr = to_device(preshuffle(d, E, H, I));
    std::vector<uint16_t> z_o2(T * H, 0);
    args2.o_ptr = to_device(z_o2);
    if(mi355::fused_moe(shuffled, args2, mi355::stream_config{}) != 0.f) { std::fprintf(stderr, "pre-shuffled call failed\n"); return 5; }
    HIP_OK(hipDeviceSynchronize());
    std::vector<uint16_t> o2(T * H);
    HIP_OK(hipMemcpy(o2.data(), args2.o_ptr, o2.size() * 2, hipMemcpyDeviceToHost));
    if(std::memcmp(o.data(), o2.data(), o.size() * 2) != 0) { std::fprintf(stderr, "pre-shuffled weights give other bits\n"); return 6; }
    // moe_sorting() with the example's trait: experts without tokens keep a unit of padding (expert E - 1 gets no token
    // here), once per dispatch policy; sizes as reference_moe_sorting lays them out without the skip
    {
        std::vector<int32_t> ids2(ids);
        for(auto& v : ids2) v = v % (E - 1);
        for(int t = 0; t < T; t++)
            if(ids2[t * K + 1] == ids2[t * K]) ids2[t * K + 1] = (ids2[t * K] + 1) % (E - 1);
        const int cells = T * K + E * U, units = cells / U + 1;
        std::vector<int32_t> r_ids(cells, -1), r_eid(units, -1);
        std::vector<float> r_w(cells, -1.f);
        int32_t r_pp = 0;
        moe_oracle_sorting(ids2.data(), w.data(), nullptr, T, K, E, U, /*skip_empty=*/0, r_ids.data(), r_w.data(), r_eid.data(), &r_pp);
        for(int policy = 0; policy < 3; policy++)
        {
            mi355::moe_sorting_trait st;
            st.dispatch_policy = policy;
            st.skip_experts_with_zero_tokens = false;
            mi355::moe_sorting_args sa{};
            std::vector<int32_t> q_ids(cells, -1), q_eid(units, -1), q_tot(2, 0);
            std::vector<float> q_w(cells, -1.f);
            sa.p_topk_ids = to_device(ids2);
            sa.p_weights = to_device(w);
            sa.p_sorted_token_ids = to_device(q_ids);
            sa.p_sorted_weights = to_device(q_w);
            sa.p_sorted_expert_ids = to_device(q_eid);
            sa.p_total_tokens_post_pad = to_device(q_tot);
            const int ws_bytes = mi355::moe_sorting_get_workspace_size(T, E, K, policy);
            if((ws_bytes == 0) != (policy != 2)) { std::fprintf(stderr, "workspace size %d with policy %d\n", ws_bytes, policy); return 7; }
            void* ws = nullptr;
            if(ws_bytes > 0) HIP_OK(hipMalloc(&ws, ws_bytes));
            sa.p_ws = ws;
            sa.tokens = T; sa.unit_size = U; sa.num_experts = E; sa.topk = K;
            if(mi355::moe_sorting(st, sa) != 0.f) { std::fprintf(stderr, "moe_sorting failed\n"); return 7; }
            HIP_OK(hipDeviceSynchronize());
            HIP_OK(hipMemcpy(q_ids.data(), sa.p_sorted_token_ids, q_ids.size() * 4, hipMemcpyDeviceToHost));
            HIP_OK(hipMemcpy(q_eid.data(), sa.p_sorted_expert_ids, q_eid.size() * 4, hipMemcpyDeviceToHost));
            HIP_OK(hipMemcpy(q_tot.data(), sa.p_total_tokens_post_pad, 8, hipMemcpyDeviceToHost));
            if(q_tot[0] != r_pp || std::memcmp(q_ids.data(), r_ids.data(), sizeof(int32_t) * r_pp) != 0 ||
               std::memcmp(q_eid.data(), r_eid.data(), sizeof(int32_t) * (r_pp / U)) != 0 || q_eid[r_pp / U - 1] != E - 1)
            { std::fprintf(stderr, "moe_sorting without the empty-expert skip differs from the oracle (policy %d)\n", policy); return 8; }
        }
    }
    // unsupported traits report -1 like CK's dispatcher; timing returns milliseconds
    mi355::fused_moe_traits bad = traits; bad.prec_i = "fp16"; bad.prec_w = "fp16";
    const float unsupported = mi355::fused_moe(bad, args);
    mi355::stream_config timed; timed.time_kernel_ = true; timed.cold_niters_ = 1; timed.nrepeat_ = 3;
    const float ms = mi355::fused_moe(traits, args, timed);
    std::printf("host_api_check: post_pad=%d rel-L2=%.3e unsupported=%g timed_ms=%.4f\n", post_pad, err, unsupported, ms);
    return (err <= 1e-2 && unsupported == -1.f && ms > 0.f) ? 0 : 1;
}
