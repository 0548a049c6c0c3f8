// Thin C wrapper that instantiates Composable Kernel's own host reference for the fused-MoE
// path, straight from the ck_tile headers installed with ROCm (/opt/rocm/include/ck_tile,
// CK 1.2.0 @ 69f44ce42ce0a5f46fba094695a1e7948d5c6679).  Nothing from ck_tile is copied here:
// the headers are compiled where they lie and the result goes to oracle/_ref/libck_ref.so.
//
// TEST INFRASTRUCTURE ONLY: used to validate oracle/moe_oracle.c, to write the golden
// fixtures, and as the "reference" CPU baseline.  The product never loads it.
//
//   ck_ref_moe_sorting   -> ck_tile::reference_moe_sorting  (host/reference/reference_moe_sorting.hpp:14)
//   ck_ref_fused_moe_*   -> ck_tile::reference_fused_moe    (host/reference/reference_fused_moe.hpp:42)
#include <cstring> // must precede the ck_tile headers (host memcpy overload)
#include <cstdint>
#include <vector>

#include "ck_tile/core.hpp"
#include "ck_tile/host/host_tensor.hpp"
#include "ck_tile/ops/elementwise/unary_element_wise_operation.hpp"
#include "ck_tile/host/reference/reference_moe_sorting.hpp"
#include "ck_tile/host/reference/reference_fused_moe.hpp"
#include "ck_tile/host/reference/reference_softmax.hpp"
#include "ck_tile/host/reference/reference_topk.hpp"
#include "ck_tile/host/reference/reference_rowwise_quantization2d.hpp"
#include "ck_tile/host/reference/reference_permute.hpp"
#include "ck_tile/host/device_prop.hpp"
#include "ck_tile/host/tensor_shuffle_utils.hpp"


using ck_tile::HostTensor;
using ck_tile::index_t;

namespace {

template <typename T>
HostTensor<T> make_tensor(std::vector<std::size_t> lens, const void* src)
{
    HostTensor<T> t(lens);
    if(src)
        std::memcpy(t.data(), src, t.get_element_space_size_in_bytes());
    return t;
}

template <typename AT, typename GT, typename DT, typename Act, typename OT = ck_tile::bf16_t>
int run_fused(const void* a, const void* g, const void* d, void* o_bf16,
              const int32_t* sorted_ids, const float* sorted_w, const int32_t* sorted_eid,
              int32_t post_pad, int32_t block_m, int32_t T, int32_t E, int32_t H, int32_t I,
              int32_t K, int32_t gate_only)
{
    const std::size_t n0      = static_cast<std::size_t>(I) * (gate_only ? 1 : 2);
    const std::size_t max_pad = static_cast<std::size_t>(K) * T + static_cast<std::size_t>(E) * block_m - K;
    const std::size_t tiles   = (max_pad + block_m - 1) / block_m;

    auto a_h = make_tensor<AT>({(std::size_t)T, (std::size_t)H}, a);
    auto g_h = make_tensor<GT>({(std::size_t)E, n0, (std::size_t)H}, g);
    auto d_h = make_tensor<DT>({(std::size_t)E, (std::size_t)H, (std::size_t)I}, d);
    HostTensor<float> sa({(std::size_t)T}), sg({(std::size_t)E, n0}), sd({(std::size_t)E, (std::size_t)H}),
        sy({(std::size_t)E, (std::size_t)I});
    HostTensor<OT> o_h({(std::size_t)T, (std::size_t)H});
    static_assert(sizeof(OT) == 2, "16-bit output types");
    auto ids_h = make_tensor<index_t>({max_pad}, nullptr);
    auto w_h   = make_tensor<float>({max_pad}, nullptr);
    auto eid_h = make_tensor<index_t>({tiles}, nullptr);
    // only the written prefix is defined; the reference never looks past post_pad
    std::memcpy(ids_h.data(), sorted_ids, sizeof(int32_t) * post_pad);
    std::memcpy(w_h.data(), sorted_w, sizeof(float) * post_pad);
    std::memcpy(eid_h.data(), sorted_eid, sizeof(int32_t) * (post_pad / block_m));
    HostTensor<index_t> nst({1});
    nst.mData[0] = post_pad;
    HostTensor<index_t> topk_ids({(std::size_t)T, (std::size_t)K}); // unused under MOCK_ID

    ck_tile::reference_fused_moe<float, Act>(
        a_h, g_h, d_h, sa, sg, sd, sy, o_h, ids_h, w_h, eid_h, nst, topk_ids, block_m, T, E, H, I, K,
        gate_only);
    std::memcpy(o_bf16, o_h.data(), sizeof(uint16_t) * (std::size_t)T * H);
    return 0;
}

template <int NW, int KW>
struct WarpTile
{
    static constexpr int N_Warp_Tile = NW;
    static constexpr int K_Warp_Tile = KW;
};
template <typename T, int NW, int KW>
void shuffle_b_into(const void* x, int32_t n, int32_t k, void* y)
{
    // (shuffle_b reads the lengths as [k, n] and copies the elements in storage order, n-major)
    auto t = make_tensor<T>({(std::size_t)k, (std::size_t)n}, x);
    auto s = ck_tile::shuffle_b<WarpTile<NW, KW>>(t);
    std::memcpy(y, s.data(), sizeof(T) * (std::size_t)n * k);
}

} // namespace

extern "C" {

__attribute__((visibility("default"))) int ck_ref_mock_id_enabled()
{
    return CK_TILE_REFERENCE_MOE_SORTING_MOCK_ID;
}

// returns post_pad (tokens after padding); outputs sized max_pad / ceil(max_pad/unit)
__attribute__((visibility("default"))) int
ck_ref_moe_sorting(const int32_t* topk_ids, const float* weights, const int32_t* local_expert_mask,
                   int32_t T, int32_t K, int32_t E, int32_t unit_size, int32_t local_expert_masking,
                   int32_t skip_empty, int32_t* sorted_ids, float* sorted_w, int32_t* sorted_eid)
{
    const std::size_t max_pad = static_cast<std::size_t>(K) * T + static_cast<std::size_t>(E) * unit_size - K;
    const std::size_t tiles   = (max_pad + unit_size - 1) / unit_size;
    auto ids_h  = make_tensor<index_t>({(std::size_t)T, (std::size_t)K}, topk_ids);
    auto w_h    = make_tensor<float>({(std::size_t)T, (std::size_t)K}, weights);
    auto mask_h = make_tensor<index_t>({(std::size_t)E}, local_expert_mask);
    if(!local_expert_mask)
        for(auto& m : mask_h.mData)
            m = 1;
    // the reference leaves cells past the written prefix untouched: pre-fill with the caller's
    auto so = make_tensor<index_t>({max_pad}, sorted_ids);
    auto sw = make_tensor<float>({max_pad}, sorted_w);
    auto se = make_tensor<index_t>({tiles}, sorted_eid);
    index_t cnt = 0;
    ck_tile::reference_moe_sorting<float, index_t>(ids_h, w_h, mask_h, so, sw, se, cnt, E, unit_size,
                                                   T, local_expert_masking != 0, skip_empty != 0);
    std::memcpy(sorted_ids, so.data(), sizeof(int32_t) * max_pad);
    std::memcpy(sorted_w, sw.data(), sizeof(float) * max_pad);
    std::memcpy(sorted_eid, se.data(), sizeof(int32_t) * tiles);
    return cnt;
}

// bf16 activations and weights, bf16 output (the bf16 benchmark configurations)
__attribute__((visibility("default"))) int
ck_ref_fused_moe_bf16(const void* a, const void* g, const void* d, void* o, const int32_t* sorted_ids,
                      const float* sorted_w, const int32_t* sorted_eid, int32_t post_pad,
                      int32_t block_m, int32_t T, int32_t E, int32_t H, int32_t I, int32_t K,
                      int32_t gate_only, int32_t activation)
{
    // activation codes of the example's fused_moe_traits: 0 = gelu, 1 = silu
    if(activation == 0)
        return run_fused<ck_tile::bf16_t, ck_tile::bf16_t, ck_tile::bf16_t, ck_tile::element_wise::Gelu>(
            a, g, d, o, sorted_ids, sorted_w, sorted_eid, post_pad, block_m, T, E, H, I, K, gate_only);
    return run_fused<ck_tile::bf16_t, ck_tile::bf16_t, ck_tile::bf16_t, ck_tile::element_wise::Silu>(
        a, g, d, o, sorted_ids, sorted_w, sorted_eid, post_pad, block_m, T, E, H, I, K, gate_only);
}

// fp16 activations, weights and output (ck_tile's other fused-MoE instance)
__attribute__((visibility("default"))) int
ck_ref_fused_moe_f16(const void* a, const void* g, const void* d, void* o, const int32_t* sorted_ids,
                     const float* sorted_w, const int32_t* sorted_eid, int32_t post_pad,
                     int32_t block_m, int32_t T, int32_t E, int32_t H, int32_t I, int32_t K,
                     int32_t gate_only, int32_t activation)
{
    using h = ck_tile::half_t;
    if(activation == 0)
        return run_fused<h, h, h, ck_tile::element_wise::Gelu, h>(a, g, d, o, sorted_ids, sorted_w, sorted_eid, post_pad,
                                                                  block_m, T, E, H, I, K, gate_only);
    return run_fused<h, h, h, ck_tile::element_wise::Silu, h>(a, g, d, o, sorted_ids, sorted_w, sorted_eid, post_pad,
                                                              block_m, T, E, H, I, K, gate_only);
}

// fp32 (de-quantised) activations and weights, bf16 output: the definition used for the
// quantised configs, because the reference ignores its scale tensors
__attribute__((visibility("default"))) int
ck_ref_fused_moe_f32(const void* a, const void* g, const void* d, void* o, const int32_t* sorted_ids,
                     const float* sorted_w, const int32_t* sorted_eid, int32_t post_pad,
                     int32_t block_m, int32_t T, int32_t E, int32_t H, int32_t I, int32_t K,
                     int32_t gate_only, int32_t activation)
{
    if(activation == 0)
        return run_fused<float, float, float, ck_tile::element_wise::Gelu>(
            a, g, d, o, sorted_ids, sorted_w, sorted_eid, post_pad, block_m, T, E, H, I, K, gate_only);
    return run_fused<float, float, float, ck_tile::element_wise::Silu>(
        a, g, d, o, sorted_ids, sorted_w, sorted_eid, post_pad, block_m, T, E, H, I, K, gate_only);
}

// router: reference_softmax over the experts of each row, then reference_topk (sorted, largest)
__attribute__((visibility("default"))) int
ck_ref_topk_softmax(const float* x, int32_t rows, int32_t experts, int32_t topk, float* out_w, int32_t* out_idx)
{
    auto x_h = make_tensor<float>({(std::size_t)rows, (std::size_t)experts}, x);
    HostTensor<float> y_h({(std::size_t)rows, (std::size_t)experts});
    ck_tile::reference_softmax<float, float, float>(x_h, y_h);
    HostTensor<float> v_h({(std::size_t)rows, (std::size_t)topk});
    HostTensor<index_t> i_h({(std::size_t)rows, (std::size_t)topk});
    ck_tile::reference_topk<float, index_t>(y_h, v_h, i_h, topk);
    std::memcpy(out_w, v_h.data(), sizeof(float) * (std::size_t)rows * topk);
    std::memcpy(out_idx, i_h.data(), sizeof(int32_t) * (std::size_t)rows * topk);
    return 0;
}

// reference_rowwise_quantization2d on fp32 rows with caller-provided scales; q_is_fp8: e4m3 else int8
__attribute__((visibility("default"))) int
ck_ref_rowwise_quant(const float* x, const float* scale, int32_t M, int32_t N, int32_t q_is_fp8, void* q)
{
    auto x_h = make_tensor<float>({(std::size_t)M, (std::size_t)N}, x);
    auto s_h = make_tensor<float>({(std::size_t)M}, scale);
    if(q_is_fp8)
    {
        HostTensor<ck_tile::fp8_t> q_h({(std::size_t)M, (std::size_t)N});
        ck_tile::reference_rowwise_quantization2d<float, float, ck_tile::fp8_t>(x_h, s_h, q_h);
        std::memcpy(q, q_h.data(), (std::size_t)M * N);
    }
    else
    {
        HostTensor<ck_tile::int8_t> q_h({(std::size_t)M, (std::size_t)N});
        ck_tile::reference_rowwise_quantization2d<float, float, ck_tile::int8_t>(x_h, s_h, q_h);
        std::memcpy(q, q_h.data(), (std::size_t)M * N);
    }
    return 0;
}

// reference_permute with (0, 1, 3, 4, 2, 5) on the byte view [e, nr, nw, kr, kw, kv_bytes]
__attribute__((visibility("default"))) int
ck_ref_permute_b_nr_kr_kw_nw_kv(const uint8_t* x, int32_t e, int32_t nr, int32_t nw, int32_t kr, int32_t kw,
                                int32_t kv_bytes, uint8_t* y)
{
    auto x_h = make_tensor<uint8_t>({(std::size_t)e, (std::size_t)nr, (std::size_t)nw, (std::size_t)kr, (std::size_t)kw,
                                     (std::size_t)kv_bytes}, x);
    auto y_h = ck_tile::reference_permute(x_h, {0, 1, 3, 4, 2, 5});
    std::memcpy(y, y_h.data(), (std::size_t)e * nr * nw * kr * kw * kv_bytes);
    return 0;
}

// ck_tile::shuffle_b (host/tensor_shuffle_utils.hpp:26-68), what a flatmm caller applies to B before the call, for
// one [n, k] matrix of 1-byte or 2-byte elements and a GemmConfig with the given warp tile (16 x 32 or 32 x 16
// elements for 2-byte types, 16 x 64 for 1-byte types).  Without a device the gfx9 branch runs, which is gfx950's.
__attribute__((visibility("default"))) int
ck_ref_shuffle_b(const void* x, int32_t n, int32_t k, int32_t elem_bytes, int32_t n_warp, int32_t k_warp, void* y)
{
    if(elem_bytes == 2 && n_warp == 16 && k_warp == 32)
        shuffle_b_into<uint16_t, 16, 32>(x, n, k, y);
    else if(elem_bytes == 2 && n_warp == 32 && k_warp == 16)
        shuffle_b_into<uint16_t, 32, 16>(x, n, k, y);
    else if(elem_bytes == 1 && n_warp == 16 && k_warp == 64)
        shuffle_b_into<uint8_t, 16, 64>(x, n, k, y);
    else
        return -1;
    return 0;
}

// scalar conversions of the reference, for pinning the oracle's bf16 / e4m3 tables
__attribute__((visibility("default"))) uint16_t ck_ref_f32_to_bf16(float f)
{
    return ck_tile::bit_cast<uint16_t>(ck_tile::type_convert<ck_tile::bf16_t>(f));
}
__attribute__((visibility("default"))) uint8_t ck_ref_f32_to_fp8(float f)
{
    return ck_tile::bit_cast<uint8_t>(ck_tile::type_convert<ck_tile::fp8_t>(f));
}
__attribute__((visibility("default"))) float ck_ref_fp8_to_f32(uint8_t v)
{
    return ck_tile::type_convert<float>(ck_tile::bit_cast<ck_tile::fp8_t>(v));
}
__attribute__((visibility("default"))) float ck_ref_silu(float x)
{
    float y;
    ck_tile::element_wise::Silu{}(y, x);
    return y;
}
__attribute__((visibility("default"))) float ck_ref_gelu(float x)
{
    float y;
    ck_tile::element_wise::Gelu{}(y, x);
    return y;
}
}
