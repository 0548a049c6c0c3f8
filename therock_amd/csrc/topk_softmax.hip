// Router front-end: softmax (or sigmoid) over the expert logits of a token, then the top-k experts
// and their weights.  Replaces ck_tile::TopkSoftmaxKernel behind TopkSoftmaxHostArgs
// (ops/topk_softmax/kernel/topk_softmax_kernel.hpp:15-25, pipeline
// ops/topk_softmax/pipeline/topk_softmax_warp_per_row_pipeline.hpp:25-140); numerics follow
// ck_tile::reference_softmax + reference_topk (host/reference/reference_softmax.hpp:12-78,
// host/reference/reference_topk.hpp:30-103): fp32 throughout, values in descending order.  Equal
// values are ordered by expert id, lowest first (the reference leaves ties to std::nth_element).
//
// One wave per token: lane l holds experts l, l + 64, ... in registers (up to 1024 experts), the row
// maximum, the sum and each of the k arg-max rounds are wave reductions.  The work is a single pass
// over tokens * experts logits, so it is bound by reading them.
#include "common.hpp"

#include <type_traits>
#include "device_utils.hpp"

namespace mi355 {
namespace {

constexpr int kRouterBlock = 256;
constexpr int kRouterWaves = kRouterBlock / kWave;
constexpr int kMaxPerLane  = 16; // experts per lane: 1024 experts at most

struct RouterParams
{
    const void* input;
    float* output;
    int* indices;
    int rows, experts, topk, stride_in, stride_out;
    int sigmoid, renorm;
};

__device__ inline float wave_max(float v)
{
#pragma unroll
    for(int d = 32; d > 0; d >>= 1)
        v = fmaxf(v, __shfl_xor(v, d));
    return v;
}
__device__ inline float wave_sum(float v)
{
#pragma unroll
    for(int d = 32; d > 0; d >>= 1)
        v += __shfl_xor(v, d);
    return v;
}

template <typename In, int PER_LANE>
__global__ __launch_bounds__(kRouterBlock) void topk_softmax_kernel(const RouterParams p)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int row  = blockIdx.x * kRouterWaves + (threadIdx.x / kWave);
    if(row >= p.rows)
        return;
    const In* x = static_cast<const In*>(p.input) + (int64_t)row * p.stride_in;
    float v[PER_LANE];
#pragma unroll
    for(int j = 0; j < PER_LANE; j++)
    {
        const int e = lane + j * kWave;
        float t     = -INFINITY;
        if(e < p.experts)
        {
            if constexpr(std::is_same_v<In, float>)
                t = x[e];
            else if constexpr(std::is_same_v<In, _Float16>)
                t = static_cast<float>(x[e]);
            else
                t = bf16_bits_to_float(x[e]);
        }
        v[j] = t;
    }
    if(p.sigmoid)
    {
#pragma unroll
        for(int j = 0; j < PER_LANE; j++)
            v[j] = lane + j * kWave < p.experts ? 1.0f / (1.0f + expf(-v[j])) : -INFINITY;
    }
    else
    {
        float m = -INFINITY;
#pragma unroll
        for(int j = 0; j < PER_LANE; j++)
            m = fmaxf(m, v[j]);
        m       = wave_max(m);
        float s = 0.f;
#pragma unroll
        for(int j = 0; j < PER_LANE; j++)
        {
            v[j] = lane + j * kWave < p.experts ? expf(v[j] - m) : 0.f;
            s += v[j];
        }
        s = wave_sum(s);
#pragma unroll
        for(int j = 0; j < PER_LANE; j++)
            v[j] = lane + j * kWave < p.experts ? v[j] / s : -INFINITY;
    }
    // k rounds of arg-max.  The probabilities are non-negative, so their bit patterns order like unsigned integers:
    // key = bits + 1 for a live entry, 0 for one that is struck out or beyond the expert count.  A round is two
    // wave reductions: the largest key, then the lowest expert id among the entries that hold it.  The winner is
    // struck out of its lane's registers and kept by lane i.
    uint32_t key[PER_LANE];
#pragma unroll
    for(int j = 0; j < PER_LANE; j++)
        key[j] = v[j] >= 0.f ? __float_as_uint(v[j]) + 1u : 0u;
    float my_w = 0.f;
    int my_e   = 0;
    float sum  = 0.f;
    for(int i = 0; i < p.topk; i++)
    {
        uint32_t bk = 0u;
        int be      = 0x7fffffff;
#pragma unroll
        for(int j = 0; j < PER_LANE; j++)
            if(key[j] > bk)
            {
                bk = key[j];
                be = lane + j * kWave;
            }
        const uint32_t top = wave_reduce_u32<true>(bk);
        const int win      = static_cast<int>(wave_reduce_u32<false>(bk == top ? static_cast<uint32_t>(be) : 0x7fffffffu));
        const float best   = top != 0u ? __uint_as_float(top - 1u) : -INFINITY;
#pragma unroll
        for(int j = 0; j < PER_LANE; j++)
            if(lane + j * kWave == win)
                key[j] = 0u;
        sum += best;
        if(lane == i)
        {
            my_w = best;
            my_e = win;
        }
    }
    if(lane < p.topk)
    {
        p.output[(int64_t)row * p.stride_out + lane]  = p.renorm ? my_w / sum : my_w;
        p.indices[(int64_t)row * p.stride_out + lane] = my_e;
    }
}

template <typename In>
int launch_t(const RouterParams& p, hipStream_t stream)
{
    const int grid = ceil_div(p.rows, kRouterWaves);
    KernelTimer timer(MI355_MOE_K_ROUTER, stream);
    const int per_lane = ceil_div(p.experts, kWave);
    if(per_lane <= 1)
        hipLaunchKernelGGL((topk_softmax_kernel<In, 1>), dim3(grid), dim3(kRouterBlock), 0, stream, p);
    else if(per_lane <= 2)
        hipLaunchKernelGGL((topk_softmax_kernel<In, 2>), dim3(grid), dim3(kRouterBlock), 0, stream, p);
    else if(per_lane <= 4)
        hipLaunchKernelGGL((topk_softmax_kernel<In, 4>), dim3(grid), dim3(kRouterBlock), 0, stream, p);
    else if(per_lane <= 8)
        hipLaunchKernelGGL((topk_softmax_kernel<In, 8>), dim3(grid), dim3(kRouterBlock), 0, stream, p);
    else
        hipLaunchKernelGGL((topk_softmax_kernel<In, kMaxPerLane>), dim3(grid), dim3(kRouterBlock), 0, stream, p);
    MI355_HIP_TRY(hipGetLastError());
    return MI355_MOE_OK;
}

} // namespace

int launch_topk_softmax(const mi355_topk_softmax_traits& t, const mi355_topk_softmax_args& a, hipStream_t stream)
{
    if(t.input_type != MI355_MOE_FP32 && t.input_type != MI355_MOE_BF16 && t.input_type != MI355_MOE_FP16)
        return fail(MI355_MOE_E_UNSUPPORTED, "topk_softmax: input type %d (fp32, bf16 and fp16 are implemented)", t.input_type);
    if(t.weight_type != MI355_MOE_FP32)
        return fail(MI355_MOE_E_UNSUPPORTED, "topk_softmax: weight type must be fp32");
    if(t.activation != 0 && t.activation != 1)
        return fail(MI355_MOE_E_UNSUPPORTED, "topk_softmax: activation %d (0 = softmax, 1 = sigmoid)", t.activation);
    if(a.num_rows < 0 || a.num_experts <= 0 || a.num_experts > kWave * kMaxPerLane || a.topk <= 0 ||
       a.topk > a.num_experts || a.topk > kWave || a.stride_input < a.num_experts || a.stride_output < a.topk)
        return fail(MI355_MOE_E_INVALID, "topk_softmax: bad sizes (rows=%d experts=%d topk=%d strides=%d,%d)", a.num_rows,
                    a.num_experts, a.topk, a.stride_input, a.stride_output);
    if(a.num_rows == 0)
        return MI355_MOE_OK;
    if(!a.p_input || !a.p_output || !a.p_indices)
        return fail(MI355_MOE_E_INVALID, "topk_softmax: null pointer");
    RouterParams p{a.p_input, static_cast<float*>(a.p_output), static_cast<int*>(a.p_indices), a.num_rows, a.num_experts,
                   a.topk,    a.stride_input, a.stride_output, t.activation, t.renormalize};
    if(t.input_type == MI355_MOE_FP32)
        return launch_t<float>(p, stream);
    return t.input_type == MI355_MOE_FP16 ? launch_t<_Float16>(p, stream) : launch_t<uint16_t>(p, stream);
}

} // namespace mi355
