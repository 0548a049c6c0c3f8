// Data-preparation kernels around the fused-MoE GEMMs for gfx950: per-row dynamic quantisation, ck_tile's
// MoE smooth-quant, and the conversion to and from ck_tile's pre-shuffled weight layout.  All of them are
// HBM-bound byte movers: one pass over the input, coalesced 16-byte accesses, no LDS beyond the row reductions.
#include "moe_gemm_device.hpp"

#include <algorithm>

namespace mi355 {
using namespace gemm;
namespace {

// one value -> e4m3 (round to nearest even, saturating) or int8 (saturate, then ck_tile's float -> int8
// static_cast: truncation toward zero)
template <bool FP8>
__device__ inline unsigned char quantise_one(float v)
{
    if constexpr(FP8)
    {
        const float cl = fminf(fmaxf(v, -448.f), 448.f);
        return static_cast<unsigned char>(__builtin_amdgcn_cvt_pk_fp8_f32(cl, cl, 0, false) & 0xff);
    }
    else
    {
        const float cl = fminf(fmaxf(v, -128.f), 127.f);
        return static_cast<unsigned char>(static_cast<signed char>(static_cast<int>(cl)));
    }
}

// eight quotients o[i] * (1 / s) -> eight codes in two dwords.  e4m3: the conversion instruction packs two codes
// into a chosen half of a dword, so four of them fill both dwords with no masking or shifting.
template <bool FP8>
__device__ inline uint2 quantise_8(const float (&o)[8], double s_rcp)
{
    if constexpr(FP8)
    {
        float c[8];
#pragma unroll
        for(int i = 0; i < 8; i++)
            c[i] = fminf(fmaxf(div_by_row_scale(o[i], s_rcp), -448.f), 448.f);
        int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], 0, false);
        w0     = __builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], w0, true);
        int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(c[4], c[5], 0, false);
        w1     = __builtin_amdgcn_cvt_pk_fp8_f32(c[6], c[7], w1, true);
        return make_uint2(static_cast<uint32_t>(w0), static_cast<uint32_t>(w1));
    }
    else
    {
        uint32_t w[2] = {0u, 0u};
#pragma unroll
        for(int i = 0; i < 8; i++)
            w[i >> 2] |= static_cast<uint32_t>(quantise_one<false>(div_by_row_scale(o[i], s_rcp))) << (8 * (i & 3));
        return make_uint2(w[0], w[1]);
    }
}

__device__ inline float block_max_256(float v, float* s_red)
{
#pragma unroll
    for(int d = 32; d > 0; d >>= 1)
        v = fmaxf(v, __shfl_xor(v, d));
    if((threadIdx.x & 63) == 0)
        s_red[threadIdx.x >> 6] = v;
    __syncthreads();
    return fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
}

// Per-row dynamic quantisation of one row by one 256-thread workgroup: xr bf16 (times sr fp32 when SMOOTH),
// scale = amax / qmax, q = quantise(value / scale).  With VEC the row is walked in 16-byte pieces of 8 elements
// (cols % 8 == 0, 16-byte aligned rows); the first kCache pieces of every thread stay in registers between the
// two passes, so rows of up to 8192 columns are read once.  Returns the row's amax to every thread.
constexpr int kQuantCache = 4;
template <bool FP8, bool SMOOTH, bool VEC>
__device__ inline float quantise_row(const uint16_t* __restrict__ xr, const float* __restrict__ sr, int cols,
                                     unsigned char* __restrict__ qr, float* s_red, bool unit_scale_when_zero, float* scale_out)
{
    const float qmx = FP8 ? 448.0f : 127.0f;
    if constexpr(VEC)
    {
        const int chunks = cols >> 3;
        float v[kQuantCache][8];
        auto load = [&](int c, float (&o)[8]) {
            const uint4 r = *reinterpret_cast<const uint4*>(xr + c * 8);
            const uint32_t d[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
            for(int i = 0; i < 4; i++)
            {
                o[2 * i]     = __uint_as_float(d[i] << 16);
                o[2 * i + 1] = __uint_as_float(d[i] & 0xffff0000u);
            }
            if constexpr(SMOOTH)
            {
                const float4 s0 = *reinterpret_cast<const float4*>(sr + c * 8);
                const float4 s1 = *reinterpret_cast<const float4*>(sr + c * 8 + 4);
                o[0] *= s0.x; o[1] *= s0.y; o[2] *= s0.z; o[3] *= s0.w;
                o[4] *= s1.x; o[5] *= s1.y; o[6] *= s1.z; o[7] *= s1.w;
            }
        };
        float amax = 0.f;
#pragma unroll
        for(int j = 0; j < kQuantCache; j++)
        {
            const int c = threadIdx.x + 256 * j;
            if(c < chunks)
            {
                load(c, v[j]);
#pragma unroll
                for(int i = 0; i < 8; i++)
                    amax = fmaxf(amax, fabsf(v[j][i]));
            }
        }
        for(int c = threadIdx.x + 256 * kQuantCache; c < chunks; c += 256)
        {
            float t[8];
            load(c, t);
#pragma unroll
            for(int i = 0; i < 8; i++)
                amax = fmaxf(amax, fabsf(t[i]));
        }
        amax          = block_max_256(amax, s_red);
        // a row of zeros: the scale written is 1 (row-wise quant) or 0 (smooth-quant, as amax / qmax gives);
        // either way the row's codes are 0, never the 0 / 0 the plain formula would convert
        const float s_out = (amax > 0.f || !unit_scale_when_zero) ? amax / qmx : 1.0f;
        const float s     = amax > 0.f ? s_out : 1.0f;
        if(threadIdx.x == 0)
            *scale_out = s_out;
        const double s_rcp = row_reciprocal(s);
        auto store = [&](int c, const float (&o)[8]) { *reinterpret_cast<uint2*>(qr + c * 8) = quantise_8<FP8>(o, s_rcp); };
#pragma unroll
        for(int j = 0; j < kQuantCache; j++)
        {
            const int c = threadIdx.x + 256 * j;
            if(c < chunks)
                store(c, v[j]);
        }
        for(int c = threadIdx.x + 256 * kQuantCache; c < chunks; c += 256)
        {
            float t[8];
            load(c, t);
            store(c, t);
        }
        return amax;
    }
    else
    {
        float amax = 0.f;
        for(int c = threadIdx.x; c < cols; c += 256)
            amax = fmaxf(amax, fabsf(bf16_bits_to_float(xr[c]) * (SMOOTH ? sr[c] : 1.0f)));
        amax          = block_max_256(amax, s_red);
        // a row of zeros: the scale written is 1 (row-wise quant) or 0 (smooth-quant, as amax / qmax gives);
        // either way the row's codes are 0, never the 0 / 0 the plain formula would convert
        const float s_out = (amax > 0.f || !unit_scale_when_zero) ? amax / qmx : 1.0f;
        const float s     = amax > 0.f ? s_out : 1.0f;
        if(threadIdx.x == 0)
            *scale_out = s_out;
        const double s_rcp = row_reciprocal(s);
        for(int c = threadIdx.x; c < cols; c += 256)
            qr[c] = quantise_one<FP8>(div_by_row_scale(bf16_bits_to_float(xr[c]) * (SMOOTH ? sr[c] : 1.0f), s_rcp));
        return amax;
    }
}

// per-row dynamic quantisation bf16 -> e4m3 / int8
template <bool FP8, bool VEC>
__global__ __launch_bounds__(256) void rowwise_quant_kernel(const uint16_t* __restrict__ x, int cols,
                                                             int64_t stride_x, unsigned char* __restrict__ q,
                                                             float* __restrict__ scale)
{
    __shared__ float s_red[4];
    const int64_t row = blockIdx.x;
    quantise_row<FP8, false, VEC>(x + row * stride_x, nullptr, cols, q + row * cols, s_red, true, scale + row);
}

// MoE smooth-quant: row (slot k, token t) = x[t, :] * smscale[expert(t, k), :], per-row dynamic quantisation.
// Scalar form: one workgroup per (token, slot).
template <bool FP8>
__global__ __launch_bounds__(256) void moe_smoothquant_kernel(const uint16_t* __restrict__ x,
                                                               const float* __restrict__ smscale,
                                                               const int* __restrict__ topk_ids, int tokens, int hidden,
                                                               int experts, int topk, int64_t x_stride, int64_t y_stride,
                                                               unsigned char* __restrict__ qy, float* __restrict__ yscale)
{
    __shared__ float s_red[4];
    const int t = blockIdx.x;
    const int k = blockIdx.y;
    int e       = topk_ids[(int64_t)t * topk + k];
    e           = min(max(e, 0), experts - 1);
    const int64_t r = (int64_t)k * tokens + t;
    quantise_row<FP8, true, false>(x + (int64_t)t * x_stride, smscale + (int64_t)e * hidden, hidden, qy + r * y_stride, s_red,
                                   false, yscale + r);
}

// Vector form (hidden % 8 == 0, aligned rows): one workgroup per token walks its slots, so the token's row is
// read once (its first kQuantCache pieces per thread stay in registers) and only the experts' smooth scales and
// the quantised rows move per slot.
template <bool FP8>
__global__ __launch_bounds__(256) void moe_smoothquant_vec_kernel(const uint16_t* __restrict__ x,
                                                                   const float* __restrict__ smscale,
                                                                   const int* __restrict__ topk_ids, int tokens,
                                                                   int hidden, int experts, int topk, int64_t x_stride,
                                                                   int64_t y_stride, unsigned char* __restrict__ qy,
                                                                   float* __restrict__ yscale)
{
    __shared__ float s_red[2][4];
    const int t        = blockIdx.x;
    const uint16_t* xr = x + (int64_t)t * x_stride;
    const int chunks   = hidden >> 3;
    const float qmx    = FP8 ? 448.0f : 127.0f;
    auto load_x = [&](int c, float (&o)[8]) {
        const uint4 r = *reinterpret_cast<const uint4*>(xr + c * 8);
        const uint32_t d[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for(int i = 0; i < 4; i++)
        {
            o[2 * i]     = __uint_as_float(d[i] << 16);
            o[2 * i + 1] = __uint_as_float(d[i] & 0xffff0000u);
        }
    };
    auto times_sm = [&](const float* sr, int c, const float (&in)[8], float (&o)[8]) {
        const float4 s0 = *reinterpret_cast<const float4*>(sr + c * 8);
        const float4 s1 = *reinterpret_cast<const float4*>(sr + c * 8 + 4);
        o[0] = in[0] * s0.x; o[1] = in[1] * s0.y; o[2] = in[2] * s0.z; o[3] = in[3] * s0.w;
        o[4] = in[4] * s1.x; o[5] = in[5] * s1.y; o[6] = in[6] * s1.z; o[7] = in[7] * s1.w;
    };
    auto scales_of_slot = [&](int k) {
        const int e = topk_ids[(int64_t)t * topk + k];
        return smscale + (int64_t)min(max(e, 0), experts - 1) * hidden;
    };
    // the smooth scales of the cached pieces, for the slot about to be processed: fetched one slot ahead, so that
    // their latency passes under the previous slot's reduction, conversions and stores
    float4 sm[kQuantCache][2];
    auto fetch_scales = [&](const float* sr) {
#pragma unroll
        for(int j = 0; j < kQuantCache; j++)
            if(threadIdx.x + 256 * j < chunks)
            {
                sm[j][0] = *reinterpret_cast<const float4*>(sr + (threadIdx.x + 256 * j) * 8);
                sm[j][1] = *reinterpret_cast<const float4*>(sr + (threadIdx.x + 256 * j) * 8 + 4);
            }
    };
    float xv[kQuantCache][8];
#pragma unroll
    for(int j = 0; j < kQuantCache; j++)
        if(threadIdx.x + 256 * j < chunks)
            load_x(threadIdx.x + 256 * j, xv[j]);
    if(topk > 0)
        fetch_scales(scales_of_slot(0));
    for(int k = 0; k < topk; k++)
    {
        const float* sr = scales_of_slot(k);
        float v[kQuantCache][8];
        float amax = 0.f;
#pragma unroll
        for(int j = 0; j < kQuantCache; j++)
        {
            const int c = threadIdx.x + 256 * j;
            if(c < chunks)
            {
                const float4 s0 = sm[j][0], s1 = sm[j][1];
                v[j][0] = xv[j][0] * s0.x; v[j][1] = xv[j][1] * s0.y; v[j][2] = xv[j][2] * s0.z; v[j][3] = xv[j][3] * s0.w;
                v[j][4] = xv[j][4] * s1.x; v[j][5] = xv[j][5] * s1.y; v[j][6] = xv[j][6] * s1.z; v[j][7] = xv[j][7] * s1.w;
#pragma unroll
                for(int i = 0; i < 8; i++)
                    amax = fmaxf(amax, fabsf(v[j][i]));
            }
        }
        if(k + 1 < topk)
            fetch_scales(scales_of_slot(k + 1));
        for(int c = threadIdx.x + 256 * kQuantCache; c < chunks; c += 256)
        {
            float a[8], b[8];
            load_x(c, a);
            times_sm(sr, c, a, b);
#pragma unroll
            for(int i = 0; i < 8; i++)
                amax = fmaxf(amax, fabsf(b[i]));
        }
        amax            = block_max_256(amax, s_red[k & 1]); // two buffers: one barrier per slot suffices
        const float ys_out = amax / qmx;
        const float ys     = amax > 0.f ? ys_out : 1.0f; // a row of zeros: scale 0, codes 0 (not 0 / 0)
        const int64_t r    = (int64_t)k * tokens + t;
        if(threadIdx.x == 0)
            yscale[r] = ys_out;
        unsigned char* qr = qy + r * y_stride;
        const double ys_rcp = row_reciprocal(ys);
        // (streaming stores: the quantised rows are written once and should not push the experts' scales out of L2)
        auto store = [&](int c, const float (&o)[8]) {
            typedef __attribute__((ext_vector_type(2))) unsigned u32x2_t;
            const uint2 q = quantise_8<FP8>(o, ys_rcp);
            __builtin_nontemporal_store(u32x2_t{q.x, q.y}, reinterpret_cast<u32x2_t*>(qr + c * 8));
        };
#pragma unroll
        for(int j = 0; j < kQuantCache; j++)
            if(threadIdx.x + 256 * j < chunks)
                store(threadIdx.x + 256 * j, v[j]);
        for(int c = threadIdx.x + 256 * kQuantCache; c < chunks; c += 256)
        {
            float a[8], b[8];
            load_x(c, a);
            times_sm(sr, c, a, b);
            store(c, b);
        }
    }
}

// Expert-grouped form, for expert tables that do not stay in an XCD's L2 beside the rows streaming through it
// (256 experts x 7168 columns of fp32 are 7.3 MB against 4 MB): a workgroup owns one expert and one range of
// kSqRange tokens.  It keeps the expert's smooth scales in registers (read once per workgroup instead of once per
// row), finds the range's routing entries that name its expert, and quantises those rows one after the other, the
// next row's activations fetched while the current one is reduced and stored.  The workgroups of one token range sit
// on one XCD and run together there (workgroup ids go round the eight XCDs: id = (range / 8 * experts + expert) * 8 +
// range % 8), so that the range's activations come from HBM once and from that XCD's L2 for the other slots.  Each row
// is computed by the same expressions as in the per-token form: the results are the same bits.
constexpr int kSqRange   = 128;  // tokens per range
constexpr int kSqMaxList = 8192; // routing entries of a range (kSqRange x topk)
template <bool FP8>
__global__ __launch_bounds__(256) void moe_smoothquant_grouped_kernel(const uint16_t* __restrict__ x,
                                                                       const float* __restrict__ smscale,
                                                                       const int* __restrict__ topk_ids, int tokens,
                                                                       int hidden, int experts, int topk, int64_t x_stride,
                                                                       int64_t y_stride, unsigned char* __restrict__ qy,
                                                                       float* __restrict__ yscale)
{
    __shared__ float s_red[2][4];
    __shared__ int s_count;
    __shared__ int s_list[kSqMaxList];
    const int xcd   = blockIdx.x & 7;
    const int e     = (blockIdx.x >> 3) % experts;
    const int range = (blockIdx.x >> 3) / experts * 8 + xcd;
    const int t0    = range * kSqRange;
    if(t0 >= tokens)
        return;
    const int nt     = min(kSqRange, tokens - t0);
    const int chunks = hidden >> 3;
    const float qmx  = FP8 ? 448.0f : 127.0f;
    if(threadIdx.x == 0)
        s_count = 0;
    __syncthreads();
    // entries of the range that name this expert (ids outside [0, experts) are clamped like in the other forms)
    const int* ids = topk_ids + (int64_t)t0 * topk;
    for(int i = threadIdx.x; i < nt * topk; i += 256)
        if(min(max(ids[i], 0), experts - 1) == e)
            s_list[atomicAdd(&s_count, 1)] = i;
    __syncthreads();
    const int n = s_count;
    if(n == 0)
        return;
    const float* sr = smscale + (int64_t)e * hidden;
    float4 sm[kQuantCache][2];
#pragma unroll
    for(int j = 0; j < kQuantCache; j++)
        if(threadIdx.x + 256 * j < chunks)
        {
            sm[j][0] = *reinterpret_cast<const float4*>(sr + (threadIdx.x + 256 * j) * 8);
            sm[j][1] = *reinterpret_cast<const float4*>(sr + (threadIdx.x + 256 * j) * 8 + 4);
        }
    auto unpack = [&](const uint4& r, float (&o)[8]) {
        const uint32_t d[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for(int i = 0; i < 4; i++)
        {
            o[2 * i]     = __uint_as_float(d[i] << 16);
            o[2 * i + 1] = __uint_as_float(d[i] & 0xffff0000u);
        }
    };
    auto times_sm = [&](int c, const float (&in)[8], float (&o)[8]) {
        const float4 s0 = *reinterpret_cast<const float4*>(sr + c * 8);
        const float4 s1 = *reinterpret_cast<const float4*>(sr + c * 8 + 4);
        o[0] = in[0] * s0.x; o[1] = in[1] * s0.y; o[2] = in[2] * s0.z; o[3] = in[3] * s0.w;
        o[4] = in[4] * s1.x; o[5] = in[5] * s1.y; o[6] = in[6] * s1.z; o[7] = in[7] * s1.w;
    };
    uint4 raw[kQuantCache];
    auto fetch_row = [&](int entry) {
        const uint16_t* xr = x + (int64_t)(t0 + entry / topk) * x_stride;
#pragma unroll
        for(int j = 0; j < kQuantCache; j++)
            if(threadIdx.x + 256 * j < chunks)
                raw[j] = *reinterpret_cast<const uint4*>(xr + (threadIdx.x + 256 * j) * 8);
    };
    fetch_row(s_list[0]);
    for(int m = 0; m < n; m++)
    {
        const int entry    = s_list[m];
        const int t        = t0 + entry / topk;
        const int k        = entry - (entry / topk) * topk;
        const uint16_t* xr = x + (int64_t)t * x_stride;
        float v[kQuantCache][8];
        float amax = 0.f;
#pragma unroll
        for(int j = 0; j < kQuantCache; j++)
            if(threadIdx.x + 256 * j < chunks)
            {
                float xv[8];
                unpack(raw[j], xv);
                const float4 s0 = sm[j][0], s1 = sm[j][1];
                v[j][0] = xv[0] * s0.x; v[j][1] = xv[1] * s0.y; v[j][2] = xv[2] * s0.z; v[j][3] = xv[3] * s0.w;
                v[j][4] = xv[4] * s1.x; v[j][5] = xv[5] * s1.y; v[j][6] = xv[6] * s1.z; v[j][7] = xv[7] * s1.w;
#pragma unroll
                for(int i = 0; i < 8; i++)
                    amax = fmaxf(amax, fabsf(v[j][i]));
            }
        if(m + 1 < n)
            fetch_row(s_list[m + 1]);
        for(int c = threadIdx.x + 256 * kQuantCache; c < chunks; c += 256)
        {
            float a[8], b[8];
            unpack(*reinterpret_cast<const uint4*>(xr + c * 8), a);
            times_sm(c, a, b);
#pragma unroll
            for(int i = 0; i < 8; i++)
                amax = fmaxf(amax, fabsf(b[i]));
        }
        amax               = block_max_256(amax, s_red[m & 1]); // two buffers: one barrier per row suffices
        const float ys_out = amax / qmx;
        const float ys     = amax > 0.f ? ys_out : 1.0f; // a row of zeros: scale 0, codes 0 (not 0 / 0)
        const int64_t r    = (int64_t)k * tokens + t;
        if(threadIdx.x == 0)
            yscale[r] = ys_out;
        unsigned char* qr   = qy + r * y_stride;
        const double ys_rcp = row_reciprocal(ys);
        auto store = [&](int c, const float (&o)[8]) {
            typedef __attribute__((ext_vector_type(2))) unsigned u32x2_t;
            const uint2 q = quantise_8<FP8>(o, ys_rcp);
            __builtin_nontemporal_store(u32x2_t{q.x, q.y}, reinterpret_cast<u32x2_t*>(qr + c * 8));
        };
#pragma unroll
        for(int j = 0; j < kQuantCache; j++)
            if(threadIdx.x + 256 * j < chunks)
                store(threadIdx.x + 256 * j, v[j]);
        for(int c = threadIdx.x + 256 * kQuantCache; c < chunks; c += 256)
        {
            float a[8], b[8];
            unpack(*reinterpret_cast<const uint4*>(xr + c * 8), a);
            times_sm(c, a, b);
            store(c, b);
        }
    }
}

// Re-quantisation of the intermediate activations between the two GEMMs of the int8 path (fused_quant 1 / 2 of
// ck_tile's fused_moe_traits; y_smooth_scale of FusedMoeGemmHostArgs, fused_moegemm_kernel.hpp:103): sorted row r
// of Y (bf16, row-major) times the smooth scale of its expert (SMOOTH), per-row dynamic quantisation to int8:
// scale = amax / 127, codes rounded to nearest even (|value / scale| <= 127 needs no clamp).  ck_tile has no
// instance of these variants to match bit for bit, so the rounding is chosen for accuracy: truncation, which the
// stand-alone smooth-quant kernel above has to use to match ck_tile's, doubles the error of the down GEMM's
// input.  One wave per row; a row of up to 2048 columns is read once.
// Output row-major, or slab-major when segs > 0 (y_slab_offset); padding rows become zeros with scale 0, rows past
// the sorted prefix are left alone.
// FP8 (the fp8 path with fused_quant): e4m3 codes instead, scale = amax / 448, rounded to nearest even by the
// conversion instruction.
template <bool SMOOTH, bool FP8>
__global__ __launch_bounds__(256) void moe_requant_y_kernel(const uint16_t* __restrict__ y, int inter,
                                                             const float* __restrict__ smooth,
                                                             const int* __restrict__ sorted_ids,
                                                             const int* __restrict__ sorted_expert_ids,
                                                             const int* __restrict__ total, int unit, int tokens, int segs,
                                                             unsigned char* __restrict__ yq, float* __restrict__ yscale)
{
    const int lane    = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if(row >= total[0])
        return;
    const int chunks = inter >> 3;
    auto dst = [&](int c) {
        return yq + (segs > 0 ? y_slab_offset(row, c * 8, segs) : row * inter + c * 8);
    };
    const bool real = (sorted_ids[row] & 0xffffff) < tokens;
    if(!real)
    {
        for(int c = lane; c < chunks; c += 64)
            *reinterpret_cast<uint2*>(dst(c)) = make_uint2(0u, 0u);
        if(lane == 0)
            yscale[row] = 0.f;
        return;
    }
    const uint16_t* yr = y + row * inter;
    const float* sr    = SMOOTH ? smooth + (int64_t)sorted_expert_ids[row / unit] * inter : nullptr;
    auto load = [&](int c, float (&o)[8]) {
        const uint4 r = *reinterpret_cast<const uint4*>(yr + c * 8);
        const uint32_t d[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for(int i = 0; i < 4; i++)
        {
            o[2 * i]     = __uint_as_float(d[i] << 16);
            o[2 * i + 1] = __uint_as_float(d[i] & 0xffff0000u);
        }
        if constexpr(SMOOTH)
        {
            const float4 s0 = *reinterpret_cast<const float4*>(sr + c * 8);
            const float4 s1 = *reinterpret_cast<const float4*>(sr + c * 8 + 4);
            o[0] *= s0.x; o[1] *= s0.y; o[2] *= s0.z; o[3] *= s0.w;
            o[4] *= s1.x; o[5] *= s1.y; o[6] *= s1.z; o[7] *= s1.w;
        }
    };
    float v[kQuantCache][8];
    float amax = 0.f;
#pragma unroll
    for(int j = 0; j < kQuantCache; j++)
    {
        const int c = lane + 64 * j;
        if(c < chunks)
        {
            load(c, v[j]);
#pragma unroll
            for(int i = 0; i < 8; i++)
                amax = fmaxf(amax, fabsf(v[j][i]));
        }
    }
    for(int c = lane + 64 * kQuantCache; c < chunks; c += 64)
    {
        float t[8];
        load(c, t);
#pragma unroll
        for(int i = 0; i < 8; i++)
            amax = fmaxf(amax, fabsf(t[i]));
    }
#pragma unroll
    for(int d = 32; d > 0; d >>= 1)
        amax = fmaxf(amax, __shfl_xor(amax, d));
    const float ys_out = amax / (FP8 ? 448.0f : 127.0f);
    const float ys     = amax > 0.f ? ys_out : 1.0f; // a row of zeros: scale 0, codes 0
    if(lane == 0)
        yscale[row] = ys_out;
    const double ys_rcp = row_reciprocal(ys);
    auto store = [&](int c, const float (&o)[8]) {
        if constexpr(FP8)
            *reinterpret_cast<uint2*>(dst(c)) = quantise_8<true>(o, ys_rcp);
        else
        {
            uint32_t w[2] = {0u, 0u};
#pragma unroll
            for(int i = 0; i < 8; i++)
                w[i >> 2] |= (static_cast<uint32_t>(static_cast<int>(__builtin_rintf(div_by_row_scale(o[i], ys_rcp)))) & 0xffu) << (8 * (i & 3));
            *reinterpret_cast<uint2*>(dst(c)) = make_uint2(w[0], w[1]);
        }
    };
#pragma unroll
    for(int j = 0; j < kQuantCache; j++)
        if(lane + 64 * j < chunks)
            store(lane + 64 * j, v[j]);
    for(int c = lane + 64 * kQuantCache; c < chunks; c += 64)
    {
        float t[8];
        load(c, t);
        store(c, t);
    }
}

// ck_tile's pre-shuffled weight layout b_nr_kr_kw_nw_kv: the row-major [e, n, k] tensor viewed as
// [e, nr, nw, kr, kw, kv] and permuted to [e, nr, kr, kw, nw, kv].  One thread moves one kv granule.
template <typename G>
__global__ __launch_bounds__(256) void permute_weights_kernel(const G* __restrict__ src, G* __restrict__ dst,
                                                               int64_t granules, int n, int kgran, int nw, int kw,
                                                               int inverse)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if(i >= granules)
        return;
    // i enumerates the permuted layout: (e, nr, kr, kw, nw)
    const int kr_n = kgran / kw;
    int64_t r      = i;
    const int a_nw = (int)(r % nw);
    r /= nw;
    const int a_kw = (int)(r % kw);
    r /= kw;
    const int a_kr = (int)(r % kr_n);
    r /= kr_n;
    const int a_nr = (int)(r % (n / nw));
    const int64_t e = r / (n / nw);
    const int64_t row_major = (e * n + (int64_t)a_nr * nw + a_nw) * kgran + (int64_t)a_kr * kw + a_kw;
    if(inverse)
        dst[row_major] = src[i];
    else
        dst[i] = src[row_major];
}

} // namespace

int launch_permute_weights(const void* src, void* dst, int32_t experts, int32_t n, int32_t k, int32_t elem_bytes,
                           int32_t nw, int32_t kw, int32_t kv, int32_t inverse, hipStream_t stream)
{
    if(!src || !dst || src == dst || experts <= 0 || n <= 0 || k <= 0 || nw <= 0 || kw <= 0 || kv <= 0 ||
       (elem_bytes != 1 && elem_bytes != 2))
        return fail(MI355_MOE_E_INVALID, "permute_weights: bad arguments");
    const int gran = kv * elem_bytes;
    if(n % nw != 0 || k % (kw * kv) != 0 || (gran != 4 && gran != 8 && gran != 16))
        return fail(MI355_MOE_E_UNSUPPORTED,
                    "permute_weights: n %% nw, k %% (kw*kv) must be 0 and kv*elem_bytes 4, 8 or 16 (n=%d k=%d nw=%d kw=%d kv=%d)",
                    n, k, nw, kw, kv);
    const int kgran        = k / kv;
    const int64_t granules = (int64_t)experts * n * kgran;
    const unsigned grid    = (unsigned)ceil_div<int64_t>(granules, 256);
    if(gran == 16)
        hipLaunchKernelGGL(permute_weights_kernel<uint4>, dim3(grid), dim3(256), 0, stream, static_cast<const uint4*>(src),
                           static_cast<uint4*>(dst), granules, n, kgran, nw, kw, inverse);
    else if(gran == 8)
        hipLaunchKernelGGL(permute_weights_kernel<uint2>, dim3(grid), dim3(256), 0, stream, static_cast<const uint2*>(src),
                           static_cast<uint2*>(dst), granules, n, kgran, nw, kw, inverse);
    else
        hipLaunchKernelGGL(permute_weights_kernel<uint32_t>, dim3(grid), dim3(256), 0, stream,
                           static_cast<const uint32_t*>(src), static_cast<uint32_t*>(dst), granules, n, kgran, nw, kw, inverse);
    MI355_HIP_TRY(hipGetLastError());
    return MI355_MOE_OK;
}

int launch_moe_smoothquant(const mi355_moe_smoothquant_args& a, int32_t q_dtype, hipStream_t stream)
{
    if(q_dtype != MI355_MOE_FP8 && q_dtype != MI355_MOE_INT8)
        return fail(MI355_MOE_E_UNSUPPORTED, "moe_smoothquant: q_dtype must be fp8 or int8");
    if(a.tokens < 0 || a.hidden_size <= 0 || a.experts <= 0 || a.topk <= 0 || a.topk > 65535 || a.x_stride < a.hidden_size ||
       a.y_stride < a.hidden_size)
        return fail(MI355_MOE_E_INVALID, "moe_smoothquant: bad sizes (tokens=%d hidden=%d experts=%d topk=%d strides=%d,%d)",
                    a.tokens, a.hidden_size, a.experts, a.topk, a.x_stride, a.y_stride);
    if(a.tokens == 0)
        return MI355_MOE_OK;
    if(!a.p_x || !a.p_smscale || !a.p_topk_ids || !a.p_yscale || !a.p_qy)
        return fail(MI355_MOE_E_INVALID, "moe_smoothquant: null pointer");
    KernelTimer timer(MI355_MOE_K_QUANT, stream);
    // 16-byte pieces of 8 elements when every row starts on a 16-byte (output: 8-byte) boundary
    const bool vec = a.hidden_size % 8 == 0 && a.x_stride % 8 == 0 && a.y_stride % 8 == 0 &&
                     reinterpret_cast<uintptr_t>(a.p_x) % 16 == 0 && reinterpret_cast<uintptr_t>(a.p_smscale) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(a.p_qy) % 8 == 0;
    auto launch = [&](auto kernel, dim3 grid) {
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, static_cast<const uint16_t*>(a.p_x),
                           static_cast<const float*>(a.p_smscale), static_cast<const int*>(a.p_topk_ids), a.tokens,
                           a.hidden_size, a.experts, a.topk, (int64_t)a.x_stride, (int64_t)a.y_stride,
                           static_cast<unsigned char*>(a.p_qy), static_cast<float*>(a.p_yscale));
    };
    const dim3 per_token((unsigned)a.tokens), per_row((unsigned)a.tokens, (unsigned)a.topk);
    // expert tables beyond 3 MB do not stay in the 4 MB L2 of an XCD: rows grouped by expert, scales in registers
    const int64_t ranges8 = ceil_div<int64_t>(ceil_div(a.tokens, kSqRange), 8);
    const bool grouped    = vec && (int64_t)a.experts * a.hidden_size * (int64_t)sizeof(float) > (3ll << 20) &&
                         kSqRange * a.topk <= kSqMaxList && ranges8 * a.experts * 8 < (1ll << 31);
    if(grouped)
    {
        const dim3 grid((unsigned)(ranges8 * a.experts * 8));
        q_dtype == MI355_MOE_FP8 ? launch(moe_smoothquant_grouped_kernel<true>, grid)
                                 : launch(moe_smoothquant_grouped_kernel<false>, grid);
    }
    else if(q_dtype == MI355_MOE_FP8)
        vec ? launch(moe_smoothquant_vec_kernel<true>, per_token) : launch(moe_smoothquant_kernel<true>, per_row);
    else
        vec ? launch(moe_smoothquant_vec_kernel<false>, per_token) : launch(moe_smoothquant_kernel<false>, per_row);
    MI355_HIP_TRY(hipGetLastError());
    return MI355_MOE_OK;
}

int launch_rowwise_quant(const void* x, int64_t rows, int32_t cols, int64_t stride_x, int32_t q_dtype, void* q,
                         void* scale, hipStream_t stream)
{
    if(!x || !q || !scale || rows < 0 || cols <= 0 || stride_x < cols)
        return fail(MI355_MOE_E_INVALID, "rowwise_quant: bad arguments");
    if(q_dtype != MI355_MOE_FP8 && q_dtype != MI355_MOE_INT8)
        return fail(MI355_MOE_E_UNSUPPORTED, "rowwise_quant: q_dtype must be fp8 or int8");
    if(rows == 0)
        return MI355_MOE_OK;
    if(rows > 0x7fffffff)
        return fail(MI355_MOE_E_INVALID, "rowwise_quant: too many rows");
    KernelTimer timer(MI355_MOE_K_QUANT, stream);
    const bool vec = cols % 8 == 0 && stride_x % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(q) % 8 == 0;
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)rows), dim3(256), 0, stream, static_cast<const uint16_t*>(x), cols,
                           stride_x, static_cast<unsigned char*>(q), static_cast<float*>(scale));
    };
    if(q_dtype == MI355_MOE_FP8)
        vec ? launch(rowwise_quant_kernel<true, true>) : launch(rowwise_quant_kernel<true, false>);
    else
        vec ? launch(rowwise_quant_kernel<false, true>) : launch(rowwise_quant_kernel<false, false>);
    MI355_HIP_TRY(hipGetLastError());
    return MI355_MOE_OK;
}

int launch_requant_y(const void* y, int32_t inter, const float* smooth, const int* sorted_ids, const int* sorted_expert_ids,
                     const int* total, int32_t unit, int32_t tokens, int32_t segs, int64_t max_rows, void* yq, float* yscale,
                     hipStream_t stream, bool fp8)
{
    if(max_rows <= 0)
        return MI355_MOE_OK;
    KernelTimer timer(MI355_MOE_K_QUANT, stream);
    const dim3 grid((unsigned)ceil_div<int64_t>(max_rows, 4));
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, static_cast<const uint16_t*>(y), inter, smooth, sorted_ids,
                           sorted_expert_ids, total, unit, tokens, segs, static_cast<unsigned char*>(yq), yscale);
    };
    if(fp8)
        smooth != nullptr ? launch(moe_requant_y_kernel<true, true>) : launch(moe_requant_y_kernel<false, true>);
    else
        smooth != nullptr ? launch(moe_requant_y_kernel<true, false>) : launch(moe_requant_y_kernel<false, false>);
    MI355_HIP_TRY(hipGetLastError());
    return MI355_MOE_OK;
}

} // namespace mi355
