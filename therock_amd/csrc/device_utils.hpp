// Device-side helpers shared by the sorting and GEMM kernels (gfx950, wave64).
#pragma once

#include "common.hpp"

namespace mi355 {

__device__ inline void wave_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Inclusive prefix sum over the 64 lanes of a wave (every lane active), with data-parallel primitives instead of
// LDS-routed shuffles: row_shr 1, 2, 4, 8 scan each row of 16 lanes (a lane shifted in from outside its row reads
// 0), row_bcast:15 adds the total of rows 0 and 2 to rows 1 and 3, row_bcast:31 the total of rows 0-1 to rows 2-3.
__device__ inline int wave_inclusive_scan(int x)
{
    x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xf, 0xf, false); // row_shr:1
    x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xf, 0xf, false); // row_shr:2
    x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xf, 0xf, false); // row_shr:4
    x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xf, 0xf, false); // row_shr:8
    x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xa, 0xf, false); // row_bcast:15 into rows 1 and 3
    x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xc, 0xf, false); // row_bcast:31 into rows 2 and 3
    return x;
}

// Wave-wide maximum / minimum of a 32-bit unsigned value, the same in every lane afterwards.  Data-parallel
// primitives instead of LDS-routed shuffles: an inclusive scan over each row of 16 lanes (row_shr 1, 2, 4, 8; lanes
// shifted in from outside a row read the identity), then lane 15 of rows 0 and 2 is combined into rows 1 and 3
// (row_bcast:15) and lane 31 into rows 2 and 3 (row_bcast:31): lane 63 holds the result.
template <bool MAX>
__device__ inline uint32_t wave_reduce_u32(uint32_t v)
{
    constexpr int ident = MAX ? 0 : -1;
    auto combine = [](uint32_t a, uint32_t b) { return MAX ? max(a, b) : min(a, b); };
    int x = static_cast<int>(v);
    x = static_cast<int>(combine(x, __builtin_amdgcn_update_dpp(ident, x, 0x111, 0xf, 0xf, false))); // row_shr:1
    x = static_cast<int>(combine(x, __builtin_amdgcn_update_dpp(ident, x, 0x112, 0xf, 0xf, false))); // row_shr:2
    x = static_cast<int>(combine(x, __builtin_amdgcn_update_dpp(ident, x, 0x114, 0xf, 0xf, false))); // row_shr:4
    x = static_cast<int>(combine(x, __builtin_amdgcn_update_dpp(ident, x, 0x118, 0xf, 0xf, false))); // row_shr:8
    x = static_cast<int>(combine(x, __builtin_amdgcn_update_dpp(ident, x, 0x142, 0xa, 0xf, false))); // row_bcast:15
    x = static_cast<int>(combine(x, __builtin_amdgcn_update_dpp(ident, x, 0x143, 0xc, 0xf, false))); // row_bcast:31
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(x, 63));
}

// Exclusive scan of one int per thread over a block of NWAVES*64 threads.  s_wave needs
// NWAVES+1 ints of LDS.  Every thread of the block must call it; `total` gets the block sum.
template <int NWAVES>
__device__ inline int block_exclusive_scan(int v, int* s_wave, int& total)
{
    static_assert(NWAVES <= kWave, "one wave scans the wave totals");
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int x    = wave_inclusive_scan(v);
    if(lane == kWave - 1)
        s_wave[wave] = x;
    __syncthreads();
    if(wave == 0)
    {
        const int w  = lane < NWAVES ? s_wave[lane] : 0;
        const int xx = wave_inclusive_scan(w);
        if(lane < NWAVES)
            s_wave[lane] = xx - w;
        if(lane == NWAVES - 1)
            s_wave[NWAVES] = xx;
    }
    __syncthreads();
    const int r = s_wave[wave] + x - v;
    total       = s_wave[NWAVES];
    __syncthreads();
    return r;
}

// N such scans at once (N values per thread), sharing the three barriers.  s_wave: N x (NWAVES + 1) ints of LDS.
template <int NWAVES, int N>
__device__ inline void block_exclusive_scan_n(const int (&v)[N], int (*s_wave)[NWAVES + 1], int (&excl)[N], int (&total)[N])
{
    static_assert(NWAVES <= kWave, "one wave scans the wave totals");
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    int x[N];
#pragma unroll
    for(int q = 0; q < N; q++)
    {
        x[q] = wave_inclusive_scan(v[q]);
        if(lane == kWave - 1)
            s_wave[q][wave] = x[q];
    }
    __syncthreads();
    if(wave == 0)
    {
#pragma unroll
        for(int q = 0; q < N; q++)
        {
            const int w  = lane < NWAVES ? s_wave[q][lane] : 0;
            const int xx = wave_inclusive_scan(w);
            if(lane < NWAVES)
                s_wave[q][lane] = xx - w;
            if(lane == NWAVES - 1)
                s_wave[q][NWAVES] = xx;
        }
    }
    __syncthreads();
#pragma unroll
    for(int q = 0; q < N; q++)
    {
        excl[q]  = s_wave[q][wave] + x[q] - v[q];
        total[q] = s_wave[q][NWAVES];
    }
    __syncthreads();
}

__device__ inline float bf16_bits_to_float(uint32_t h) { return __uint_as_float(h << 16); }

// round-to-nearest-even float -> bf16 bits (NaN stays NaN)
__device__ inline uint32_t float_to_bf16_bits(float f)
{
    uint32_t u = __float_as_uint(f);
    if((u & 0x7fffffffu) > 0x7f800000u)
        return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}

// two floats -> packed fp16 (round to nearest even, overflow to infinity: the IEEE conversion)
__device__ inline uint32_t pack_f16x2(float lo, float hi)
{
    const _Float16 a = static_cast<_Float16>(lo), b = static_cast<_Float16>(hi);
    return static_cast<uint32_t>(__builtin_bit_cast(unsigned short, a)) |
           (static_cast<uint32_t>(__builtin_bit_cast(unsigned short, b)) << 16);
}
__device__ inline float f16_bits_to_float(uint32_t h)
{
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(h)));
}

// two floats -> packed bf16 pair, round-to-nearest-even: a single v_cvt_pk_bf16_f32 on gfx950
__device__ inline uint32_t pack_bf16x2(float lo, float hi)
{
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
    typedef __attribute__((ext_vector_type(2))) float f32x2_t;
    const f32x2_t v  = {lo, hi};
    const bf16x2_t b = __builtin_convertvector(v, bf16x2_t);
    uint32_t r;
    __builtin_memcpy(&r, &b, sizeof(r));
    return r;
}

// x / s for many dividends x and one divisor s (a row's quantisation scale), with the result of the fp32 division
// and a third of its instructions: one fp64 reciprocal per row, then per element an fp64 product rounded to fp32.
// Why the rounding agrees: the product is within 2^-51.9 (relative) of the real quotient z (two fp64 roundings).
// The fp32 result can only differ if a midpoint m of two neighbouring fp32 numbers lies that close to z.  Write
// x = X 2^a, s = S 2^c with 24-bit integers X, S and m = M 2^b with an odd 25-bit M: z - m = (X 2^a - M S 2^(b+c)) / s
// is not zero (M S = X 2^k would need the odd M > 2^24 to divide X < 2^24), so it is at least one unit of that
// integer difference, |z - m| >= m / (M S) > m 2^-49.  Below 2^-126 midpoints have fewer bits and a quotient can hit
// one exactly; there the two results may be neighbouring subnormals of the same sign, which every quantiser here
// turns into the same zero.  Infinities, NaNs and zeros behave as in the division (1 / inf = 0, inf * 0 = NaN).
__device__ inline double row_reciprocal(float s) { return 1.0 / static_cast<double>(s); }
__device__ inline float div_by_row_scale(float x, double s_reciprocal)
{
    return static_cast<float>(static_cast<double>(x) * s_reciprocal);
}

} // namespace mi355
