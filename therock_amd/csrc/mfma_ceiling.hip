// Diagnostic behind mi355_moe_mfma_sustained(): the matrix-core rate a device sustains under its power and current
// limits, measured with the same MFMA instruction the grouped GEMMs issue for a precision.
//
// Why it exists.  The published dense peaks (5.0 PFLOP/s fp8, 2.5 bf16) are "every SIMD issues back to back at
// 2.4 GHz" figures.  A loop of nothing but independent MFMAs on register operands reaches them on this chip only when
// the operands are zeros: with operands that toggle like real data the package runs into its power limit, the
// firmware lowers the clock to about 1.9 GHz, and the same loop sustains about 3.9 PFLOP/s of fp8.  A kernel that
// also moves data has less than that to spend on MFMAs.  The benchmark reports this rate, measured on the device it
// runs on, beside the published peak.
//
// The kernel: 256 workgroups per launch round x 8 waves (two per SIMD), each wave 10 independent accumulator tiles
// (two weight fragments x five token fragments, the register blocking of the large-tile GEMM), operands generated in
// registers from a hash (finite e4m3 / bf16 / int8 values with random signs, mantissas and a spread of exponents),
// no LDS or global traffic inside the loop.  The accumulators are folded into one value per lane that is stored only
// if a kernel argument that the host always passes as 0 says so, so nothing is written and nothing is optimised away.
#include "moe_gemm_device.hpp"

namespace mi355 {
using namespace gemm;
namespace {

// volatile: a store to it is never removed, although nothing reads it
__device__ volatile int g_sink[64];

__device__ inline uint32_t hash32(uint32_t x)
{
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}

// four random finite 8-bit codes (e4m3: exponent field 4 .. 9 of 15; as int8 simply four values) or two bf16 / fp16
// values of magnitude 2^-3 .. 2^2
template <int MODE>
__device__ inline uint32_t random_operand_word(uint32_t seed)
{
    const uint32_t h = hash32(seed);
    if constexpr(MODE == kFp8)
    {
        uint32_t r = 0;
#pragma unroll
        for(int b = 0; b < 4; b++)
        {
            const uint32_t byte = (h >> (8 * b)) & 0xffu;
            const uint32_t e    = 4u + ((byte >> 3) & 0xfu) % 6u;
            r |= ((byte & 0x87u) | (e << 3)) << (8 * b);
        }
        return r;
    }
    else if constexpr(MODE == kI8)
        return h;
    else if constexpr(MODE == kF16)
    {
        // sign, exponent 12 .. 17 of 31 (bias 15), 10 random mantissa bits
        const uint32_t lo = (h & 0x83ffu) | ((12u + ((h >> 10) & 0x1fu) % 6u) << 10);
        const uint32_t hi = ((h >> 16) & 0x83ffu) | ((12u + ((h >> 26) & 0x1fu) % 6u) << 10);
        return lo | (hi << 16);
    }
    else
    {
        // bf16: sign, exponent 124 .. 129 of 255 (bias 127), 7 random mantissa bits
        const uint32_t lo = (h & 0x807fu) | ((124u + ((h >> 7) & 0xffu) % 6u) << 7);
        const uint32_t hi = ((h >> 16) & 0x807fu) | ((124u + ((h >> 23) & 0xffu) % 6u) << 7);
        return lo | (hi << 16);
    }
}

template <int MODE>
__global__ __launch_bounds__(512) void mfma_ceiling_kernel(int iters, uint32_t seed, int zeros, int never)
{
    using Acc = typename ModeTraits<MODE>::Acc;
    Frag w[2], x[5];
    const uint32_t id = (blockIdx.x * 512u + threadIdx.x) * 64u + seed;
    auto fill = [&](Frag& f, uint32_t k) {
        uint32_t v[8];
#pragma unroll
        for(int j = 0; j < 8; j++)
            v[j] = zeros ? 0u : random_operand_word<MODE>(id + k * 8u + j);
        f.lo = make_uint4(v[0], v[1], v[2], v[3]);
        f.hi = make_uint4(v[4], v[5], v[6], v[7]);
    };
    fill(w[0], 0);
    fill(w[1], 1);
#pragma unroll
    for(int i = 0; i < 5; i++)
        fill(x[i], 2 + i);
    Acc acc[5][2];
#pragma unroll
    for(int i = 0; i < 5; i++)
#pragma unroll
        for(int b = 0; b < 2; b++)
#pragma unroll
            for(int v = 0; v < 16; v++)
                acc[i][b][v] = 0;
    for(int it = 0; it < iters; it++)
    {
        // 16-bit modes: one K step of 64 bytes is two MFMAs (lo and hi halves of the fragments), issued round the ten
        // tiles so that consecutive MFMAs never share an accumulator
#pragma unroll
        for(int h = 0; h < (ModeTraits<MODE>::kOpB == 16 ? 2 : 1); h++)
#pragma unroll
            for(int i = 0; i < 5; i++)
#pragma unroll
                for(int b = 0; b < 2; b++)
                {
                    if constexpr(MODE == kFp8)
                        acc[i][b] = mfma_fp8_unscaled(w[b], x[i], acc[i][b]);
                    else
                    {
                        Frag a = w[b], c = x[i];
                        if(h == 1)
                        {
                            a.lo = w[b].hi;
                            c.lo = x[i].hi;
                        }
                        acc[i][b] = mfma<MODE>(a, c, 127, acc[i][b]);
                    }
                }
    }
    // integer accumulators may wrap and float ones grow; only the bit pattern matters here
    uint32_t fold = 0;
#pragma unroll
    for(int i = 0; i < 5; i++)
#pragma unroll
        for(int b = 0; b < 2; b++)
#pragma unroll
            for(int v = 0; v < 16; v++)
                fold ^= bit_cast_dev<uint32_t>(acc[i][b][v]) + 0x9e3779b9u * (uint32_t)(i * 32 + b * 16 + v);
    if(fold == 0x5bd1e995u && never != 0) // the host passes 0: nothing is ever stored, and the compiler cannot know
        g_sink[threadIdx.x & 63] = (int)fold;
}

template <int MODE>
int run(int ms_target, int zeros, double* tflops, hipStream_t stream)
{
    struct Events // destroyed on every way out
    {
        hipEvent_t a = nullptr, b = nullptr;
        ~Events()
        {
            if(a)
                (void)hipEventDestroy(a);
            if(b)
                (void)hipEventDestroy(b);
        }
    } ev;
    MI355_HIP_TRY(hipEventCreate(&ev.a));
    MI355_HIP_TRY(hipEventCreate(&ev.b));
    const hipEvent_t e0 = ev.a, e1 = ev.b;
    const int grid  = device_info().num_cu;
    // MFMAs of one K step of 64 bytes per tile, FLOP of each
    constexpr int kPerStep     = ModeTraits<MODE>::kOpB == 16 ? 2 : 1;
    constexpr double kFlopStep = 2.0 * 32 * 32 * 64 / (MODE == kFp8 || MODE == kI8 ? 1 : 2);
    (void)kPerStep;
    int iters       = 2000;
    double total_ms = 0.0, flop = 0.0;
    uint32_t seed   = 1;
    // the first launches run before the power controller has settled: they count as warm-up, the rate is taken from
    // the second half of the requested time
    for(int phase = 0; phase < 2; phase++)
    {
        total_ms = 0.0;
        flop     = 0.0;
        while(total_ms < 0.5 * ms_target)
        {
            MI355_HIP_TRY(hipEventRecord(e0, stream));
            hipLaunchKernelGGL((mfma_ceiling_kernel<MODE>), dim3(grid), dim3(512), 0, stream, iters, seed++, zeros, 0);
            MI355_HIP_TRY(hipGetLastError());
            MI355_HIP_TRY(hipEventRecord(e1, stream));
            MI355_HIP_TRY(hipEventSynchronize(e1));
            float ms = 0.f;
            MI355_HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
            total_ms += ms;
            flop += (double)grid * 8 * iters * 10 * kFlopStep;
            if(ms < 2.0f && iters < (1 << 20))
                iters *= 2; // launches of a few milliseconds: the launch gap does not show
        }
    }
    *tflops = flop / (total_ms * 1e-3) / 1e12;
    return MI355_MOE_OK;
}

} // namespace

int mfma_sustained(int prec, int milliseconds, int zeros, double* tflops, hipStream_t stream)
{
    if(tflops == nullptr || milliseconds <= 0 || milliseconds > 60000)
        return fail(MI355_MOE_E_INVALID, "mfma_sustained: bad arguments");
    switch(prec)
    {
    case MI355_MOE_FP8: return run<kFp8>(milliseconds, zeros, tflops, stream);
    case MI355_MOE_BF16: return run<kBf16>(milliseconds, zeros, tflops, stream);
    case MI355_MOE_FP16: return run<kF16>(milliseconds, zeros, tflops, stream);
    case MI355_MOE_INT8: return run<kI8>(milliseconds, zeros, tflops, stream);
    default: return fail(MI355_MOE_E_UNSUPPORTED, "mfma_sustained: precision %d", prec);
    }
}

} // namespace mi355
