/*
 * CPU oracle for the fused-MoE path (moe_sorting + gate/up GEMM + SiLU*up + down GEMM +
 * top-k weighted combine).
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, the smoke check and the
 * cpu_baseline leg of bench.py may load it; the product path never links or calls it.
 *
 * It restates, in plain C, the host reference that ships with Composable Kernel ck_tile 1.2.0
 * (commit 69f44ce42ce0a5f46fba094695a1e7948d5c6679, installed under /opt/rocm/include/ck_tile;
 * paths below are relative to that directory):
 *
 *   moe_oracle_sorting        <- host/reference/reference_moe_sorting.hpp:14-117
 *   moe_oracle_fused_moe      <- host/reference/reference_fused_moe.hpp:42-204
 *   silu                      <- ops/elementwise/unary_element_wise_operation.hpp:1013-1026
 *   bf16 round-to-nearest-even<- core/numeric/bfloat16.hpp:284-291 (builtin __bf16 cast, RNE)
 *   e4m3 (OCP) encode/decode  <- core/numeric/float8.hpp:600-660 (saturating RNE, +-448)
 *   row-wise quantisation     <- host/reference/reference_rowwise_quantization2d.hpp:12-31
 *   scale placement           <- host/reference/reference_moe_gemm.hpp:94-113,202-203
 *   moe_oracle_moe_gemm       <- host/reference/reference_moe_gemm.hpp:18-241 (ck_tile's unfused grouped GEMMs)
 *   moe_oracle_topk_softmax   <- host/reference/reference_softmax.hpp:12-78 + host/reference/reference_topk.hpp:30-103
 *                                (sigmoid variant: ops/topk_softmax/pipeline/topk_softmax_warp_per_row_pipeline.hpp:88-92)
 *
 * ck_tile's reference_fused_moe ignores its four scale tensors (:200-203).  For quantised
 * inputs the oracle is therefore *defined* as "de-quantise every operand to fp32 (q * scale)
 * and run the fp32 reference"; moe_oracle_fused_moe does that de-quantisation on the fly.
 *
 * Pinning status (what checks each function, beyond this file):
 *   sorting     - the three worked examples in ops/fused_moe/kernel/moe_sorting_kernel.hpp:55-117,
 *                 brute force over every routing of tiny problems, ck_tile's own
 *                 reference_moe_sorting compiled into oracle/_ref (bit-exact).
 *   fused moe   - ck_tile's reference_fused_moe in oracle/_ref on the same inputs; an
 *                 independent dense (sorting-free) float64 formulation in numpy.
 *   bf16 / e4m3 - exhaustive comparison with torch's bfloat16 / float8_e4m3fn casts.
 *   moe gemm    - a dense float64 formulation that never sorts, the composition gate+up -> down against
 *                 moe_oracle_fused_moe (itself bit-exact with ck_tile); ck_tile's reference for these is a
 *                 device kernel (oracle/_ref/libck_ref_gpu.so), compared in a GPU test.
 *   topk softmax- ck_tile's reference_softmax + reference_topk in oracle/_ref; closed forms (equal
 *                 logits, shift invariance, weights of all experts sum to one), scipy's softmax and
 *                 numpy's argsort on random rows.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

enum
{
    MOE_DT_F32  = 0,
    MOE_DT_BF16 = 1,
    MOE_DT_E4M3 = 2,
    MOE_DT_I8   = 3,
    MOE_DT_F16  = 4
};

/* ------------------------------------------------------------------ scalar conversions */

static inline float bits_to_f32(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint32_t f32_to_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

ORACLE_API float moe_oracle_bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

/* round-to-nearest-even, NaN kept quiet (core/numeric/bfloat16.hpp:118-140 / :284-291) */
ORACLE_API uint16_t moe_oracle_f32_to_bf16(float f)
{
    uint32_t u = f32_to_bits(f);
    if((u & 0x7fffffffu) > 0x7f800000u)
        return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* IEEE binary16 (ck_tile::half_t = _Float16, core/numeric/half.hpp): every value is an fp32 value */
ORACLE_API float moe_oracle_f16_to_f32(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h >> 15) << 31, ex = (h >> 10) & 0x1fu, man = h & 0x3ffu;
    float r;
    if(ex == 0x1f)
        return bits_to_f32(sign | 0x7f800000u | (man << 13)); /* infinity, or NaN with its payload */
    r = ex == 0 ? ldexpf((float)man, -24) : ldexpf(1.0f + (float)man / 1024.0f, (int)ex - 15);
    return sign ? -r : r;
}

/* round to nearest even, overflow to infinity, subnormals kept (the _Float16 cast of the compiler) */
ORACLE_API uint16_t moe_oracle_f32_to_f16(float f)
{
    const uint32_t u = f32_to_bits(f), sign = (u >> 16) & 0x8000u, mag = u & 0x7fffffffu;
    if(mag > 0x7f800000u)
        return (uint16_t)(sign | 0x7e00u); /* quiet NaN */
    if(mag >= 0x477ff000u) /* 65520 = halfway between the largest finite value and 2^16: rounds to infinity */
        return (uint16_t)(sign | 0x7c00u);
    if(mag < 0x33000001u) /* at most 2^-25: rounds to zero (2^-25 itself is a tie with the even code 0) */
        return (uint16_t)sign;
    {
        const int e      = (int)(mag >> 23) - 127;                 /* unbiased exponent, -25 .. 15 */
        const uint32_t m = (mag & 0x7fffffu) | 0x800000u;          /* 24-bit significand */
        const int shift  = e >= -14 ? 13 : 13 + (-14 - e);         /* bits dropped (subnormal results drop more) */
        uint32_t q       = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if(rem > half || (rem == half && (q & 1u)))
            q++;
        /* normal: q has the hidden bit at 2^10, adding the exponent field carries correctly when q = 2^11 */
        return (uint16_t)(sign | (e >= -14 ? (((uint32_t)(e + 14) << 10) + q) : q));
    }
}

/* OCP e4m3 ("e4m3fn"): bias 7, no inf, 0x7f/0xff = NaN, max finite 448 */
ORACLE_API float moe_oracle_e4m3_to_f32(uint8_t v)
{
    uint32_t sign = (v >> 7) & 1u;
    uint32_t ex   = (v >> 3) & 0xfu;
    uint32_t man  = v & 7u;
    float r;
    if(ex == 0xf && man == 7)
        r = NAN;
    else if(ex == 0)
        r = ldexpf((float)man, -9); /* subnormal: man/8 * 2^-6 */
    else
        r = ldexpf(1.0f + (float)man / 8.0f, (int)ex - 7);
    return sign ? -r : r;
}

/* saturating round-to-nearest-even float -> e4m3 (core/numeric/float8.hpp:600-660: clip to
 * +-448 first, then RNE).  NaN -> 0x7f. */
ORACLE_API uint8_t moe_oracle_f32_to_e4m3(float f)
{
    if(isnan(f))
        return 0x7f;
    uint8_t sign = signbit(f) ? 0x80 : 0;
    float a      = fabsf(f);
    if(a >= 448.0f)
        return sign | 0x7e;
    if(a == 0.0f)
        return sign;
    int e;
    (void)frexpf(a, &e); /* a = m * 2^e, m in [0.5,1) -> exponent of leading bit is e-1 */
    int ex = e - 1;
    if(ex < -6)
        ex = -6;                          /* subnormal range shares the 2^-6 scale */
    float q   = ldexpf(a, 3 - ex);        /* in units of one mantissa ulp */
    float rq  = nearbyintf(q);            /* default rounding mode: RNE */
    int   iq  = (int)rq;
    int biased;
    if(ex == -6 && iq < 8)
    {
        biased = 0; /* subnormal */
    }
    else
    {
        if(iq == 16)
        {
            iq = 8;
            ex += 1;
        }
        biased = ex + 7;
        iq -= 8;
    }
    if(biased > 15 || (biased == 15 && iq > 6))
        return sign | 0x7e;
    return (uint8_t)(sign | (biased << 3) | iq);
}

static inline float silu_f32(float x) { return x * (1.0f / (1.0f + expf(-x))); }
/* ck_tile::element_wise::Gelu, the exact (erf) form: unary_element_wise_operation.hpp:975-986.  Its host
 * expression `0.5f * x * (1.f + erf(float(0.70710678118f * x)))` picks the double erf, so the sum and the last
 * product are evaluated in double and rounded to float once */
static inline float gelu_f32(float x)
{
    return (float)((double)(0.5f * x) * (1.0 + erf((double)(0.70710678118f * x))));
}
/* activation codes of fused_moe_traits: 0 = gelu, 1 = silu */
static inline float act_f32(float x, int activation) { return activation == 0 ? gelu_f32(x) : silu_f32(x); }

ORACLE_API float moe_oracle_silu(float x) { return silu_f32(x); }
ORACLE_API float moe_oracle_gelu(float x) { return gelu_f32(x); }

/* -------------------------------------------------------------------------- quantisation */

/* one quantised element: saturate, then ck_tile's type_convert (core/numeric/int8.hpp:101: a plain
 * static_cast for int8, i.e. truncation toward zero; core/numeric/float8.hpp: saturating RNE for e4m3).
 * nearest != 0 rounds int8 to nearest-even instead (what the synthetic-input generator uses). */
static inline void quant_store(void* q, int64_t i, float v, int dt, int nearest)
{
    if(dt == MOE_DT_E4M3)
        ((uint8_t*)q)[i] = moe_oracle_f32_to_e4m3(v);
    else
    {
        float c          = v > 127.f ? 127.f : (v < -128.f ? -128.f : v);
        ((int8_t*)q)[i]  = nearest ? (int8_t)nearbyintf(c) : (int8_t)c;
    }
}

/* per-row dynamic quantisation: scale[m] = amax(row)/qmax, q = convert(saturate(x/scale))
 * (host/reference/reference_rowwise_quantization2d.hpp:12-31 with the scale the smooth-quant pipeline
 * computes, ops/smoothquant/pipeline/smoothquant_pipeline_one_pass.hpp:103-117).
 * x is fp32 [M,N] (caller up-converts bf16).  dt = MOE_DT_E4M3 (qmax 448) or MOE_DT_I8 (127).
 * A row of zeros gets scale 1 so that no division by zero happens. */
ORACLE_API int moe_oracle_rowwise_quant2(const float* x, int64_t M, int64_t N, int dt, int nearest, void* q,
                                         float* scale)
{
    if(dt != MOE_DT_E4M3 && dt != MOE_DT_I8)
        return -1;
    const float qmax = dt == MOE_DT_E4M3 ? 448.0f : 127.0f;
#pragma omp parallel for schedule(static)
    for(int64_t m = 0; m < M; m++)
    {
        const float* r = x + m * N;
        float amax     = 0.f;
        for(int64_t n = 0; n < N; n++)
        {
            float a = fabsf(r[n]);
            if(a > amax)
                amax = a;
        }
        float s  = amax > 0.f ? amax / qmax : 1.0f;
        scale[m] = s;
        for(int64_t n = 0; n < N; n++)
            quant_store(q, m * N + n, r[n] / s, dt, nearest);
    }
    return 0;
}

/* nearest-even variant kept under the old name: the quantiser of the synthetic benchmark inputs */
ORACLE_API int moe_oracle_rowwise_quant(const float* x, int64_t M, int64_t N, int dt, void* q, float* scale)
{
    return moe_oracle_rowwise_quant2(x, M, N, dt, 1, q, scale);
}

/* MoE smooth-quant (ops/smoothquant/kernel/moe_smoothquant_kernel.hpp:12-27, 152-175 and
 * pipeline/smoothquant_pipeline_one_pass.hpp:73-118): for slot k of token t routed to expert e,
 * y = x[t,:] * smscale[e,:] in fp32, yscale[k*tokens + t] = amax|y| / qmax, qy[k*tokens + t, :] =
 * convert(saturate(y / yscale)).  Outputs are [topk, tokens, hidden] and [topk, tokens].
 * A row of zeros (ck_tile converts 0 / 0 there, which is undefined behaviour) gets scale 0 and codes 0. */
ORACLE_API int moe_oracle_smoothquant(const float* x, const float* smscale, const int32_t* topk_ids, int32_t tokens,
                                      int32_t hidden, int32_t experts, int32_t topk, int dt, void* qy, float* yscale)
{
    if(dt != MOE_DT_E4M3 && dt != MOE_DT_I8)
        return -1;
    const float qmax = dt == MOE_DT_E4M3 ? 448.0f : 127.0f;
    for(int64_t k = 0; k < topk; k++)
        for(int64_t t = 0; t < tokens; t++)
        {
            const int e = topk_ids[t * topk + k];
            if(e < 0 || e >= experts)
                return -2;
            const float* xr = x + t * hidden;
            const float* sr = smscale + (int64_t)e * hidden;
            float amax      = 0.f;
            for(int64_t h = 0; h < hidden; h++)
            {
                const float a = fabsf(xr[h] * sr[h]);
                amax          = a > amax ? a : amax;
            }
            const float ys           = amax / qmax;
            yscale[k * tokens + t]   = ys;
            const float div          = amax > 0.f ? ys : 1.0f;
            for(int64_t h = 0; h < hidden; h++)
                quant_store(qy, (k * tokens + t) * hidden + h, (xr[h] * sr[h]) / div, dt, 0);
        }
    return 0;
}

/* ------------------------------------------------------------------------------- sorting */

static inline int32_t mock_id(int32_t t, int32_t k)
{
    return (int32_t)(((uint32_t)t & 0x00ffffffu) | (((uint32_t)k & 0xffu) << 24));
}

/*
 * reference_moe_sorting.hpp:14-117 with CK_TILE_REFERENCE_MOE_SORTING_MOCK_ID = 1.
 * Outputs past the written prefix are left untouched.  *post_pad is overwritten (the ck_tile
 * function accumulates into a caller-zeroed counter; the result is the same).
 * local_expert_mask may be NULL (no masking).  Returns the number of unit tiles written.
 */
ORACLE_API int moe_oracle_sorting(const int32_t* topk_ids, const float* weights,
                                  const int32_t* local_expert_mask, int32_t tokens, int32_t topk,
                                  int32_t experts, int32_t unit_size, int32_t skip_empty,
                                  int32_t* sorted_token_ids, float* sorted_weights,
                                  int32_t* sorted_expert_ids, int32_t* post_pad)
{
    int64_t* cnt = (int64_t*)calloc((size_t)experts, sizeof(int64_t));
    int64_t* off = (int64_t*)calloc((size_t)experts + 1, sizeof(int64_t));
    if(!cnt || !off)
        return -1;
    for(int64_t i = 0; i < (int64_t)tokens * topk; i++)
    {
        int32_t e = topk_ids[i];
        if(e < 0 || e >= experts)
        {
            free(cnt);
            free(off);
            return -2;
        }
        cnt[e]++;
    }
    /* per expert: slices = max(1, ceil(cnt/unit)) (:42 starts every expert with one slice) */
    const int32_t pad = mock_id(tokens, topk);
    int64_t out = 0, tile = 0;
    int32_t out_eid = 0;
    int64_t* base   = (int64_t*)malloc(sizeof(int64_t) * (size_t)experts);
    for(int32_t e = 0; e < experts; e++)
    {
        base[e] = -1;
        if(local_expert_mask && local_expert_mask[e] == 0)
            continue; /* :86-90, does not advance the output expert id */
        if(skip_empty && cnt[e] == 0)
        {
            out_eid++; /* :91-98 */
            continue;
        }
        int64_t slices = (cnt[e] + unit_size - 1) / unit_size;
        if(slices < 1)
            slices = 1;
        base[e] = out;
        for(int64_t i = cnt[e]; i < slices * unit_size; i++)
        {
            sorted_token_ids[out + i] = pad;
            sorted_weights[out + i]   = 0.f;
        }
        for(int64_t s = 0; s < slices; s++)
            sorted_expert_ids[tile + s] = out_eid;
        out += slices * unit_size;
        tile += slices;
        out_eid++;
    }
    /* t-major, k-minor fill => ascending token id inside an expert (:47-78) */
    memset(cnt, 0, sizeof(int64_t) * (size_t)experts);
    for(int32_t t = 0; t < tokens; t++)
        for(int32_t k = 0; k < topk; k++)
        {
            int32_t e = topk_ids[(int64_t)t * topk + k];
            if(base[e] < 0)
                continue;
            int64_t p           = base[e] + cnt[e]++;
            sorted_token_ids[p] = mock_id(t, k);
            sorted_weights[p]   = weights[(int64_t)t * topk + k];
        }
    *post_pad = (int32_t)out;
    free(cnt);
    free(off);
    free(base);
    return (int)tile;
}

/* --------------------------------------------------------------------------- fused MoE */

static inline float load_as_f32(const void* p, int dt, int64_t i)
{
    switch(dt)
    {
    case MOE_DT_F32: return ((const float*)p)[i];
    case MOE_DT_BF16: return moe_oracle_bf16_to_f32(((const uint16_t*)p)[i]);
    case MOE_DT_E4M3: return moe_oracle_e4m3_to_f32(((const uint8_t*)p)[i]);
    default: return (float)((const int8_t*)p)[i];
    }
}

/* de-quantise a row of n elements starting at element offset `off`, times `scale` */
static void dequant_row(float* dst, const void* p, int dt, int64_t off, int64_t n, float scale)
{
    for(int64_t i = 0; i < n; i++)
        dst[i] = load_as_f32(p, dt, off + i) * scale;
}

/* sequential fp32 dot product in ck_tile's order (strict) or with 8 partial sums (fast) */
static inline float dot_f32(const float* a, const float* b, int64_t n, int strict)
{
    if(strict)
    {
        float acc = 0.f;
        for(int64_t i = 0; i < n; i++)
            acc += a[i] * b[i];
        return acc;
    }
    float p[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    int64_t i  = 0;
    for(; i + 8 <= n; i += 8)
        for(int j = 0; j < 8; j++)
            p[j] += a[i + j] * b[i + j];
    float acc = ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
    for(; i < n; i++)
        acc += a[i] * b[i];
    return acc;
}

/*
 * reference_fused_moe.hpp:42-204.
 *   a   [tokens, hidden]          dtype a_dt, optional per-token scale a_scale[tokens]
 *   g   [experts, 2*inter, hidden] (gate rows [0,inter), up rows [inter,2*inter); or
 *       [experts, inter, hidden] when gate_only), optional g_scale[experts, n0]
 *   d   [experts, hidden, inter]  optional d_scale[experts, hidden]
 *   sorted_* / post_pad           as written by moe_oracle_sorting with unit_size = block_m
 *   o   [tokens, hidden]          o_dt = MOE_DT_BF16 (one RNE at the end) or MOE_DT_F32
 *   out_topk (optional, may be NULL) fp32 [tokens, topk, hidden] partials before the reduce
 * strict != 0 keeps ck_tile's exact summation order (slow, bit-comparable with oracle/_ref).
 * De-quantised operands are formed as float(q)*scale before the multiply, which is what
 * feeding ck_tile's reference the de-quantised tensors does.
 */
ORACLE_API int moe_oracle_fused_moe(const void* a, int a_dt, const float* a_scale, const void* g,
                                    int g_dt, const float* g_scale, const void* d, int d_dt,
                                    const float* d_scale, void* o, int o_dt,
                                    const int32_t* sorted_token_ids, const float* sorted_weights,
                                    const int32_t* sorted_expert_ids, int32_t post_pad,
                                    int32_t block_m, int32_t tokens, int32_t experts,
                                    int32_t hidden, int32_t inter, int32_t topk, int32_t gate_only,
                                    int32_t strict, float* out_topk, int32_t activation)
{
    (void)experts;
    const int64_t n0       = (int64_t)inter * (gate_only ? 1 : 2);
    const int64_t n_rows   = post_pad; /* rows past post_pad are never visited (:92-94) */
    const size_t part_elts = (size_t)tokens * topk * hidden;
    float* part            = out_topk ? out_topk : (float*)malloc(part_elts * sizeof(float));
    if(!part)
        return -1;
    memset(part, 0, part_elts * sizeof(float)); /* HostTensor storage is value-initialised */

    /* rows of one expert are contiguous: de-quantise that expert's weights once */
    int rc = 0;
    int64_t row = 0;
    while(row < n_rows)
    {
        const int32_t e = sorted_expert_ids[row / block_m];
        int64_t end     = row;
        while(end < n_rows && sorted_expert_ids[end / block_m] == e)
            end += block_m;
        float* gw = (float*)malloc(sizeof(float) * (size_t)n0 * hidden);
        float* dw = (float*)malloc(sizeof(float) * (size_t)hidden * inter);
        if(!gw || !dw)
        {
            free(gw);
            free(dw);
            rc = -1;
            break;
        }
#pragma omp parallel for schedule(static)
        for(int64_t n = 0; n < n0; n++)
            dequant_row(gw + n * hidden, g, g_dt, ((int64_t)e * n0 + n) * hidden, hidden,
                        g_scale ? g_scale[(int64_t)e * n0 + n] : 1.0f);
#pragma omp parallel for schedule(static)
        for(int64_t h = 0; h < hidden; h++)
            dequant_row(dw + h * inter, d, d_dt, ((int64_t)e * hidden + h) * inter, inter,
                        d_scale ? d_scale[(int64_t)e * hidden + h] : 1.0f);

#pragma omp parallel
        {
            float* x    = (float*)malloc(sizeof(float) * (size_t)hidden);
            float* acc0 = (float*)malloc(sizeof(float) * (size_t)n0);
            float* y    = (float*)malloc(sizeof(float) * (size_t)inter);
#pragma omp for schedule(dynamic, 1)
            for(int64_t i = row; i < end; i++)
            {
                int32_t id    = sorted_token_ids[i];
                int32_t slot  = (int32_t)((uint32_t)id >> 24);
                int32_t token = id & 0xffffff;
                if(token >= tokens)
                    continue; /* padding row (:97-99) */
                float w = sorted_weights[i];
                dequant_row(x, a, a_dt, (int64_t)token * hidden, hidden,
                            a_scale ? a_scale[token] : 1.0f);
                for(int64_t n = 0; n < n0; n++) /* first gemm :125-135 */
                    acc0[n] = dot_f32(x, gw + n * hidden, hidden, strict);
                if(gate_only)
                    for(int64_t n = 0; n < inter; n++)
                        y[n] = act_f32(acc0[n], activation);
                else
                    for(int64_t n = 0; n < inter; n++) /* :156-161 */
                        y[n] = act_f32(acc0[n], activation) * acc0[n + inter];
                float* dst = part + ((int64_t)token * topk + slot) * hidden;
                for(int64_t h = 0; h < hidden; h++) /* second gemm :166-174 */
                    dst[h] = dot_f32(y, dw + h * inter, inter, strict) * w;
            }
            free(x);
            free(acc0);
            free(y);
        }
        free(gw);
        free(dw);
        row = end;
    }

    if(rc == 0)
    {
        /* reduce over slots in order 0..topk-1, one final conversion (:186-197) */
#pragma omp parallel for schedule(static)
        for(int64_t t = 0; t < tokens; t++)
            for(int64_t h = 0; h < hidden; h++)
            {
                float acc = 0.f;
                for(int64_t k = 0; k < topk; k++)
                    acc += part[(t * topk + k) * hidden + h];
                if(o_dt == MOE_DT_BF16)
                    ((uint16_t*)o)[t * hidden + h] = moe_oracle_f32_to_bf16(acc);
                else
                    ((float*)o)[t * hidden + h] = acc;
            }
    }
    if(!out_topk)
        free(part);
    return rc;
}

/* ---------------------------------------------------------------------- unfused grouped GEMMs
 * reference_moe_gemm.hpp:41-241 with row-major A and C, B as [experts, N, K], one scale per row of A
 * (scale_a, may be NULL) and per output channel (scale_b [experts, N], may be NULL), an optional expert
 * bias [experts, N] added to the scaled dot products (:205-211).
 *   kind 1 (gate+up): row r of the sorted list with token t, slot s: A row t, C row t*topk+s,
 *       C[., n] = bf16( act(acc_gate + bias, acc_up + bias_up) ), gate = B rows [0, N/2), up = B rows [N/2, N)
 *   kind 0 (gate only): the same rows, C[., n] = bf16( act(acc + bias, 1) ) over all N rows of B (:216-219)
 *   kind 2 (down)   : A row t*topk+s, C row t; ck_tile adds bf16((acc + bias) * w[r]) to C with packed bf16
 *       atomics (:214-238).  Here a token's slots are summed in fp32 in slot order on top of the bf16 value C
 *       holds and rounded once: the same quantity without the order-dependent bf16 rounding of every partial sum.
 * act: 0 = ck_tile::moe::MoeSilu, silu(gate) * linear; 1 = ck_tile::moe::Swiglu{alpha, limit}:
 *       gate' = min(gate, limit), linear' = clamp(linear, -limit, limit), gate' * sigmoid(alpha * gate') * (linear' + 1)
 *       (ops/flatmm/kernel/moe_flatmm_kernel.hpp:139-183, host branch: a true division, no rcp).
 * n_padded_zeros / k_padded_zeros (MoeFlatmmHostArgs, moe_flatmm_kernel.hpp:29-30): the last rows of every
 * expert's B, respectively the last columns of A and B, are padding that the device kernel never fetches (its
 * tensor views end before them, :600-606): they count as zeros.
 * A and B are fp32 (the caller up-converts), C holds bf16 bits, or fp16 bits with c_dt = MOE_DT_F16
 * (moe_oracle_moe_gemm_dt; ck_tile's MoeFlatmm is instantiated for both, CDataType of its kernel). */
static inline float moe_act_f32(int act, float gate, float linear, float alpha, float limit)
{
    if(act == 0)
        return silu_f32(gate) * linear;
    gate   = gate < limit ? gate : limit;
    linear = linear < limit ? (linear > -limit ? linear : -limit) : limit;
    return gate * (1.0f / (1.0f + expf(alpha * -gate))) * (linear + 1.0f);
}

ORACLE_API float moe_oracle_moe_act(int act, float gate, float linear, float alpha, float limit)
{
    return moe_act_f32(act, gate, linear, alpha, limit);
}

static inline uint16_t c_from_f32(int32_t c_dt, float f)
{
    return c_dt == MOE_DT_F16 ? moe_oracle_f32_to_f16(f) : moe_oracle_f32_to_bf16(f);
}

ORACLE_API int moe_oracle_moe_gemm_dt(int kind, const int32_t* sorted_ids, const int32_t* sorted_eid, const float* sorted_w,
                                      int32_t max_token_id, int32_t tokens_per_block, const float* A, const float* B,
                                      uint16_t* C, int32_t num_tokens, int32_t topk, int32_t N, int32_t K, int32_t stride_a,
                                      int32_t stride_c, const float* scale_a, const float* scale_b, const float* exp_bias,
                                      int32_t act, float alpha, float limit, int32_t n_padded_zeros, int32_t k_padded_zeros,
                                      int32_t c_dt)
{
    if(kind < 0 || kind > 2 || act < 0 || act > 1 || n_padded_zeros < 0 || n_padded_zeros > N || k_padded_zeros < 0 ||
       k_padded_zeros > K || (c_dt != MOE_DT_BF16 && c_dt != MOE_DT_F16))
        return -1;
    const int32_t pn = kind == 1 ? N / 2 : N;
    const int32_t nv = N - n_padded_zeros; /* rows of B that exist */
    const int32_t kv = K - k_padded_zeros; /* columns that exist */
    float* acc2      = NULL; /* kind 2: fp32 sums [tokens, N], started from C */
    if(kind == 2)
    {
        acc2 = (float*)malloc(sizeof(float) * (size_t)num_tokens * N);
        if(!acc2)
            return -2;
        for(int64_t t = 0; t < num_tokens; t++)
            for(int64_t n = 0; n < N; n++)
                acc2[t * N + n] = c_dt == MOE_DT_F16 ? moe_oracle_f16_to_f32(C[t * stride_c + n])
                                                     : moe_oracle_bf16_to_f32(C[t * stride_c + n]);
    }
    /* slot order inside a token = the order of the reference's reduction: walk slots, then rows */
    for(int32_t s = 0; s < (kind == 2 ? topk : 1); s++)
        for(int64_t r = 0; r < max_token_id; r++)
        {
            const int32_t id  = sorted_ids[r];
            const int32_t tok = id & 0xffffff, slot = (int32_t)((uint32_t)id >> 24);
            if(tok >= num_tokens || (kind == 2 && slot != s))
                continue;
            const int64_t e      = sorted_eid[r / tokens_per_block];
            const int64_t a_row  = kind == 2 ? (int64_t)tok * topk + slot : tok;
            const int64_t c_row  = kind == 2 ? tok : (int64_t)tok * topk + slot;
            const float* a       = A + a_row * stride_a;
            const float sa       = scale_a ? scale_a[a_row] : 1.0f;
#pragma omp parallel for schedule(static)
            for(int32_t n = 0; n < pn; n++)
            {
                const float* b = B + (e * N + n) * K;
                float acc      = 0.f;
                if(n < nv)
                    for(int32_t k = 0; k < kv; k++)
                        acc += a[k] * b[k];
                acc *= sa * (scale_b ? scale_b[e * N + n] : 1.0f);
                acc += exp_bias ? exp_bias[e * N + n] : 0.f;
                if(kind == 1)
                {
                    const float* bu = B + (e * N + n + pn) * K;
                    float up        = 0.f;
                    if(n + pn < nv)
                        for(int32_t k = 0; k < kv; k++)
                            up += a[k] * bu[k];
                    up *= sa * (scale_b ? scale_b[e * N + n + pn] : 1.0f);
                    up += exp_bias ? exp_bias[e * N + n + pn] : 0.f;
                    C[c_row * stride_c + n] = c_from_f32(c_dt, moe_act_f32(act, acc, up, alpha, limit));
                }
                else if(kind == 0)
                    C[c_row * stride_c + n] = c_from_f32(c_dt, moe_act_f32(act, acc, 1.0f, alpha, limit));
                else
                    acc2[c_row * N + n] += acc * sorted_w[r];
            }
        }
    if(kind == 2)
    {
        for(int64_t t = 0; t < num_tokens; t++)
            for(int64_t n = 0; n < N; n++)
                C[t * stride_c + n] = c_from_f32(c_dt, acc2[t * N + n]);
        free(acc2);
    }
    return 0;
}

ORACLE_API int moe_oracle_moe_gemm(int kind, const int32_t* sorted_ids, const int32_t* sorted_eid, const float* sorted_w,
                                   int32_t max_token_id, int32_t tokens_per_block, const float* A, const float* B,
                                   uint16_t* C, int32_t num_tokens, int32_t topk, int32_t N, int32_t K, int32_t stride_a,
                                   int32_t stride_c, const float* scale_a, const float* scale_b, const float* exp_bias,
                                   int32_t act, float alpha, float limit, int32_t n_padded_zeros, int32_t k_padded_zeros)
{
    return moe_oracle_moe_gemm_dt(kind, sorted_ids, sorted_eid, sorted_w, max_token_id, tokens_per_block, A, B, C, num_tokens,
                                  topk, N, K, stride_a, stride_c, scale_a, scale_b, exp_bias, act, alpha, limit,
                                  n_padded_zeros, k_padded_zeros, MOE_DT_BF16);
}

/* ------------------------------------------------------------------------------ router
 * reference_softmax.hpp:39-74 (row maximum, sum of exp(x - max) in ascending expert order, exp / sum)
 * followed by reference_topk.hpp:73-95 (the k largest, descending).  sigmoid != 0 replaces the softmax
 * by 1 / (1 + exp(-x)) as the device pipeline does.  Ties, which the reference leaves to
 * std::nth_element, go to the lower expert id.  x is fp32 [rows, experts] (the caller up-converts);
 * renorm != 0 divides the k weights by their sum (an extension of this build's router, not in ck_tile). */
ORACLE_API int moe_oracle_topk_softmax(const float* x, int32_t rows, int32_t experts, int32_t topk, int32_t sigmoid,
                                       int32_t renorm, float* out_w, int32_t* out_idx)
{
    if(rows < 0 || experts <= 0 || topk <= 0 || topk > experts)
        return -1;
    float* y = (float*)malloc(sizeof(float) * (size_t)experts);
    if(!y)
        return -2;
    for(int64_t r = 0; r < rows; r++)
    {
        const float* xr = x + r * experts;
        if(sigmoid)
        {
            for(int e = 0; e < experts; e++)
                y[e] = 1.0f / (1.0f + expf(-xr[e]));
        }
        else
        {
            float m = -INFINITY;
            for(int e = 0; e < experts; e++)
                m = m < xr[e] ? xr[e] : m;
            float sum = 0.f;
            for(int e = 0; e < experts; e++)
                sum += expf(xr[e] - m);
            for(int e = 0; e < experts; e++)
                y[e] = expf(xr[e] - m) / sum;
        }
        float wsum = 0.f;
        for(int i = 0; i < topk; i++)
        {
            int be = 0;
            for(int e = 1; e < experts; e++)
                if(y[e] > y[be])
                    be = e;
            out_w[r * topk + i]   = y[be];
            out_idx[r * topk + i] = be;
            wsum += y[be];
            y[be] = -INFINITY;
        }
        if(renorm)
            for(int i = 0; i < topk; i++)
                out_w[r * topk + i] /= wsum;
    }
    free(y);
    return 0;
}

/* threads the OpenMP loops above will use (reported as "cores" by the CPU baseline) */
ORACLE_API int moe_oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

ORACLE_API void moe_oracle_set_num_threads(int n)
{
#ifdef _OPENMP
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}
