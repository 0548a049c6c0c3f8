// oracle/_ref/libck_ref_gpu.so: ck_tile's DEVICE reference of the unfused MoE GEMMs
// (host/reference/reference_moe_gemm.hpp), compiled from the headers installed with ROCm.  Test
// infrastructure only; kept apart from libck_ref.so because a library with device code initialises the
// HIP runtime when it is loaded, which must not happen before the process under test has set up its own.
#include <cstring> // must precede the ck_tile headers (host memcpy overload)
#include <cstdint>

#include <hip/hip_runtime.h>

#include "ck_tile/core.hpp"
#include "ck_tile/host/host_tensor.hpp"
#include "ck_tile/ops/elementwise/unary_element_wise_operation.hpp"
#include "ck_tile/ops/common/tensor_layout.hpp"
#include "ck_tile/host/reference/reference_moe_gemm.hpp"
#include "ck_tile/host/kernel_launch.hpp"
#include "ck_tile/ops/flatmm/kernel/moe_flatmm_kernel.hpp" // ck_tile::moe::MoeSilu, ck_tile::moe::Swiglu

using ck_tile::index_t;

namespace {

// ck_tile's reference of the unfused MoE GEMMs is a device kernel (reference_moe_gemm.hpp:18-330): this
// wrapper stages host buffers through device memory and runs it on the current GPU.  A, B, C hold bf16
// bits; scale_a [rows of A] and scale_b [E, N] are fp32 (pass ones for "no scale": the kernel always reads
// them); bias [E, N] fp32 or null.  The activation is ck_tile's own functor, default-constructed by the
// kernel: ck_tile::moe::MoeSilu or ck_tile::moe::Swiglu (alpha 1.702, limit 7;
// ops/flatmm/kernel/moe_flatmm_kernel.hpp:139-183).  Returns 0, or a negative HIP error code.
template <int KIND, typename Act>
static int run_moe_gemm_gpu(const int32_t* ids, const int32_t* eid, int32_t max_token_id, const uint16_t* A,
                            const uint16_t* B, uint16_t* C, const float* w, int32_t T, int32_t block, int32_t topk,
                            int32_t M, int32_t E, int32_t N, int32_t K, int64_t a_rows, int64_t c_rows, int32_t c_cols,
                            const float* sa, const float* sb, const float* bias)
{
    using bf16 = ck_tile::bf16_t;
    using Row  = ck_tile::tensor_layout::gemm::RowMajor;
    using Col  = ck_tile::tensor_layout::gemm::ColumnMajor;
    int32_t *d_ids = nullptr, *d_eid = nullptr, *d_max = nullptr;
    bf16 *d_a = nullptr, *d_b = nullptr, *d_c = nullptr;
    float *d_w = nullptr, *d_sa = nullptr, *d_sb = nullptr, *d_bias = nullptr;
    const size_t tiles = (size_t)(M + block - 1) / block;
#define CKR(x)                      \
    do                              \
    {                               \
        hipError_t e_ = (x);        \
        if(e_ != hipSuccess)        \
            return -(int)e_ - 1000; \
    } while(0)
    CKR(hipMalloc(&d_ids, sizeof(int32_t) * M));
    CKR(hipMalloc(&d_eid, sizeof(int32_t) * tiles));
    CKR(hipMalloc(&d_max, sizeof(int32_t)));
    CKR(hipMalloc(&d_a, 2 * (size_t)a_rows * K));
    CKR(hipMalloc(&d_b, 2 * (size_t)E * N * K));
    CKR(hipMalloc(&d_c, 2 * (size_t)c_rows * c_cols));
    CKR(hipMalloc(&d_w, sizeof(float) * M));
    CKR(hipMalloc(&d_sa, sizeof(float) * a_rows));
    CKR(hipMalloc(&d_sb, sizeof(float) * (size_t)E * N));
    CKR(hipMemcpy(d_ids, ids, sizeof(int32_t) * M, hipMemcpyHostToDevice));
    CKR(hipMemcpy(d_eid, eid, sizeof(int32_t) * tiles, hipMemcpyHostToDevice));
    CKR(hipMemcpy(d_max, &max_token_id, sizeof(int32_t), hipMemcpyHostToDevice));
    CKR(hipMemcpy(d_a, A, 2 * (size_t)a_rows * K, hipMemcpyHostToDevice));
    CKR(hipMemcpy(d_b, B, 2 * (size_t)E * N * K, hipMemcpyHostToDevice));
    CKR(hipMemcpy(d_c, C, 2 * (size_t)c_rows * c_cols, hipMemcpyHostToDevice));
    CKR(hipMemcpy(d_w, w, sizeof(float) * M, hipMemcpyHostToDevice));
    CKR(hipMemcpy(d_sa, sa, sizeof(float) * a_rows, hipMemcpyHostToDevice));
    CKR(hipMemcpy(d_sb, sb, sizeof(float) * (size_t)E * N, hipMemcpyHostToDevice));
    if(bias != nullptr)
    {
        CKR(hipMalloc(&d_bias, sizeof(float) * (size_t)E * N));
        CKR(hipMemcpy(d_bias, bias, sizeof(float) * (size_t)E * N, hipMemcpyHostToDevice));
    }
    ck_tile::reference_moe_gemm_gpu<bf16, bf16, float, bf16, Row, Col, Row, KIND, Act>(
        d_ids, d_eid, d_max, d_a, d_b, d_c, d_w, T, block, topk, M, N, K, K, K, c_cols, 1, 1, K, d_sa, d_sb, d_bias);
    CKR(hipGetLastError());
    CKR(hipDeviceSynchronize());
    CKR(hipMemcpy(C, d_c, 2 * (size_t)c_rows * c_cols, hipMemcpyDeviceToHost));
#undef CKR
    for(void* ptr : {(void*)d_ids, (void*)d_eid, (void*)d_max, (void*)d_a, (void*)d_b, (void*)d_c, (void*)d_w,
                     (void*)d_sa, (void*)d_sb, (void*)d_bias})
        (void)hipFree(ptr);
    return 0;
}

template <typename Act>
static int dispatch_kind(int32_t kind, const int32_t* ids, const int32_t* eid, int32_t max_token_id, const uint16_t* A,
                         const uint16_t* B, uint16_t* C, const float* w, int32_t T, int32_t block, int32_t topk, int32_t M,
                         int32_t E, int32_t N, int32_t K, const float* sa, const float* sb, const float* bias)
{
    if(kind == 0)
        return run_moe_gemm_gpu<0, Act>(ids, eid, max_token_id, A, B, C, w, T, block, topk, M, E, N, K, T, (int64_t)T * topk,
                                        N, sa, sb, bias);
    if(kind == 1)
        return run_moe_gemm_gpu<1, Act>(ids, eid, max_token_id, A, B, C, w, T, block, topk, M, E, N, K, T, (int64_t)T * topk,
                                        N / 2, sa, sb, bias);
    if(kind == 2)
        return run_moe_gemm_gpu<2, Act>(ids, eid, max_token_id, A, B, C, w, T, block, topk, M, E, N, K, (int64_t)T * topk, T,
                                        N, sa, sb, bias);
    return -1;
}

} // namespace

extern "C" {

// act: 0 = ck_tile::moe::MoeSilu, 1 = ck_tile::moe::Swiglu (default alpha and limit); bias may be null
__attribute__((visibility("default"))) int
ck_ref_moe_gemm_gpu(int32_t kind, const int32_t* ids, const int32_t* eid, int32_t max_token_id, const uint16_t* A,
                    const uint16_t* B, uint16_t* C, const float* w, int32_t T, int32_t block, int32_t topk, int32_t M,
                    int32_t E, int32_t N, int32_t K, const float* sa, const float* sb, const float* bias, int32_t act)
{
    if(act == 1)
        return dispatch_kind<ck_tile::moe::Swiglu>(kind, ids, eid, max_token_id, A, B, C, w, T, block, topk, M, E, N, K, sa, sb,
                                                   bias);
    return dispatch_kind<ck_tile::moe::MoeSilu>(kind, ids, eid, max_token_id, A, B, C, w, T, block, topk, M, E, N, K, sa, sb,
                                                bias);
}
}
