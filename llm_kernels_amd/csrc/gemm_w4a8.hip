// W4A8 GEMM: int8 activations x row-packed uint4 weights with two-level scales.
#include "gemm_direct.hpp"

using namespace llmk;

namespace {

// packed [N/8, K] int32 -> b8 [N, K] int8 with b8 = int8(int8(q - z4) * s4) (two's-complement wrap)
__global__ void w4a8_expand_kernel(const int32_t* __restrict__ packed, const int8_t* __restrict__ s4,
                                   const int8_t* __restrict__ z4, int8_t* __restrict__ out,
                                   int64_t N, int64_t K, int group) {
    // one thread: 8 rows x 4 consecutive k
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t kq = K / 4;
    if (idx >= (N / 8) * kq) return;
    const int64_t pr = idx / kq, k = (idx - pr * kq) * 4;
    const v4i w = *(const v4i*)(packed + pr * K + k);
    const int64_t kg = K / group;
    const int64_t gi = k / group;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int64_t n = pr * 8 + i;
        const int z = z4[n * kg + gi], s = s4[n * kg + gi];
        unsigned o = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int q = (w[j] >> (4 * i)) & 0xf;
            const int d = (int)(int8_t)(q - z);
            o |= ((unsigned)((d * s) & 0xff)) << (8 * j);
        }
        *(unsigned*)(out + n * K + k) = o;
    }
}

}  // namespace

extern "C" int llmk_gemm_w4a8(const int8_t* a, const void* a_s, const int32_t* b_packed, const void* b_s, int s_dtype,
                              const int8_t* b_s4, const int8_t* b_z4, void* c, int c_dtype, int64_t M, int64_t N,
                              int64_t K, int group_int4, void* workspace, int64_t workspace_bytes, void* stream) {
    if (M < 0 || N < 0 || K < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_w4a8: negative dimension");
    if (K % 128 || N % 8) LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_w4a8: need K %% 128 == 0 and N %% 8 == 0 (K=%lld N=%lld)", (long long)K, (long long)N);
    if (group_int4 < 4 || group_int4 % 4 || K % group_int4) LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_w4a8: group_int4=%d must divide K and be a multiple of 4", group_int4);
    if (M == 0 || N == 0) return LLMK_OK;
    if (!a || !a_s || !b_packed || !b_s || !b_s4 || !b_z4 || !c) LLMK_FAIL(LLMK_ERR_ARG, "gemm_w4a8: null pointer");
    if (!workspace || workspace_bytes < N * K) LLMK_FAIL(LLMK_ERR_ARG, "gemm_w4a8: workspace of N*K=%lld bytes required", (long long)(N * K));
    if (K > 0) {
        dim3 grid((unsigned)cdiv64((N / 8) * (K / 4), 256)), blk(256);
        w4a8_expand_kernel<<<grid, blk, 0, (hipStream_t)stream>>>(b_packed, b_s4, b_z4, (int8_t*)workspace, N, K, group_int4);
        LLMK_CHECK_LAUNCH("gemm_w4a8(expand)");
    }
    // what is left of the workspace behind the expanded weights (16-byte aligned) serves the int8 GEMM
    const int64_t used = (N * K + 15) & ~(int64_t)15;
    void* rest = workspace_bytes > used ? (void*)((uint8_t*)workspace + used) : nullptr;
    const int64_t rest_bytes = rest ? workspace_bytes - used : 0;
    return llmk_gemm_i8_block(a, a_s, (const int8_t*)workspace, b_s, s_dtype, c, c_dtype, M, N, K, rest, rest_bytes, stream);
}
