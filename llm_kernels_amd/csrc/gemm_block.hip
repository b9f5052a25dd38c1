// Dense block-scaled fp8 / int8 GEMM entry points.
#include <algorithm>
#include <mutex>

#include "gemm_wide.hpp"

using namespace llmk;

namespace {

int check_common(const char* name, const void* a, const void* b, int64_t M, int64_t N, int64_t K, int c_dtype) {
    if (M < 0 || N < 0 || K < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "%s: negative dimension", name);
    if (K % 128 != 0) LLMK_FAIL(LLMK_ERR_SHAPE, "%s: K=%lld must be a multiple of 128", name, (long long)K);
    if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) LLMK_FAIL(LLMK_ERR_SHAPE, "%s: dimension exceeds int32", name);
    if (c_dtype != LLMK_F32 && c_dtype != LLMK_F16 && c_dtype != LLMK_BF16) LLMK_FAIL(LLMK_ERR_DTYPE, "%s: c_dtype %d", name, c_dtype);
    if (M && N && K && (!a || !b)) LLMK_FAIL(LLMK_ERR_ARG, "%s: null operand", name);
    if ((((uintptr_t)a) | ((uintptr_t)b)) & 15) LLMK_FAIL(LLMK_ERR_ARG, "%s: operands must be 16-byte aligned", name);
    return LLMK_OK;
}

// Decode-sized M with K beyond one resident batch per wave (32 steps): the weight-streaming kernel runs on
// K ranges of at most 32 steps side by side (gridDim.z) and a second kernel adds their fp32 partial sums.
inline int stream_k_ranges(int64_t M, int64_t N, int64_t K) {
    if (M > 64 || K <= 4096 || mid_m_prefers_tiles(M, N, K)) return 1;
    return (int)((K / 128 + 31) / 32);
}

template <int KIND>
int launch_stream(DirectArgs& p, void* workspace, int64_t workspace_bytes, hipStream_t stream, const char* name) {
    const int nz = stream_k_ranges(p.M, p.N, p.K);
    const int64_t mn = (int64_t)p.M * p.N;
    if (nz > 1 && workspace && workspace_bytes >= nz * mn * 4) {
        const int steps = p.K / 128;
        p.kc_steps = ((steps + nz - 1) / nz + 3) & ~3;         // even ranges, whole 4-step groups
        p.partial = (float*)workspace;
        p.ksplit = (steps + p.kc_steps - 1) / p.kc_steps;
        int rc = launch_direct<KIND, false>(p, p.M, stream, name);
        if (rc) return rc;
        const unsigned blocks = (unsigned)((mn + 1023) / 1024);
        if (p.c_dtype == LLMK_BF16) splitk_sum_kernel<LLMK_BF16><<<blocks, 256, 0, stream>>>(p.partial, p.c, mn, p.ksplit);
        else if (p.c_dtype == LLMK_F16) splitk_sum_kernel<LLMK_F16><<<blocks, 256, 0, stream>>>(p.partial, p.c, mn, p.ksplit);
        else splitk_sum_kernel<LLMK_F32><<<blocks, 256, 0, stream>>>(p.partial, p.c, mn, p.ksplit);
        LLMK_CHECK_LAUNCH(name);
        return LLMK_OK;
    }
    return launch_direct<KIND, false>(p, p.M, stream, name);
}

}  // namespace

// scratch without the (fixed-size) part for a split last round of 256-column tiles
static int64_t workspace_core_bytes(int64_t M, int64_t N, int64_t K) {
    // large-M kernels stream fp32 activation scales; 16-bit scales are widened into the workspace first;
    // mid-size M with few tiles adds the fp32 split-K partials behind them
    if (K <= 0) return 0;
    if (M <= 64 && !mid_m_prefers_tiles(M, N, K)) {
        const int nz = stream_k_ranges(M, N, K);
        return nz > 1 ? (int64_t)nz * M * N * 4 : 0;
    }
    const int64_t scales = (M * (K / 128) * 4 + 255) & ~(int64_t)255;
    int z = splitk_factor(M, N, K);
    if (M <= 512) z = std::max({z, mid_plan(M, N, K).z, midw_plan(M, N, K).z});      // the mid-size kernels' K slices
    return scales + (z > 1 ? (int64_t)z * M * N * 4 : 0);
}

extern "C" int64_t llmk_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    // more than 512 rows and at least W_TAIL_MIN_KT K steps of 128 bytes (shorter tiles are never split): room for
    // the partial sums of a split last round of 256-column tiles behind the rest
    return workspace_core_bytes(M, N, K) + (K >= W_TAIL_MIN_KT * 128 && M > 512 ? w_tail_bytes() : 0);
}

extern "C" int llmk_gemm_fp8_block(const void* a, const float* a_s, const void* b, const float* b_s, void* c,
                                   int c_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                   int64_t workspace_bytes, void* stream) {
    int rc = check_common("gemm_fp8_block", a, b, M, N, K, c_dtype);
    if (rc) return rc;
    if (M == 0 || N == 0) return LLMK_OK;
    if (!c || (K && (!a_s || !b_s))) LLMK_FAIL(LLMK_ERR_ARG, "gemm_fp8_block: null pointer");
    DirectArgs p{};
    p.a = (const uint8_t*)a; p.b = (const uint8_t*)b; p.c = c; p.a_s = a_s; p.b_s = b_s;
    p.c_dtype = c_dtype; p.s_dtype = LLMK_F32; p.M = (int)M; p.N = (int)N; p.K = (int)K; p.E = 1;
    if (M > 64 || (mid_m_prefers_tiles(M, N, K) && workspace && workspace_bytes >= llmk_gemm_workspace_bytes(M, N, K)))
        return launch_big<K_FP8_BLOCK, false>(p, workspace, workspace_bytes, (hipStream_t)stream, "gemm_fp8_block(tiled)");
    return launch_stream<K_FP8_BLOCK>(p, workspace, workspace_bytes, (hipStream_t)stream, "gemm_fp8_block");
}

// llmk_gemm_fp8_block for the benchmark's calibration: the same launch, and workgroup 0 of the 256-column tile kernel
// reports the ticks of the shader clock and of the 100 MHz clock it lived (clocks[0], clocks[1]); shapes that run on
// other kernels leave clocks untouched.
extern "C" int llmk_calib_gemm_fp8_clock(const void* a, const float* a_s, const void* b, const float* b_s, void* c,
                                         int c_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                         int64_t workspace_bytes, long long* clocks, void* stream) {
    int rc = check_common("calib_gemm_fp8_clock", a, b, M, N, K, c_dtype);
    if (rc) return rc;
    if (M <= 64 || N == 0 || !c || !a_s || !b_s || !clocks) LLMK_FAIL(LLMK_ERR_ARG, "calib_gemm_fp8_clock: needs M > 512 and every pointer");
    DirectArgs p{};
    p.a = (const uint8_t*)a; p.b = (const uint8_t*)b; p.c = c; p.a_s = a_s; p.b_s = b_s; p.clocks = clocks;
    p.c_dtype = c_dtype; p.s_dtype = LLMK_F32; p.M = (int)M; p.N = (int)N; p.K = (int)K; p.E = 1;
    return launch_big<K_FP8_BLOCK, false>(p, workspace, workspace_bytes, (hipStream_t)stream, "calib_gemm_fp8_clock");
}

extern "C" int llmk_gemm_i8_block(const int8_t* a, const void* a_s, const int8_t* b, const void* b_s, int s_dtype,
                                  void* c, int c_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                  int64_t workspace_bytes, void* stream) {
    int rc = check_common("gemm_i8_block", a, b, M, N, K, c_dtype);
    if (rc) return rc;
    if (s_dtype != LLMK_F32 && s_dtype != LLMK_F16 && s_dtype != LLMK_BF16) LLMK_FAIL(LLMK_ERR_DTYPE, "gemm_i8_block: s_dtype %d", s_dtype);
    if (M == 0 || N == 0) return LLMK_OK;
    if (!c || (K && (!a_s || !b_s))) LLMK_FAIL(LLMK_ERR_ARG, "gemm_i8_block: null pointer");
    DirectArgs p{};
    p.a = (const uint8_t*)a; p.b = (const uint8_t*)b; p.c = c; p.a_s = a_s; p.b_s = b_s;
    p.c_dtype = c_dtype; p.s_dtype = s_dtype; p.M = (int)M; p.N = (int)N; p.K = (int)K; p.E = 1;
    if (M > 64 || (mid_m_prefers_tiles(M, N, K) && workspace && workspace_bytes >= llmk_gemm_workspace_bytes(M, N, K)))
        return launch_big<K_I8_BLOCK, false>(p, workspace, workspace_bytes, (hipStream_t)stream, "gemm_i8_block(tiled)");
    return launch_stream<K_I8_BLOCK>(p, workspace, workspace_bytes, (hipStream_t)stream, "gemm_i8_block");
}

extern "C" int llmk_gemm_i8_rowcol(const int8_t* a, const float* a_s, const int8_t* b, const float* b_s, void* c,
                                   int c_dtype, int32_t* c_i32, int64_t M, int64_t N, int64_t K, void* workspace,
                                   int64_t workspace_bytes, void* stream) {
    int rc = check_common("gemm_i8_rowcol", a, b, M, N, K, c_dtype);
    if (rc) return rc;
    if (M == 0 || N == 0) return LLMK_OK;
    if (!c && !c_i32) LLMK_FAIL(LLMK_ERR_ARG, "gemm_i8_rowcol: no output buffer");
    if (c && (!a_s || !b_s)) LLMK_FAIL(LLMK_ERR_ARG, "gemm_i8_rowcol: scales required for the scaled output");
    DirectArgs p{};
    p.a = (const uint8_t*)a; p.b = (const uint8_t*)b; p.c = c; p.c_i32 = c_i32; p.a_s = a_s; p.b_s = b_s;
    p.c_dtype = c_dtype; p.s_dtype = LLMK_F32; p.M = (int)M; p.N = (int)N; p.K = (int)K; p.E = 1;
    // large M: the tile kernels accumulate int32 over the whole K range inside the MFMA and scale in the epilogue
    if (M > 64 && dma_eligible(p)) {
        // few tiles and a long K: K slices over the CUs, int32 partial sums in the workspace, one pass that adds
        // them as integers and scales (same bits as the unsplit kernel)
        if (mid_wanted(M, N, K)) {
            MidPlan pl = mid_plan(M, N, K);
            if (pl.z > 1 && !(workspace && workspace_bytes >= (int64_t)pl.z * M * N * 4 && !((uintptr_t)workspace & 15))) pl.z = 1;
            if (mid_eligible<K_I8_ROWCOL>(p, pl.mt, pl.z)) {
                if (pl.z > 1) { p.partial = (float*)workspace; p.ksplit = pl.z; }
                return pl.mt == 4 ? launch_mid<K_I8_ROWCOL, 4>(p, (hipStream_t)stream, "gemm_i8_rowcol(mid)")
                                  : launch_mid<K_I8_ROWCOL, 2>(p, (hipStream_t)stream, "gemm_i8_rowcol(mid)");
            }
        }
        const int z = splitk_factor(M, N, K);
        if (z > 1 && workspace && workspace_bytes >= (int64_t)z * M * N * 4 && !((uintptr_t)workspace & 15)) {
            p.partial = (float*)workspace;
            p.ksplit = z;
        }
        return launch_dma<K_I8_ROWCOL, false>(p, (hipStream_t)stream, "gemm_i8_rowcol(tiled)");
    }
    return launch_direct<K_I8_ROWCOL, false>(p, (int)M, (hipStream_t)stream, "gemm_i8_rowcol");
}

// ------------------------------------------------------------------ llmk_gemm_fp8_block without a scratch argument
// For callers that cannot allocate device memory (HIP graph capture, serving loops, harnesses that forbid
// hipMalloc): the fp32 partial sums of the split-K / K-range kernels live in a file-scope device array instead
// of a caller-provided buffer.  Every GPU the library runs on holds its own copy of the array until the
// process ends; its address on a device is looked up once, with that device current, and only that address
// (never the array's name, which is a host-side stand-in) is handed to kernels.
namespace {

static __device__ __align__(256) unsigned char scratch[LLMK_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

int static_scratch(void** out, const char* name) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) LLMK_FAIL(LLMK_ERR_LAUNCH, "%s: hipGetDevice: %s", name, hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) LLMK_FAIL(LLMK_ERR_ARG, "%s: device ordinal %d out of range", name, dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            LLMK_FAIL(LLMK_ERR_LAUNCH, "%s: hipGetSymbolAddress(scratch) on device %d: %s", name, dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return LLMK_OK;
}

}  // namespace

extern "C" int llmk_gemm_fp8_block_static(const void* a, const float* a_s, const void* b, const float* b_s, void* c,
                                          int c_dtype, int64_t M, int64_t N, int64_t K, void* stream) {
    int rc = check_common("gemm_fp8_block_static", a, b, M, N, K, c_dtype);
    if (rc) return rc;
    // (the built-in array serves the scratch a shape cannot do without efficiently; the optional partial sums of a
    // split last round of tiles, 64 MiB, are left out: large shapes run unsplit here)
    const int64_t need = workspace_core_bytes(M, N, K);
    if (need > (int64_t)LLMK_STATIC_SCRATCH_BYTES)
        LLMK_FAIL(LLMK_ERR_SHAPE, "gemm_fp8_block_static: M=%lld N=%lld K=%lld needs %lld bytes of scratch, the built-in "
                  "buffer holds %lld; use llmk_gemm_fp8_block with a caller-provided workspace",
                  (long long)M, (long long)N, (long long)K, (long long)need, (long long)LLMK_STATIC_SCRATCH_BYTES);
    void* ws = nullptr;
    if (need > 0) {
        rc = static_scratch(&ws, "gemm_fp8_block_static");
        if (rc) return rc;
    }
    // Every plane of partial sums is written in full by the first kernel before the summing kernel reads it,
    // so nothing in the array has to start at zero; what a previous (possibly larger) call left is never read.
    return llmk_gemm_fp8_block(a, a_s, b, b_s, c, c_dtype, M, N, K, ws, need > 0 ? need : 0, stream);
}
