// n-bit pack / unpack kernels (pure streaming integer work; HBM bound).
#include "common.hpp"

namespace {

__device__ __forceinline__ uint64_t load_uint(const void* p, int64_t i, int bytes) {
    switch (bytes) {
        case 1: return ((const uint8_t*)p)[i];
        case 2: return ((const uint16_t*)p)[i];
        case 4: return ((const uint32_t*)p)[i];
        default: return ((const uint64_t*)p)[i];
    }
}
__device__ __forceinline__ void store_uint(void* p, int64_t i, int bytes, uint64_t v) {
    switch (bytes) {
        case 1: ((uint8_t*)p)[i] = (uint8_t)v; break;
        case 2: ((uint16_t*)p)[i] = (uint16_t)v; break;
        case 4: ((uint32_t*)p)[i] = (uint32_t)v; break;
        default: ((uint64_t*)p)[i] = v; break;
    }
}

// one thread per packed word; lanes run along the contiguous column axis of both matrices
template <int IN_BYTES, int OUT_BYTES>
__global__ void pack_rows_kernel(const void* __restrict__ in, void* __restrict__ out,
                                 int64_t rows_out, int64_t cols, int nbits, int e) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows_out * cols) return;
    int64_t r = idx / cols, c = idx - r * cols;
    uint64_t acc = 0;
    for (int i = 0; i < e; ++i)
        acc |= load_uint(in, (r * e + i) * cols + c, IN_BYTES) << (i * nbits);
    store_uint(out, idx, OUT_BYTES, acc);
}

template <int IN_BYTES, int OUT_BYTES>
__global__ void pack_cols_kernel(const void* __restrict__ in, void* __restrict__ out,
                                 int64_t rows, int64_t cols_out, int nbits, int e) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * cols_out) return;
    uint64_t acc = 0;
    const int64_t base = idx * e;            // in is [rows, cols_out*e] contiguous
    for (int i = 0; i < e; ++i)
        acc |= load_uint(in, base + i, IN_BYTES) << (i * nbits);
    store_uint(out, idx, OUT_BYTES, acc);
}

// one thread per unpacked element
template <int PK_BYTES, int OUT_BYTES>
__global__ void unpack_rows_kernel(const void* __restrict__ packed, void* __restrict__ out,
                                   int64_t rows_packed, int64_t cols, int nbits, int e) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows_packed * e * cols) return;
    int64_t ro = idx / cols, c = idx - ro * cols;
    int64_t r = ro / e;
    int i = (int)(ro - r * e);
    uint64_t w = load_uint(packed, r * cols + c, PK_BYTES);
    uint64_t mask = (nbits >= 64) ? ~0ull : ((1ull << nbits) - 1ull);
    store_uint(out, idx, OUT_BYTES, (w >> (i * nbits)) & mask);
}

template <int PK_BYTES, int OUT_BYTES>
__global__ void unpack_cols_kernel(const void* __restrict__ packed, void* __restrict__ out,
                                   int64_t rows, int64_t cols_packed, int nbits, int e) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows * cols_packed * e) return;
    int64_t w_idx = idx / e;
    int i = (int)(idx - w_idx * e);
    uint64_t w = load_uint(packed, w_idx, PK_BYTES);
    uint64_t mask = (nbits >= 64) ? ~0ull : ((1ull << nbits) - 1ull);
    store_uint(out, idx, OUT_BYTES, (w >> (i * nbits)) & mask);
}

bool valid_bytes(int b) { return b == 1 || b == 2 || b == 4 || b == 8; }
bool valid_pack(int nbits, int pack_bits) {
    return (pack_bits == 8 || pack_bits == 16 || pack_bits == 32 || pack_bits == 64) &&
           (nbits == 1 || nbits == 2 || nbits == 4 || nbits == 8);
}

#define LLMK_BYTES_SWITCH2(a, b, CALL)                                         \
    switch ((a) * 16 + (b)) {                                                  \
        case 0x11: CALL(1, 1); break; case 0x12: CALL(1, 2); break;            \
        case 0x14: CALL(1, 4); break; case 0x18: CALL(1, 8); break;            \
        case 0x21: CALL(2, 1); break; case 0x22: CALL(2, 2); break;            \
        case 0x24: CALL(2, 4); break; case 0x28: CALL(2, 8); break;            \
        case 0x41: CALL(4, 1); break; case 0x42: CALL(4, 2); break;            \
        case 0x44: CALL(4, 4); break; case 0x48: CALL(4, 8); break;            \
        case 0x81: CALL(8, 1); break; case 0x82: CALL(8, 2); break;            \
        case 0x84: CALL(8, 4); break; case 0x88: CALL(8, 8); break;            \
        default: LLMK_FAIL(LLMK_ERR_DTYPE, "unsupported element widths %d/%d", (a), (b)); \
    }

}  // namespace

extern "C" int llmk_pack_rows(const void* in, int in_bytes, void* out, int64_t rows_out, int64_t cols,
                              int nbits, int pack_bits, void* stream) {
    if (!valid_pack(nbits, pack_bits) || !valid_bytes(in_bytes))
        LLMK_FAIL(LLMK_ERR_DTYPE, "pack_rows: nbits=%d pack_bits=%d in_bytes=%d", nbits, pack_bits, in_bytes);
    if (rows_out < 0 || cols < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "pack_rows: negative shape");
    int64_t n = rows_out * cols;
    if (n == 0) return LLMK_OK;
    if (!in || !out) LLMK_FAIL(LLMK_ERR_ARG, "pack_rows: null pointer");
    const int e = pack_bits / nbits, ob = pack_bits / 8;
    dim3 grid((unsigned)cdiv64(n, 256)), block(256);
#define CALL(IB, OB) pack_rows_kernel<IB, OB><<<grid, block, 0, (hipStream_t)stream>>>(in, out, rows_out, cols, nbits, e)
    LLMK_BYTES_SWITCH2(in_bytes, ob, CALL)
#undef CALL
    LLMK_CHECK_LAUNCH("pack_rows");
    return LLMK_OK;
}

extern "C" int llmk_pack_cols(const void* in, int in_bytes, void* out, int64_t rows, int64_t cols_out,
                              int nbits, int pack_bits, void* stream) {
    if (!valid_pack(nbits, pack_bits) || !valid_bytes(in_bytes))
        LLMK_FAIL(LLMK_ERR_DTYPE, "pack_cols: nbits=%d pack_bits=%d in_bytes=%d", nbits, pack_bits, in_bytes);
    if (rows < 0 || cols_out < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "pack_cols: negative shape");
    int64_t n = rows * cols_out;
    if (n == 0) return LLMK_OK;
    if (!in || !out) LLMK_FAIL(LLMK_ERR_ARG, "pack_cols: null pointer");
    const int e = pack_bits / nbits, ob = pack_bits / 8;
    dim3 grid((unsigned)cdiv64(n, 256)), block(256);
#define CALL(IB, OB) pack_cols_kernel<IB, OB><<<grid, block, 0, (hipStream_t)stream>>>(in, out, rows, cols_out, nbits, e)
    LLMK_BYTES_SWITCH2(in_bytes, ob, CALL)
#undef CALL
    LLMK_CHECK_LAUNCH("pack_cols");
    return LLMK_OK;
}

extern "C" int llmk_unpack_rows(const void* packed, int pack_bits, void* out, int out_bytes,
                                int64_t rows_packed, int64_t cols, int nbits, int e, void* stream) {
    if (!valid_pack(nbits, pack_bits) || !valid_bytes(out_bytes) || e < 1 || e * nbits > pack_bits)
        LLMK_FAIL(LLMK_ERR_DTYPE, "unpack_rows: nbits=%d pack_bits=%d out_bytes=%d e=%d", nbits, pack_bits, out_bytes, e);
    if (rows_packed < 0 || cols < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "unpack_rows: negative shape");
    int64_t n = rows_packed * e * cols;
    if (n == 0) return LLMK_OK;
    if (!packed || !out) LLMK_FAIL(LLMK_ERR_ARG, "unpack_rows: null pointer");
    const int pb = pack_bits / 8;
    dim3 grid((unsigned)cdiv64(n, 256)), block(256);
#define CALL(PB, OB) unpack_rows_kernel<PB, OB><<<grid, block, 0, (hipStream_t)stream>>>(packed, out, rows_packed, cols, nbits, e)
    LLMK_BYTES_SWITCH2(pb, out_bytes, CALL)
#undef CALL
    LLMK_CHECK_LAUNCH("unpack_rows");
    return LLMK_OK;
}

extern "C" int llmk_unpack_cols(const void* packed, int pack_bits, void* out, int out_bytes,
                                int64_t rows, int64_t cols_packed, int nbits, int e, void* stream) {
    if (!valid_pack(nbits, pack_bits) || !valid_bytes(out_bytes) || e < 1 || e * nbits > pack_bits)
        LLMK_FAIL(LLMK_ERR_DTYPE, "unpack_cols: nbits=%d pack_bits=%d out_bytes=%d e=%d", nbits, pack_bits, out_bytes, e);
    if (rows < 0 || cols_packed < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "unpack_cols: negative shape");
    int64_t n = rows * cols_packed * e;
    if (n == 0) return LLMK_OK;
    if (!packed || !out) LLMK_FAIL(LLMK_ERR_ARG, "unpack_cols: null pointer");
    const int pb = pack_bits / 8;
    dim3 grid((unsigned)cdiv64(n, 256)), block(256);
#define CALL(PB, OB) unpack_cols_kernel<PB, OB><<<grid, block, 0, (hipStream_t)stream>>>(packed, out, rows, cols_packed, nbits, e)
    LLMK_BYTES_SWITCH2(pb, out_bytes, CALL)
#undef CALL
    LLMK_CHECK_LAUNCH("unpack_cols");
    return LLMK_OK;
}
