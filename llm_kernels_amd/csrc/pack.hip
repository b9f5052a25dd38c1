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

// ---- uint8 elements, 16 bytes per load and store.  The kernels above move one element (or one word) per thread and
// request; at 4 bits in 32-bit words they reach 0.8 to 2.4 TB/s.  NBITS / PB (bytes of a packed word) are compile-time so
// that every shift is an immediate and the element loops run in registers.
typedef unsigned v4u __attribute__((ext_vector_type(4)));

template <int PB> struct WordOf { typedef uint32_t T; };
template <> struct WordOf<8> { typedef uint64_t T; };

// byte j (0 .. 15) of a 16-byte vector
__device__ __forceinline__ unsigned byte_of(const v4u& v, int j) { return (v[j >> 2] >> (8 * (j & 3))) & 0xffu; }

// out[r][c] = sum_i in[r e + i][c] << (i NBITS): a thread takes 16 consecutive columns of one packed row
template <int NBITS, int PB>
__global__ void pack_rows_vec_kernel(const uint8_t* __restrict__ in, uint8_t* __restrict__ out, int64_t rows_out, int64_t cols) {
    typedef typename WordOf<PB>::T W;
    constexpr int E = PB * 8 / NBITS;
    const int64_t cv = cols >> 4;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows_out * cv) return;
    const int64_t r = idx / cv, c0 = (idx - r * cv) << 4;
    W acc[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[j] = 0;
#pragma unroll 8
    for (int i = 0; i < E; ++i) {
        const v4u v = *(const v4u*)(in + (r * E + i) * cols + c0);
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[j] |= (W)byte_of(v, j) << (i * NBITS);
    }
    uint8_t* dst = out + (r * cols + c0) * PB;
    if constexpr (PB == 8) {
#pragma unroll
        for (int j = 0; j < 16; j += 2) *(v4u*)(dst + j * 8) = (v4u){(unsigned)acc[j], (unsigned)(acc[j] >> 32), (unsigned)acc[j + 1], (unsigned)(acc[j + 1] >> 32)};
    } else if constexpr (PB == 4) {
#pragma unroll
        for (int j = 0; j < 16; j += 4) *(v4u*)(dst + j * 4) = (v4u){(unsigned)acc[j], (unsigned)acc[j + 1], (unsigned)acc[j + 2], (unsigned)acc[j + 3]};
    } else if constexpr (PB == 2) {
        v4u a, b;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            a[q] = (unsigned)acc[2 * q] | ((unsigned)acc[2 * q + 1] << 16);
            b[q] = (unsigned)acc[8 + 2 * q] | ((unsigned)acc[9 + 2 * q] << 16);
        }
        *(v4u*)dst = a;
        *(v4u*)(dst + 16) = b;
    } else {
        v4u a;
#pragma unroll
        for (int q = 0; q < 4; ++q)
            a[q] = (unsigned)acc[4 * q] | ((unsigned)acc[4 * q + 1] << 8) | ((unsigned)acc[4 * q + 2] << 16) | ((unsigned)acc[4 * q + 3] << 24);
        *(v4u*)dst = a;
    }
}

// out[w] = sum_i in[w e + i] << (i NBITS) over the flat arrays: a thread takes max(16, e) input bytes
template <int NBITS, int PB>
__global__ void pack_cols_vec_kernel(const uint8_t* __restrict__ in, uint8_t* __restrict__ out, int64_t words) {
    typedef typename WordOf<PB>::T W;
    constexpr int E = PB * 8 / NBITS;
    constexpr int LOADS = E > 16 ? E / 16 : 1;            // 16-byte loads per thread
    constexpr int WPT = E > 16 ? 1 : 16 / E;              // words per thread
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx * WPT >= words) return;
    W w[WPT];
#pragma unroll
    for (int q = 0; q < WPT; ++q) w[q] = 0;
    const uint8_t* src = in + idx * (LOADS * 16);
#pragma unroll
    for (int l = 0; l < LOADS; ++l) {
        const v4u v = *(const v4u*)(src + 16 * l);
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int k = 16 * l + j;                     // element of this thread's run
            w[k / E] |= (W)byte_of(v, j) << ((k % E) * NBITS);
        }
    }
    uint8_t* dst = out + idx * (WPT * PB);
#pragma unroll
    for (int q = 0; q < WPT; ++q) *(W*)(dst + q * PB) = w[q];          // (runs of up to 16 bytes; the compiler merges them)
}
template <> struct WordOf<1> { typedef uint8_t T; };
template <> struct WordOf<2> { typedef uint16_t T; };

// out[r e + i][c] = (packed[r][c] >> (i NBITS)) & mask: a thread takes 16 bytes of packed words of one row and writes,
// for every i, the 16 / PB elements they hold
template <int NBITS, int PB>
__global__ void unpack_rows_vec_kernel(const uint8_t* __restrict__ packed, uint8_t* __restrict__ out, int64_t rows_packed, int64_t cols, int e) {
    constexpr int WPT = 16 / PB;
    constexpr unsigned MASK = (1u << NBITS) - 1u;
    const int64_t cv = cols / WPT;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= rows_packed * cv) return;
    const int64_t r = idx / cv, c0 = (idx - r * cv) * WPT;
    const v4u v = *(const v4u*)(packed + (r * cols + c0) * PB);
    uint64_t w[WPT];
#pragma unroll
    for (int q = 0; q < WPT; ++q) {
        if constexpr (PB == 8) w[q] = (uint64_t)v[2 * q] | ((uint64_t)v[2 * q + 1] << 32);
        else if constexpr (PB == 4) w[q] = v[q];
        else if constexpr (PB == 2) w[q] = (v[q >> 1] >> (16 * (q & 1))) & 0xffffu;
        else w[q] = byte_of(v, q);
    }
    for (int i = 0; i < e; ++i) {
        uint8_t* dst = out + (r * e + i) * cols + c0;
        if constexpr (WPT == 2) {
            *(uint16_t*)dst = (uint16_t)(((w[0] >> (i * NBITS)) & MASK) | (((w[1] >> (i * NBITS)) & MASK) << 8));
        } else {
#pragma unroll
            for (int d = 0; d < WPT / 4; ++d) {
                unsigned o = 0;
#pragma unroll
                for (int b = 0; b < 4; ++b) o |= (unsigned)((w[4 * d + b] >> (i * NBITS)) & MASK) << (8 * b);
                *(unsigned*)(dst + 4 * d) = o;
            }
        }
    }
}

// out[w e + i] = (packed[w] >> (i NBITS)) & mask over the flat arrays: a thread takes 16 bytes of packed words
template <int NBITS, int PB>
__global__ void unpack_cols_vec_kernel(const uint8_t* __restrict__ packed, uint8_t* __restrict__ out, int64_t words) {
    constexpr int WPT = 16 / PB, E = PB * 8 / NBITS;
    constexpr unsigned MASK = (1u << NBITS) - 1u;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx * WPT >= words) return;
    const v4u v = *(const v4u*)(packed + idx * 16);
    uint8_t* dst = out + idx * (WPT * E);
#pragma unroll
    for (int q = 0; q < WPT; ++q) {
        uint64_t w;
        if constexpr (PB == 8) w = (uint64_t)v[2 * q] | ((uint64_t)v[2 * q + 1] << 32);
        else if constexpr (PB == 4) w = v[q];
        else if constexpr (PB == 2) w = (v[q >> 1] >> (16 * (q & 1))) & 0xffffu;
        else w = byte_of(v, q);
        // E output bytes of this word, four at a time (E = 1, 2 for the narrowest words: single bytes)
        if constexpr (E >= 4) {
#pragma unroll
            for (int d = 0; d < E / 4; ++d) {
                unsigned o = 0;
#pragma unroll
                for (int b = 0; b < 4; ++b) o |= (unsigned)((w >> ((4 * d + b) * NBITS)) & MASK) << (8 * b);
                *(unsigned*)(dst + q * E + 4 * d) = o;
            }
        } else {
#pragma unroll
            for (int b = 0; b < E; ++b) dst[q * E + b] = (uint8_t)((w >> (b * NBITS)) & MASK);
        }
    }
}

#define LLMK_NBITS_PB_SWITCH(nbits, pb, CALL)                                                            \
    switch ((nbits) * 16 + (pb)) {                                                                       \
        case 0x11: CALL(1, 1); break; case 0x12: CALL(1, 2); break; case 0x14: CALL(1, 4); break; case 0x18: CALL(1, 8); break; \
        case 0x21: CALL(2, 1); break; case 0x22: CALL(2, 2); break; case 0x24: CALL(2, 4); break; case 0x28: CALL(2, 8); break; \
        case 0x41: CALL(4, 1); break; case 0x42: CALL(4, 2); break; case 0x44: CALL(4, 4); break; case 0x48: CALL(4, 8); break; \
        case 0x81: CALL(8, 1); break; case 0x82: CALL(8, 2); break; case 0x84: CALL(8, 4); break; case 0x88: CALL(8, 8); break; \
        default: break;                                                                                  \
    }

bool aligned16(const void* a, const void* b) { return ((((uintptr_t)a) | ((uintptr_t)b)) & 15) == 0; }

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
    if (in_bytes == 1 && cols % 16 == 0 && aligned16(in, out)) {        // 16 columns per thread
        dim3 vgrid((unsigned)cdiv64(rows_out * (cols / 16), 256));
#define CALL(NB, PB) pack_rows_vec_kernel<NB, PB><<<vgrid, 256, 0, (hipStream_t)stream>>>((const uint8_t*)in, (uint8_t*)out, rows_out, cols)
        LLMK_NBITS_PB_SWITCH(nbits, ob, CALL)
#undef CALL
        LLMK_CHECK_LAUNCH("pack_rows");
        return LLMK_OK;
    }
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
    {
        const int wpt = e > 16 ? 1 : 16 / e;                              // words per thread of the 16-byte kernel
        if (in_bytes == 1 && n % wpt == 0 && aligned16(in, out)) {
            dim3 vgrid((unsigned)cdiv64(n / wpt, 256));
#define CALL(NB, PB) pack_cols_vec_kernel<NB, PB><<<vgrid, 256, 0, (hipStream_t)stream>>>((const uint8_t*)in, (uint8_t*)out, n)
            LLMK_NBITS_PB_SWITCH(nbits, ob, CALL)
#undef CALL
            LLMK_CHECK_LAUNCH("pack_cols");
            return LLMK_OK;
        }
    }
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
    if (out_bytes == 1 && cols % (16 / pb) == 0 && cols % 4 == 0 && aligned16(packed, out)) {     // 16 bytes of packed words per thread
        dim3 vgrid((unsigned)cdiv64(rows_packed * (cols / (16 / pb)), 256));
#define CALL(NB, PB) unpack_rows_vec_kernel<NB, PB><<<vgrid, 256, 0, (hipStream_t)stream>>>((const uint8_t*)packed, (uint8_t*)out, rows_packed, cols, e)
        LLMK_NBITS_PB_SWITCH(nbits, pb, CALL)
#undef CALL
        LLMK_CHECK_LAUNCH("unpack_rows");
        return LLMK_OK;
    }
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
    if (out_bytes == 1 && e == pack_bits / nbits && (rows * cols_packed) % (16 / pb) == 0 && aligned16(packed, out)) {   // full words, 16 bytes per thread
        dim3 vgrid((unsigned)cdiv64(rows * cols_packed / (16 / pb), 256));
#define CALL(NB, PB) unpack_cols_vec_kernel<NB, PB><<<vgrid, 256, 0, (hipStream_t)stream>>>((const uint8_t*)packed, (uint8_t*)out, rows * cols_packed)
        LLMK_NBITS_PB_SWITCH(nbits, pb, CALL)
#undef CALL
        LLMK_CHECK_LAUNCH("unpack_cols");
        return LLMK_OK;
    }
    dim3 grid((unsigned)cdiv64(n, 256)), block(256);
#define CALL(PB, OB) unpack_cols_kernel<PB, OB><<<grid, block, 0, (hipStream_t)stream>>>(packed, out, rows, cols_packed, nbits, e)
    LLMK_BYTES_SWITCH2(pb, out_bytes, CALL)
#undef CALL
    LLMK_CHECK_LAUNCH("unpack_cols");
    return LLMK_OK;
}
