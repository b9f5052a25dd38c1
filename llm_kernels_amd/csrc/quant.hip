// Activation / weight quantizers and dequantizers (streaming kernels, HBM bound).
//
// Arithmetic follows the reference kernels exactly: fp32 math, IEEE division by the
// un-rounded fp32 scale, then the scale is stored in its (possibly narrower) type.
#include "quant_util.hpp"

namespace {

// ---------------------------------------------------------------- 1 x block activation quant
// LPG lanes cooperate on one group of LPG*8 contiguous elements.
template <int DT, int LPG, bool FP8>
__global__ void act_quant_kernel(const void* __restrict__ x, void* __restrict__ y, void* __restrict__ s,
                                 int64_t n_groups, int mode, bool fp8_scale_f16 = false) {
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t grp = tid / LPG;
    const bool live = grp < n_groups;
    const int64_t gsafe = live ? grp : 0;
    const int64_t off = gsafe * (LPG * EPL) + (tid % LPG) * EPL;
    float v[EPL];
    load8<DT>(x, off, v);
    float m = 0.f;
#pragma unroll
    for (int j = 0; j < EPL; ++j) m = fmaxf(m, fabsf(v[j]));
    m = group_max<LPG>(m);
    if (!live) return;
    quant_store8<FP8>(v, m, y, off, s, grp, tid % LPG == 0, mode, fp8_scale_f16);
}

// ---------------------------------------------------------------- 1 x block dequant of a communication payload
// x = cast(y -> scale dtype) * s, the product rounded in the scale dtype (fp16 in the reference), then cast
// to the output dtype.  LPG lanes per group, 8 elements each.
template <int SDT, int ODT, int LPG, bool FP8>
__global__ void block_dequant_kernel(const uint8_t* __restrict__ y, const void* __restrict__ s, void* __restrict__ x,
                                     int64_t n_groups) {
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t grp = tid / LPG;
    if (grp >= n_groups) return;
    const int64_t off = grp * (LPG * EPL) + (tid % LPG) * EPL;
    const float sc = FloatIO<SDT>::ld(s, grp);
    const uint2 raw = *(const uint2*)(y + off);
    const unsigned w[2] = {raw.x, raw.y};
    float v[EPL];
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
        const unsigned b = (w[j >> 2] >> (8 * (j & 3))) & 0xff;
        float q;
        if constexpr (FP8) {
            // e4m3fn decode (exact in fp16 and fp32): NaN patterns 0x7f / 0xff stay NaN
            const unsigned e = (b >> 3) & 0xf, mnt = b & 7;
            float mag = e ? __uint_as_float(((e + 120u) << 23) | (mnt << 20)) : (float)mnt * 0.001953125f;
            if ((b & 0x7f) == 0x7f) mag = __uint_as_float(0x7fc00000u);
            q = (b & 0x80) ? -mag : mag;
        } else {
            q = (float)(int)(int8_t)b;
        }
        v[j] = rnd<SDT>(q * sc);
    }
    if ((((uintptr_t)x) & (ODT == LLMK_F32 ? 31 : 15)) == 0) {
        store8<ODT>(x, off, v);
    } else {
#pragma unroll
        for (int j = 0; j < EPL; ++j) FloatIO<ODT>::st(x, off + j, v[j]);
    }
}

// ---------------------------------------------------------------- one group per row (per-token / per-channel int8)
// One 256-thread workgroup per row of any length: absmax over the row, s = absmax / 127 in fp32 (stored
// fp32), y = round-half-away(x / s).  The second pass re-reads the row, which the first pass left in cache.
template <int DT>
__global__ __launch_bounds__(256) void row_quant_i8_kernel(const void* __restrict__ x, int8_t* __restrict__ y,
                                                           float* __restrict__ s, int64_t cols, bool vec) {
    __shared__ float red[4];
    const int64_t row = blockIdx.x, base = row * cols;
    const int t = threadIdx.x;
    float m = 0.f;
    if (vec) {
        for (int64_t c = (int64_t)t * EPL; c < cols; c += 256 * EPL) {
            float v[EPL];
            load8<DT>(x, base + c, v);
#pragma unroll
            for (int j = 0; j < EPL; ++j) m = fmaxf(m, fabsf(v[j]));
        }
    } else {
        for (int64_t c = t; c < cols; c += 256) m = fmaxf(m, fabsf(FloatIO<DT>::ld(x, base + c)));
    }
    m = wave_max(m);
    if ((t & 63) == 0) red[t >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float sc = m / 127.f;
    const bool fast = div_by_ok(sc);
    const float r = fast ? 1.0f / sc : 0.f;
    if (vec) {
        for (int64_t c = (int64_t)t * EPL; c < cols; c += 256 * EPL) {
            float v[EPL];
            load8<DT>(x, base + c, v);
            unsigned w[2] = {0, 0};
#pragma unroll
            for (int j = 0; j < EPL; ++j) {
                const int qi = (int)roundf(fast ? div_by(v[j], sc, r) : v[j] / sc);
                w[j >> 2] |= ((unsigned)(qi & 0xff)) << (8 * (j & 3));
            }
            *(uint2*)(y + base + c) = make_uint2(w[0], w[1]);
        }
    } else {
        for (int64_t c = t; c < cols; c += 256) {
            const float v = FloatIO<DT>::ld(x, base + c);
            y[base + c] = (int8_t)(int)roundf(fast ? div_by(v, sc, r) : v / sc);
        }
    }
    if (t == 0) s[row] = sc;
}

// ---------------------------------------------------------------- block x block weight quant
// one 256-thread workgroup per (BLOCK x BLOCK) tile, BLOCK <= 128, BLOCK % 8 == 0.
// thread t: column chunk (t % 16) * 8, rows t / 16 + 16 * j.
template <int DT, bool FP8>
__global__ void weight_quant_block_kernel(const void* __restrict__ x, void* __restrict__ y, void* __restrict__ s,
                                          int64_t M, int64_t N, int block, float qmax, int mode, int clamp) {
    __shared__ float red[4];
    const int nb = (int)((N + block - 1) / block);
    const int64_t r0 = (int64_t)blockIdx.y * block, c0 = (int64_t)blockIdx.x * block;
    const int t = threadIdx.x;
    const int cc = (t & 15) * EPL;
    // whole tiles of rows that are whole 16-byte chunks: 8 elements per load and per store
    const bool vec = r0 + block <= M && c0 + block <= N && N % EPL == 0 && ((((uintptr_t)x) | ((uintptr_t)y)) & 15) == 0;
    float v[8][EPL];
    float m = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int rr = (t >> 4) + 16 * j;
        const int64_t r = r0 + rr;
        if (vec) {
            if (rr < block && cc < block) {
                load8<DT>(x, r * N + c0 + cc, v[j]);
            } else {
#pragma unroll
                for (int e = 0; e < EPL; ++e) v[j][e] = 0.f;
            }
        } else {
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const int64_t c = c0 + cc + e;
                float val = 0.f;
                if (rr < block && cc + e < block && r < M && c < N) val = FloatIO<DT>::ld(x, r * N + c);
                v[j][e] = val;
            }
        }
#pragma unroll
        for (int e = 0; e < EPL; ++e) m = fmaxf(m, fabsf(v[j][e]));
    }
    m = wave_max(m);
    if ((t & 63) == 0) red[t >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float sc = m / qmax;
    // v / sc by the shared reciprocal and one residual correction where the operands allow it (see div_by)
    const bool fast = div_by_ok(sc);
    const float rcp = fast ? 1.0f / sc : 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const int rr = (t >> 4) + 16 * j;
        const int64_t r = r0 + rr;
        float q[EPL];
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            q[e] = fast ? div_by(v[j][e], sc, rcp) : v[j][e] / sc;
            if constexpr (!FP8) {
                q[e] = round_mode(q[e], mode);
                if (clamp) q[e] = fminf(fmaxf(q[e], -qmax), qmax);
            }
        }
        if (vec) {
            if (rr < block && cc < block) {
                uint2 o;
                if constexpr (FP8) {
                    o.x = pack_fp8x4(q[0], q[1], q[2], q[3]);
                    o.y = pack_fp8x4(q[4], q[5], q[6], q[7]);
                } else {
                    unsigned w[2] = {0, 0};
#pragma unroll
                    for (int e = 0; e < EPL; ++e) w[e >> 2] |= ((unsigned)((int)q[e] & 0xff)) << (8 * (e & 3));
                    o.x = w[0];
                    o.y = w[1];
                }
                *(uint2*)((uint8_t*)y + r * N + c0 + cc) = o;
            }
        } else {
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const int64_t c = c0 + cc + e;
                if (rr < block && cc + e < block && r < M && c < N) {
                    if constexpr (FP8) ((uint8_t*)y)[r * N + c] = (uint8_t)(pack_fp8x4(q[e], 0.f, 0.f, 0.f) & 0xff);
                    else ((int8_t*)y)[r * N + c] = (int8_t)(int)q[e];
                }
            }
        }
    }
    if (t == 0) {
        if constexpr (FP8) ((float*)s)[(int64_t)blockIdx.y * nb + blockIdx.x] = sc;
        else ((unsigned short*)s)[(int64_t)blockIdx.y * nb + blockIdx.x] = f32_to_f16(sc);
    }
}

// ---------------------------------------------------------------- w4a8 second level (in place)
template <int LPG>
__global__ void w4a8_level2_kernel(int8_t* __restrict__ y, int8_t* __restrict__ s4, int8_t* __restrict__ z4,
                                   int64_t n_groups) {
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t grp = tid / LPG;
    const bool live = grp < n_groups;
    const int64_t off = (live ? grp : 0) * (LPG * EPL) + (tid % LPG) * EPL;
    uint2 u = *(const uint2*)(y + off);
    float v[EPL];
    unsigned w[2] = {u.x, u.y};
#pragma unroll
    for (int j = 0; j < EPL; ++j) v[j] = (float)(int8_t)((w[j >> 2] >> (8 * (j & 3))) & 0xff);
    float mx = v[0], mn = v[0];
#pragma unroll
    for (int j = 1; j < EPL; ++j) { mx = fmaxf(mx, v[j]); mn = fminf(mn, v[j]); }
    mx = group_max<LPG>(mx);
    mn = group_min<LPG>(mn);
    if (!live) return;
    const float fs4 = floorf((mx - mn) / 15.0f + 0.5f);
    const float fz4 = floorf(-mn / fs4 + 0.5f);
    unsigned o[2] = {0, 0};
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
        float q = floorf(v[j] / fs4 + 0.5f) + fz4;
        q = fminf(fmaxf(q, 0.f), 15.f);
        o[j >> 2] |= ((unsigned)((int)q & 0xff)) << (8 * (j & 3));
    }
    *(uint2*)(y + off) = make_uint2(o[0], o[1]);
    if (tid % LPG == 0) { s4[grp] = (int8_t)(int)fs4; z4[grp] = (int8_t)(int)fz4; }
}

// ---------------------------------------------------------------- dequantizers
template <int ODT, int SDT, bool FP8>
__global__ void weight_dequant_block_kernel(const uint8_t* __restrict__ x, const void* __restrict__ s,
                                            void* __restrict__ y, int64_t M, int64_t N, int block) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= M * N) return;
    const int64_t r = idx / N, c = idx - r * N;
    const int64_t nb = (N + block - 1) / block;
    const float sc = FloatIO<SDT>::ld(s, (r / block) * nb + c / block);
    float xv;
    if constexpr (FP8) {
        xv = __builtin_amdgcn_cvt_f32_fp8((int)x[idx], 0);
    } else {
        xv = (float)(int8_t)x[idx];
    }
    FloatIO<ODT>::st(y, idx, xv * sc);
}

// One workgroup per 4096 columns of a row, every store instruction of a wave one contiguous KB: a lane takes
// the 4 (fp32 output) or 8 (16-bit output) elements at 256 E q + E tid of the span, q = 0 .. 16 / E - 1.  With
// 16 consecutive elements per lane the four 16-byte stores of a lane leave partly written lines between the
// instructions (fp32 output: 77 us for 14336 x 4096 against 49.5 us; 6.6 TB/s is what the byte -> fp16
// converter reaches with contiguous 16-byte stores).  N and the block size multiples of 16.
template <int ODT, int SDT, bool FP8>
__global__ void weight_dequant_block_row_kernel(const uint8_t* __restrict__ x, const void* __restrict__ s,
                                                void* __restrict__ y, int64_t N, int block) {
    constexpr int E = ODT == LLMK_F32 ? 4 : 8, CH = 16 / E;
    const int64_t r = blockIdx.x;
    const int nb = (int)((N + block - 1) / block);
    const int64_t srow = (r / block) * nb;
    const int c0 = blockIdx.y * 4096 + threadIdx.x * E;
    unsigned w[CH][E / 4];
    float sc[CH];
#pragma unroll
    for (int q = 0; q < CH; ++q) {
        const int c = c0 + q * 256 * E;
        const bool live = c < N;
        const int cs = live ? c : 0;
        if constexpr (E == 4) {
            w[q][0] = *(const unsigned*)(x + r * N + cs);
        } else {
            const uint2 t = *(const uint2*)(x + r * N + cs);
            w[q][0] = t.x; w[q][1] = t.y;
        }
        sc[q] = FloatIO<SDT>::ld(s, srow + cs / block);
    }
#pragma unroll
    for (int q = 0; q < CH; ++q) {
        const int c = c0 + q * 256 * E;
        if (c >= N) continue;
        float v[E];
#pragma unroll
        for (int h = 0; h < E / 4; ++h) {
            if constexpr (FP8) {
                v[4 * h + 0] = __builtin_amdgcn_cvt_f32_fp8((int)w[q][h], 0) * sc[q];
                v[4 * h + 1] = __builtin_amdgcn_cvt_f32_fp8((int)w[q][h], 1) * sc[q];
                v[4 * h + 2] = __builtin_amdgcn_cvt_f32_fp8((int)w[q][h], 2) * sc[q];
                v[4 * h + 3] = __builtin_amdgcn_cvt_f32_fp8((int)w[q][h], 3) * sc[q];
            } else {
#pragma unroll
                for (int b = 0; b < 4; ++b) v[4 * h + b] = (float)(int8_t)(w[q][h] >> (8 * b)) * sc[q];
            }
        }
        if constexpr (ODT == LLMK_F16) {            // the products are fp32 values of their own: round twice, as the reference does
#pragma unroll
            for (int e = 0; e < E; ++e) v[e] = keep_f32(v[e]);
        }
        if constexpr (ODT == LLMK_F32) {
            *(float4*)((float*)y + r * N + c) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
            unsigned o[4];
#pragma unroll
            for (int h = 0; h < 4; ++h)
                o[h] = ODT == LLMK_F16 ? ((unsigned)f32_to_f16(v[2 * h]) | ((unsigned)f32_to_f16(v[2 * h + 1]) << 16))
                                       : ((unsigned)f32_to_bf16(v[2 * h]) | ((unsigned)f32_to_bf16(v[2 * h + 1]) << 16));
            *(uint4*)((unsigned short*)y + r * N + c) = make_uint4(o[0], o[1], o[2], o[3]);
        }
    }
}

__global__ void w4a8_dequant_kernel(const int32_t* __restrict__ packed, const unsigned short* __restrict__ s,
                                    const int8_t* __restrict__ s4, const int8_t* __restrict__ z4,
                                    unsigned short* __restrict__ y, int64_t N, int64_t K, int block, int group) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t np = N / 8;
    if (idx >= np * K) return;
    const int64_t pr = idx / K, k = idx - pr * K;
    const unsigned w = (unsigned)packed[idx];
    const int64_t kg = (K + group - 1) / group, kb = (K + block - 1) / block;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int64_t n = pr * 8 + i;
        const int8_t q = (int8_t)((w >> (4 * i)) & 0xf);
        const int8_t d = (int8_t)(q - z4[n * kg + k / group]);
        const int8_t d8 = (int8_t)(d * s4[n * kg + k / group]);   // int8 wrap-around, as the reference evaluates it
        const float sc = f16_to_f32(s[(n / block) * kb + k / block]);
        y[n * K + k] = f32_to_f16((float)d8 * sc);
    }
}

// the same with 8 consecutive k per thread: 8 packed words in, one 16-byte store per row out (K, the group
// and 16-byte alignment of the words and of y are the caller's to check)
__global__ void w4a8_dequant_vec_kernel(const int32_t* __restrict__ packed, const unsigned short* __restrict__ s,
                                        const int8_t* __restrict__ s4, const int8_t* __restrict__ z4,
                                        unsigned short* __restrict__ y, int64_t N, int64_t K, int block, int group) {
    const int64_t idx = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 8;
    const int64_t np = N / 8;
    if (idx >= np * K) return;
    const int64_t pr = idx / K, k = idx - pr * K;
    const uint4 a = *(const uint4*)(packed + idx), b = *(const uint4*)(packed + idx + 4);
    const unsigned w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    const int64_t kg = (K + group - 1) / group, kb = (K + block - 1) / block;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int64_t n = pr * 8 + i;
        const int8_t z = z4[n * kg + k / group], m = s4[n * kg + k / group];
        const float sc = f16_to_f32(s[(n / block) * kb + k / block]);
        unsigned o[4];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int8_t q = (int8_t)((w[j] >> (4 * i)) & 0xf);
            const int8_t d8 = (int8_t)((int8_t)(q - z) * m);          // int8 wrap-around, as the reference evaluates it
            const unsigned h = f32_to_f16((float)d8 * sc);
            o[j >> 1] = (j & 1) ? (o[j >> 1] | (h << 16)) : h;
        }
        *(uint4*)(y + n * K + k) = make_uint4(o[0], o[1], o[2], o[3]);
    }
}

// ---------------------------------------------------------------- symmetric int4 along K for W [N, K] (W4A16)
// s = absmax / 7 rounded to fp16; q = clamp(rne(w / s), -8, 7) + 8 with the division by the rounded scale in
// fp32.  A lane owns 8 consecutive k: its 8 nibbles are exactly one int32 of the [N, K/8] bit-packed layout
// (nibble i of a word is k = 8 word + i), so the packed word, the 8 bytes of q and the group's scale leave in
// one pass over W.  A group of zeros has scale 0 and stores q = 8 (the value 0).
template <int DT, int LPG>
__global__ void w4_quant_nk_kernel(const void* __restrict__ w, int32_t* __restrict__ packed,
                                   unsigned short* __restrict__ s, uint8_t* __restrict__ q, int64_t n_groups) {
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t grp = tid / LPG;
    const bool live = grp < n_groups;
    const int64_t off = live ? tid * EPL : 0;
    float v[EPL];
    load8<DT>(w, off, v);
    float m = 0.f;
#pragma unroll
    for (int j = 0; j < EPL; ++j) m = fmaxf(m, fabsf(v[j]));
    m = group_max<LPG>(m);
    if (!live) return;
    const unsigned short sh = f32_to_f16(m / 7.0f);
    const float sc = f16_to_f32(sh);
    const bool fast = div_by_ok(sc);
    const float r = fast ? 1.0f / sc : 0.f;
    unsigned word = 0, b[2] = {0, 0};
#pragma unroll
    for (int j = 0; j < EPL; ++j) {
        const float t = fast ? div_by(v[j], sc, r) : v[j] / sc;
        const float c = fminf(fmaxf(rintf(t), -8.f), 7.f);        // fmin / fmax drop a NaN (0 / 0): the value 0
        const unsigned n = (unsigned)((int)(t != t ? 0.f : c) + 8);
        word |= n << (4 * j);
        b[j >> 2] |= n << (8 * (j & 3));
    }
    packed[tid] = (int32_t)word;
    if (q) *(uint2*)(q + off) = make_uint2(b[0], b[1]);
    if (tid % LPG == 0) s[grp] = sh;
}

bool lpg_ok(int block) {
    return block == 8 || block == 16 || block == 32 || block == 64 || block == 128 || block == 256 || block == 512;
}

}  // namespace

#define LPG_SWITCH(block, CALL)                                                       \
    switch ((block) / EPL) {                                                          \
        case 1: CALL(1); break;  case 2: CALL(2); break;  case 4: CALL(4); break;     \
        case 8: CALL(8); break;  case 16: CALL(16); break; case 32: CALL(32); break;  \
        default: CALL(64); break;                                                     \
    }

extern "C" int llmk_act_quant_fp8(const void* x, int x_dtype, void* y, float* s, int64_t n_groups,
                                  int block, void* stream) {
    if (!lpg_ok(block)) LLMK_FAIL(LLMK_ERR_SHAPE, "act_quant_fp8: block %d unsupported (power of two in 8..512)", block);
    if (n_groups == 0) return LLMK_OK;
    if (!x || !y || !s || n_groups < 0) LLMK_FAIL(LLMK_ERR_ARG, "act_quant_fp8: bad argument");
    const int64_t threads = n_groups * (block / EPL);
    dim3 grid((unsigned)cdiv64(threads, 256)), blk(256);
#define CALL(L) LLMK_DISPATCH_FLOAT(x_dtype, DT, (act_quant_kernel<DT, L, true><<<grid, blk, 0, (hipStream_t)stream>>>(x, y, s, n_groups, 0)))
    LPG_SWITCH(block, CALL)
#undef CALL
    LLMK_CHECK_LAUNCH("act_quant_fp8");
    return LLMK_OK;
}

/* W [N, K] float -> int32 [N, K/8] nibbles along K, fp16 scales [N, K/group], optionally q uint8 [N, K] */
extern "C" int llmk_quant_w4_nk(const void* w, int w_dtype, int32_t* packed, void* scales, uint8_t* q, int64_t N,
                                int64_t K, int group, void* stream) {
    if (!lpg_ok(group)) LLMK_FAIL(LLMK_ERR_SHAPE, "quant_w4_nk: group %d unsupported (power of two in 8..512)", group);
    if (N < 0 || K < 0 || K % group) LLMK_FAIL(LLMK_ERR_SHAPE, "quant_w4_nk: K %lld is not a multiple of the group %d", (long long)K, group);
    if (N == 0 || K == 0) return LLMK_OK;
    if (!w || !packed || !scales) LLMK_FAIL(LLMK_ERR_ARG, "quant_w4_nk: bad argument");
    if (((uintptr_t)w & 15) || ((uintptr_t)q & 7)) LLMK_FAIL(LLMK_ERR_ARG, "quant_w4_nk: W needs 16-byte and q 8-byte alignment");
    const int64_t n_groups = N * (K / group);
    const int64_t threads = n_groups * (group / EPL);
    dim3 grid((unsigned)cdiv64(threads, 256)), blk(256);
#define CALL(L) LLMK_DISPATCH_FLOAT(w_dtype, DT, (w4_quant_nk_kernel<DT, L><<<grid, blk, 0, (hipStream_t)stream>>>(w, packed, (unsigned short*)scales, q, n_groups)))
    LPG_SWITCH(group, CALL)
#undef CALL
    LLMK_CHECK_LAUNCH("quant_w4_nk");
    return LLMK_OK;
}

/* 1 x block e4m3 quantizer with the scale stored as fp16 or fp32 (communication payload format) */
extern "C" int llmk_comm_quant_fp8(const void* x, int x_dtype, void* y, void* s, int s_dtype, int64_t n_groups,
                                   int block, void* stream) {
    if (!lpg_ok(block)) LLMK_FAIL(LLMK_ERR_SHAPE, "comm_quant_fp8: block %d unsupported (power of two in 8..512)", block);
    if (s_dtype != LLMK_F16 && s_dtype != LLMK_F32) LLMK_FAIL(LLMK_ERR_DTYPE, "comm_quant_fp8: s_dtype %d", s_dtype);
    if (n_groups == 0) return LLMK_OK;
    if (!x || !y || !s || n_groups < 0) LLMK_FAIL(LLMK_ERR_ARG, "comm_quant_fp8: bad argument");
    const int64_t threads = n_groups * (block / EPL);
    dim3 grid((unsigned)cdiv64(threads, 256)), blk(256);
    const bool f16s = s_dtype == LLMK_F16;
#define CALL(L) LLMK_DISPATCH_FLOAT(x_dtype, DT, (act_quant_kernel<DT, L, true><<<grid, blk, 0, (hipStream_t)stream>>>(x, y, s, n_groups, 0, f16s)))
    LPG_SWITCH(block, CALL)
#undef CALL
    LLMK_CHECK_LAUNCH("comm_quant_fp8");
    return LLMK_OK;
}

extern "C" int llmk_comm_dequant(const void* y, int kind, const void* s, int s_dtype, void* x, int x_dtype,
                                 int64_t n_groups, int block, void* stream) {
    if (!lpg_ok(block)) LLMK_FAIL(LLMK_ERR_SHAPE, "comm_dequant: block %d unsupported (power of two in 8..512)", block);
    if (kind != LLMK_KIND_I8 && kind != LLMK_KIND_FP8) LLMK_FAIL(LLMK_ERR_DTYPE, "comm_dequant: kind %d", kind);
    if (n_groups == 0) return LLMK_OK;
    if (!x || !y || !s || n_groups < 0) LLMK_FAIL(LLMK_ERR_ARG, "comm_dequant: bad argument");
    const int64_t threads = n_groups * (block / EPL);
    dim3 grid((unsigned)cdiv64(threads, 256)), blk(256);
#define CALL(L) LLMK_DISPATCH_FLOAT(s_dtype, SDT, LLMK_DISPATCH_FLOAT(x_dtype, ODT, {                                              \
        if (kind == LLMK_KIND_FP8) block_dequant_kernel<SDT, ODT, L, true><<<grid, blk, 0, (hipStream_t)stream>>>((const uint8_t*)y, s, x, n_groups); \
        else block_dequant_kernel<SDT, ODT, L, false><<<grid, blk, 0, (hipStream_t)stream>>>((const uint8_t*)y, s, x, n_groups); }))
    LPG_SWITCH(block, CALL)
#undef CALL
    LLMK_CHECK_LAUNCH("comm_dequant");
    return LLMK_OK;
}

extern "C" int llmk_act_quant_i8(const void* x, int x_dtype, int8_t* y, void* s, int64_t n_groups,
                                 int block, int round_mode, void* stream) {
    if (!lpg_ok(block)) LLMK_FAIL(LLMK_ERR_SHAPE, "act_quant_i8: block %d unsupported (power of two in 8..512)", block);
    if (round_mode != LLMK_ROUND_HALF_AWAY && round_mode != LLMK_ROUND_HALF_UP)
        LLMK_FAIL(LLMK_ERR_DTYPE, "act_quant_i8: round_mode %d", round_mode);
    if (n_groups == 0) return LLMK_OK;
    if (!x || !y || !s || n_groups < 0) LLMK_FAIL(LLMK_ERR_ARG, "act_quant_i8: bad argument");
    const int64_t threads = n_groups * (block / EPL);
    dim3 grid((unsigned)cdiv64(threads, 256)), blk(256);
#define CALL(L) LLMK_DISPATCH_FLOAT(x_dtype, DT, (act_quant_kernel<DT, L, false><<<grid, blk, 0, (hipStream_t)stream>>>(x, y, s, n_groups, round_mode)))
    LPG_SWITCH(block, CALL)
#undef CALL
    LLMK_CHECK_LAUNCH("act_quant_i8");
    return LLMK_OK;
}

extern "C" int llmk_quant_i8_rowwise(const void* x, int x_dtype, int8_t* y, float* s, int64_t rows, int64_t cols,
                                     void* stream) {
    if (rows < 0 || cols < 0 || rows > 0x7fffffff) LLMK_FAIL(LLMK_ERR_SHAPE, "quant_i8_rowwise: bad shape");
    if (rows == 0) return LLMK_OK;
    if (!y || !s || (cols && !x)) LLMK_FAIL(LLMK_ERR_ARG, "quant_i8_rowwise: null pointer");
    const int esz = x_dtype == LLMK_F32 ? 4 : 2;
    // 8 elements per lane when every row starts on a 16-byte (input) and 8-byte (output) boundary
    const bool vec = cols % EPL == 0 && (((uintptr_t)x) & 15) == 0 && (((uintptr_t)y) & 7) == 0 && (cols * esz) % 16 == 0;
    LLMK_DISPATCH_FLOAT(x_dtype, DT, (row_quant_i8_kernel<DT><<<dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream>>>(x, y, s, cols, vec)));
    LLMK_CHECK_LAUNCH("quant_i8_rowwise");
    return LLMK_OK;
}

extern "C" int llmk_weight_quant_i8_block(const void* x, int x_dtype, int8_t* y, void* s, int64_t M, int64_t N,
                                          int block, float qmax, int round_mode, int clamp, void* stream) {
    if (block < 8 || block > 128 || block % 8) LLMK_FAIL(LLMK_ERR_SHAPE, "weight_quant_i8_block: block %d (need 8..128, %%8)", block);
    if (M == 0 || N == 0) return LLMK_OK;
    if (!x || !y || !s || M < 0 || N < 0) LLMK_FAIL(LLMK_ERR_ARG, "weight_quant_i8_block: bad argument");
    dim3 grid((unsigned)cdiv64(N, block), (unsigned)cdiv64(M, block)), blk(256);
    LLMK_DISPATCH_FLOAT(x_dtype, DT, (weight_quant_block_kernel<DT, false><<<grid, blk, 0, (hipStream_t)stream>>>(x, y, s, M, N, block, qmax, round_mode, clamp)));
    LLMK_CHECK_LAUNCH("weight_quant_i8_block");
    return LLMK_OK;
}

extern "C" int llmk_weight_quant_fp8_block(const void* x, int x_dtype, void* y, float* s, int64_t M, int64_t N,
                                           int block, void* stream) {
    if (block < 8 || block > 128 || block % 8) LLMK_FAIL(LLMK_ERR_SHAPE, "weight_quant_fp8_block: block %d (need 8..128, %%8)", block);
    if (M == 0 || N == 0) return LLMK_OK;
    if (!x || !y || !s || M < 0 || N < 0) LLMK_FAIL(LLMK_ERR_ARG, "weight_quant_fp8_block: bad argument");
    dim3 grid((unsigned)cdiv64(N, block), (unsigned)cdiv64(M, block)), blk(256);
    LLMK_DISPATCH_FLOAT(x_dtype, DT, (weight_quant_block_kernel<DT, true><<<grid, blk, 0, (hipStream_t)stream>>>(x, y, s, M, N, block, 448.f, 0, 0)));
    LLMK_CHECK_LAUNCH("weight_quant_fp8_block");
    return LLMK_OK;
}

extern "C" int llmk_weight_quant_w4a8_level2(int8_t* y, int8_t* s4, int8_t* z4, int64_t M, int64_t N, int group,
                                             void* stream) {
    if (!lpg_ok(group) || N % group) LLMK_FAIL(LLMK_ERR_SHAPE, "w4a8_level2: group %d / N %lld", group, (long long)N);
    if (M == 0 || N == 0) return LLMK_OK;
    if (!y || !s4 || !z4) LLMK_FAIL(LLMK_ERR_ARG, "w4a8_level2: null pointer");
    const int64_t n_groups = M * (N / group);
    const int64_t threads = n_groups * (group / EPL);
    dim3 grid((unsigned)cdiv64(threads, 256)), blk(256);
#define CALL(L) w4a8_level2_kernel<L><<<grid, blk, 0, (hipStream_t)stream>>>(y, s4, z4, n_groups)
    LPG_SWITCH(group, CALL)
#undef CALL
    LLMK_CHECK_LAUNCH("w4a8_level2");
    return LLMK_OK;
}

extern "C" int llmk_weight_dequant_fp8_block(const void* x, const float* s, void* y, int y_dtype, int64_t M, int64_t N,
                                             int block, void* stream) {
    if (block < 1) LLMK_FAIL(LLMK_ERR_SHAPE, "weight_dequant_fp8_block: block %d", block);
    if (M == 0 || N == 0) return LLMK_OK;
    if (!x || !s || !y) LLMK_FAIL(LLMK_ERR_ARG, "weight_dequant_fp8_block: null pointer");
    dim3 grid((unsigned)cdiv64(M * N, 256)), blk(256);
    if (N % 16 == 0 && block % 16 == 0 && ((((uintptr_t)x) | ((uintptr_t)y)) & 15) == 0 && M < (1ll << 31) && N <= 4096ll * 65535) {
        dim3 rgrid((unsigned)M, (unsigned)cdiv64(N, 4096));
        LLMK_DISPATCH_FLOAT(y_dtype, ODT, (weight_dequant_block_row_kernel<ODT, LLMK_F32, true><<<rgrid, blk, 0, (hipStream_t)stream>>>((const uint8_t*)x, s, y, N, block)));
        LLMK_CHECK_LAUNCH("weight_dequant_fp8_block");
        return LLMK_OK;
    }
    LLMK_DISPATCH_FLOAT(y_dtype, ODT, (weight_dequant_block_kernel<ODT, LLMK_F32, true><<<grid, blk, 0, (hipStream_t)stream>>>((const uint8_t*)x, s, y, M, N, block)));
    LLMK_CHECK_LAUNCH("weight_dequant_fp8_block");
    return LLMK_OK;
}

extern "C" int llmk_weight_dequant_i8_block(const int8_t* x, const void* s, int s_dtype, void* y, int y_dtype,
                                            int64_t M, int64_t N, int block, void* stream) {
    if (block < 1) LLMK_FAIL(LLMK_ERR_SHAPE, "weight_dequant_i8_block: block %d", block);
    if (M == 0 || N == 0) return LLMK_OK;
    if (!x || !s || !y) LLMK_FAIL(LLMK_ERR_ARG, "weight_dequant_i8_block: null pointer");
    dim3 grid((unsigned)cdiv64(M * N, 256)), blk(256);
    if (N % 16 == 0 && block % 16 == 0 && ((((uintptr_t)x) | ((uintptr_t)y)) & 15) == 0 && M < (1ll << 31) && N <= 4096ll * 65535) {
        dim3 rgrid((unsigned)M, (unsigned)cdiv64(N, 4096));
        LLMK_DISPATCH_FLOAT(y_dtype, ODT, LLMK_DISPATCH_FLOAT(s_dtype, SDT, (weight_dequant_block_row_kernel<ODT, SDT, false><<<rgrid, blk, 0, (hipStream_t)stream>>>((const uint8_t*)x, s, y, N, block))));
        LLMK_CHECK_LAUNCH("weight_dequant_i8_block");
        return LLMK_OK;
    }
    LLMK_DISPATCH_FLOAT(y_dtype, ODT, LLMK_DISPATCH_FLOAT(s_dtype, SDT, (weight_dequant_block_kernel<ODT, SDT, false><<<grid, blk, 0, (hipStream_t)stream>>>((const uint8_t*)x, s, y, M, N, block))));
    LLMK_CHECK_LAUNCH("weight_dequant_i8_block");
    return LLMK_OK;
}

extern "C" int llmk_weight_dequant_w4a8(const int32_t* packed, const void* s, const int8_t* s4, const int8_t* z4,
                                        void* y, int64_t N, int64_t K, int block, int group, void* stream) {
    if (N % 8 || block < 1 || group < 1) LLMK_FAIL(LLMK_ERR_SHAPE, "weight_dequant_w4a8: N %% 8 != 0 or bad block/group");
    if (N == 0 || K == 0) return LLMK_OK;
    if (!packed || !s || !s4 || !z4 || !y) LLMK_FAIL(LLMK_ERR_ARG, "weight_dequant_w4a8: null pointer");
    dim3 grid((unsigned)cdiv64((N / 8) * K, 256)), blk(256);
    if (K % 8 == 0 && group % 8 == 0 && block % 8 == 0 && ((((uintptr_t)packed) | ((uintptr_t)y)) & 15) == 0) {
        dim3 vgrid((unsigned)cdiv64((N / 8) * K / 8, 256));
        w4a8_dequant_vec_kernel<<<vgrid, blk, 0, (hipStream_t)stream>>>(packed, (const unsigned short*)s, s4, z4,
                                                                       (unsigned short*)y, N, K, block, group);
        LLMK_CHECK_LAUNCH("weight_dequant_w4a8");
        return LLMK_OK;
    }
    w4a8_dequant_kernel<<<grid, blk, 0, (hipStream_t)stream>>>(packed, (const unsigned short*)s, s4, z4,
                                                               (unsigned short*)y, N, K, block, group);
    LLMK_CHECK_LAUNCH("weight_dequant_w4a8");
    return LLMK_OK;
}
