// Large-M block-scaled fp8 / int8 GEMM with a three-stage global->LDS pipeline fed by the
// direct-to-LDS loads of gfx950 (global_load_lds_dwordx4: no staging registers, no ds_write).
//
// Workgroup: 512 threads = 8 waves (4 along M x 2 along N), output tile 256 x 128, K step 128
// (one scale block).  Wave tile 64 x 64 = 4 x 4 MFMA tiles, two waves per SIMD.
//
// LDS stage (50176 B for 256 rows): A rows x 128 B, B 128 rows x 128 B, and the fp32 activation-scale column
// of this K step.  A direct-to-LDS load writes lane l's 16 bytes at base + 16 l, so rows cannot be
// padded; instead the 16-byte chunk index is XOR-swizzled with ((row >> 1) & 7) on the global side:
// LDS slot s of row R holds global chunk s ^ ((R >> 1) & 7).  Two 128-byte rows span the 64 banks, so
// the b128 fragment reads of 16 consecutive lanes (16 rows, same chunk) land in 16 different
// 16-byte bank groups.
//
// Pipeline: stages kt+1 and kt+2 are in flight while stage kt is multiplied; the memory counter is
// waited on by hand (the loads are issued from inline asm, so the compiler does not drain them
// before every LDS read).  Each thread issues 7 loads per stage, hence vmcnt(7).
// The loop contains no other vector-memory instruction: weight scales are copied to LDS up front.
#pragma once
#include "gemm_tiled.hpp"

namespace llmk {

constexpr int D_BN = 128, D_THREADS = 512, D_NSTAGE = 3;
constexpr int D_B = D_BN * 128, D_S = 256 * 4;
constexpr int D_MAX_KT = 256;                            // weight-scale table entries (K <= 32768)
// stage bytes and LDS per tile height (MI 16-row tiles per wave, 64 * MI rows): 50176 / 33792 / 25600 per
// stage, 151552 / 102400 / 77824 bytes in all, so that two workgroups of the 64-row tile share a CU
constexpr int d_a(int mi) { return 64 * mi * 128; }
constexpr int d_stage(int mi) { return d_a(mi) + D_B + D_S; }
constexpr int d_lds(int mi) { return D_NSTAGE * d_stage(mi) + D_MAX_KT * 4; }

// Direct-to-LDS loads: M0 holds the LDS base.  A load that reads M0 needs one wait state after the scalar write
// to it, which the compiler inserts for its own instructions and not inside an asm statement: hence the s_nop.
__device__ __forceinline__ void dma16(uint32_t lds_addr, uint32_t voff, const void* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory", "m0");
}
__device__ __forceinline__ void dma4(uint32_t lds_addr, uint32_t voff, const void* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory", "m0");
}
// 16-bit element -> one dword per lane in LDS (zero-extended)
__device__ __forceinline__ void dma2(uint32_t lds_addr, uint32_t voff, const void* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_ushort %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory", "m0");
}
// s_waitcnt immediates for gfx9: vmcnt = imm[3:0] | imm[15:14] << 4, expcnt = imm[6:4] (7 = no wait),
// lgkmcnt = imm[11:8] (15 = no wait)
#define LLMK_WAIT_VMCNT_7 0x0F77
#define LLMK_WAIT_VMCNT_6 0x0F76
#define LLMK_WAIT_VMCNT_0 0x0F70


// Unscaled kinds accumulate inside the MFMA over the whole K range: two 16x16x32 half-precision MFMAs, or two
// 16x16x64 int8 MFMAs whose int32 accumulators travel as raw bits in the fp32 accumulator registers.
template <int KIND>
__device__ __forceinline__ v4f mma_plain(const v8i& x, const v8i& y, v4f c) {
    if constexpr (KIND == K_I8_ROWCOL) {
        v4i ci;
        __builtin_memcpy(&ci, &c, 16);
        const v4i x0 = {x[0], x[1], x[2], x[3]}, x1 = {x[4], x[5], x[6], x[7]};
        const v4i y0 = {y[0], y[1], y[2], y[3]}, y1 = {y[4], y[5], y[6], y[7]};
        ci = mfma_i8_16x16x64(x0, y0, ci);
        ci = mfma_i8_16x16x64(x1, y1, ci);
        __builtin_memcpy(&c, &ci, 16);
        return c;
    } else if constexpr (KIND == K_F16 || KIND == K_W4NK || KIND == K_W4MARLIN) {
        v8h x0, x1, y0, y1;
        __builtin_memcpy(&x0, &x, 16); __builtin_memcpy(&x1, ((const char*)&x) + 16, 16);
        __builtin_memcpy(&y0, &y, 16); __builtin_memcpy(&y1, ((const char*)&y) + 16, 16);
        c = mfma_f16_16x16x32(x0, y0, c);
        return mfma_f16_16x16x32(x1, y1, c);
    } else {
        v8bf x0, x1, y0, y1;
        __builtin_memcpy(&x0, &x, 16); __builtin_memcpy(&x1, ((const char*)&x) + 16, 16);
        __builtin_memcpy(&y0, &y, 16); __builtin_memcpy(&y1, ((const char*)&y) + 16, 16);
        c = mfma_bf16_16x16x32(x0, y0, c);
        return mfma_bf16_16x16x32(x1, y1, c);
    }
}

// ---- 4-bit weights inside the tile kernel (K_W4NK) ----
// nibble -> fp16 without integer->float converts: (q | 0x6400) is the fp16 number 1024 + q,
// ((q << 4) | 0x6400) is 1024 + 16 q; one packed subtract / fma gives q - 8 exactly.
__device__ __forceinline__ v2h w4_as_h2(unsigned u) { v2h r; __builtin_memcpy(&r, &u, 4); return r; }
__device__ __forceinline__ unsigned w4_as_u32(v2h h) { unsigned r; __builtin_memcpy(&r, &h, 4); return r; }
// one packed word (nibble j = element 8*word + j of the row) -> eight fp16 (q - 8) * scale in K order
__device__ __forceinline__ v4i w4_word_to_f16x8(unsigned w, v2h sc) {
    const v2h k1032 = {(_Float16)1032.f, (_Float16)1032.f};
    const v2h k16 = {(_Float16)0.0625f, (_Float16)0.0625f};
    const v2h k72 = {(_Float16)72.f, (_Float16)72.f};
    const unsigned w8 = w >> 8;
    const unsigned p04 = w4_as_u32((w4_as_h2((w & 0x000f000fu) | 0x64006400u) - k1032) * sc);
    const unsigned p15 = w4_as_u32((w4_as_h2((w & 0x00f000f0u) | 0x64006400u) * k16 - k72) * sc);
    const unsigned p26 = w4_as_u32((w4_as_h2((w8 & 0x000f000fu) | 0x64006400u) - k1032) * sc);
    const unsigned p37 = w4_as_u32((w4_as_h2((w8 & 0x00f000f0u) | 0x64006400u) * k16 - k72) * sc);
    v4i o;
    o[0] = (int)__builtin_amdgcn_perm(p15, p04, 0x05040100u);
    o[1] = (int)__builtin_amdgcn_perm(p37, p26, 0x05040100u);
    o[2] = (int)__builtin_amdgcn_perm(p15, p04, 0x07060302u);
    o[3] = (int)__builtin_amdgcn_perm(p37, p26, 0x07060302u);
    return o;
}
// ---- uint4 weights packed eight rows per word, dequantised to int8 (K_W4A8) ----
// A word holds the nibbles of eight weight rows at one k.  b8 = int8(int8(q - z) * s) with two's-complement wrap is
// the low byte of (q - z) * s in any wider arithmetic, i.e. of q * s + c with c = -(z * s): one packed 16-bit
// multiply-add handles two rows of a word at once (row j in the low half, row j + 4 in the high half, each with
// its own s and c), and byte permutes gather four consecutive k of a row into one dword.
typedef unsigned short w4_us2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ w4_us2 w4_as_us2(unsigned u) { w4_us2 r; __builtin_memcpy(&r, &u, 4); return r; }
__device__ __forceinline__ unsigned w4_us2_bits(w4_us2 v) { unsigned r; __builtin_memcpy(&r, &v, 4); return r; }
// sp[j], cp[j]: (s, c) of rows j | j + 4 as 16-bit pairs, from the eight scale / zero-point bytes of a packed row
__device__ __forceinline__ void w4a8_row_consts(uint2 sb, uint2 zb, unsigned (&sp)[4], unsigned (&cp)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const unsigned sel = 0x0c000c00u | (unsigned)j | ((unsigned)(4 + j) << 16);      // [byte j of .x, 0, byte j of .y, 0]
        sp[j] = __builtin_amdgcn_perm(sb.y, sb.x, sel);
        const unsigned zp = __builtin_amdgcn_perm(zb.y, zb.x, sel);
        cp[j] = w4_us2_bits((w4_us2){0, 0} - w4_as_us2(zp) * w4_as_us2(sp[j]));
    }
}
// four consecutive words (k, k + 1, k + 2, k + 3) of a packed row -> out[i] = the four int8 weights of row i at
// those k (byte order = k order)
__device__ __forceinline__ void w4a8_words_to_i8(const v4i& w, const unsigned (&sp)[4], const unsigned (&cp)[4], unsigned (&out)[8]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        unsigned r[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const unsigned x = (((unsigned)w[i]) >> (4 * j)) & 0x000f000fu;
            r[i] = w4_us2_bits(w4_as_us2(x) * w4_as_us2(sp[j]) + w4_as_us2(cp[j]));
        }
        const unsigned t01 = __builtin_amdgcn_perm(r[1], r[0], 0x06020400u);
        const unsigned t23 = __builtin_amdgcn_perm(r[3], r[2], 0x06020400u);
        out[j] = __builtin_amdgcn_perm(t23, t01, 0x05040100u);
        out[j + 4] = __builtin_amdgcn_perm(t23, t01, 0x07060302u);
    }
}

// Register loads issued from inline asm like the direct-to-LDS loads, so that they take part in the same
// hand-counted vmcnt scheme (a compiler-tracked load would make the compiler wait for every load in flight).
// The destination is only read behind an explicit s_waitcnt that names it as a read-write operand.  The
// compiler takes the register for ready as soon as the load is issued, so the scheme holds only while it
// neither copies, spills nor reuses the register before that wait: check_asm.py proves exactly that on the
// assembly of every build (all control-flow paths from each such load), and the build fails otherwise.
__device__ __forceinline__ uint64_t asm_load_b64(uint32_t voff, const void* sbase) {
    uint64_t v;
    asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
    return v;
}
__device__ __forceinline__ v4i asm_load_b128(uint32_t voff, const void* sbase) {
    v4i v;
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
    return v;
}
__device__ __forceinline__ unsigned asm_load_u16(uint32_t voff, const void* sbase) {
    unsigned v;
    asm volatile("global_load_ushort %0, %1, %2" : "=v"(v) : "v"(voff), "s"(sbase) : "memory");
    return v;
}

// ---- epilogue helpers.  A lane owns two runs of 8 consecutive outputs (two MFMA results each) per row, so that
// the four lane groups of a row write 64 contiguous bytes per store instruction (vector stores when the row
// segment is 16-byte aligned).
template <int ODT>
__device__ __forceinline__ void store_run8(void* c, int64_t off, const v4f& a, const v4f& b, int n_valid, bool vec_ok) {
    if (vec_ok && n_valid >= 8) {
        if constexpr (ODT == LLMK_F32) {
            v4f* dst = (v4f*)((float*)c + off);
            dst[0] = a;
            dst[1] = b;
        } else {
            v4i w;
            w[0] = (int)(ODT == LLMK_F16 ? pack_f16x2(a[0], a[1]) : pack_bf16x2(a[0], a[1]));
            w[1] = (int)(ODT == LLMK_F16 ? pack_f16x2(a[2], a[3]) : pack_bf16x2(a[2], a[3]));
            w[2] = (int)(ODT == LLMK_F16 ? pack_f16x2(b[0], b[1]) : pack_bf16x2(b[0], b[1]));
            w[3] = (int)(ODT == LLMK_F16 ? pack_f16x2(b[2], b[3]) : pack_bf16x2(b[2], b[3]));
            *(v4i*)((unsigned short*)c + off) = w;
        }
    } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (q < n_valid) FloatIO<ODT>::st(c, off + q, a[q]);
            if (4 + q < n_valid) FloatIO<ODT>::st(c, off + 4 + q, b[q]);
        }
    }
}
__device__ __forceinline__ void store_run8_i32(int32_t* c, int64_t off, const v4f& a, const v4f& b, int n_valid, bool vec_ok) {
    if (vec_ok && n_valid >= 8) {
        v4f* dst = (v4f*)(c + off);
        dst[0] = a;          // raw bits
        dst[1] = b;
    } else {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (q < n_valid) c[off + q] = __float_as_int(a[q]);
            if (4 + q < n_valid) c[off + 4 + q] = __float_as_int(b[q]);
        }
    }
}
__device__ __forceinline__ void rowcol_epilogue8(const DirectArgs& p, v4f& a, v4f& b, int m, int64_t off, int nb, int n_valid) {
    if (p.c_i32) {
        const bool vec_i = ((((uintptr_t)p.c_i32) & 15) == 0) && (p.N % 4 == 0);
        store_run8_i32(p.c_i32, off, a, b, n_valid, vec_i);
    }
    if (!p.c) return;
    const float as = ((const float*)p.a_s)[m];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        a[q] = (float)__float_as_int(a[q]) * as * ((const float*)p.b_s)[nb + min(q, n_valid - 1)];
        b[q] = (float)__float_as_int(b[q]) * as * ((const float*)p.b_s)[nb + min(4 + q, n_valid - 1)];
    }
}

// MI = 16-row tiles per wave along M (4, 2 or 1): the workgroup tile is 64*MI rows x 128 columns.
// AS16: the activation scales are 16-bit (fp16 or bf16 by p.s_dtype) and are staged as they are, one zero-extended
// element per dword slot of the scale column (global_load_lds_ushort), instead of being widened by a pass of their own.
template <int KIND, bool GROUPED, int MI, bool AS16 = false>
__global__ __launch_bounds__(D_THREADS) void gemm_dma_kernel(DirectArgs p) {
    constexpr int BM = 64 * MI;              // tile rows
    constexpr int WR = 16 * MI;              // rows per wave
    constexpr int D_A = d_a(MI), D_STAGE = d_stage(MI);
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;
    // SCALED: 8-bit operands with per-128-K block scales.  Otherwise no scales inside the K loop (fp16 / bf16
    // operands, or int8 with per-token and per-channel scales applied in the epilogue): a K step is still
    // one 128-byte row segment (two MFMAs per tile) and the MFMAs accumulate directly.
    // K_W4NK: fp16 activations by direct-to-LDS loads as for K_F16; the weight rows of a stage are expanded
    // from the packed words by the threads themselves (one 8-byte load, 16 weights, two 16-byte LDS writes per
    // thread and K step), one K step behind the loads and one ahead of the multiplication.
    constexpr bool SCALED = (KIND == K_FP8_BLOCK || KIND == K_I8_BLOCK || KIND == K_W4A8);
    // K_W4MARLIN: the same for the Marlin layout (16-byte units of 32 values: 4 k x 8 columns): a thread takes
    // half a unit and scatters its eight fp16 pairs over the weight rows.
    // K_W4A8: int8 activations and block scales as for K_I8_BLOCK; the int8 weight rows of a stage are expanded
    // from words that pack eight rows each: a thread loads four consecutive words of one packed row (16 bytes)
    // and writes four int8 weights of each of the eight rows; the zero points and second-level scales of the
    // tile's 128 rows for every K step sit in an LDS table filled before the pipeline starts.
    constexpr bool W4NK = (KIND == K_W4NK), W4M = (KIND == K_W4MARLIN), W4A8 = (KIND == K_W4A8);
    constexpr bool W4H = W4NK || W4M, W4 = W4H || W4A8;
    constexpr int ESZ = (KIND == K_F16 || KIND == K_BF16 || W4H) ? 2 : 1;
    const int N = p.N;
    const int K = p.K * ESZ;                 // row length in bytes
    const int KT_all = K >> 7;
    // split-K: workgroup z multiplies K steps [kt0, kt0 + KT) and writes fp32 partial sums
    int kt0 = 0, KT = KT_all;
    if (!GROUPED && p.ksplit > 1) {
        const int per = (KT_all + p.ksplit - 1) / p.ksplit;
        kt0 = (int)blockIdx.z * per;
        KT = max(0, min(per, KT_all - kt0));
    }
    const int n0 = blockIdx.x * D_BN;

    int m_start, m_end;
    const uint8_t* bbase = p.b;
    int64_t bs_off = 0;
    if constexpr (GROUPED) {
        int tile = blockIdx.y, e = 0, cum = 0;
        int64_t s0 = p.seg_indptr[0];
        bool found = false;
        for (; e < p.E; ++e) {
            const int64_t s1 = p.seg_indptr[e + 1];
            const int t = (int)((s1 - s0 + BM - 1) / BM);
            if (tile < cum + t) { found = true; m_start = (int)s0 + (tile - cum) * BM; m_end = min((int)s1, m_start + BM); break; }
            cum += t;
            s0 = s1;
        }
        if (!found) return;
        const int64_t widx = p.weight_indices ? p.weight_indices[e] : e;
        bbase += widx * (int64_t)N * K;
        bs_off = widx * (int64_t)((N + 127) / 128) * KT_all;
    } else {
        m_start = blockIdx.y * BM;
        m_end = min(p.M, m_start + BM);
    }

    float* bsl = (float*)(lds + D_NSTAGE * D_STAGE);
    const int64_t bs_row = bs_off + (int64_t)blockIdx.x * KT_all + kt0;

    // ---- per-thread source offsets (bytes, 32 bit) of the 7 loads of a stage.
    // Load i of a wave fills LDS rows 8q .. 8q+7 with q = wave*4+i (A) or wave*2+i (B), q & 1 == i & 1.
    // A: LDS row R holds tile row R.  B: within each 64-row half, LDS row rho holds tile column
    // 32*(rho >> 5) + 8*((rho & 15) >> 2) + 4*((rho >> 4) & 1) + (rho & 3): MFMA j then produces, in lane group g,
    // the four columns 32*(j >> 1) + 8g + 4*(j & 1) + (0..3), so that a lane ends up with two runs of 8 consecutive
    // columns of one output row and a store instruction writes 64 contiguous bytes per row.
    const int row8 = lane >> 3;
    uint32_t aoff[MI], boff[2];
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int R = 8 * (wave * MI + i) + row8;
        const uint32_t chunk = (uint32_t)((lane & 7) ^ ((R >> 1) & 7)) * 16u;
        aoff[i] = (uint32_t)min(m_start + R, m_end - 1) * (uint32_t)K + chunk;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t chunk = (uint32_t)((lane & 7) ^ (((i & 1) * 4 + (row8 >> 1)) & 7)) * 16u;
        const int R = 8 * (wave * 2 + i) + row8, rho = R & 63;
        const int col = (R & 64) + 32 * (rho >> 5) + 8 * ((rho & 15) >> 2) + 4 * ((rho >> 4) & 1) + (rho & 3);
        boff[i] = (uint32_t)min(n0 + col, N - 1) * (uint32_t)K + chunk;
    }
    const uint32_t soff = (uint32_t)min(m_start + min((wave & 3) * 64 + lane, BM - 1), m_end - 1) * (uint32_t)KT_all * (AS16 ? 2u : 4u);
    auto dma_scale = [&](uint32_t lds_addr, int kt_abs) {
        if constexpr (AS16) dma2(lds_addr, soff, (const uint8_t*)p.a_s + (int64_t)kt_abs * 2);
        else dma4(lds_addr, soff, (const uint8_t*)p.a_s + (int64_t)kt_abs * 4);
    };
    // K_W4NK: thread t expands quarter (t & 3) of LDS row t >> 2 (16 weights of a 64-element K step)
    uint32_t w4_off = 0, w4_soff = 0, w4_lds = 0;
    if constexpr (W4M) {
        // A K step of 64 is four strips of 16 k; the tile's 128 columns are two 64-column chunks: 256 units.
        // Thread t: unit (strip sl, chunk ch, lane ml = 8 columns c x 4 k-pairs q), words 2h and 2h + 1.
        // Word j, byte pair b of a unit: column 16 j + 8 b + c of the chunk, k = 2 q, 2 q + 1 (low nibbles of
        // the two halfwords) and 2 q + 8, 2 q + 9 (high nibbles) of the strip.
        const int h = tid & 1, ml = (tid >> 1) & 31, ch = (tid >> 6) & 1, sl = tid >> 7, c = ml >> 2, q = ml & 3;
        const int nchunks = N >> 6;
        const int chunk = min((n0 >> 6) + ch, nchunks - 1);
        w4_off = (uint32_t)((sl * nchunks + chunk) * 32 + ml) * 16u + (uint32_t)h * 8u;      // + 4 strips per K step
        w4_soff = (uint32_t)(64 * chunk + 8 * c + 4 * h) * 2u;                              // + scale row per K step
        // first of the eight pairs (j = 2h, b = 0, low nibbles): LDS row of column 16 j + c, K chunk 2 sl
        w4_lds = (uint32_t)(ch * 8 + h * 2) | ((uint32_t)c << 8) | ((uint32_t)sl << 16) | ((uint32_t)q << 24);   // packed fields
    }
    if constexpr (W4NK) {
        const int R = tid >> 2, q = tid & 3, rho = R & 63;
        const int col = (R & 64) + 32 * (rho >> 5) + 8 * ((rho & 15) >> 2) + 4 * ((rho >> 4) & 1) + (rho & 3);
        const uint32_t n = (uint32_t)min(n0 + col, N - 1);
        w4_off = n * (uint32_t)(p.K >> 1) + (uint32_t)q * 8u;                  // bytes into the packed matrix
        w4_soff = n * (uint32_t)(p.K / p.group) * 2u;                          // bytes into the scale matrix
        w4_lds = (uint32_t)R * 128u + (uint32_t)((2 * q) ^ ((R >> 1) & 7)) * 16u;   // chunk 2q; chunk 2q+1 is at ^16
    }
    // K_W4A8: zero points and second-level scales of the tile, raw bytes [K step][row] behind the weight-scale table
    uint8_t* w4tab = lds + D_NSTAGE * D_STAGE + D_MAX_KT * 4;
    if constexpr (W4A8) {
        // thread t: packed row pr = t >> 5 of the tile's sixteen, words 4 kc .. 4 kc + 3 (kc = t & 31) of the K step
        const int pr = tid >> 5, kc = tid & 31, np = N >> 3;
        w4_off = (uint32_t)min((n0 >> 3) + pr, np - 1) * (uint32_t)(p.K * 4) + (uint32_t)kc * 16u;
        // the eight rows of a packed row are tile columns 8 pr + i; column c of a 64-column half sits in LDS row
        // 32 (c >> 5) + 16 ((c >> 2) & 1) + 4 ((c >> 3) & 3) + (c & 3): rows i = 0..3 are consecutive LDS rows from
        // `base`, rows 4..7 the same 16 LDS rows further on; every pair of rows shares the swizzle of `base`
        const int ph = pr & 7, base = 64 * (pr >> 3) + 32 * (ph >> 2) + 4 * (ph & 3);
        w4_lds = (uint32_t)base | ((uint32_t)kc << 16) | ((uint32_t)pr << 24);
    }

    // the same loads in two bursts for the block-scaled kinds on the taller tiles: activation rows before the
    // step is multiplied, weight rows and scale column between its two phases (the buffer they go to was
    // released by the barrier of the previous step; 2-5 % faster for int8, even for fp8)
    auto issue_b_half = [&](int kt) {
        const uint32_t st = lds_base + (uint32_t)(kt % D_NSTAGE) * D_STAGE;
        const uint8_t* gb = bbase + (int64_t)(kt0 + kt) * 128;
        if constexpr (!W4) {
#pragma unroll
            for (int i = 0; i < 2; ++i) dma16(st + D_A + (uint32_t)(wave * 2 + i) * 1024u, boff[i], gb);
        }
        if constexpr (SCALED) dma_scale(st + D_A + D_B + (uint32_t)(wave & 3) * 256u, kt0 + kt);
    };
    auto issue_a_half = [&](int kt) {
        const uint32_t st = lds_base + (uint32_t)(kt % D_NSTAGE) * D_STAGE;
        const uint8_t* ga = p.a + (int64_t)(kt0 + kt) * 128;
#pragma unroll
        for (int i = 0; i < MI; ++i) dma16(st + (uint32_t)(wave * MI + i) * 1024u, aoff[i], ga);
    };
    auto issue = [&](int kt) {
        const uint32_t st = lds_base + (uint32_t)(kt % D_NSTAGE) * D_STAGE;
        const uint8_t* ga = p.a + (int64_t)(kt0 + kt) * 128;
        const uint8_t* gb = bbase + (int64_t)(kt0 + kt) * 128;
#pragma unroll
        for (int i = 0; i < MI; ++i) dma16(st + (uint32_t)(wave * MI + i) * 1024u, aoff[i], ga);
        if constexpr (!W4) {
#pragma unroll
            for (int i = 0; i < 2; ++i) dma16(st + D_A + (uint32_t)(wave * 2 + i) * 1024u, boff[i], gb);
        }
        if constexpr (SCALED) dma_scale(st + D_A + D_B + (uint32_t)(wave & 3) * 256u, kt0 + kt);
    };
    // K_W4NK: packed words and group scale of K step kt -> registers (requested before the activation loads
    // of the same step, so that waiting for them leaves exactly those MI loads in flight) ...
    // (the group scale is one halfword for the row-packed layout and four for a Marlin half unit: separate
    // variables of the exact register width, so that no widening move is ever placed between load and wait)
    uint64_t w4_words = 0, w4_scale = 0;
    unsigned w4_scale16 = 0;
    v4i w4_words4 = {0, 0, 0, 0};
    auto w4_request = [&](int kt) {
        if constexpr (W4A8) w4_words4 = asm_load_b128(w4_off, (const uint8_t*)p.b + (int64_t)(kt0 + kt) * 512);
        if constexpr (W4NK) {
            w4_words = asm_load_b64(w4_off, (const uint8_t*)p.b + (int64_t)(kt0 + kt) * 32);
            w4_scale16 = asm_load_u16(w4_soff, (const uint8_t*)p.b_s + (int64_t)(((kt0 + kt) * 64) / p.group) * 2);
        }
        if constexpr (W4M) {
            w4_words = asm_load_b64(w4_off, (const uint8_t*)p.b + (int64_t)(kt0 + kt) * 4 * (N >> 6) * 512);
            w4_scale = asm_load_b64(w4_soff, (const uint8_t*)p.b_s + (int64_t)(((kt0 + kt) * 64) / p.group) * N * 2);
        }
    };
    // ... and from there, expanded, into the weight rows of stage kt
    auto w4_expand = [&](int kt) {
        if constexpr (W4) {
            // everything but the MI youngest (activation) loads (and the scale column behind them for the
            // block-scaled kind).  The registers pass through the wait as read-write operands: the compiler must
            // have them in VGPRs here and takes every later use from this statement, so no use can be scheduled
            // above the wait.
            if constexpr (W4NK) asm volatile("s_waitcnt vmcnt(%2)" : "+v"(w4_words), "+v"(w4_scale16) : "n"(MI) : "memory");
            else if constexpr (W4M) asm volatile("s_waitcnt vmcnt(%2)" : "+v"(w4_words), "+v"(w4_scale) : "n"(MI) : "memory");
            else asm volatile("s_waitcnt vmcnt(%1)" : "+v"(w4_words4) : "n"(MI + 1) : "memory");
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (W4A8) {
            const int base = (int)(w4_lds & 0xffffu), kc = (int)((w4_lds >> 16) & 0xffu), pr = (int)(w4_lds >> 24);
            const uint8_t* tabk = w4tab + kt * 128 + 8 * pr;
            unsigned sp[4], cp[4], rows[8];
            w4a8_row_consts(*(const uint2*)tabk, *(const uint2*)(tabk + 128 * KT), sp, cp);
            w4a8_words_to_i8(w4_words4, sp, cp, rows);
            uint8_t* dst = lds + (kt % D_NSTAGE) * D_STAGE + D_A + (kc & 3) * 4;
            const int chunk = kc >> 2;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int R = base + (i & 3) + 16 * (i >> 2);
                *(unsigned*)(dst + R * 128 + ((chunk ^ ((R >> 1) & 7)) * 16)) = rows[i];
            }
        }
        if constexpr (W4NK) {
            const unsigned s16 = w4_scale16;
            const v2h sc = w4_as_h2(s16 | (s16 << 16));
            uint8_t* dst = lds + (kt % D_NSTAGE) * D_STAGE + D_A + w4_lds;
            *(v4i*)dst = w4_word_to_f16x8((unsigned)w4_words, sc);
            *(v4i*)(dst + ((w4_lds & 16u) ? -16 : 16)) = w4_word_to_f16x8((unsigned)(w4_words >> 32), sc);
        }
        if constexpr (W4M) {
            const v2h k1032 = {(_Float16)1032.f, (_Float16)1032.f};
            const v2h k16 = {(_Float16)0.0625f, (_Float16)0.0625f};
            const v2h k72 = {(_Float16)72.f, (_Float16)72.f};
            const int j0 = (int)(w4_lds & 7u), ch8 = (int)(w4_lds & 8u), c = (int)((w4_lds >> 8) & 7u);
            const int sl = (int)((w4_lds >> 16) & 3u), q = (int)(w4_lds >> 24);
            uint8_t* bst = lds + (kt % D_NSTAGE) * D_STAGE + D_A;
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                for (int b = 0; b < 2; ++b) {
                    const unsigned u = ((unsigned)(w4_words >> (32 * jj))) >> (8 * b);
                    const unsigned s16 = (unsigned)(w4_scale >> (16 * (2 * jj + b))) & 0xffffu;
                    const v2h sc = w4_as_h2(s16 | (s16 << 16));
                    const int col = 16 * (j0 + jj) + 8 * b + c;                                 // column in the chunk
                    const int R = (ch8 ? 64 : 0) + (col >> 5) * 32 + ((col >> 2) & 1) * 16 + ((col >> 3) & 3) * 4 + (col & 3);   // its LDS row
                    uint8_t* row = bst + R * 128 + 4 * q;
                    const int sw = (R >> 1) & 7;
                    *(v2h*)(row + ((2 * sl) ^ sw) * 16) = (w4_as_h2((u & 0x000f000fu) | 0x64006400u) - k1032) * sc;
                    *(v2h*)(row + ((2 * sl + 1) ^ sw) * 16) = (w4_as_h2((u & 0x00f000f0u) | 0x64006400u) * k16 - k72) * sc;
                }
        }
    };
    // Nothing is in flight when the last K step begins (the step before it ended with vmcnt(0)); this wait costs
    // nothing and puts a covering wait on every static path into that step, also on those that the trip counts
    // rule out (a request in the loop followed by a skipped middle step), which the check of the assembly walks.
    auto w4_drain = [&]() {
        if constexpr (W4A8) asm volatile("s_waitcnt vmcnt(0)" : "+v"(w4_words4) : : "memory");
    };
    // loads per stage per thread: MI (A) + 2 (B, or words + scale for K_W4NK; one load of words for K_W4A8) + 1 (scale column);
    // imm = vmcnt | no expcnt/lgkmcnt wait
    constexpr int WAIT_ONE_STAGE = 0x0F70 | (MI + (W4A8 ? 1 : 2) + (SCALED ? 1 : 0));

    // acc[i][j][q] = C[row 16i + r][col 32*(j >> 1) + 8g + 4*(j & 1) + q] of the wave's 64 x 64 tile
    v4f acc[MI][4];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

    if constexpr (W4A8) {
        // the table first (ordinary loads; the wait for them also drains stage 0, whose words are expanded next).
        // KT is the same for every thread of the workgroup, so the barrier is reached by all or by none.
        if (KT > 0) {
            w4_request(0);
            issue(0);
            for (int i = tid; i < 128 * KT; i += D_THREADS) {
                const int row = i / KT, kk = i - row * KT;
                const int64_t at = (int64_t)min(n0 + row, N - 1) * KT_all + kt0 + kk;
                w4tab[kk * 128 + row] = (uint8_t)p.w4_s4[at];
                w4tab[(KT + kk) * 128 + row] = (uint8_t)p.w4_z4[at];
            }
            __syncthreads();
            w4_expand(0);
        }
    } else if (KT > 0) { w4_request(0); issue(0); w4_expand(0); }
    if (KT > 1) { w4_request(1); issue(1); }
    // weight scales of this tile for every K step -> LDS.  These are the only compiler-tracked vector
    // loads; they sit behind the first two stages in the memory queue, so waiting for them also waits
    // for stage 0 and 1 (an acceptable one-off: the pipeline is being filled anyway).
    if constexpr (SCALED)
        for (int i = tid; i < KT; i += D_THREADS) bsl[i] = ld_scale(p.b_s, bs_row + i, p.s_dtype);
    __builtin_amdgcn_s_waitcnt(LLMK_WAIT_VMCNT_0);
    __syncthreads();

    // fragment read offsets inside a 16-row slab: chunks g and g + 4 of row r, swizzled (same K order for
    // both operands; the four lane groups of a b128 read then hit disjoint bank sets)
    const int lo = r * 128 + ((g ^ ((r >> 1) & 7)) * 16);
    const int hi = r * 128 + (((g + 4) ^ ((r >> 1) & 7)) * 16);
    auto ldfrag = [&](const uint8_t* base) {
        const v4i x = *(const v4i*)(base + lo), y = *(const v4i*)(base + hi);
        return (v8i){x[0], x[1], x[2], x[3], y[0], y[1], y[2], y[3]};
    };

    // Software pipeline inside the wave: the 16 partial products of a K step live in two register sets,
    // X (tile rows 0,1) and Y (tile rows 2,3).  While the MFMAs of one set run, the scale-and-accumulate
    // FMAs of the other set (finished half a step earlier) issue on the VALU: one MFMA (32 cycles) covers
    // the four FMAs (16 cycles) of one tile.
    constexpr int H = MI >= 2 ? MI / 2 : 1;   // tile rows per register set (MI == 1: set X only, no overlap)
    v4f tx[H][4], ty[H][4];
    float sy[H];
#pragma unroll
    for (int i = 0; i < H; ++i) {
        sy[i] = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) tx[i][j] = ty[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
    }

    // fragments of the K step being multiplied (zero before the first load: multiplying them is a no-op)
    v8i bf[4], af[MI];
    float sa[MI];
#pragma unroll
    for (int j = 0; j < 4; ++j) bf[j] = (v8i){0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        af[i] = (v8i){0, 0, 0, 0, 0, 0, 0, 0};
        sa[i] = 0.f;
    }
    auto load_frags = [&](int kt) {
        const uint8_t* st = lds + (kt % D_NSTAGE) * D_STAGE;
        const uint8_t* As = st + (wm * WR) * 128;
        const uint8_t* Bs = st + D_A + (wn * 64) * 128;
        const float* Ss = (const float*)(st + D_A + D_B) + wm * WR + r;
#pragma unroll
        for (int j = 0; j < 4; ++j) bf[j] = ldfrag(Bs + j * 2048);
#pragma unroll
        for (int i = 0; i < MI; ++i) af[i] = ldfrag(As + i * 2048);
        if constexpr (SCALED) {
            const float bs = bsl[kt];
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                if constexpr (AS16) {
                    const unsigned raw = ((const unsigned*)Ss)[i * 16];
                    sa[i] = (p.s_dtype == LLMK_F16 ? f16_to_f32((unsigned short)raw) : bf16_to_f32((unsigned short)raw)) * bs;
                } else {
                    sa[i] = Ss[i * 16] * bs;
                }
            }
        }
    };
    // The weight fragment is the MFMA row operand and the activation fragment the column operand, i.e.
    // the tile is produced transposed: a lane owns output row r and four consecutive columns per MFMA.
    // Branch-free so that the whole body is a single scheduling region.
    int mid_kt = -1;                    // >= 0: stage whose second half of loads goes out between the phases
    auto compute = [&]() {
        if constexpr (!SCALED) {
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = mma_plain<KIND>(bf[j], af[i], acc[i][j]);
        } else if constexpr (MI == 1) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[0][j] += tx[0][j] * sy[0];                  // retire the previous step while this one multiplies
                tx[0][j] = step_dot<KIND>(bf[j], af[0]);
            }
            sy[0] = sa[0];
        } else {
            // phase 1: X <- upper tile rows of this step; retire Y of the previous step into the lower acc rows
#pragma unroll
            for (int i = 0; i < H; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[H + i][j] += ty[i][j] * sy[i];
                    tx[i][j] = step_dot<KIND>(bf[j], af[i]);
                    __builtin_amdgcn_sched_group_barrier(0x008, KIND == K_FP8_BLOCK ? 1 : 2, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, KIND == K_FP8_BLOCK ? 4 : 8, 0);
                }
            if (mid_kt >= 0) { issue_b_half(mid_kt); mid_kt = -1; }
            // phase 2: Y <- lower tile rows of this step; retire X into the upper acc rows
#pragma unroll
            for (int i = 0; i < H; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    ty[i][j] = step_dot<KIND>(bf[j], af[H + i]);
                    acc[i][j] += tx[i][j] * sa[i];
                    __builtin_amdgcn_sched_group_barrier(0x008, KIND == K_FP8_BLOCK ? 1 : 2, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, KIND == K_FP8_BLOCK ? 4 : 8, 0);
                }
#pragma unroll
            for (int i = 0; i < H; ++i) sy[i] = sa[H + i];
        }
    };

    // Ping-pong between the two wave groups that share every SIMD (waves 0-3 and 4-7): group 0 reads the
    // fragments of step kt and multiplies them in the same iteration, group 1 multiplies the fragments it
    // read one iteration earlier and then reads step kt.  While one wave of a SIMD waits for LDS, the other
    // one keeps the matrix pipe busy.  Both groups hit the same barriers.
    // Steady state: stage kt+2 is issued, stage kt consumed, stage kt+1 awaited.
    int kt = 0;
    if (wave < 4) {
        for (; kt + 2 < KT; ++kt) {
            w4_expand(kt + 1);
            w4_request(kt + 2);
            if constexpr (SCALED && MI >= 2) { issue_a_half(kt + 2); mid_kt = kt + 2; } else issue(kt + 2);
            load_frags(kt);
            compute();
            __builtin_amdgcn_s_waitcnt(WAIT_ONE_STAGE);
            __syncthreads();
        }
        if (kt + 1 < KT) {
            w4_expand(kt + 1);
            load_frags(kt);
            compute();
            __builtin_amdgcn_s_waitcnt(LLMK_WAIT_VMCNT_0);
            __syncthreads();
            ++kt;
        }
        w4_drain();
        if (kt < KT) {
            load_frags(kt);
            compute();
        }
    } else {
        for (; kt + 2 < KT; ++kt) {
            w4_expand(kt + 1);
            w4_request(kt + 2);
            if constexpr (SCALED && MI >= 2) { issue_a_half(kt + 2); mid_kt = kt + 2; } else issue(kt + 2);
            compute();
            __builtin_amdgcn_sched_barrier(0);
            load_frags(kt);
            __builtin_amdgcn_s_waitcnt(WAIT_ONE_STAGE);
            __syncthreads();
        }
        if (kt + 1 < KT) {
            w4_expand(kt + 1);
            compute();
            __builtin_amdgcn_sched_barrier(0);
            load_frags(kt);
            __builtin_amdgcn_s_waitcnt(LLMK_WAIT_VMCNT_0);
            __syncthreads();
            ++kt;
        }
        w4_drain();
        if (kt < KT) {
            compute();
            __builtin_amdgcn_sched_barrier(0);
            load_frags(kt);
        }
        compute();
    }
    if constexpr (SCALED && MI >= 2) {
#pragma unroll
        for (int i = 0; i < H; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[H + i][j] += ty[i][j] * sy[i];
    }
    if constexpr (SCALED && MI == 1) {
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[0][j] += tx[0][j] * sy[0];
    }

    // ---- epilogue: every lane writes two runs of 8 consecutive outputs of each of its rows
    const bool split = !GROUPED && p.ksplit > 1;
    void* cout = split ? (void*)(p.partial + (int64_t)blockIdx.z * p.M * N) : p.c;
    const int cdt = split ? LLMK_F32 : p.c_dtype;
    const int esz = cdt == LLMK_F32 ? 4 : 2;
    const bool vec_ok = ((((uintptr_t)cout) & 15) == 0) && (((int64_t)N * esz) % 16 == 0);
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int m = m_start + wm * WR + 16 * i + r;
        if (m >= m_end) continue;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int nbh = n0 + wn * 64 + 32 * h + 8 * g;
            const int nv = N - nbh;
            if (nv <= 0) continue;
            const int64_t off = (int64_t)m * N + nbh;
            if constexpr (KIND == K_I8_ROWCOL) {
                // (a K slice leaves its int32 sums, bit for bit, in the fp32 partial buffer: the summing pass
                // adds them as integers and scales once, so the result does not depend on the split)
                if (!split) {
                    rowcol_epilogue8(p, acc[i][2 * h], acc[i][2 * h + 1], m, off, nbh, nv);
                    if (!p.c) continue;
                }
            }
            if (cdt == LLMK_BF16) store_run8<LLMK_BF16>(cout, off, acc[i][2 * h], acc[i][2 * h + 1], nv, vec_ok);
            else if (cdt == LLMK_F16) store_run8<LLMK_F16>(cout, off, acc[i][2 * h], acc[i][2 * h + 1], nv, vec_ok);
            else store_run8<LLMK_F32>(cout, off, acc[i][2 * h], acc[i][2 * h + 1], nv, vec_ok);
        }
    }
}

// sum of the split-K partials -> output dtype
template <int ODT>
__global__ void splitk_sum_kernel(const float* __restrict__ partial, void* __restrict__ c, int64_t mn, int z) {
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= mn) return;
    if (i + 4 <= mn && mn % 4 == 0) {
        // four independent loads at a time (the partials come from other CUs' writes: every load is a long
        // round trip), added in slice order
        v4f s = {0.f, 0.f, 0.f, 0.f};
        int k = 0;
        for (; k + 4 <= z; k += 4) {
            v4f t[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) t[j] = *(const v4f*)(partial + (int64_t)(k + j) * mn + i);
#pragma unroll
            for (int j = 0; j < 4; ++j) s += t[j];
        }
        for (; k < z; ++k) s += *(const v4f*)(partial + (int64_t)k * mn + i);
#pragma unroll
        for (int q = 0; q < 4; ++q) FloatIO<ODT>::st(c, i + q, s[q]);
    } else {
        for (int64_t j = i; j < min(i + 4, mn); ++j) {
            float s = 0.f;
            for (int k = 0; k < z; ++k) s += partial[(int64_t)k * mn + j];
            FloatIO<ODT>::st(c, j, s);
        }
    }
}

// The same for the per-token x per-channel int8 kind: the partials are int32 sums over K slices; they are
// added as integers (exactly what one workgroup over all of K would have held), written out raw when the
// caller asked for them, and scaled by a_s[m] * b_s[n] into the output dtype.
template <int ODT>
__global__ void splitk_sum_rowcol_kernel(const int32_t* __restrict__ partial, DirectArgs p, int64_t mn, int z) {
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= mn) return;
    const float* as = (const float*)p.a_s;
    const float* bs = (const float*)p.b_s;
    if (p.N % 4 == 0) {                       // the four elements share a row, every slice is 16-byte aligned
        v4i s = {0, 0, 0, 0};
        int k = 0;
        for (; k + 4 <= z; k += 4) {
            v4i t[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) t[j] = *(const v4i*)(partial + (int64_t)(k + j) * mn + i);
#pragma unroll
            for (int j = 0; j < 4; ++j) s += t[j];
        }
        for (; k < z; ++k) s += *(const v4i*)(partial + (int64_t)k * mn + i);
        if (p.c_i32) {
            if ((((uintptr_t)p.c_i32) & 15) == 0) *(v4i*)(p.c_i32 + i) = s;
            else {
#pragma unroll
                for (int q = 0; q < 4; ++q) p.c_i32[i + q] = s[q];
            }
        }
        if (p.c) {
            const int m = (int)(i / p.N), n = (int)(i % p.N);
            const float am = as[m];
#pragma unroll
            for (int q = 0; q < 4; ++q) FloatIO<ODT>::st(p.c, i + q, (float)s[q] * am * bs[n + q]);
        }
    } else {
        for (int64_t j = i; j < min(i + 4, mn); ++j) {
            int s = 0;
            for (int k = 0; k < z; ++k) s += partial[(int64_t)k * mn + j];
            if (p.c_i32) p.c_i32[j] = s;
            if (p.c) FloatIO<ODT>::st(p.c, j, (float)s * as[j / p.N] * bs[j % p.N]);
        }
    }
}

// fp16 / bf16 activation scales -> fp32 (the pipeline above streams 4-byte scale elements)
template <int SDT>
__global__ void scales_to_f32_kernel(const void* __restrict__ src, float* __restrict__ dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = FloatIO<SDT>::ld(src, i);
}

// true when the three-stage kernel can take this problem (32-bit source offsets, scale table size)
inline bool dma_eligible(const DirectArgs& p, int esz = 1) {
    const int64_t kb = (int64_t)p.K * esz;              // row bytes
    return (int64_t)p.M * kb < (1ll << 32) && (int64_t)p.N * kb < (1ll << 32) && kb % 128 == 0 &&
           (int64_t)p.M * (kb >> 7) * 4 < (1ll << 32) && (kb >> 7) <= D_MAX_KT && p.K > 0;
}

// K steps one workgroup of the K_W4A8 kind walks (its share of a split K range): sizes its LDS table
constexpr int D_LDS_MAX = 160 * 1024;
inline int w4a8_table_steps(const DirectArgs& p) {
    const int KT = p.K >> 7;
    return p.ksplit > 1 ? (KT + p.ksplit - 1) / p.ksplit : KT;
}
// tallest tile (MI) whose stages leave room for that table
inline int w4a8_max_mi(const DirectArgs& p) {
    const int tab = 256 * w4a8_table_steps(p);
    // (the 256-row tile has no registers to spare for the expansion: the kind runs on the 128- and 64-row tiles)
    return d_lds(2) + tab <= D_LDS_MAX ? 2 : (d_lds(1) + tab <= D_LDS_MAX ? 1 : 0);
}

// p.a_s: fp32, or with AS16 the 16-bit scales of dtype p.s_dtype as the caller passed them; p.s_dtype describes b_s.
template <int KIND, bool GROUPED, int MI, bool AS16 = false>
int launch_dma_mi(const DirectArgs& p, hipStream_t stream, const char* name) {
    static std::atomic<uint64_t> configured{0};
    auto kern = gemm_dma_kernel<KIND, GROUPED, MI, AS16>;
    constexpr int BM = 64 * MI;
    const int tiles_m = GROUPED ? grouped_row_tiles(p.M, p.E, BM) : (p.M + BM - 1) / BM;
    const bool split = !GROUPED && p.ksplit > 1 && p.partial;
    // K_W4A8: the table of zero points and second-level scales (256 bytes per K step of the workgroup) behind the stages
    const int lds_bytes = d_lds(MI) + (KIND == K_W4A8 ? 256 * w4a8_table_steps(p) : 0);
    if (lds_bytes > D_LDS_MAX) LLMK_FAIL(LLMK_ERR_SHAPE, "%s: %d bytes of LDS needed", name, lds_bytes);
    if (int rc = llmk_reserve_lds((const void*)kern, KIND == K_W4A8 ? D_LDS_MAX : d_lds(MI), configured, name)) return rc;
    dim3 grid((unsigned)((p.N + D_BN - 1) / D_BN), (unsigned)tiles_m, split ? (unsigned)p.ksplit : 1u);
    if (grid.x == 0 || grid.y == 0) return LLMK_OK;
    kern<<<grid, D_THREADS, lds_bytes, stream>>>(p);
    LLMK_CHECK_LAUNCH(name);
    if (split) {
        const int64_t mn = (int64_t)p.M * p.N;
        const unsigned blocks = (unsigned)cdiv64(cdiv64(mn, 4), 256);
        if constexpr (KIND == K_I8_ROWCOL) {
            const int32_t* part = (const int32_t*)p.partial;
            if (p.c_dtype == LLMK_BF16) splitk_sum_rowcol_kernel<LLMK_BF16><<<blocks, 256, 0, stream>>>(part, p, mn, p.ksplit);
            else if (p.c_dtype == LLMK_F16) splitk_sum_rowcol_kernel<LLMK_F16><<<blocks, 256, 0, stream>>>(part, p, mn, p.ksplit);
            else splitk_sum_rowcol_kernel<LLMK_F32><<<blocks, 256, 0, stream>>>(part, p, mn, p.ksplit);
            LLMK_CHECK_LAUNCH(name);
            return LLMK_OK;
        }
        if (p.c_dtype == LLMK_BF16) splitk_sum_kernel<LLMK_BF16><<<blocks, 256, 0, stream>>>(p.partial, p.c, mn, p.ksplit);
        else if (p.c_dtype == LLMK_F16) splitk_sum_kernel<LLMK_F16><<<blocks, 256, 0, stream>>>(p.partial, p.c, mn, p.ksplit);
        else splitk_sum_kernel<LLMK_F32><<<blocks, 256, 0, stream>>>(p.partial, p.c, mn, p.ksplit);
        LLMK_CHECK_LAUNCH(name);
    }
    return LLMK_OK;
}

}  // namespace llmk
