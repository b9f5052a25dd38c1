// Single-GPU expert-parallel MoE path: segment bookkeeping, token permute / un-permute,
// gated activation, and the grouped GEMM over one GPU's experts.
#include "gemm_wide.hpp"
#include "quant_util.hpp"

using namespace llmk;

namespace {

// seg_indptr[e + 1] = number of sorted ids <= e (binary search for the right boundary)
__global__ void seg_indptr_kernel(const int64_t* __restrict__ sorted_ids, int64_t* __restrict__ seg_indptr,
                                  int64_t num_toks, int num_experts) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= num_experts) return;
    int64_t lo = 0, hi = num_toks;       // first index with id > e
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (sorted_ids[mid] > e) hi = mid; else lo = mid + 1;
    }
    seg_indptr[e + 1] = lo;
    if (e == 0) seg_indptr[0] = 0;
}

__global__ void src2dst_kernel(const int64_t* __restrict__ reorder_ids, int32_t* __restrict__ src2dst, int64_t n) {
    const int64_t d = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (d < n) src2dst[reorder_ids[d]] = (int32_t)d;
}

__device__ __forceinline__ int64_t ld_id(const void* p, int64_t i, int bytes) {
    return bytes == 8 ? ((const int64_t*)p)[i] : (int64_t)((const int32_t*)p)[i];
}

// Stable counting sort of the flattened expert ids, with the segment pointers and the source -> destination
// map as by-products: what torch.sort(stable) + seg_indptr_kernel + src2dst_kernel produce in eight launches.
// Bucket 0 takes negative ids, bucket e + 1 expert e, bucket E + 1 ids >= E (both out-of-range buckets keep
// their arrival order; a well-formed input leaves them empty).
// Workgroup g places the ids [1024 g, 1024 g + 1024).  It counts, per bucket, all ids (-> bucket starts) and
// the ids in front of its chunk, by reading the whole id list (at most PP_MAX_IDS ids, from L2); a lane's
// position is then bucket start + ids of the bucket in earlier chunks + those in the lower waves of the
// chunk + its rank among the equal ids of its own wave.  No workgroup waits for another.
constexpr int PP_THREADS = 1024, PP_WAVES = PP_THREADS / 64, PP_MAX_EXPERTS = 512, PP_BUCKETS = PP_MAX_EXPERTS + 2;

__global__ __launch_bounds__(PP_THREADS) void ep_preprocess_kernel(const void* __restrict__ ids, int ids_bytes, int n, int E,
                                                                   void* __restrict__ sorted_out, int32_t* __restrict__ src2dst,
                                                                   int64_t* __restrict__ seg_indptr) {
    __shared__ int tot[PP_BUCKETS];      // ids per bucket, then the bucket's first position
    __shared__ int pre[PP_BUCKETS];      // ids per bucket in front of this workgroup's chunk
    __shared__ int wcount[PP_WAVES][PP_BUCKETS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nb = E + 2;
    const int c0 = blockIdx.x * PP_THREADS;
    auto bucket_at = [&](int i) {
        if (i >= n) return -1;
        const int64_t id = ld_id(ids, i, ids_bytes);
        return id < 0 ? 0 : (id >= E ? E + 1 : (int)id + 1);
    };
    for (int b = tid; b < nb; b += PP_THREADS) { tot[b] = 0; pre[b] = 0; }
    for (int i = tid; i < PP_WAVES * nb; i += PP_THREADS) wcount[i / nb][i % nb] = 0;
    __syncthreads();
    constexpr int U = 4;                 // rounds whose loads are in flight together
    if (nb <= 64) {
        // few buckets: lane k of every wave counts bucket k from ballots (one LDS atomic per id would
        // serialise on the few addresses)
        int acc_t = 0, acc_p = 0;
        for (int r0 = 0; r0 < n; r0 += U * PP_THREADS) {
            int b[U];
#pragma unroll
            for (int u = 0; u < U; ++u) b[u] = bucket_at(r0 + u * PP_THREADS + tid);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const bool before = r0 + u * PP_THREADS < c0;        // whole rounds lie in front of the chunk or not
                for (int k = 0; k < nb; ++k) {
                    const int c = __popcll(__ballot(b[u] == k));
                    if (lane == k) { acc_t += c; if (before) acc_p += c; }
                }
            }
        }
        if (lane < nb) { atomicAdd(&tot[lane], acc_t); atomicAdd(&pre[lane], acc_p); }
    } else {
        for (int r0 = 0; r0 < n; r0 += U * PP_THREADS) {
            int b[U];
#pragma unroll
            for (int u = 0; u < U; ++u) b[u] = bucket_at(r0 + u * PP_THREADS + tid);
#pragma unroll
            for (int u = 0; u < U; ++u) if (b[u] >= 0) {
                atomicAdd(&tot[b[u]], 1);
                if (r0 + u * PP_THREADS < c0) atomicAdd(&pre[b[u]], 1);
            }
        }
    }
    __syncthreads();
    if (wave == 0) {
        // exclusive scan of the bucket counts: a run of buckets per lane, then a scan over the lanes
        const int per = (nb + 63) / 64, b0 = lane * per;
        int sum = 0;
        for (int k = 0; k < per; ++k) if (b0 + k < nb) sum += tot[b0 + k];
        int incl = sum;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int t = __shfl_up(incl, o, 64);
            if (lane >= o) incl += t;
        }
        int run = incl - sum;
        for (int k = 0; k < per; ++k) if (b0 + k < nb) {
            const int c = tot[b0 + k];
            tot[b0 + k] = run;
            run += c;
        }
    }
    __syncthreads();
    // seg_indptr[e + 1] = number of ids <= e = start of bucket e + 2; seg_indptr[0] = 0
    if (blockIdx.x == 0)
        for (int e = tid; e <= E; e += PP_THREADS) seg_indptr[e] = e == 0 ? 0 : (int64_t)tot[e + 1];

    // rank of a lane among the lanes of its wave with the same bucket, one leader per bucket publishes the count
    const int i = c0 + tid;
    const int b = bucket_at(i);
    int rank = 0;
    uint64_t todo = __ballot(b >= 0);
    while (todo) {                                       // one pass per distinct bucket of the wave
        const int l = __ffsll((unsigned long long)todo) - 1;
        const int v = __builtin_amdgcn_readlane(b, l);
        const uint64_t m = __ballot(b == v);
        if (b == v) {
            rank = __popcll(m & ((1ull << lane) - 1ull));
            if (lane == l) wcount[wave][b] = __popcll(m);
        }
        todo &= ~m;
    }
    __syncthreads();
    if (b >= 0) {
        int pos = tot[b] + pre[b] + rank;
        for (int w = 0; w < wave; ++w) pos += wcount[w][b];
        const int64_t id = (b >= 1 && b <= E) ? (int64_t)(b - 1) : ld_id(ids, i, ids_bytes);
        if (ids_bytes == 8) ((int64_t*)sorted_out)[pos] = id; else ((int32_t*)sorted_out)[pos] = (int32_t)id;
        src2dst[i] = pos;
    }
}

// one workgroup per token: copy (x * 1/a1_scale[e]) into each destination row of its local experts
template <int IDT, int ODT>
__global__ void pre_reorder_kernel(const void* __restrict__ x, void* __restrict__ out, const int32_t* __restrict__ src2dst,
                                   const void* __restrict__ topk_ids, int ids_bytes, const float* __restrict__ a1_scales,
                                   int start_e, int end_e, int topk, int64_t hidden) {
    const int64_t t = blockIdx.x;
    for (int j = 0; j < topk; ++j) {
        const int64_t e = ld_id(topk_ids, t * topk + j, ids_bytes);
        if (e < start_e || e > end_e) continue;
        const float scale = a1_scales ? 1.0f / a1_scales[e - start_e] : 1.0f;
        const int64_t dst = src2dst[t * topk + j];
        for (int64_t c = threadIdx.x; c < hidden; c += blockDim.x)
            FloatIO<ODT>::st(out, dst * hidden + c, FloatIO<IDT>::ld(x, t * hidden + c) * scale);
    }
}

// groups per thread of the fused activation + quantisation kernel (8192 x 28672 bf16 -> e4m3: 121 us with 1,
// 117 us with 2, 131 us with 4, 146 us with 8)
constexpr int AMQ_UNROLL = 2;

template <int IDT, int ODT>
__global__ void act_and_mul_kernel(const void* __restrict__ gateup, void* __restrict__ out,
                                   const void* __restrict__ reorder_topk_ids, int ids_bytes,
                                   const float* __restrict__ scales, int start_e, int end_e, int64_t two_i, int act) {
    const int64_t row = blockIdx.x;
    const int64_t e = ld_id(reorder_topk_ids, row, ids_bytes);
    if (e < start_e || e > end_e) return;
    const int64_t I = two_i / 2;
    const bool has_scale = scales != nullptr;
    const float scale = has_scale ? rnd<IDT>(1.0f / scales[e - start_e]) : 1.0f;
    for (int64_t c = threadIdx.x; c < I; c += blockDim.x) {
        const float gv = FloatIO<IDT>::ld(gateup, row * two_i + c);
        const float up = FloatIO<IDT>::ld(gateup, row * two_i + I + c);
        const float r = gated_act<IDT>(gv, up, act, has_scale, scale);
        FloatIO<ODT>::st(out, row * I + c, r);
    }
}

// the same with 8 outputs per thread and pass (I a multiple of 8, 16-byte aligned tensors); a thread requests
// the operands of two passes before it converts the first
template <int IDT, int ODT>
__global__ void act_and_mul_vec_kernel(const void* __restrict__ gateup, void* __restrict__ out,
                                       const void* __restrict__ reorder_topk_ids, int ids_bytes,
                                       const float* __restrict__ scales, int start_e, int end_e, int64_t two_i, int act) {
    const int64_t row = blockIdx.x;
    const int64_t e = ld_id(reorder_topk_ids, row, ids_bytes);
    if (e < start_e || e > end_e) return;
    const int64_t I = two_i / 2;
    const bool has_scale = scales != nullptr;
    const float scale = has_scale ? rnd<IDT>(1.0f / scales[e - start_e]) : 1.0f;
    const int64_t step = (int64_t)blockDim.x * EPL;
    for (int64_t c0 = (int64_t)threadIdx.x * EPL; c0 < I; c0 += 2 * step) {
        const int64_t c1 = c0 + step;
        const bool two = c1 < I;
        float gv[2][EPL], up[2][EPL], r[EPL];
        load8<IDT>(gateup, row * two_i + c0, gv[0]);
        load8<IDT>(gateup, row * two_i + I + c0, up[0]);
        if (two) {
            load8<IDT>(gateup, row * two_i + c1, gv[1]);
            load8<IDT>(gateup, row * two_i + I + c1, up[1]);
        }
#pragma unroll
        for (int j = 0; j < EPL; ++j) r[j] = gated_act<IDT>(gv[0][j], up[0][j], act, has_scale, scale);
        store8<ODT>(out, row * I + c0, r);
        if (two) {
#pragma unroll
            for (int j = 0; j < EPL; ++j) r[j] = gated_act<IDT>(gv[1][j], up[1][j], act, has_scale, scale);
            store8<ODT>(out, row * I + c1, r);
        }
    }
}

// Gated activation and 1 x 128 activation quantisation in one pass: 16 lanes own one group of 128 outputs,
// 8 each.  The values quantised are exactly those the separate activation kernel would have stored in the
// tensor dtype, so q and s equal those of the two-kernel sequence bit for bit.
template <int IDT, bool FP8>
__global__ void act_mul_quant_kernel(const void* __restrict__ gateup, void* __restrict__ q_out, void* __restrict__ s_out,
                                     const void* __restrict__ reorder_topk_ids, int ids_bytes,
                                     const float* __restrict__ scales, int start_e, int end_e, int64_t M, int64_t two_i,
                                     int act, int mode) {
    // a workgroup owns AMQ_UNROLL x 16 consecutive groups; a thread requests the operands of all its groups
    // before it converts the first one
    const int64_t I = two_i / 2, gpr = I / 128;
    const int sub = threadIdx.x & 15;
    int64_t grp[AMQ_UNROLL], row[AMQ_UNROLL], col[AMQ_UNROLL];
    bool live[AMQ_UNROLL];
    float gv[AMQ_UNROLL][EPL], up[AMQ_UNROLL][EPL];
#pragma unroll
    for (int k = 0; k < AMQ_UNROLL; ++k) {
        grp[k] = ((int64_t)blockIdx.x * AMQ_UNROLL + k) * (blockDim.x >> 4) + (threadIdx.x >> 4);
        live[k] = grp[k] < M * gpr;
        const int64_t gs = live[k] ? grp[k] : 0;
        row[k] = gs / gpr;
        col[k] = (gs - row[k] * gpr) * 128 + sub * EPL;
        load8<IDT>(gateup, row[k] * two_i + col[k], gv[k]);
        load8<IDT>(gateup, row[k] * two_i + I + col[k], up[k]);
    }
#pragma unroll
    for (int k = 0; k < AMQ_UNROLL; ++k) {
        const int64_t e = ld_id(reorder_topk_ids, row[k], ids_bytes);
        const bool local = e >= start_e && e <= end_e;
        const bool has_scale = scales != nullptr && local;
        const float scale = has_scale ? rnd<IDT>(1.0f / scales[e - start_e]) : 1.0f;
        float r[EPL];
        float m = 0.f;
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
            r[j] = gated_act<IDT>(gv[k][j], up[k][j], act, has_scale, scale);
            m = fmaxf(m, fabsf(r[j]));
        }
        m = group_max<16>(m);
        if (!live[k] || !local) continue;
        quant_store8<FP8>(r, m, q_out, row[k] * I + col[k], s_out, grp[k], sub == 0, mode);
    }
}

// Token permutation and 1 x 128 activation quantisation in one pass: a token's row is read once, quantised
// (after the optional per-expert scale, rounded to the tensor dtype as the separate kernels do) and written
// to the destination row of each of its local experts.
constexpr int PRQ_UNROLL = 1;      // groups per thread of the fused permutation + quantisation kernel (2 and 4: no faster)

template <int IDT, bool FP8>
__global__ void pre_reorder_quant_kernel(const void* __restrict__ x, void* __restrict__ q_out, void* __restrict__ s_out,
                                         const int32_t* __restrict__ src2dst, const void* __restrict__ topk_ids,
                                         int ids_bytes, const float* __restrict__ a1_scales, int start_e, int end_e,
                                         int topk, int64_t T, int64_t hidden, int mode) {
    const int64_t gpr = hidden / 128;
    const int sub = threadIdx.x & 15;
    int64_t t[PRQ_UNROLL], gi[PRQ_UNROLL];
    bool live[PRQ_UNROLL];
    float v[PRQ_UNROLL][EPL];
#pragma unroll
    for (int u = 0; u < PRQ_UNROLL; ++u) {
        const int64_t grp = ((int64_t)blockIdx.x * PRQ_UNROLL + u) * (blockDim.x >> 4) + (threadIdx.x >> 4);
        live[u] = grp < T * gpr;
        const int64_t gs = live[u] ? grp : 0;
        t[u] = gs / gpr;
        gi[u] = gs - t[u] * gpr;
        load8<IDT>(x, t[u] * hidden + gi[u] * 128 + sub * EPL, v[u]);
    }
#pragma unroll
    for (int u = 0; u < PRQ_UNROLL; ++u) {
        const int64_t col = gi[u] * 128 + sub * EPL;
        for (int j = 0; j < topk; ++j) {
            const int64_t e = ld_id(topk_ids, t[u] * topk + j, ids_bytes);
            const bool local = e >= start_e && e <= end_e;
            const float scale = (a1_scales && local) ? 1.0f / a1_scales[e - start_e] : 1.0f;
            float w[EPL];
            float m = 0.f;
#pragma unroll
            for (int k = 0; k < EPL; ++k) {
                w[k] = rnd<IDT>(v[u][k] * scale);
                m = fmaxf(m, fabsf(w[k]));
            }
            m = group_max<16>(m);
            if (!live[u] || !local) continue;
            const int64_t dst = src2dst[t[u] * topk + j];
            quant_store8<FP8>(w, m, q_out, dst * hidden + col, s_out, dst * gpr + gi[u], sub == 0, mode);
        }
    }
}

template <int DT, int WDT>
__global__ void post_reorder_kernel(const void* __restrict__ down, void* __restrict__ out, const int32_t* __restrict__ src2dst,
                                    const void* __restrict__ topk_ids, int ids_bytes, const void* __restrict__ topk_w,
                                    int start_e, int end_e, int topk, int64_t hidden) {
    const int64_t t = blockIdx.x;
    if constexpr (DT != LLMK_F32) {
        // 16-bit rows of whole 16-byte chunks: 8 columns per lane and load
        if (hidden % EPL == 0 && (((uintptr_t)down | (uintptr_t)out) & 15) == 0) {
            for (int64_t c = (int64_t)threadIdx.x * EPL; c < hidden; c += (int64_t)blockDim.x * EPL) {
                float sum[EPL] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                for (int j = 0; j < topk; ++j) {
                    const int64_t e = ld_id(topk_ids, t * topk + j, ids_bytes);
                    if (e < start_e || e > end_e) continue;
                    const int64_t dst = src2dst[t * topk + j];
                    const float w = rnd<DT>(FloatIO<WDT>::ld(topk_w, t * topk + j));
                    float v[EPL];
                    load8<DT>(down, dst * hidden + c, v);
#pragma unroll
                    for (int k = 0; k < EPL; ++k) sum[k] = rnd<DT>(sum[k] + rnd<DT>(v[k] * w));
                }
                uint4 o;
                if constexpr (DT == LLMK_BF16) {
                    o.x = pack_bf16x2(sum[0], sum[1]); o.y = pack_bf16x2(sum[2], sum[3]);
                    o.z = pack_bf16x2(sum[4], sum[5]); o.w = pack_bf16x2(sum[6], sum[7]);
                } else {
                    o.x = pack_f16x2(sum[0], sum[1]); o.y = pack_f16x2(sum[2], sum[3]);
                    o.z = pack_f16x2(sum[4], sum[5]); o.w = pack_f16x2(sum[6], sum[7]);
                }
                *(uint4*)((unsigned short*)out + t * hidden + c) = o;
            }
            return;
        }
    }
    for (int64_t c = threadIdx.x; c < hidden; c += blockDim.x) {
        float sum = 0.f;
        for (int j = 0; j < topk; ++j) {
            const int64_t e = ld_id(topk_ids, t * topk + j, ids_bytes);
            if (e < start_e || e > end_e) continue;
            const int64_t dst = src2dst[t * topk + j];
            const float w = rnd<DT>(FloatIO<WDT>::ld(topk_w, t * topk + j));
            const float v = FloatIO<DT>::ld(down, dst * hidden + c);
            sum = rnd<DT>(sum + rnd<DT>(v * w));     // product and running sum both live in the tensor dtype
        }
        FloatIO<DT>::st(out, t * hidden + c, sum);
    }
}

// ---------------------------------------------------------------- per-expert scalar scales -> block-scale layout
// scale_a[r, :] = sa[e(r)] for the rows of segment e, scale_b[w, :, :] = sb[w]; rows outside every segment get 0.
// Blocks [0, M) write one activation-scale row each, blocks [M, M + Eb) one expert's weight scales.
template <int SDT>
__global__ void expert_scales_kernel(const float* __restrict__ sa, const float* __restrict__ sb,
                                     const int64_t* __restrict__ seg, int E, int64_t M, int kb, int64_t nbkb,
                                     void* __restrict__ scale_a, void* __restrict__ scale_b) {
    const int64_t blk = blockIdx.x;
    if (blk < M) {
        float v = 0.f;
        for (int e = 0; e < E; ++e)
            if (blk >= seg[e] && blk < seg[e + 1]) { v = sa[e]; break; }
        for (int i = threadIdx.x; i < kb; i += blockDim.x) FloatIO<SDT>::st(scale_a, blk * kb + i, v);
    } else {
        const int64_t w = blk - M;
        const float v = sb[w];
        for (int64_t i = threadIdx.x; i < nbkb; i += blockDim.x) FloatIO<SDT>::st(scale_b, w * nbkb + i, v);
    }
}

}  // namespace

extern "C" int llmk_moe_expert_scales(const float* sa, const float* sb, const int64_t* seg_indptr, int E, int Eb,
                                      int64_t M, int64_t N, int64_t K, void* scale_a, void* scale_b, int s_dtype,
                                      void* stream) {
    if (M < 0 || N < 0 || K < 0 || E < 0 || Eb < 0 || K % 128) LLMK_FAIL(LLMK_ERR_SHAPE, "moe_expert_scales: bad shape");
    if (M + Eb == 0 || K == 0) return LLMK_OK;
    if (!sa || !sb || !seg_indptr || !scale_a || !scale_b) LLMK_FAIL(LLMK_ERR_ARG, "moe_expert_scales: null pointer");
    const int kb = (int)(K / 128);
    const int64_t nbkb = ((N + 127) / 128) * kb;
    LLMK_DISPATCH_FLOAT(s_dtype, SDT, (expert_scales_kernel<SDT><<<(unsigned)(M + Eb), 64, 0, (hipStream_t)stream>>>(
        sa, sb, seg_indptr, E, M, kb, nbkb, scale_a, scale_b)));
    LLMK_CHECK_LAUNCH("moe_expert_scales");
    return LLMK_OK;
}

extern "C" int llmk_moe_seg_indptr(const int64_t* sorted_ids, int64_t* seg_indptr, int64_t num_toks, int num_experts,
                                   void* stream) {
    if (num_experts < 0 || num_toks < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "moe_seg_indptr: negative size");
    if (!seg_indptr || (num_toks && !sorted_ids)) LLMK_FAIL(LLMK_ERR_ARG, "moe_seg_indptr: null pointer");
    if (num_experts == 0) return LLMK_OK;
    seg_indptr_kernel<<<(unsigned)cdiv64(num_experts, 64), 64, 0, (hipStream_t)stream>>>(sorted_ids, seg_indptr, num_toks, num_experts);
    LLMK_CHECK_LAUNCH("moe_seg_indptr");
    return LLMK_OK;
}

extern "C" int llmk_moe_src2dst(const int64_t* reorder_ids, int32_t* src2dst, int64_t num_toks, void* stream) {
    if (num_toks < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "moe_src2dst: negative size");
    if (num_toks == 0) return LLMK_OK;
    if (!reorder_ids || !src2dst) LLMK_FAIL(LLMK_ERR_ARG, "moe_src2dst: null pointer");
    src2dst_kernel<<<(unsigned)cdiv64(num_toks, 256), 256, 0, (hipStream_t)stream>>>(reorder_ids, src2dst, num_toks);
    LLMK_CHECK_LAUNCH("moe_src2dst");
    return LLMK_OK;
}

extern "C" int llmk_moe_ep_preprocess(const void* topk_ids, int ids_bytes, int64_t num_toks, int num_experts,
                                      void* sorted_ids, int32_t* src2dst, int64_t* seg_indptr, void* stream) {
    if (num_experts < 0 || num_toks < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "moe_ep_preprocess: negative size");
    if (num_experts > LLMK_MOE_PREPROCESS_MAX_EXPERTS || num_toks > LLMK_MOE_PREPROCESS_MAX_IDS)
        LLMK_FAIL(LLMK_ERR_SHAPE, "moe_ep_preprocess: %lld ids of %d experts exceed the limits %d / %d of the one-workgroup sort",
                  (long long)num_toks, num_experts, LLMK_MOE_PREPROCESS_MAX_IDS, LLMK_MOE_PREPROCESS_MAX_EXPERTS);
    if (ids_bytes != 4 && ids_bytes != 8) LLMK_FAIL(LLMK_ERR_DTYPE, "moe_ep_preprocess: ids_bytes %d", ids_bytes);
    if (!seg_indptr || (num_toks && (!topk_ids || !sorted_ids || !src2dst))) LLMK_FAIL(LLMK_ERR_ARG, "moe_ep_preprocess: null pointer");
    static_assert(LLMK_MOE_PREPROCESS_MAX_EXPERTS == PP_MAX_EXPERTS, "header limit and kernel table size differ");
    const unsigned grid = (unsigned)(num_toks > 0 ? cdiv64(num_toks, PP_THREADS) : 1);
    ep_preprocess_kernel<<<grid, PP_THREADS, 0, (hipStream_t)stream>>>(topk_ids, ids_bytes, (int)num_toks, num_experts, sorted_ids, src2dst, seg_indptr);
    LLMK_CHECK_LAUNCH("moe_ep_preprocess");
    return LLMK_OK;
}

extern "C" int llmk_moe_pre_reorder(const void* x, int x_dtype, void* out, int out_dtype, const int32_t* src2dst,
                                    const void* topk_ids, int ids_bytes, const float* a1_scales, int start_expert,
                                    int end_expert, int topk, int64_t T, int64_t hidden, void* stream) {
    if (T < 0 || hidden < 0 || topk < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "moe_pre_reorder: negative size");
    if (ids_bytes != 4 && ids_bytes != 8) LLMK_FAIL(LLMK_ERR_DTYPE, "moe_pre_reorder: ids_bytes %d", ids_bytes);
    if (T == 0 || hidden == 0 || topk == 0) return LLMK_OK;
    if (!x || !out || !src2dst || !topk_ids) LLMK_FAIL(LLMK_ERR_ARG, "moe_pre_reorder: null pointer");
    LLMK_DISPATCH_FLOAT(x_dtype, IDT, LLMK_DISPATCH_FLOAT(out_dtype, ODT,
        (pre_reorder_kernel<IDT, ODT><<<(unsigned)T, 256, 0, (hipStream_t)stream>>>(x, out, src2dst, topk_ids, ids_bytes, a1_scales, start_expert, end_expert, topk, hidden))));
    LLMK_CHECK_LAUNCH("moe_pre_reorder");
    return LLMK_OK;
}

extern "C" int llmk_moe_act_and_mul(const void* gateup, int in_dtype, void* out, int out_dtype,
                                    const void* reorder_topk_ids, int ids_bytes, const float* scales, int start_expert,
                                    int end_expert, int64_t M, int64_t two_i, int act, void* stream) {
    if (M < 0 || two_i < 0 || two_i % 2) LLMK_FAIL(LLMK_ERR_SHAPE, "moe_act_and_mul: bad shape");
    if (ids_bytes != 4 && ids_bytes != 8) LLMK_FAIL(LLMK_ERR_DTYPE, "moe_act_and_mul: ids_bytes %d", ids_bytes);
    if (act != 0 && act != 1) LLMK_FAIL(LLMK_ERR_DTYPE, "moe_act_and_mul: act %d", act);
    if (M == 0 || two_i == 0) return LLMK_OK;
    if (!gateup || !out || !reorder_topk_ids) LLMK_FAIL(LLMK_ERR_ARG, "moe_act_and_mul: null pointer");
    const int in_al = in_dtype == LLMK_F32 ? 31 : 15, out_al = out_dtype == LLMK_F32 ? 31 : 15;
    if ((two_i / 2) % 8 == 0 && ((uintptr_t)gateup & in_al) == 0 && ((uintptr_t)out & out_al) == 0) {
        LLMK_DISPATCH_FLOAT(in_dtype, IDT, LLMK_DISPATCH_FLOAT(out_dtype, ODT,
            (act_and_mul_vec_kernel<IDT, ODT><<<(unsigned)M, 256, 0, (hipStream_t)stream>>>(gateup, out, reorder_topk_ids, ids_bytes, scales, start_expert, end_expert, two_i, act))));
        LLMK_CHECK_LAUNCH("moe_act_and_mul");
        return LLMK_OK;
    }
    LLMK_DISPATCH_FLOAT(in_dtype, IDT, LLMK_DISPATCH_FLOAT(out_dtype, ODT,
        (act_and_mul_kernel<IDT, ODT><<<(unsigned)M, 256, 0, (hipStream_t)stream>>>(gateup, out, reorder_topk_ids, ids_bytes, scales, start_expert, end_expert, two_i, act))));
    LLMK_CHECK_LAUNCH("moe_act_and_mul");
    return LLMK_OK;
}

extern "C" int llmk_moe_act_and_mul_quant(const void* gateup, int in_dtype, void* q_out, void* s_out, int kind,
                                          int round_mode, const void* reorder_topk_ids, int ids_bytes,
                                          const float* scales, int start_expert, int end_expert, int64_t M,
                                          int64_t two_i, int act, void* stream) {
    if (M < 0 || two_i < 0 || two_i % 256) LLMK_FAIL(LLMK_ERR_SHAPE, "moe_act_and_mul_quant: 2I=%lld must be a multiple of 256", (long long)two_i);
    if (ids_bytes != 4 && ids_bytes != 8) LLMK_FAIL(LLMK_ERR_DTYPE, "moe_act_and_mul_quant: ids_bytes %d", ids_bytes);
    if (act != 0 && act != 1) LLMK_FAIL(LLMK_ERR_DTYPE, "moe_act_and_mul_quant: act %d", act);
    if (kind != LLMK_KIND_I8 && kind != LLMK_KIND_FP8) LLMK_FAIL(LLMK_ERR_DTYPE, "moe_act_and_mul_quant: kind %d", kind);
    if (round_mode != LLMK_ROUND_HALF_AWAY && round_mode != LLMK_ROUND_HALF_UP) LLMK_FAIL(LLMK_ERR_DTYPE, "moe_act_and_mul_quant: round_mode %d", round_mode);
    if (in_dtype == LLMK_F32) LLMK_FAIL(LLMK_ERR_DTYPE, "moe_act_and_mul_quant: fp16 / bf16 inputs only");
    if (M == 0 || two_i == 0) return LLMK_OK;
    if (!gateup || !q_out || !s_out || !reorder_topk_ids) LLMK_FAIL(LLMK_ERR_ARG, "moe_act_and_mul_quant: null pointer");
    if (((uintptr_t)gateup | (uintptr_t)q_out) & 15) LLMK_FAIL(LLMK_ERR_ARG, "moe_act_and_mul_quant: buffers must be 16-byte aligned");
    const int64_t threads = M * (two_i / 256) * 16;
    const unsigned grid = (unsigned)cdiv64(threads, 256 * AMQ_UNROLL);
    LLMK_DISPATCH_FLOAT(in_dtype, IDT, {
        if (kind == LLMK_KIND_FP8) act_mul_quant_kernel<IDT, true><<<grid, 256, 0, (hipStream_t)stream>>>(gateup, q_out, s_out, reorder_topk_ids, ids_bytes, scales, start_expert, end_expert, M, two_i, act, round_mode);
        else act_mul_quant_kernel<IDT, false><<<grid, 256, 0, (hipStream_t)stream>>>(gateup, q_out, s_out, reorder_topk_ids, ids_bytes, scales, start_expert, end_expert, M, two_i, act, round_mode);
    });
    LLMK_CHECK_LAUNCH("moe_act_and_mul_quant");
    return LLMK_OK;
}

extern "C" int llmk_moe_pre_reorder_quant(const void* x, int x_dtype, void* q_out, void* s_out, int kind, int round_mode,
                                          const int32_t* src2dst, const void* topk_ids, int ids_bytes,
                                          const float* a1_scales, int start_expert, int end_expert, int topk,
                                          int64_t T, int64_t hidden, void* stream) {
    if (T < 0 || hidden < 0 || topk < 0 || hidden % 128) LLMK_FAIL(LLMK_ERR_SHAPE, "moe_pre_reorder_quant: hidden=%lld must be a multiple of 128", (long long)hidden);
    if (ids_bytes != 4 && ids_bytes != 8) LLMK_FAIL(LLMK_ERR_DTYPE, "moe_pre_reorder_quant: ids_bytes %d", ids_bytes);
    if (kind != LLMK_KIND_I8 && kind != LLMK_KIND_FP8) LLMK_FAIL(LLMK_ERR_DTYPE, "moe_pre_reorder_quant: kind %d", kind);
    if (round_mode != LLMK_ROUND_HALF_AWAY && round_mode != LLMK_ROUND_HALF_UP) LLMK_FAIL(LLMK_ERR_DTYPE, "moe_pre_reorder_quant: round_mode %d", round_mode);
    if (x_dtype == LLMK_F32) LLMK_FAIL(LLMK_ERR_DTYPE, "moe_pre_reorder_quant: fp16 / bf16 inputs only");
    if (T == 0 || hidden == 0 || topk == 0) return LLMK_OK;
    if (!x || !q_out || !s_out || !src2dst || !topk_ids) LLMK_FAIL(LLMK_ERR_ARG, "moe_pre_reorder_quant: null pointer");
    if (((uintptr_t)x | (uintptr_t)q_out) & 15) LLMK_FAIL(LLMK_ERR_ARG, "moe_pre_reorder_quant: buffers must be 16-byte aligned");
    const int64_t threads = T * (hidden / 128) * 16;
    const unsigned grid = (unsigned)cdiv64(threads, 256 * PRQ_UNROLL);
    LLMK_DISPATCH_FLOAT(x_dtype, IDT, {
        if (kind == LLMK_KIND_FP8) pre_reorder_quant_kernel<IDT, true><<<grid, 256, 0, (hipStream_t)stream>>>(x, q_out, s_out, src2dst, topk_ids, ids_bytes, a1_scales, start_expert, end_expert, topk, T, hidden, round_mode);
        else pre_reorder_quant_kernel<IDT, false><<<grid, 256, 0, (hipStream_t)stream>>>(x, q_out, s_out, src2dst, topk_ids, ids_bytes, a1_scales, start_expert, end_expert, topk, T, hidden, round_mode);
    });
    LLMK_CHECK_LAUNCH("moe_pre_reorder_quant");
    return LLMK_OK;
}

extern "C" int llmk_moe_post_reorder(const void* down_out, void* out, int dtype, const int32_t* src2dst,
                                     const void* topk_ids, int ids_bytes, const void* topk_weights, int w_dtype,
                                     int start_expert, int end_expert, int topk, int64_t T, int64_t hidden,
                                     void* stream) {
    if (T < 0 || hidden < 0 || topk < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "moe_post_reorder: negative size");
    if (ids_bytes != 4 && ids_bytes != 8) LLMK_FAIL(LLMK_ERR_DTYPE, "moe_post_reorder: ids_bytes %d", ids_bytes);
    if (T == 0 || hidden == 0) return LLMK_OK;
    if (!down_out || !out || !src2dst || !topk_ids || !topk_weights) LLMK_FAIL(LLMK_ERR_ARG, "moe_post_reorder: null pointer");
    LLMK_DISPATCH_FLOAT(dtype, DT, LLMK_DISPATCH_FLOAT(w_dtype, WDT,
        (post_reorder_kernel<DT, WDT><<<(unsigned)T, 256, 0, (hipStream_t)stream>>>(down_out, out, src2dst, topk_ids, ids_bytes, topk_weights, start_expert, end_expert, topk, hidden))));
    LLMK_CHECK_LAUNCH("moe_post_reorder");
    return LLMK_OK;
}

extern "C" int llmk_grouped_gemm(const void* a, const void* b, void* c, int kind, int c_dtype, int E, int64_t M,
                                 int64_t N, int64_t K, const int64_t* seg_indptr, const int64_t* weight_indices,
                                 const void* scale_a, const void* scale_b, int s_dtype, void* workspace,
                                 int64_t workspace_bytes, void* stream) {
    if (M < 0 || N < 0 || K < 0 || E < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "grouped_gemm: negative dimension");
    if (c_dtype != LLMK_F32 && c_dtype != LLMK_F16 && c_dtype != LLMK_BF16) LLMK_FAIL(LLMK_ERR_DTYPE, "grouped_gemm: c_dtype %d", c_dtype);
    const bool scaled = (kind == LLMK_KIND_I8 || kind == LLMK_KIND_FP8);
    const int kstep = scaled ? 128 : 64;
    if (K % kstep) LLMK_FAIL(LLMK_ERR_SHAPE, "grouped_gemm: K=%lld must be a multiple of %d for this element kind", (long long)K, kstep);
    if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) LLMK_FAIL(LLMK_ERR_SHAPE, "grouped_gemm: dimension exceeds int32");
    if (M == 0 || N == 0 || E == 0) return LLMK_OK;
    if (!a || !b || !c || !seg_indptr) LLMK_FAIL(LLMK_ERR_ARG, "grouped_gemm: null pointer");
    if (scaled && (!scale_a || !scale_b)) LLMK_FAIL(LLMK_ERR_ARG, "grouped_gemm: block scales required for int8 / fp8 operands");
    if ((((uintptr_t)a) | ((uintptr_t)b)) & 15) LLMK_FAIL(LLMK_ERR_ARG, "grouped_gemm: operands must be 16-byte aligned");
    DirectArgs p{};
    p.a = (const uint8_t*)a; p.b = (const uint8_t*)b; p.c = c; p.a_s = scale_a; p.b_s = scale_b;
    p.seg_indptr = seg_indptr; p.weight_indices = weight_indices;
    p.c_dtype = c_dtype; p.s_dtype = s_dtype; p.M = (int)M; p.N = (int)N; p.K = (int)K; p.E = E;
    hipStream_t st = (hipStream_t)stream;
    // Tile kernels when the average segment is longer than 64 rows, and from two rows per expert up when the
    // expert weights are large (measured on 8 experts of 4096 x 14336, whole forward, tile vs weight-streaming
    // kernel: 256 vs 158 us at 1 token, 295 vs 289 us at 8, 344 vs 374 us at 16, 362 vs 481 us at 64).
    // Also with several short segments: the weight-streaming kernel spreads its workgroups over the row tiles and
    // leaves each of them a fraction of the column workgroups (measured: tile kernels faster from six row tiles).
    const bool big = M > 64 * (int64_t)E || (M > 2 * (int64_t)E && N * K >= ((int64_t)20 << 20)) ||
                     grouped_row_tiles((int)M, E, 16) >= 6;
    if (big && kind == LLMK_KIND_I8) return launch_big<K_I8_BLOCK, true>(p, workspace, workspace_bytes, st, "grouped_gemm(i8, tiled)");
    if (big && kind == LLMK_KIND_FP8) return launch_big<K_FP8_BLOCK, true>(p, workspace, workspace_bytes, st, "grouped_gemm(fp8, tiled)");
    if (big && kind == LLMK_KIND_F16 && dma_eligible(p, 2)) return launch_big_half<K_F16, true>(p, st, "grouped_gemm(f16, tiled)");
    if (big && kind == LLMK_KIND_BF16 && dma_eligible(p, 2)) return launch_big_half<K_BF16, true>(p, st, "grouped_gemm(bf16, tiled)");
    switch (kind) {
        case LLMK_KIND_I8:   return launch_direct<K_I8_BLOCK, true>(p, (int)M, st, "grouped_gemm(i8)");
        case LLMK_KIND_FP8:  return launch_direct<K_FP8_BLOCK, true>(p, (int)M, st, "grouped_gemm(fp8)");
        case LLMK_KIND_F16:  return launch_direct<K_F16, true>(p, (int)M, st, "grouped_gemm(f16)");
        case LLMK_KIND_BF16: return launch_direct<K_BF16, true>(p, (int)M, st, "grouped_gemm(bf16)");
        default: LLMK_FAIL(LLMK_ERR_DTYPE, "grouped_gemm: kind %d", kind);
    }
}

// which tile kernel the gated-activation form would run on for this shape: 8 / 4 = tile rows per wave of the 256-column
// kernel, 0 = none (the caller runs the grouped GEMM and the activation kernel instead)
static int swiglu_tile_rows(int kind, const DirectArgs& p) {
    if (p.N % 256 || p.K % 128 || !dma_eligible(p)) return 0;
    const bool big = p.M > 64 * (int64_t)p.E || (p.M > 2 * (int64_t)p.E && (int64_t)p.N * p.K >= ((int64_t)20 << 20)) ||
                     grouped_row_tiles(p.M, p.E, 16) >= 6;
    if (!big) return 0;
    const int choice = kind == LLMK_KIND_FP8 ? dma_tile_choice<K_FP8_BLOCK, true>(p) : dma_tile_choice<K_I8_BLOCK, true>(p);
    return choice == 8 ? 8 : (choice == 9 ? 4 : 0);
}

extern "C" int llmk_grouped_gemm_swiglu_quant_fused(int kind, int E, int64_t M, int64_t two_i, int64_t K) {
    if ((kind != LLMK_KIND_I8 && kind != LLMK_KIND_FP8) || E <= 0 || M <= 0 || two_i <= 0 || K <= 0) return 0;
    if (M > 0x7fffffff || two_i > 0x7fffffff || K > 0x7fffffff) return 0;
    DirectArgs p{};
    p.M = (int)M; p.N = (int)two_i; p.K = (int)K; p.E = E;
    return swiglu_tile_rows(kind, p) ? 1 : 0;
}

extern "C" int llmk_grouped_gemm_swiglu_quant(const void* a, const void* b, void* q_out, void* s_out, int kind, int mid_dtype,
                                              int round_mode, int E, int64_t M, int64_t two_i, int64_t K,
                                              const int64_t* seg_indptr, const int64_t* weight_indices, const void* scale_a,
                                              const void* scale_b, int s_dtype, int act, void* workspace,
                                              int64_t workspace_bytes, void* stream) {
    if (M < 0 || two_i < 0 || K < 0 || E < 0) LLMK_FAIL(LLMK_ERR_SHAPE, "grouped_gemm_swiglu_quant: negative dimension");
    if (kind != LLMK_KIND_I8 && kind != LLMK_KIND_FP8) LLMK_FAIL(LLMK_ERR_DTYPE, "grouped_gemm_swiglu_quant: kind %d", kind);
    if (mid_dtype != LLMK_F16 && mid_dtype != LLMK_BF16) LLMK_FAIL(LLMK_ERR_DTYPE, "grouped_gemm_swiglu_quant: mid_dtype %d (the dtype the gate / up sums are rounded to: fp16 or bf16)", mid_dtype);
    if (act != 0 && act != 1) LLMK_FAIL(LLMK_ERR_ARG, "grouped_gemm_swiglu_quant: act %d", act);
    if (round_mode != LLMK_ROUND_HALF_AWAY && round_mode != LLMK_ROUND_HALF_UP) LLMK_FAIL(LLMK_ERR_DTYPE, "grouped_gemm_swiglu_quant: round_mode %d", round_mode);
    if (M > 0x7fffffff || two_i > 0x7fffffff || K > 0x7fffffff) LLMK_FAIL(LLMK_ERR_SHAPE, "grouped_gemm_swiglu_quant: dimension exceeds int32");
    if (M == 0 || two_i == 0 || E == 0) return LLMK_OK;
    if (!a || !b || !q_out || !s_out || !seg_indptr || !scale_a || !scale_b) LLMK_FAIL(LLMK_ERR_ARG, "grouped_gemm_swiglu_quant: null pointer");
    if ((((uintptr_t)a) | ((uintptr_t)b)) & 15 || ((uintptr_t)q_out & 7)) LLMK_FAIL(LLMK_ERR_ARG, "grouped_gemm_swiglu_quant: operands must be 16-byte aligned, q_out 8-byte aligned");
    DirectArgs p{};
    p.a = (const uint8_t*)a; p.b = (const uint8_t*)b; p.c = q_out; p.q_scale = s_out; p.a_s = scale_a; p.b_s = scale_b;
    p.seg_indptr = seg_indptr; p.weight_indices = weight_indices;
    p.c_dtype = mid_dtype; p.s_dtype = s_dtype; p.M = (int)M; p.N = (int)two_i; p.K = (int)K; p.E = E;
    p.act = act; p.round_mode = round_mode;
    const int rows = swiglu_tile_rows(kind, p);
    if (!rows) LLMK_FAIL(LLMK_ERR_SHAPE, "grouped_gemm_swiglu_quant: shape E=%d M=%lld 2I=%lld K=%lld is not one the fused kernel takes (ask llmk_grouped_gemm_swiglu_quant_fused first)", E, (long long)M, (long long)two_i, (long long)K);
    hipStream_t st = (hipStream_t)stream;
    if (s_dtype != LLMK_F32) {
        // 16-bit activation scales are widened first, as in front of the plain kernel
        const int64_t n = M * (K >> 7);
        if (!workspace || workspace_bytes < n * 4 || ((uintptr_t)workspace & 15)) LLMK_FAIL(LLMK_ERR_ARG, "grouped_gemm_swiglu_quant: 16-bit activation scales need %lld bytes of workspace", (long long)(n * 4));
        const unsigned blocks = (unsigned)cdiv64(n, 256);
        if (s_dtype == LLMK_F16) scales_to_f32_kernel<LLMK_F16><<<blocks, 256, 0, st>>>(scale_a, (float*)workspace, n);
        else if (s_dtype == LLMK_BF16) scales_to_f32_kernel<LLMK_BF16><<<blocks, 256, 0, st>>>(scale_a, (float*)workspace, n);
        else LLMK_FAIL(LLMK_ERR_DTYPE, "grouped_gemm_swiglu_quant: s_dtype %d", s_dtype);
        LLMK_CHECK_LAUNCH("grouped_gemm_swiglu_quant(scales)");
        p.a_s = workspace;
    }
    if (kind == LLMK_KIND_FP8)
        return rows == 8 ? launch_wide_swiglu<K_FP8_BLOCK, 8>(p, st, "grouped_gemm_swiglu_quant(fp8)") : launch_wide_swiglu<K_FP8_BLOCK, 4>(p, st, "grouped_gemm_swiglu_quant(fp8)");
    return rows == 8 ? launch_wide_swiglu<K_I8_BLOCK, 8>(p, st, "grouped_gemm_swiglu_quant(i8)") : launch_wide_swiglu<K_I8_BLOCK, 4>(p, st, "grouped_gemm_swiglu_quant(i8)");
}
