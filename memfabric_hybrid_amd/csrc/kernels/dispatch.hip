/*
 * Expert-major permutation with fused per-token quantisation.
 *
 * One workgroup owns one source token: the row is read from HBM once (two
 * 16-byte loads per lane per 16 elements), reduced to its absmax (whole row
 * for int8, per 128 columns for e4m3), quantised once in registers and then
 * stored to each of the token's K destination rows with 16-byte stores, so
 * HBM traffic is the algorithmic minimum of one read and K quantised writes.
 * With per-expert smooth scales the quantised row differs per pick and is
 * recomputed per pick from the registers.
 */
#include "zbal_device.h"
#include "zbal_hip_kernels.h"

int32_t zbalhip_layout_ranges_internal(const int32_t *idx, int64_t tokens, int64_t experts, int64_t topk,
                                       const uint8_t *active_mask, int32_t *send_token_idx, int32_t *hist, int nblk,
                                       int tokens_per_block, hipStream_t st);

int32_t zbalhip_ll_counts_internal(const int32_t *const *ids, int ranks, int me, int64_t tokens, int64_t topk,
                                   int64_t experts, int32_t token_nums_type, int32_t *all_counts, int32_t *ep_recv_counts,
                                   int64_t *expert_token_nums, hipStream_t st);

int32_t zbalhip_layout_fused_internal(const int32_t *idx, int64_t tokens, int64_t experts, int64_t topk,
                                      int32_t token_nums_type, const uint8_t *active_mask, int32_t *send_token_idx,
                                      int32_t *incl_i32, int32_t *row_off, int64_t *counts_i64, int64_t *nums_typed,
                                      hipStream_t st);

namespace {

constexpr int kThreads = 256;
constexpr int kElemsPerLane = 16;

enum { QM_COPY = 0, QM_INT8_EPS = 1, QM_FP8 = 2, QM_INT8_NOEPS = 3 };

/*
 * Where the rows go. Expert e belongs to rank e / e_loc, whose receive window is dest[that rank] (and scale[that
 * rank] for the quantisation scales); on one GPU the windows are local allocations, over xGMI they would be
 * mapped peer memory, the kernel is the same. Offsets are looked up as base[e * ranks + my_rank]: the slot of
 * this sender in the receiver's expert-major, then source-rank order (reference
 * zbal_kernel_notify_dispatch.h:356-378, zbal_kernel_dispatch_normal.h:528-533). rows_cap is the number of rows
 * each window holds; a pick that would land past it is dropped rather than written out of bounds.
 */
struct PeerRows {
    uint8_t *dest[ZBALHIP_MAX_REDUCE_PEERS];
    float *scale[ZBALHIP_MAX_REDUCE_PEERS];
    int ranks, my_rank, e_loc;
    int64_t rows_cap;
};

__device__ __forceinline__ int64_t pick_row(const int32_t *__restrict__ base, int base_inclusive, const PeerRows &pr, int e,
                                            int32_t rank_in_expert)
{
    /* running sums start anew with every destination rank's block of `experts` entries (low-latency counts) */
    const int slot = e * pr.ranks + pr.my_rank;
    const int32_t b = base_inclusive ? (slot % (pr.e_loc * pr.ranks) == 0 ? 0 : base[slot - 1]) : base[slot];
    const int64_t row = (int64_t)b + rank_in_expert;
    return row < pr.rows_cap ? row : -1;
}

/*
 * Small batches: the permute kernel works the layout out itself. With at most kInlineMaxPicks picks in all, every
 * workgroup counts the whole index array (a few KiB that sit in L2) into an LDS histogram, scans it into the
 * exclusive row offsets and counts the same-expert picks that precede each of its own token's picks: no layout
 * launch in front of the permute, and no dependency between workgroups. Workgroup 0 also writes the layout's
 * outputs (any of them may be null); every workgroup writes its token's expand_idx entries.
 */
constexpr int kInlineMaxPicks = 4096;
constexpr int kInlineMaxTopk = 32;
constexpr int kInlineMaxExperts = 1024;

struct InlineLayout {
    const uint8_t *active_mask;   /* optional: only the first sum(mask) tokens are routed */
    int tokens, token_nums_type;
    int32_t *expand_idx;          /* [T, K] */
    int32_t *incl_i32;            /* [E] running sums */
    int32_t *row_off;             /* [E + 1] exclusive offsets */
    int64_t *counts_i64;          /* [E] */
    int64_t *nums_typed;          /* [E] counts (type 1) or running sums (type 0) */
};

/*
 * On return s_off[e] = rows before expert e, s_e[k] / s_rk[k] = expert and rank of pick k of token t. Negative ranks are
 * not routed: -1 an invalid expert id, -2 a token past the active ones (the combine leaves such a token's row alone).
 */
__device__ __forceinline__ void inline_layout(const int32_t *__restrict__ idx, int t, int topk, int experts,
                                              const InlineLayout &il, int32_t *s_off, int32_t *s_e, int32_t *s_rk, int32_t *s_tmp)
{
    const int tid = threadIdx.x, nthr = blockDim.x, lane = tid & 63, wave = tid >> 6;
    for (int e = tid; e < experts; e += nthr) s_off[e] = 0;
    /* the first four indices of this lane are requested together with the token's own picks (no mask: every token counts) */
    int first[4] = {-1, -1, -1, -1};
    if (il.active_mask == nullptr) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (tid + u * nthr < il.tokens * topk) first[u] = idx[tid + u * nthr];
    }
    if (tid < topk) {
        s_e[tid] = idx[(int64_t)t * topk + tid];
        s_rk[tid] = 0;
    }
    if (tid == 0) s_tmp[0] = 0;
    __syncthreads();
    int active = il.tokens;
    if (il.active_mask) {
        int part = 0;
        for (int tt = tid; tt < il.tokens; tt += nthr) part += il.active_mask[tt] != 0;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) part += __shfl_xor(part, off, 64);
        if (lane == 0 && part) atomicAdd(&s_tmp[0], part);
        __syncthreads();
        active = s_tmp[0];
    }
    const int n = active * topk, mine0 = t * topk;
    /* four indices per lane are requested before the first is used: the loop is a chain of round trips to L2 otherwise */
    for (int i0 = tid; i0 < n; i0 += 4 * nthr) {
        int ev[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (i0 == tid && il.active_mask == nullptr) ev[u] = first[u];
            else ev[u] = i0 + u * nthr < n ? idx[i0 + u * nthr] : -1;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int e = ev[u], i = i0 + u * nthr;
            if (e < 0 || e >= experts) continue;
            atomicAdd(&s_off[e], 1);
            if (i < mine0 + topk)
                for (int k = 0; k < topk; ++k)
                    if (e == s_e[k] && i < mine0 + k) atomicAdd(&s_rk[k], 1);
        }
    }
    __syncthreads();
    /* exclusive scan of the counts, in place: a thread owns `chunk` consecutive experts */
    const int chunk = (experts + nthr - 1) / nthr, b0 = tid * chunk;
    int32_t sum = 0;
    for (int j = 0; j < chunk; ++j)
        if (b0 + j < experts) sum += s_off[b0 + j];
    int32_t incl = sum;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int32_t o = __shfl_up(incl, off, 64);
        if (lane >= off) incl += o;
    }
    if (lane == 63) s_tmp[1 + wave] = incl;
    __syncthreads();
    for (int w = 0; w < wave; ++w) incl += s_tmp[1 + w];
    int32_t run = incl - sum;
    const bool writer = blockIdx.x == 0;
    for (int j = 0; j < chunk; ++j) {
        const int e = b0 + j;
        if (e >= experts) break;
        const int32_t c = s_off[e];
        s_off[e] = run;
        if (writer) {
            if (il.row_off) il.row_off[e] = run;
            if (il.incl_i32) il.incl_i32[e] = run + c;
            if (il.counts_i64) il.counts_i64[e] = c;
            if (il.nums_typed) il.nums_typed[e] = il.token_nums_type == 0 ? (int64_t)(run + c) : (int64_t)c;
        }
        run += c;
        if (writer && e == experts - 1 && il.row_off) il.row_off[experts] = run;
    }
    if (tid < topk) {
        const int e = s_e[tid];
        const int32_t rk = t >= active ? -2 : ((e >= 0 && e < experts) ? s_rk[tid] : -1);
        s_rk[tid] = rk;
        il.expand_idx[(int64_t)t * topk + tid] = rk;
    }
    __syncthreads();
}

/*
 * Large batches: the layout launch in front of the permute only ranks the picks within token ranges and leaves one
 * histogram per range (layout_ranges_kernel); what is left of the layout -- how many picks of an expert the ranges
 * before a token's own hold, and the experts' first rows -- every permute workgroup works out for itself from that
 * small table while its row is on its way from HBM: no workgroup of either launch waits for another, and the layout
 * launch is a third of what it was. Workgroup 0 also writes the offsets and counts the stages after the permute read.
 */
constexpr int kTableMaxEntries = 2048;        /* ranges x experts */
constexpr int kTableMaxExperts = 256;         /* one expert per thread in the scan */

struct RangeTable {
    const int32_t *hist;          /* [ranges][experts] */
    int ranges, tokens_per_range;
    int32_t *expand_idx;          /* [T, K]: in, the rank within the range; out, the rank within the expert */
    int32_t *row_off;             /* [E + 1] */
    int64_t *counts_i64;          /* [E] */
};

constexpr int kTablePerThread = kTableMaxEntries / kThreads;

/* the table's entries tid, tid + kThreads, ...: requested before the row, so that they arrive first (a wave's loads return in order) */
__device__ __forceinline__ void table_request(const RangeTable &rt, int experts, int32_t (&tabv)[kTablePerThread])
{
    const int n = rt.ranges * experts;
#pragma unroll
    for (int j = 0; j < kTablePerThread; ++j) {
        const int i = j * kThreads + (int)threadIdx.x;
        tabv[j] = i < n ? rt.hist[i] : 0;
    }
}

/* On return s_first[e] = first row of expert e, s_before[e] = picks of expert e in the ranges before `range`. */
__device__ __forceinline__ void table_layout(const RangeTable &rt, const int32_t (&tabv)[kTablePerThread], int range,
                                             int experts, bool writer, int32_t *s_tab, int32_t *s_first, int32_t *s_before,
                                             int32_t *s_tmp)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
#pragma unroll
    for (int j = 0; j < kTablePerThread; ++j) s_tab[j * kThreads + tid] = tabv[j];
    __syncthreads();
    int32_t c = 0;
    if (tid < experts) {
        int32_t bef = 0;
        for (int r = 0; r < rt.ranges; ++r) {
            const int32_t v = s_tab[r * experts + tid];
            c += v;
            if (r < range) bef += v;
        }
        s_before[tid] = bef;
    }
    int32_t incl = c;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int32_t o = __shfl_up(incl, off, 64);
        if (lane >= off) incl += o;
    }
    if (lane == 63) s_tmp[wave] = incl;
    __syncthreads();
    for (int w = 0; w < wave; ++w) incl += s_tmp[w];
    if (tid < experts) {
        s_first[tid] = incl - c;
        if (writer) {
            rt.row_off[tid] = incl - c;
            if (rt.counts_i64) rt.counts_i64[tid] = c;
            if (tid == experts - 1) rt.row_off[experts] = incl;
        }
    }
    __syncthreads();
}

/* 16 consecutive 16-bit elements (two 16-byte loads) as fp32 */
template <int XDT> __device__ __forceinline__ void cvt16(const u32x4 &a, const u32x4 &b, float (&v)[16])
{
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = zb_half_to_f32<XDT>(a[i] & 0xffffu);
        v[2 * i + 1] = zb_half_to_f32<XDT>(a[i] >> 16);
        v[8 + 2 * i] = zb_half_to_f32<XDT>(b[i] & 0xffffu);
        v[8 + 2 * i + 1] = zb_half_to_f32<XDT>(b[i] >> 16);
    }
}

__device__ __forceinline__ u32x4 pack16_i8(const float (&v)[16], float s)
{
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        uint32_t w = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) w |= ((uint32_t)zb_rint_i8(v[4 * i + j] * s) & 0xffu) << (8 * j);
        o[i] = w;
    }
    return o;
}

__device__ __forceinline__ u32x4 pack16_e4m3(const float (&v)[16], float mult)
{
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t lo = zb_cvt_pk_e4m3(v[4 * i] * mult, v[4 * i + 1] * mult);
        const uint32_t hi = zb_cvt_pk_e4m3(v[4 * i + 2] * mult, v[4 * i + 3] * mult);
        o[i] = lo | (hi << 16);
    }
    return o;
}

/*
 * SLOTS = ceil(H / 16 / blockDim): 16-element segments each lane keeps in registers.
 * QM: quant flavour. SMOOTH: per-expert fp32 multipliers [E,H] (int8 only).
 */
enum { LM_GIVEN = 0, LM_INLINE = 1, LM_TABLE = 2 };     /* where ranks and offsets come from */

template <int XDT, int QM, int SLOTS, bool SMOOTH, int LM>
__global__ void __launch_bounds__(kThreads)
permute_quant_kernel(const uint16_t *__restrict__ x, const int32_t *__restrict__ topk_idx,
                     const int32_t *__restrict__ rank_in_expert, const int32_t *__restrict__ base, int base_inclusive,
                     const float *__restrict__ smooth, int hidden, int topk, int experts, PeerRows pr, InlineLayout il,
                     RangeTable rt, uint32_t *__restrict__ clear_words, int64_t clear_count)
{
    constexpr bool INLINE = LM == LM_INLINE, TABLE = LM == LM_TABLE;
    __shared__ float red[kThreads / 64];
    __shared__ int32_t s_off[INLINE ? kInlineMaxExperts : (TABLE ? kTableMaxExperts : 1)];
    __shared__ int32_t s_before[TABLE ? kTableMaxExperts : 1], s_tab[TABLE ? kTableMaxEntries : 1];
    __shared__ int32_t s_e[kInlineMaxTopk], s_rk[INLINE ? kInlineMaxTopk : 1], s_tmp[8];
    __shared__ int64_t s_row[kInlineMaxTopk];
    const int t = blockIdx.x;
    const int nseg = hidden / kElemsPerLane;
    /* words the next stage wants at zero (the row maxima the int modes' first GEMM accumulates into) */
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < clear_count; i += (int64_t)gridDim.x * blockDim.x)
        clear_words[i] = 0u;
    /*
     * Where the token's picks go is worked out by one lane per pick while the row is on its way (the picks' index,
     * rank and offset loads depend on each other: done pick after pick inside the store loop they cost topk round
     * trips to L2 per workgroup): index and rank are requested before the row, the offset after it.
     * s_row[k] < 0: pick k is not routed.
     */
    const bool picker = !INLINE && threadIdx.x < topk && threadIdx.x < kInlineMaxTopk;
    int pick_e = -1, pick_rk = -1;
    if (picker) {
        pick_e = topk_idx[(int64_t)t * topk + threadIdx.x];
        pick_rk = TABLE ? rt.expand_idx[(int64_t)t * topk + threadIdx.x] : rank_in_expert[(int64_t)t * topk + threadIdx.x];
    }
    int32_t tabv[TABLE ? kTablePerThread : 1];
    if constexpr (TABLE) table_request(rt, experts, tabv);
    /* the row is requested here (streamed: it is read once) and first used after the picks are resolved: the two latencies overlap */
    u32x4 raw[SLOTS][2];
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
        const int seg = s * blockDim.x + threadIdx.x;
        raw[s][0] = raw[s][1] = u32x4{0u, 0u, 0u, 0u};
        if (seg < nseg) {
            raw[s][0] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x + (int64_t)t * hidden + (int64_t)seg * 16));
            raw[s][1] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x + (int64_t)t * hidden + (int64_t)seg * 16 + 8));
        }
    }
    if constexpr (INLINE) {
        inline_layout(topk_idx, t, topk, experts, il, s_off, s_e, s_rk, s_tmp);
        if (threadIdx.x < topk) {
            const int32_t rk = s_rk[threadIdx.x];
            const int64_t row = rk < 0 ? -1 : (int64_t)s_off[s_e[threadIdx.x]] + rk;
            s_row[threadIdx.x] = row < pr.rows_cap ? row : -1;
        }
    } else if constexpr (TABLE) {
        table_layout(rt, tabv, t / rt.tokens_per_range, experts, t == 0, s_tab, s_off, s_before, s_tmp);
        if (picker) {
            int64_t row = -1;
            if (pick_e >= 0 && pick_e < experts && pick_rk >= 0) {       /* rank < 0: the layout masked this token out */
                const int32_t rk = s_before[pick_e] + pick_rk;
                rt.expand_idx[(int64_t)t * topk + threadIdx.x] = rk;       /* the rank within the expert: what the combine reads */
                row = (int64_t)s_off[pick_e] + rk;
                if (row >= pr.rows_cap) row = -1;
            }
            s_e[threadIdx.x] = pick_e;
            s_row[threadIdx.x] = row;
        }
    } else if (picker) {
        const bool routed = pick_e >= 0 && pick_e < experts && pick_rk >= 0;      /* rank < 0: the layout masked this token out */
        s_e[threadIdx.x] = pick_e;
        s_row[threadIdx.x] = routed ? pick_row(base, base_inclusive, pr, pick_e, pick_rk) : -1;
    }
    __syncthreads();
    float v[SLOTS][16];
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) cvt16<XDT>(raw[s][0], raw[s][1], v[s]);
    /* destination of pick k of this token: false if the pick is not routed (uniform across the workgroup) */
    auto resolve = [&](int k, int &e, int64_t &row) __attribute__((always_inline)) -> bool {
        if (INLINE || k < kInlineMaxTopk) {
            e = s_e[k];
            row = s_row[k];
            return row >= 0;
        }
        e = topk_idx[(int64_t)t * topk + k];          /* more picks per token than the table holds: one by one */
        const int rk = rank_in_expert[(int64_t)t * topk + k];
        if (e < 0 || e >= experts || rk < 0) return false;
        row = pick_row(base, base_inclusive, pr, e, rk);
        return row >= 0;
    };

    if constexpr (QM == QM_FP8) {
        /* eight consecutive lanes share one 128-column block */
        u32x4 q[SLOTS];
        float sc[SLOTS];
#pragma unroll
        for (int s = 0; s < SLOTS; ++s) {
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(v[s][i]));
            amax = zb_group_max<3>(amax);
            amax = fmaxf(amax, 1e-4f);
            const float mult = 448.0f / amax;
            q[s] = pack16_e4m3(v[s], mult);
            sc[s] = amax * (1.0f / 448.0f);
        }
        const int nblk128 = hidden / 128;
        for (int k = 0; k < topk; ++k) {
            int e;
            int64_t row;
            if (!resolve(k, e, row)) continue;
            uint8_t *dest = pr.dest[e / pr.e_loc];
            float *dest_scale = pr.scale[e / pr.e_loc];
#pragma unroll
            for (int s = 0; s < SLOTS; ++s) {
                const int seg = s * blockDim.x + threadIdx.x;
                if (seg < nseg) {
                    *reinterpret_cast<u32x4 *>(dest + row * hidden + (int64_t)seg * 16) = q[s];
                    if ((seg & 7) == 0) dest_scale[row * nblk128 + (seg >> 3)] = sc[s];
                }
            }
        }
    } else if constexpr (!SMOOTH) {
        float amax = 0.0f;
#pragma unroll
        for (int s = 0; s < SLOTS; ++s)
#pragma unroll
            for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(v[s][i]));
        amax = zb_block_max(amax, red);
        float sq, stored;
        if (QM == QM_INT8_NOEPS && amax == 0.0f) { sq = 0.0f; stored = 0.0f; }
        else {
            sq = (QM == QM_INT8_EPS) ? 127.0f / (amax + 1e-12f) : 127.0f / amax;
            stored = 1.0f / sq;
        }
        u32x4 q[SLOTS];
#pragma unroll
        for (int s = 0; s < SLOTS; ++s) q[s] = pack16_i8(v[s], sq);
        for (int k = 0; k < topk; ++k) {
            int e;
            int64_t row;
            if (!resolve(k, e, row)) continue;
            uint8_t *dest = pr.dest[e / pr.e_loc];
#pragma unroll
            for (int s = 0; s < SLOTS; ++s) {
                const int seg = s * blockDim.x + threadIdx.x;
                if (seg < nseg)
                    *reinterpret_cast<u32x4 *>(dest + row * hidden + (int64_t)seg * 16) = q[s];
            }
            if (threadIdx.x == 0) pr.scale[e / pr.e_loc][row] = stored;
        }
    } else {
        for (int k = 0; k < topk; ++k) {
            int e;
            int64_t row;
            if (!resolve(k, e, row)) continue; /* uniform across the block */
            uint8_t *dest = pr.dest[e / pr.e_loc];
            float sv[SLOTS][16];
            float amax = 0.0f;
#pragma unroll
            for (int s = 0; s < SLOTS; ++s) {
                const int seg = s * blockDim.x + threadIdx.x;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float m = (seg < nseg) ? smooth[(int64_t)e * hidden + seg * 16 + i] : 0.0f;
                    sv[s][i] = v[s][i] * m;
                    amax = fmaxf(amax, fabsf(sv[s][i]));
                }
            }
            amax = zb_block_max(amax, red);
            float sq, stored;
            if (amax == 0.0f) { sq = 0.0f; stored = 0.0f; }
            else { sq = 127.0f / amax; stored = 1.0f / sq; }
#pragma unroll
            for (int s = 0; s < SLOTS; ++s) {
                const int seg = s * blockDim.x + threadIdx.x;
                if (seg < nseg) {
                    const u32x4 q = pack16_i8(sv[s], sq);
                    *reinterpret_cast<u32x4 *>(dest + row * hidden + (int64_t)seg * 16) = q;
                }
            }
            if (threadIdx.x == 0) pr.scale[e / pr.e_loc][row] = stored;
        }
    }
}

/* plain row copy (no quantisation): 16-byte chunks of 8 elements */
__global__ void __launch_bounds__(kThreads)
permute_copy_kernel(const uint16_t *__restrict__ x, const int32_t *__restrict__ topk_idx,
                    const int32_t *__restrict__ rank_in_expert, const int32_t *__restrict__ base, int base_inclusive,
                    int hidden, int topk, int experts, PeerRows pr)
{
    const int t = blockIdx.x;
    const int nchunk = hidden / 8;
    for (int c0 = 0; c0 < nchunk; c0 += blockDim.x * 4) {
        u32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = c0 + u * blockDim.x + threadIdx.x;
            if (c < nchunk) v[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(x + (int64_t)t * hidden + (int64_t)c * 8));
        }
        for (int k = 0; k < topk; ++k) {
            const int e = topk_idx[(int64_t)t * topk + k];
            const int rk = rank_in_expert[(int64_t)t * topk + k];
            if (e < 0 || e >= experts || rk < 0) continue;      /* rk < 0: the layout masked this token out */
            const int64_t row = pick_row(base, base_inclusive, pr, e, rk);
            if (row < 0) continue;
            uint16_t *dest = reinterpret_cast<uint16_t *>(pr.dest[e / pr.e_loc]);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int c = c0 + u * blockDim.x + threadIdx.x;
                if (c < nchunk)
                    *reinterpret_cast<u32x4 *>(dest + row * hidden + (int64_t)c * 8) = v[u];
            }
        }
    }
}

/* what a permute launch does besides permuting: work out the layout itself (small batches), clear words for the next stage */
struct PermuteExtras {
    const InlineLayout *inline_layout;     /* null: ranks and offsets come from the layout launch */
    uint32_t *clear_words;
    int64_t clear_count;
    const RangeTable *range_table;         /* non-null: ranks within token ranges + the ranges' histograms (large batches) */
};

template <int XDT, int QM, bool SMOOTH>
int32_t launch_quant(const void *x, const int32_t *topk_idx, const int32_t *rank_in_expert, const int32_t *base,
                     int base_inclusive, const float *smooth, int64_t tokens, int64_t hidden, int64_t topk,
                     int64_t experts, const PeerRows &pr, const PermuteExtras &ex, hipStream_t st)
{
    const int nseg = (int)(hidden / kElemsPerLane);
    int threads = (nseg + 63) / 64 * 64;
    if (threads > kThreads) threads = kThreads;
    if (ex.range_table) threads = kThreads;       /* the table's scan gives every expert a thread */
    const int slots = (nseg + threads - 1) / threads;
    const InlineLayout il = ex.inline_layout ? *ex.inline_layout : InlineLayout{};
    const RangeTable rt = ex.range_table ? *ex.range_table : RangeTable{};
#define ZB_LAUNCH_I(S, LMV)                                                                                       \
    permute_quant_kernel<XDT, QM, S, SMOOTH, LMV><<<(unsigned)tokens, threads, 0, st>>>(                           \
        (const uint16_t *)x, topk_idx, rank_in_expert, base, base_inclusive, smooth, (int)hidden, (int)topk,       \
        (int)experts, pr, il, rt, ex.clear_words, ex.clear_count)
#define ZB_LAUNCH(S)                                                                                              \
    do {                                                                                                          \
        if (ex.inline_layout) ZB_LAUNCH_I(S, LM_INLINE);                                                          \
        else if (ex.range_table) ZB_LAUNCH_I(S, LM_TABLE);                                                        \
        else ZB_LAUNCH_I(S, LM_GIVEN);                                                                            \
    } while (0)
    if (slots <= 1) ZB_LAUNCH(1);
    else if (slots <= 2) ZB_LAUNCH(2);
    else if (slots <= 4) ZB_LAUNCH(4);
    else return ZBALHIP_INVALID;
#undef ZB_LAUNCH
#undef ZB_LAUNCH_I
    return zbalhip_check_launch();
}

} // namespace

/*
 * Shared by the three public launchers. quant: QM_* flavour. `base` is the
 * exclusive (or inclusive) per-expert row offset table on the device; `pr`
 * says where each rank's rows go.
 */
static int32_t permute_launch(const void *x, int32_t x_dtype, const int32_t *topk_idx, const int32_t *rank_in_expert,
                              const int32_t *base, int base_inclusive, const float *smooth, int64_t tokens,
                              int64_t hidden, int64_t topk, int64_t experts, int quant, const PeerRows &pr, hipStream_t st,
                              const PermuteExtras &ex = PermuteExtras{})
{
    if (x_dtype != ZDT_BF16 && x_dtype != ZDT_FP16) return ZBALHIP_INVALID;
    if (hidden <= 0 || hidden > 16 * kThreads * 4 || topk <= 0 || tokens < 0) return ZBALHIP_INVALID;
    if (tokens == 0) return ZBALHIP_OK;
    if (quant == QM_COPY) {
        if (hidden % 8 != 0 || ex.inline_layout || ex.clear_count) return ZBALHIP_INVALID;
        permute_copy_kernel<<<(unsigned)tokens, kThreads, 0, st>>>((const uint16_t *)x, topk_idx, rank_in_expert, base,
                                                                 base_inclusive, (int)hidden, (int)topk, (int)experts, pr);
        return zbalhip_check_launch();
    }
    if (hidden % 16 != 0 || (quant == QM_FP8 && hidden % 128 != 0)) return ZBALHIP_INVALID;
    const bool bf = (x_dtype == ZDT_BF16);
#define ZB_GO(QMV, SM)                                                                                               \
    return bf ? launch_quant<ZDT_BF16, QMV, SM>(x, topk_idx, rank_in_expert, base, base_inclusive, smooth, tokens,  \
                                                 hidden, topk, experts, pr, ex, st)                                  \
              : launch_quant<ZDT_FP16, QMV, SM>(x, topk_idx, rank_in_expert, base, base_inclusive, smooth, tokens,  \
                                                 hidden, topk, experts, pr, ex, st)
    if (quant == QM_FP8) { ZB_GO(QM_FP8, false); }
    if (quant == QM_INT8_EPS) { ZB_GO(QM_INT8_EPS, false); }
    if (quant == QM_INT8_NOEPS) {
        if (smooth) { ZB_GO(QM_INT8_NOEPS, true); }
        ZB_GO(QM_INT8_NOEPS, false);
    }
#undef ZB_GO
    return ZBALHIP_INVALID;
}

/* the permute kernel can work the layout out itself when the batch is this small (inline_layout above) */
static bool layout_fits_inline(int64_t tokens, int64_t topk, int64_t experts, int quant)
{
    return quant != QM_COPY && tokens > 0 && tokens * topk <= kInlineMaxPicks && topk <= kInlineMaxTopk &&
           experts <= kInlineMaxExperts;
}

/* one rank that owns every expert: all rows go to `dest` */
static PeerRows single_window(void *dest, float *dest_scale, int64_t experts, int64_t rows_cap)
{
    PeerRows pr = {};
    pr.dest[0] = (uint8_t *)dest;
    pr.scale[0] = dest_scale;
    pr.ranks = 1;
    pr.my_rank = 0;
    pr.e_loc = (int)experts;
    pr.rows_cap = rows_cap;
    return pr;
}

extern "C" int32_t zbalhip_dispatch_normal(const void *x, int32_t x_dtype, const int32_t *topk_idx,
                                           const int32_t *send_token_idx, const int32_t *put_offset, int64_t tokens,
                                           int64_t hidden, int64_t topk, int64_t experts, int32_t quant_mode,
                                           void *const *dest, float *const *dest_scale, int32_t ranks, int32_t my_rank,
                                           int64_t dest_rows, void *stream)
{
    if (!x || !topk_idx || !send_token_idx || !put_offset || !dest) return ZBALHIP_INVALID;
    if (experts <= 0 || quant_mode < 0 || quant_mode > 2) return ZBALHIP_INVALID;
    if (ranks <= 0 || ranks > ZBALHIP_MAX_REDUCE_PEERS || my_rank < 0 || my_rank >= ranks || experts % ranks != 0 || dest_rows < 0)
        return ZBALHIP_INVALID;
    if (quant_mode != 0 && !dest_scale) return ZBALHIP_INVALID;
    PeerRows pr = {};
    for (int r = 0; r < ranks; ++r) {
        if (!dest[r] || (quant_mode != 0 && !dest_scale[r])) return ZBALHIP_INVALID;
        pr.dest[r] = (uint8_t *)dest[r];
        pr.scale[r] = quant_mode != 0 ? dest_scale[r] : nullptr;
    }
    pr.ranks = ranks;
    pr.my_rank = my_rank;
    pr.e_loc = (int)(experts / ranks);
    pr.rows_cap = dest_rows;
    const int q = quant_mode == 0 ? QM_COPY : (quant_mode == 1 ? QM_INT8_EPS : QM_FP8);
    return permute_launch(x, x_dtype, topk_idx, send_token_idx, put_offset, 0, nullptr, tokens, hidden, topk, experts, q, pr,
                          (hipStream_t)stream);
}

extern "C" int32_t zbalhip_dispatch_low_latency(const void *x, int32_t x_dtype, const int32_t *expert_ids,
                                                int64_t tokens, int64_t hidden, int64_t topk, int64_t experts,
                                                int32_t quant_mode, int32_t token_nums_type, void *expand_x,
                                                float *dynamic_scales, int32_t *expand_idx, int64_t *expert_token_nums,
                                                int32_t *ep_recv_counts, int32_t *scratch, int32_t scratch_blocks,
                                                void *stream)
{
    /* an empty batch has no per-token data: only the counts are written */
    if (!expert_token_nums || !ep_recv_counts || !scratch) return ZBALHIP_INVALID;
    if (tokens > 0 && (!x || !expert_ids || !expand_x || !expand_idx)) return ZBALHIP_INVALID;
    if (experts <= 0 || experts > 1024 || topk <= 0 || tokens < 0 || quant_mode < 0 || quant_mode > 2 ||
        scratch_blocks < 1)
        return ZBALHIP_INVALID;
    hipStream_t st = (hipStream_t)stream;
    const int q = quant_mode == 0 ? QM_COPY : (quant_mode == 1 ? QM_INT8_NOEPS : QM_FP8);
    if (tokens > 0 && q != QM_COPY && !dynamic_scales) return ZBALHIP_INVALID;
    if (layout_fits_inline(tokens, topk, experts, q)) {      /* one launch: the permute kernel derives ranks and counts itself */
        InlineLayout il = {};
        il.tokens = (int)tokens;
        il.token_nums_type = token_nums_type;
        il.expand_idx = expand_idx;
        il.incl_i32 = ep_recv_counts;
        il.nums_typed = expert_token_nums;
        const PermuteExtras ex = {&il, nullptr, 0, nullptr};
        return permute_launch(x, x_dtype, expert_ids, expand_idx, ep_recv_counts, 1, nullptr, tokens, hidden, topk, experts, q,
                              single_window(expand_x, dynamic_scales, experts, tokens * topk), st, ex);
    }
    const int32_t rc = zbalhip_layout_fused_internal(expert_ids, tokens, experts, topk, token_nums_type, nullptr, expand_idx,
                                                     ep_recv_counts, nullptr, nullptr, expert_token_nums, st);
    if (rc != ZBALHIP_OK) return rc;
    return permute_launch(x, x_dtype, expert_ids, expand_idx, ep_recv_counts, 1, nullptr, tokens, hidden, topk, experts, q,
                          single_window(expand_x, dynamic_scales, experts, tokens * topk), st);
}

extern "C" int32_t zbalhip_dispatch_low_latency_ranks(const void *x, int32_t x_dtype, const int32_t *const *expert_ids,
                                                      int64_t tokens, int64_t hidden, int64_t topk, int64_t experts,
                                                      int32_t quant_mode, int32_t token_nums_type, void *const *expand_x,
                                                      float *const *dynamic_scales, int32_t ranks, int32_t my_rank,
                                                      int64_t dest_rows, int32_t *expand_idx, int64_t *expert_token_nums,
                                                      int32_t *ep_recv_counts, int32_t *all_counts, void *stream)
{
    if (!expert_ids || !expert_token_nums || !ep_recv_counts || !all_counts) return ZBALHIP_INVALID;
    if (experts <= 0 || experts > 1024 || topk <= 0 || tokens < 0 || tokens * topk > 0x7fffffff || quant_mode < 0 ||
        quant_mode > 2 || dest_rows < 0)
        return ZBALHIP_INVALID;
    if (ranks <= 0 || ranks > ZBALHIP_MAX_REDUCE_PEERS || my_rank < 0 || my_rank >= ranks || experts % ranks != 0)
        return ZBALHIP_INVALID;
    if (tokens > 0 && (!x || !expand_x || !expand_idx || (quant_mode != 0 && !dynamic_scales))) return ZBALHIP_INVALID;
    PeerRows pr = {};
    for (int r = 0; r < ranks; ++r) {
        if (tokens > 0 && (!expert_ids[r] || !expand_x[r] || (quant_mode != 0 && !dynamic_scales[r]))) return ZBALHIP_INVALID;
        pr.dest[r] = tokens > 0 ? (uint8_t *)expand_x[r] : nullptr;
        pr.scale[r] = (tokens > 0 && quant_mode != 0) ? dynamic_scales[r] : nullptr;
    }
    pr.ranks = ranks;
    pr.my_rank = my_rank;
    pr.e_loc = (int)(experts / ranks);
    pr.rows_cap = dest_rows;
    hipStream_t st = (hipStream_t)stream;
    int32_t rc = zbalhip_ll_counts_internal(expert_ids, ranks, my_rank, tokens, topk, experts, token_nums_type, all_counts,
                                            ep_recv_counts, expert_token_nums, st);
    if (rc != ZBALHIP_OK || tokens == 0) return rc;
    /* the rank of each of my picks among my own earlier picks of the same expert */
    rc = zbalhip_layout_fused_internal(expert_ids[my_rank], tokens, experts, topk, 1, nullptr, expand_idx, nullptr, nullptr,
                                       nullptr, nullptr, st);
    if (rc != ZBALHIP_OK) return rc;
    const int q = quant_mode == 0 ? QM_COPY : (quant_mode == 1 ? QM_INT8_NOEPS : QM_FP8);
    return permute_launch(x, x_dtype, expert_ids[my_rank], expand_idx, ep_recv_counts, 1, nullptr, tokens, hidden, topk,
                          experts, q, pr, st);
}

extern "C" int32_t zbalhip_fused_permute_quant(const void *x, int32_t x_dtype, const int32_t *expert_ids,
                                               const float *smooth, const uint8_t *active_mask, int64_t tokens,
                                               int64_t hidden, int64_t topk,
                                               int64_t experts, int32_t mode, void *q1, float *xs, int32_t *expand_idx,
                                               int64_t *counts, int32_t *row_off, uint32_t *clear_words,
                                               int64_t clear_count, int32_t *scratch, int32_t scratch_blocks, void *stream)
{
    if (!counts || !row_off || clear_count < 0 || (clear_count > 0 && !clear_words)) return ZBALHIP_INVALID;
    if (tokens > 0 && (!x || !expert_ids || !q1 || !xs || !expand_idx)) return ZBALHIP_INVALID;
    if (experts <= 0 || experts > 1024 || topk <= 0 || tokens < 0 || (mode != 1 && mode != 2)) return ZBALHIP_INVALID;
    if (mode == 2 && smooth) return ZBALHIP_INVALID;
    if (scratch_blocks < 0 || (scratch_blocks > 0 && !scratch)) return ZBALHIP_INVALID;
    hipStream_t st = (hipStream_t)stream;
    const int q = mode == 2 ? QM_FP8 : QM_INT8_NOEPS;
    if (layout_fits_inline(tokens, topk, experts, q)) {      /* one launch: the permute kernel derives ranks and offsets itself */
        InlineLayout il = {};
        il.active_mask = active_mask;
        il.tokens = (int)tokens;
        il.token_nums_type = 1;
        il.expand_idx = expand_idx;
        il.row_off = row_off;
        il.counts_i64 = counts;
        const PermuteExtras ex = {&il, clear_words, clear_count, nullptr};
        return permute_launch(x, x_dtype, expert_ids, expand_idx, row_off, 0, smooth, tokens, hidden, topk, experts, q,
                              single_window(q1, xs, experts, tokens * topk), st, ex);
    }
    /* large batches with room for the ranges' histograms: a short layout launch, the rest of the layout inside the permute launch */
    int64_t ranges = (tokens * topk + 1023) / 1024;
    if (ranges > scratch_blocks) ranges = scratch_blocks;
    if (ranges > kTableMaxEntries / experts) ranges = kTableMaxEntries / experts;
    if (tokens > 0 && ranges >= 1 && experts <= kTableMaxExperts && topk <= kInlineMaxTopk && tokens * topk <= 0x7fffffff) {
        RangeTable rt = {};
        rt.tokens_per_range = (int)((tokens + ranges - 1) / ranges);
        rt.ranges = (int)((tokens + rt.tokens_per_range - 1) / rt.tokens_per_range);
        rt.hist = scratch;
        rt.expand_idx = expand_idx;
        rt.row_off = row_off;
        rt.counts_i64 = counts;
        const int32_t rc = zbalhip_layout_ranges_internal(expert_ids, tokens, experts, topk, active_mask, expand_idx, scratch,
                                                          rt.ranges, rt.tokens_per_range, st);
        if (rc != ZBALHIP_OK) return rc;
        const PermuteExtras ex = {nullptr, clear_words, clear_count, &rt};
        return permute_launch(x, x_dtype, expert_ids, nullptr, nullptr, 0, smooth, tokens, hidden, topk, experts, q,
                              single_window(q1, xs, experts, tokens * topk), st, ex);
    }
    const int32_t rc = zbalhip_layout_fused_internal(expert_ids, tokens, experts, topk, 1, active_mask, expand_idx, nullptr,
                                                     row_off, counts, nullptr, st);
    if (rc != ZBALHIP_OK) return rc;
    if (tokens == 0 && clear_count > 0) return zbalhip_fill_i32((int32_t *)clear_words, clear_count, 0, stream);
    const PermuteExtras ex = {nullptr, clear_words, clear_count, nullptr};
    return permute_launch(x, x_dtype, expert_ids, expand_idx, row_off, 0, smooth, tokens, hidden, topk, experts, q,
                          single_window(q1, xs, experts, tokens * topk), st, ex);
}
