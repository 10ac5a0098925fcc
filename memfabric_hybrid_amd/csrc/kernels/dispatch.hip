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
    const int slot = e * pr.ranks + pr.my_rank;
    const int32_t b = base_inclusive ? (slot == 0 ? 0 : base[slot - 1]) : base[slot];
    const int64_t row = (int64_t)b + rank_in_expert;
    return row < pr.rows_cap ? row : -1;
}

/* load 16 consecutive 16-bit elements as fp32 */
template <int XDT> __device__ __forceinline__ void load16(const uint16_t *__restrict__ p, float (&v)[16])
{
    const u32x4 a = *reinterpret_cast<const u32x4 *>(p);
    const u32x4 b = *reinterpret_cast<const u32x4 *>(p + 8);
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
template <int XDT, int QM, int SLOTS, bool SMOOTH>
__global__ void __launch_bounds__(kThreads)
permute_quant_kernel(const uint16_t *__restrict__ x, const int32_t *__restrict__ topk_idx,
                     const int32_t *__restrict__ rank_in_expert, const int32_t *__restrict__ base, int base_inclusive,
                     const float *__restrict__ smooth, int hidden, int topk, int experts, PeerRows pr)
{
    __shared__ float red[kThreads / 64];
    const int t = blockIdx.x;
    const int nseg = hidden / kElemsPerLane;
    float v[SLOTS][16];
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
        const int seg = s * blockDim.x + threadIdx.x;
        if (seg < nseg) load16<XDT>(x + (int64_t)t * hidden + (int64_t)seg * 16, v[s]);
        else {
#pragma unroll
            for (int i = 0; i < 16; ++i) v[s][i] = 0.0f;
        }
    }

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
            const int e = topk_idx[(int64_t)t * topk + k];
            const int rk = rank_in_expert[(int64_t)t * topk + k];
            if (e < 0 || e >= experts || rk < 0) continue;      /* rk < 0: the layout masked this token out */
            const int64_t row = pick_row(base, base_inclusive, pr, e, rk);
            if (row < 0) continue;
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
            const int e = topk_idx[(int64_t)t * topk + k];
            const int rk = rank_in_expert[(int64_t)t * topk + k];
            if (e < 0 || e >= experts || rk < 0) continue;      /* rk < 0: the layout masked this token out */
            const int64_t row = pick_row(base, base_inclusive, pr, e, rk);
            if (row < 0) continue;
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
            const int e = topk_idx[(int64_t)t * topk + k];
            const int rk = rank_in_expert[(int64_t)t * topk + k];
            if (e < 0 || e >= experts || rk < 0) continue; /* uniform across the block */
            const int64_t row = pick_row(base, base_inclusive, pr, e, rk);
            if (row < 0) continue;
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
            if (c < nchunk) v[u] = *reinterpret_cast<const u32x4 *>(x + (int64_t)t * hidden + (int64_t)c * 8);
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

template <int XDT, int QM, bool SMOOTH>
int32_t launch_quant(const void *x, const int32_t *topk_idx, const int32_t *rank_in_expert, const int32_t *base,
                     int base_inclusive, const float *smooth, int64_t tokens, int64_t hidden, int64_t topk,
                     int64_t experts, const PeerRows &pr, hipStream_t st)
{
    const int nseg = (int)(hidden / kElemsPerLane);
    int threads = (nseg + 63) / 64 * 64;
    if (threads > kThreads) threads = kThreads;
    const int slots = (nseg + threads - 1) / threads;
#define ZB_LAUNCH(S)                                                                                              \
    permute_quant_kernel<XDT, QM, S, SMOOTH><<<(unsigned)tokens, threads, 0, st>>>(                                \
        (const uint16_t *)x, topk_idx, rank_in_expert, base, base_inclusive, smooth, (int)hidden, (int)topk,       \
        (int)experts, pr)
    if (slots <= 1) ZB_LAUNCH(1);
    else if (slots <= 2) ZB_LAUNCH(2);
    else if (slots <= 4) ZB_LAUNCH(4);
    else return ZBALHIP_INVALID;
#undef ZB_LAUNCH
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
                              int64_t hidden, int64_t topk, int64_t experts, int quant, const PeerRows &pr, hipStream_t st)
{
    if (x_dtype != ZDT_BF16 && x_dtype != ZDT_FP16) return ZBALHIP_INVALID;
    if (hidden <= 0 || hidden > 16 * kThreads * 4 || topk <= 0 || tokens < 0) return ZBALHIP_INVALID;
    if (tokens == 0) return ZBALHIP_OK;
    if (quant == QM_COPY) {
        if (hidden % 8 != 0) return ZBALHIP_INVALID;
        permute_copy_kernel<<<(unsigned)tokens, kThreads, 0, st>>>((const uint16_t *)x, topk_idx, rank_in_expert, base,
                                                                 base_inclusive, (int)hidden, (int)topk, (int)experts, pr);
        return zbalhip_check_launch();
    }
    if (hidden % 16 != 0 || (quant == QM_FP8 && hidden % 128 != 0)) return ZBALHIP_INVALID;
    const bool bf = (x_dtype == ZDT_BF16);
#define ZB_GO(QMV, SM)                                                                                               \
    return bf ? launch_quant<ZDT_BF16, QMV, SM>(x, topk_idx, rank_in_expert, base, base_inclusive, smooth, tokens,  \
                                                 hidden, topk, experts, pr, st)                                      \
              : launch_quant<ZDT_FP16, QMV, SM>(x, topk_idx, rank_in_expert, base, base_inclusive, smooth, tokens,  \
                                                 hidden, topk, experts, pr, st)
    if (quant == QM_FP8) { ZB_GO(QM_FP8, false); }
    if (quant == QM_INT8_EPS) { ZB_GO(QM_INT8_EPS, false); }
    if (quant == QM_INT8_NOEPS) {
        if (smooth) { ZB_GO(QM_INT8_NOEPS, true); }
        ZB_GO(QM_INT8_NOEPS, false);
    }
#undef ZB_GO
    return ZBALHIP_INVALID;
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
    const int32_t rc = zbalhip_layout_fused_internal(expert_ids, tokens, experts, topk, token_nums_type, nullptr, expand_idx,
                                                     ep_recv_counts, nullptr, nullptr, expert_token_nums, st);
    if (rc != ZBALHIP_OK) return rc;
    const int q = quant_mode == 0 ? QM_COPY : (quant_mode == 1 ? QM_INT8_NOEPS : QM_FP8);
    if (tokens > 0 && q != QM_COPY && !dynamic_scales) return ZBALHIP_INVALID;
    return permute_launch(x, x_dtype, expert_ids, expand_idx, ep_recv_counts, 1, nullptr, tokens, hidden, topk, experts, q,
                          single_window(expand_x, dynamic_scales, experts, tokens * topk), st);
}

extern "C" int32_t zbalhip_fused_permute_quant(const void *x, int32_t x_dtype, const int32_t *expert_ids,
                                               const float *smooth, const uint8_t *active_mask, int64_t tokens,
                                               int64_t hidden, int64_t topk,
                                               int64_t experts, int32_t mode, void *q1, float *xs, int32_t *expand_idx,
                                               int64_t *counts, int32_t *row_off, int32_t *scratch,
                                               int32_t scratch_blocks, void *stream)
{
    if (!counts || !row_off || !scratch) return ZBALHIP_INVALID;
    if (tokens > 0 && (!x || !expert_ids || !q1 || !xs || !expand_idx)) return ZBALHIP_INVALID;
    if (experts <= 0 || experts > 1024 || topk <= 0 || tokens < 0 || (mode != 1 && mode != 2) || scratch_blocks < 1)
        return ZBALHIP_INVALID;
    if (mode == 2 && smooth) return ZBALHIP_INVALID;
    hipStream_t st = (hipStream_t)stream;
    const int32_t rc = zbalhip_layout_fused_internal(expert_ids, tokens, experts, topk, 1, active_mask, expand_idx, nullptr,
                                                     row_off, counts, nullptr, st);
    if (rc != ZBALHIP_OK) return rc;
    return permute_launch(x, x_dtype, expert_ids, expand_idx, row_off, 0, smooth, tokens, hidden, topk, experts,
                          mode == 2 ? QM_FP8 : QM_INT8_NOEPS, single_window(q1, xs, experts, tokens * topk), st);
}
