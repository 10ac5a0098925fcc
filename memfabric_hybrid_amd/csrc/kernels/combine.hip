/*
 * Weighted combine (gather-reduce): out[t,:] = round(sum_k w[t,k] * y[row(t,k),:]).
 *
 * One workgroup per output token (small batches: per piece of a token's row,
 * so that every CU has work). Each lane owns 16-byte chunks (8 elements)
 * of the row; for a chunk it issues the loads of up to eight picks back to
 * back so that eight 16-byte requests per lane are in flight, then folds
 * them into fp32 accumulators in pick order with a separately rounded
 * multiply and add, and stores one rounded 16-byte chunk. HBM traffic is
 * K row reads plus one row write per token.
 */
#include "zbal_device.h"
#include "zbal_hip_kernels.h"

namespace {

constexpr int kThreads = 256;
constexpr int kMaxTopk = 32;
constexpr int kGroup = 8;

/*
 * Where the rows are read from: expert e's rows sit in the window of rank e / e_loc, at the slot
 * base[e * ranks + my_rank] that this rank's dispatch wrote them to (reference zbal_kernel_combine_normal.h:437-494).
 * One GPU: the windows are local allocations; over xGMI they would be mapped peer memory. rows_cap: rows per window.
 */
struct PeerSource {
    const uint16_t *y[ZBALHIP_MAX_REDUCE_PEERS];
    int ranks, my_rank, e_loc;
    int64_t rows_cap;
};

template <int DT>
__global__ void __launch_bounds__(kThreads)
combine_kernel(PeerSource src, const int32_t *__restrict__ base, int base_inclusive,
               const float *__restrict__ w, const int32_t *__restrict__ topk_idx,
               const int32_t *__restrict__ rank_in_expert, int hidden, int topk, int experts,
               uint16_t *__restrict__ out)
{
    __shared__ const uint16_t *s_row[kMaxTopk];
    __shared__ float s_w[kMaxTopk];
    __shared__ int s_n;
    const int t = blockIdx.x;
    if (threadIdx.x < 64) {
        /*
         * One lane per pick resolves its source row (three dependent loads; done pick after pick by one lane they are
         * topk round trips in a row, which is what a small batch waits for); the valid picks are then compacted in
         * pick order. Rank -2 (or a negative rank on a valid expert id) belongs to a token that the layout masked
         * out (x_active_mask): such a token's output row is left as it is. Rank -1 on an invalid expert id is a pick
         * that goes nowhere: the token's row is still written, from its other picks, or as zeros if it has none.
         */
        const int k = threadIdx.x;
        bool keep = false, masked = false;
        const uint16_t *row_ptr = nullptr;
        float wk = 0.0f;
        if (k < topk) {
            const int e = topk_idx[(int64_t)t * topk + k];
            const int32_t rk = rank_in_expert[(int64_t)t * topk + k];
            wk = w[(int64_t)t * topk + k];
            if (rk == -2) masked = true;
            else if (e >= 0 && e < experts) {
                if (rk < 0) masked = true;
                else {
                    const int slot = e * src.ranks + src.my_rank;
                    /* running sums start anew with every rank's block of `experts` entries (low-latency counts) */
                    const int32_t b = base_inclusive ? (slot % experts == 0 ? 0 : base[slot - 1]) : base[slot];
                    const int64_t row = (int64_t)b + rk;
                    if (row < src.rows_cap) {            /* never read past the window */
                        keep = true;
                        row_ptr = src.y[e / src.e_loc] + row * hidden;
                    }
                }
            }
        }
        const uint64_t kept = __ballot(keep);
        const bool any_masked = __ballot(masked) != 0;
        if (keep && !any_masked) {
            const int pos = __popcll(kept & ((1ull << k) - 1ull));
            s_row[pos] = row_ptr;
            s_w[pos] = wk;
        }
        if (k == 0) s_n = any_masked ? -1 : __popcll(kept);
    }
    __syncthreads();
    const int n = s_n;
    if (n < 0) return;
    /* blockIdx.y: a small batch spreads each row over several workgroups, so that the whole chip takes part */
    const int nchunk_all = hidden / 8;
    const int per_split = (nchunk_all + gridDim.y - 1) / gridDim.y;
    const int c_begin = blockIdx.y * per_split;
    const int nchunk = c_begin + per_split < nchunk_all ? c_begin + per_split : nchunk_all;
    for (int c = c_begin + threadIdx.x; c < nchunk; c += blockDim.x) {
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = 0.0f;
        for (int k0 = 0; k0 < n; k0 += kGroup) {
            u32x4 v[kGroup];
#pragma unroll
            for (int u = 0; u < kGroup; ++u)
                if (k0 + u < n)
                    v[u] = __builtin_nontemporal_load(
                        reinterpret_cast<const u32x4 *>(s_row[k0 + u] + (int64_t)c * 8));
#pragma unroll
            for (int u = 0; u < kGroup; ++u) {
                if (k0 + u < n) {
                    const float wk = s_w[k0 + u];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float lo = zb_half_to_f32<DT>(v[u][i] & 0xffffu) * wk;
                        const float hi = zb_half_to_f32<DT>(v[u][i] >> 16) * wk;
                        acc[2 * i] = acc[2 * i] + lo;
                        acc[2 * i + 1] = acc[2 * i + 1] + hi;
                    }
                }
            }
        }
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = zb_pack2_half<DT>(acc[2 * i], acc[2 * i + 1]);
        __builtin_nontemporal_store(o, reinterpret_cast<u32x4 *>(out + (int64_t)t * hidden + (int64_t)c * 8));
    }
}

} // namespace

extern "C" int32_t zbalhip_combine(const void *const *y, int32_t ranks, int32_t my_rank, int64_t y_rows, int32_t dtype,
                                   const int32_t *base, int32_t base_is_inclusive, const float *w, const int32_t *topk_idx,
                                   const int32_t *send_token_idx, int64_t tokens, int64_t hidden, int64_t topk,
                                   int64_t experts, void *out, void *stream)
{
    if (!y || !base || !w || !topk_idx || !send_token_idx || !out) return ZBALHIP_INVALID;
    if (dtype != ZDT_BF16 && dtype != ZDT_FP16) return ZBALHIP_INVALID;
    if (tokens < 0 || hidden <= 0 || hidden % 8 != 0 || topk <= 0 || topk > kMaxTopk || experts <= 0)
        return ZBALHIP_INVALID;
    if (ranks <= 0 || ranks > ZBALHIP_MAX_REDUCE_PEERS || my_rank < 0 || my_rank >= ranks || experts % ranks != 0 || y_rows < 0)
        return ZBALHIP_INVALID;
    PeerSource src = {};
    for (int r = 0; r < ranks; ++r) {
        if (!y[r]) return ZBALHIP_INVALID;
        src.y[r] = (const uint16_t *)y[r];
    }
    src.ranks = ranks;
    src.my_rank = my_rank;
    src.e_loc = (int)(experts / ranks);
    src.rows_cap = y_rows;
    if (tokens == 0) return ZBALHIP_OK;
    /* fewer tokens than two per CU: cut the rows into pieces of at least one chunk per lane of a full workgroup */
    int splits = 1;
    while (tokens * splits < 512 && splits < 8 && hidden / 8 / (splits * 2) >= kThreads / 2) splits *= 2;
    const int64_t per_split = (hidden / 8 + splits - 1) / splits;
    int threads = (int)((per_split + 63) / 64 * 64);
    if (threads > kThreads) threads = kThreads;
    const dim3 grid((unsigned)tokens, (unsigned)splits);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == ZDT_BF16)
        combine_kernel<ZDT_BF16><<<grid, threads, 0, st>>>(src, base, base_is_inclusive, w, topk_idx, send_token_idx,
                                                                     (int)hidden, (int)topk, (int)experts, (uint16_t *)out);
    else
        combine_kernel<ZDT_FP16><<<grid, threads, 0, st>>>(src, base, base_is_inclusive, w, topk_idx, send_token_idx,
                                                                     (int)hidden, (int)topk, (int)experts, (uint16_t *)out);
    return zbalhip_check_launch();
}
