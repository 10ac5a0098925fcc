/*
 * Routing and layout kernels: softmax top-k router, per-expert histogram with
 * stable per-pick ranks, and the count scans that turn the histogram into row
 * offsets.
 *
 * The stable rank of a pick (its position among earlier picks of the same
 * expert, in flat (t,k) order) is computed without atomics on the result:
 * blocks own contiguous token ranges, a first pass leaves one histogram per
 * block in `scratch`, and the second pass starts each block from the sum of
 * the histograms of the blocks before it; inside a block, picks are ranked 64
 * at a time with wave ballots (lanes holding the same expert find each other
 * by intersecting one ballot per index bit) and the four waves of a block
 * commit their running counts in wave order.
 */
#include <mutex>

#include "zbal_device.h"
#include "zbal_hip_kernels.h"
#include "zbal_layout_rank.h"

#define ZB_MAX_EXPERTS 1024
#define ZB_LAYOUT_THREADS 256
#define ZB_FUSED_THREADS 1024

/*
 * Per-block histograms of zbalhip_dispatch_layout_static: the rows its kernels otherwise find in the caller's
 * `scratch` argument, for the largest case the entry point takes. Every GPU the library runs on holds its own copy
 * for the life of the process (200 KiB). Host code never uses this name as an address: it asks the runtime for the
 * device address once per device (static_scratch_of) and hands that pointer to the kernels.
 */
static __device__ __align__(256) int32_t scratch[ZBALHIP_LAYOUT_MAX_BLOCKS * ZB_MAX_EXPERTS];

namespace {

constexpr int ZB_MAX_DEVICES = 64;

/*
 * This GPU's copy of `scratch`: its device address, looked up on the first call with that GPU current, and an event
 * that marks the end of the last launch sequence that used it. Calls are issued under `mu`, each waiting for that
 * event on its own stream first and recording it again after its last launch, so two callers on different streams
 * (or threads) take turns on the array instead of racing on it.
 */
struct StaticScratch {
    std::mutex mu;
    int32_t *addr = nullptr;
    hipEvent_t last_use = nullptr;
};

StaticScratch *static_scratch_of(int dev)
{
    static StaticScratch per_device[ZB_MAX_DEVICES];
    StaticScratch &s = per_device[dev];
    std::lock_guard<std::mutex> guard(s.mu);
    if (s.addr == nullptr) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return nullptr;
        if (hipEventCreateWithFlags(&s.last_use, hipEventDisableTiming) != hipSuccess) return nullptr;
        s.addr = static_cast<int32_t *>(p);
    }
    return &s;
}

struct LayoutPlan {
    int nblk;
    int tokens_per_block;
};

inline LayoutPlan plan_layout(int64_t tokens, int64_t topk, int max_blocks)
{
    LayoutPlan p;
    int64_t want = (tokens * topk + 1023) / 1024;
    if (want < 1) want = 1;
    if (want > max_blocks) want = max_blocks;
    int64_t tpb = (tokens + want - 1) / want;
    if (tpb < 1) tpb = 1;
    p.tokens_per_block = (int)tpb;
    p.nblk = (int)((tokens + tpb - 1) / tpb);
    if (p.nblk < 1) p.nblk = 1;
    return p;
}

template <typename IdxT>
__global__ void __launch_bounds__(ZB_LAYOUT_THREADS)
layout_hist_kernel(const IdxT *__restrict__ idx, int tokens, int topk, int experts, int ranks, int tpb,
                   int32_t *__restrict__ scratch, int32_t *__restrict__ tokens_per_rank)
{
    __shared__ int32_t hist[ZB_MAX_EXPERTS];
    for (int e = threadIdx.x; e < experts; e += blockDim.x) hist[e] = 0;
    if (blockIdx.x == 0 && tokens_per_rank)
        for (int r = threadIdx.x; r < ranks; r += blockDim.x) tokens_per_rank[r] = 0;
    __syncthreads();
    const int64_t p0 = (int64_t)blockIdx.x * tpb * topk;
    int64_t p1 = p0 + (int64_t)tpb * topk;
    const int64_t pend = (int64_t)tokens * topk;
    if (p1 > pend) p1 = pend;
    for (int64_t i = p0 + threadIdx.x; i < p1; i += blockDim.x) {
        int64_t e = (int64_t)idx[i];
        if (e >= 0 && e < experts) atomicAdd(&hist[e], 1);
    }
    __syncthreads();
    for (int e = threadIdx.x; e < experts; e += blockDim.x) scratch[(int64_t)blockIdx.x * experts + e] = hist[e];
}

template <typename IdxT>
__global__ void __launch_bounds__(ZB_LAYOUT_THREADS)
layout_rank_kernel(const IdxT *__restrict__ idx, int tokens, int topk, int experts, int ranks, int tpb, int nbits,
                   const int32_t *__restrict__ scratch, int32_t *__restrict__ send_token_idx,
                   int32_t *__restrict__ tokens_per_rank)
{
    __shared__ int32_t run[ZB_MAX_EXPERTS];
    __shared__ int32_t rcnt[ZB_MAX_EXPERTS];
    __shared__ __align__(16) uint8_t cnt[ZB_LAYOUT_THREADS / 64 * ZB_MAX_EXPERTS];
    const int b = blockIdx.x;
    for (int e = threadIdx.x; e < experts; e += blockDim.x) {
        int32_t s = 0;
        for (int bb = 0; bb < b; ++bb) s += scratch[(int64_t)bb * experts + e];
        run[e] = s;
    }
    for (int r = threadIdx.x; r < ranks; r += blockDim.x) rcnt[r] = 0;
    __syncthreads();

    const int tok0 = b * tpb;
    int tok1 = tok0 + tpb;
    if (tok1 > tokens) tok1 = tokens;
    rank_picks(idx, (int64_t)tok0 * topk, (int64_t)tok1 * topk, experts, nbits, run, cnt, send_token_idx);

    /* tokens per rank: one count per (token, rank) no matter how many of the token's picks land there */
    if (tokens_per_rank) {
        const int e_loc = experts / ranks;
        for (int t = tok0 + threadIdx.x; t < tok1; t += blockDim.x) {
            for (int k = 0; k < topk; ++k) {
                int64_t e = (int64_t)idx[(int64_t)t * topk + k];
                if (e < 0 || e >= experts) continue;
                const int r = (int)(e / e_loc);
                bool first = true;
                for (int k2 = 0; k2 < k; ++k2) {
                    int64_t e2 = (int64_t)idx[(int64_t)t * topk + k2];
                    if (e2 >= 0 && e2 < experts && (int)(e2 / e_loc) == r) first = false;
                }
                if (first) atomicAdd(&rcnt[r], 1);
            }
        }
        __syncthreads();
        for (int r = threadIdx.x; r < ranks; r += blockDim.x)
            if (rcnt[r]) atomicAdd(&tokens_per_rank[r], rcnt[r]);
    }
}

/*
 * The whole layout in one launch, for the callers that need ranks and offsets but no per-rank counts: every
 * block first counts the picks that precede its own range (the index array is a few hundred KiB and sits in L2,
 * so reading it again per block is cheaper than a launch), ranks its own picks, and the last block, whose running
 * counts are then the totals, scans them into the offsets. Every output pointer except send_token_idx may be null.
 */
template <typename IdxT>
__global__ void __launch_bounds__(ZB_FUSED_THREADS)
layout_fused_kernel(const IdxT *__restrict__ idx, int tokens, int topk, int experts, int tpb, int nbits,
                    int token_nums_type, const uint8_t *__restrict__ active_mask, int32_t *__restrict__ send_token_idx,
                    int32_t *__restrict__ incl_i32, int32_t *__restrict__ row_off /* [E+1] */,
                    int64_t *__restrict__ counts_i64, int64_t *__restrict__ nums_typed)
{
    __shared__ int32_t run[ZB_MAX_EXPERTS];
    __shared__ int32_t wsum[ZB_FUSED_THREADS / 64];
    __shared__ int32_t s_active;
    __shared__ __align__(16) uint8_t cnt[ZB_FUSED_THREADS / 64 * ZB_MAX_EXPERTS];
    for (int e = threadIdx.x; e < experts; e += blockDim.x) run[e] = 0;
    if (threadIdx.x == 0) s_active = 0;
    __syncthreads();
    /*
     * x_active_mask (one bool per token): the reference processes the first sum(mask) tokens and nothing else
     * (TokenActiveMaskCal, fused_deep_moe/gemm/kernel/...swiglu_quant_multistage_workspace.h:836-863). Picks of
     * the other tokens get rank -2 here: the permute kernel skips every negative rank, and the combine kernel leaves
     * the output row of such a token alone. (-1 is a pick with an invalid expert id in a token that is routed: the
     * combine still writes that token's row, from its other picks or as zeros.)
     */
    int active = tokens;
    if (active_mask) {
        int part = 0;
        for (int t = threadIdx.x; t < tokens; t += blockDim.x) part += active_mask[t] != 0;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) part += __shfl_xor(part, off, 64);
        if ((threadIdx.x & 63) == 0 && part) atomicAdd(&s_active, part);
        __syncthreads();
        active = s_active;
    }
    int tok0 = blockIdx.x * tpb;
    int tok1 = tok0 + tpb;
    if (tok1 > tokens) tok1 = tokens;
    for (int64_t i = (int64_t)(tok0 > active ? tok0 : active) * topk + threadIdx.x; i < (int64_t)tok1 * topk; i += blockDim.x)
        send_token_idx[i] = -2;
    if (tok0 > active) tok0 = active;
    if (tok1 > active) tok1 = active;
    const int64_t p0 = (int64_t)tok0 * topk, p1 = (int64_t)tok1 * topk;
    constexpr int PER = 16 / (int)sizeof(IdxT);      /* indices per 16-byte load */
    const int64_t nvec = ((uintptr_t)idx & 15) == 0 ? p0 / PER : 0;
    /* four 16-byte loads per lane are requested before the first is counted: a chain of round trips to L2 otherwise */
    for (int64_t v0 = threadIdx.x; v0 < nvec; v0 += 4 * (int64_t)blockDim.x) {
        u32x4 raw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t v = v0 + u * (int64_t)blockDim.x;
            raw[u] = v < nvec ? *reinterpret_cast<const u32x4 *>(idx + v * PER) : u32x4{~0u, ~0u, ~0u, ~0u};
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int j = 0; j < PER; ++j) {
                int64_t e;
                if (sizeof(IdxT) == 4) e = (int32_t)raw[u][j];
                else e = (int64_t)(((uint64_t)raw[u][2 * j + 1] << 32) | raw[u][2 * j]);
                if (e >= 0 && e < experts) atomicAdd(&run[(int)e], 1);
            }
    }
    for (int64_t i = nvec * PER + threadIdx.x; i < p0; i += blockDim.x) {
        const int64_t e = (int64_t)idx[i];
        if (e >= 0 && e < experts) atomicAdd(&run[(int)e], 1);
    }
    __syncthreads();
    rank_picks(idx, p0, p1, experts, nbits, run, cnt, send_token_idx);
    if (blockIdx.x != gridDim.x - 1) return;

    /* rank_picks ends on a barrier: run[] now holds the totals */
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int32_t carry = 0;
    for (int base = 0; base < experts; base += ZB_FUSED_THREADS) {
        const int e = base + threadIdx.x;
        const int32_t c = e < experts ? run[e] : 0;
        int32_t s = c;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int32_t o = __shfl_up(s, off, 64);
            if (lane >= off) s += o;
        }
        if (lane == 63) wsum[wave] = s;
        __syncthreads();
        int32_t add = carry;
        for (int w = 0; w < wave; ++w) add += wsum[w];
        s += add;
        int32_t chunk_total = 0;
        for (int w = 0; w < ZB_FUSED_THREADS / 64; ++w) chunk_total += wsum[w];
        carry += chunk_total;
        __syncthreads();
        if (e < experts) {
            if (incl_i32) incl_i32[e] = s;
            if (row_off) { row_off[e] = s - c; if (e == experts - 1) row_off[experts] = s; }
            if (counts_i64) counts_i64[e] = c;
            if (nums_typed) nums_typed[e] = token_nums_type == 0 ? (int64_t)s : (int64_t)c;
        }
    }
}

/*
 * The part of the layout that needs no other block: the picks of a token range are ranked among themselves
 * (send_token_idx = position among the range's picks of the same expert) and the range's histogram is left in
 * hist[range][experts]. The permute kernel that follows turns the histograms into offsets on its own (dispatch.hip,
 * table mode), so this launch is all there is in front of it: no counting of the ranges before, no scan.
 * A range is worked on by `subs` blocks, each ranking one slice of it; a block counts the picks of the slices before
 * its own itself (LDS atomics: a fraction of what ranking them costs), so no block waits for another, and the block of
 * the last slice ends up with the whole range's histogram and writes it.
 */
template <typename IdxT, bool SLICED>
__global__ void __launch_bounds__(ZB_FUSED_THREADS)
layout_ranges_kernel(const IdxT *__restrict__ idx, int tokens, int topk, int experts, int tpb, int subs_arg, int nbits,
                     const uint8_t *__restrict__ active_mask, int32_t *__restrict__ send_token_idx,
                     int32_t *__restrict__ hist)
{
    __shared__ int32_t run[ZB_MAX_EXPERTS];
    __shared__ int32_t s_active;
    __shared__ __align__(16) uint8_t cnt[ZB_FUSED_THREADS / 64 * ZB_MAX_EXPERTS];
    for (int e = threadIdx.x; e < experts; e += blockDim.x) run[e] = 0;
    if (threadIdx.x == 0) s_active = 0;
    __syncthreads();
    int active = tokens;
    if (active_mask) {          /* the first sum(mask) tokens are routed, the picks of the others get rank -2 (layout_fused_kernel) */
        int part = 0;
        for (int t = threadIdx.x; t < tokens; t += blockDim.x) part += active_mask[t] != 0;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) part += __shfl_xor(part, off, 64);
        if ((threadIdx.x & 63) == 0 && part) atomicAdd(&s_active, part);
        __syncthreads();
        active = s_active;
    }
    const int subs = SLICED ? subs_arg : 1;
    const int range = SLICED ? blockIdx.x / subs : blockIdx.x, sub = SLICED ? blockIdx.x - range * subs : 0;
    int tok0 = range * tpb;
    int tok1 = tok0 + tpb;
    if (tok1 > tokens) tok1 = tokens;
    int sl0 = tok0, sl1 = tok1;
    if (SLICED) {
        const int tps = (tpb + subs - 1) / subs;            /* tokens per slice */
        sl0 = tok0 + sub * tps;
        sl1 = sl0 + tps;
        if (sl0 > tok1) sl0 = tok1;
        if (sl1 > tok1) sl1 = tok1;
    }
    for (int64_t i = (int64_t)(sl0 > active ? sl0 : active) * topk + threadIdx.x; i < (int64_t)sl1 * topk; i += blockDim.x)
        send_token_idx[i] = -2;
    if (tok0 > active) tok0 = active;
    if (sl0 > active) sl0 = active;
    if (sl1 > active) sl1 = active;
    if (SLICED) {       /* the picks of this range in front of the slice: counted only */
        for (int64_t i = (int64_t)tok0 * topk + threadIdx.x; i < (int64_t)sl0 * topk; i += blockDim.x) {
            const int64_t e = (int64_t)idx[i];
            if (e >= 0 && e < experts) atomicAdd(&run[(int)e], 1);
        }
        __syncthreads();
    }
    rank_picks(idx, (int64_t)sl0 * topk, (int64_t)sl1 * topk, experts, nbits, run, cnt, send_token_idx);
    /* rank_picks ends on a barrier: run[] counts the range up to this slice's end; the last slice's block has it all */
    if (!SLICED || sub == subs - 1)
        for (int e = threadIdx.x; e < experts; e += blockDim.x) hist[(int64_t)range * experts + e] = run[e];
}

/*
 * One block: totals per expert from the per-block histograms (or from a
 * ready histogram when nblk == 0), then an inclusive scan over experts.
 * Every output pointer may be null.
 */
__global__ void __launch_bounds__(ZB_MAX_EXPERTS)
layout_scan_kernel(const int32_t *__restrict__ hist, int nblk, int experts, int topk, int token_nums_type,
                   int32_t *__restrict__ counts_i32, int32_t *__restrict__ excl_i32, int32_t *__restrict__ incl_i32,
                   int32_t *__restrict__ row_off /* [E+1] */, int64_t *__restrict__ counts_i64,
                   int64_t *__restrict__ nums_typed, int32_t *__restrict__ total, int32_t *__restrict__ balance)
{
    __shared__ int32_t wsum[ZB_MAX_EXPERTS / 64];
    const int e = threadIdx.x;
    int32_t c = 0;
    if (e < experts) {
        if (nblk == 0) c = hist[e];
        else for (int b = 0; b < nblk; ++b) c += hist[(int64_t)b * experts + e];
    }
    int32_t s = c;
    const int lane = e & 63, wave = e >> 6;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        int32_t o = __shfl_up(s, off, 64);
        if (lane >= off) s += o;
    }
    if (lane == 63) wsum[wave] = s;
    __syncthreads();
    int32_t add = 0;
    for (int w = 0; w < wave; ++w) add += wsum[w];
    s += add;
    if (e < experts) {
        if (counts_i32) counts_i32[e] = c;
        if (excl_i32) excl_i32[e] = s - c;
        if (incl_i32) incl_i32[e] = s;
        if (row_off) { row_off[e] = s - c; if (e == experts - 1) row_off[experts] = s; }
        if (counts_i64) counts_i64[e] = c;
        if (nums_typed) nums_typed[e] = token_nums_type == 0 ? (int64_t)s : (int64_t)c;
        if (e == experts - 1) {
            if (total) *total = s;
            if (balance) {
                const int32_t bs = s / topk;
                balance[0] = bs > 0 ? 0 : -1;
                balance[1] = bs > 0 ? bs - 1 : -1;
            }
        }
    }
}

/*
 * Notify for a group of R ranks, from the point of view of rank `me` (reference zbal_kernel_notify_dispatch.h
 * ReorderRecvDataOutput :356-378, BuildTotalRecvTokens :531-564, BuildRecvTokenPerExp :566-596,
 * BuildBalanceMatrix :421-498 without re-balancing). counts.p[s] is rank s's tokens-per-expert vector, read where
 * it lies in that rank's window. For every destination rank r the offsets are the exclusive running sum of
 * counts[s][r * E_loc + le] taken local expert by local expert and, within an expert, source rank by source rank.
 * One block, one thread per (local expert, source rank) pair of a destination rank.
 */
struct CountsOfRanks {
    const int32_t *p[ZBALHIP_MAX_REDUCE_PEERS];
};

__global__ void __launch_bounds__(ZB_MAX_EXPERTS)
notify_ranks_kernel(CountsOfRanks counts, int ranks, int me, int experts, int topk, int32_t *__restrict__ recv_data,
                    int32_t *__restrict__ put_offset, int32_t *__restrict__ total_recv,
                    int64_t *__restrict__ recv_tokens_per_expert, int32_t *__restrict__ balance)
{
    __shared__ int32_t wsum[ZB_MAX_EXPERTS / 64];
    __shared__ int32_t rank_total[ZBALHIP_MAX_REDUCE_PEERS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const int e_loc = experts / ranks;
    for (int i = tid; i < ranks * experts; i += blockDim.x) recv_data[i] = counts.p[i / experts][i % experts];
    if (tid < ranks) rank_total[tid] = 0;
    __syncthreads();
    for (int r = 0; r < ranks; ++r) {
        const int le = tid / ranks, s = tid - le * ranks;
        const int32_t c = tid < experts ? counts.p[s][r * e_loc + le] : 0;
        int32_t incl = c;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int32_t o = __shfl_up(incl, off, 64);
            if (lane >= off) incl += o;
        }
        if (lane == 63) wsum[wave] = incl;
        __syncthreads();
        int32_t add = 0, all = 0;
        for (int w = 0; w < nwaves; ++w) {
            if (w < wave) add += wsum[w];
            all += wsum[w];
        }
        if (tid < experts) put_offset[r * experts + tid] = incl + add - c;
        if (r == me && tid == 0) *total_recv = all;
        /* what source rank s sends in all: the sum over destination ranks of its share */
        if (tid < experts && c) atomicAdd(&rank_total[s], c);
        __syncthreads();
    }
    for (int le = tid; le < e_loc; le += blockDim.x) {
        int64_t sum = 0;
        for (int s = 0; s < ranks; ++s) sum += counts.p[s][me * e_loc + le];
        recv_tokens_per_expert[le] = sum;
    }
    for (int i = tid; i < ranks * 2 * ranks; i += blockDim.x) {
        const int row = i / (2 * ranks), col = i - row * 2 * ranks;
        const int32_t bs = rank_total[row] / topk;
        int32_t v = -1;
        if (bs > 0 && col == 2 * row) v = 0;
        if (bs > 0 && col == 2 * row + 1) v = bs - 1;
        balance[i] = v;
    }
}

/*
 * Counts of the low-latency dispatch for a group of R ranks, from the point of view of rank `me` (reference
 * zbal_kernel_dispatch_low_latency.h: every rank's per-expert counts gathered into allExpertTokenNums :344-345,
 * ReorderRecvDataOutput :690-713, WaitNotify :641-688). ids.p[s] is rank s's [tokens, topk] expert ids, read where
 * they lie in that rank's window (the reference's ranks push their counts to each other and wait for flags; on one
 * GPU the inputs of all modelled ranks are in place before any of them is launched). all_counts[s * E + e] = picks
 * of expert e by rank s; ep_recv_counts[r * E + le * R + s] = INCLUSIVE running sum, per destination rank r, over
 * its local experts le and, within an expert, the source ranks s (a consumer takes index i's start from entry i - 1,
 * 0 at the start of a rank's block); expert_token_nums[le] = rows rank `me` receives for its local expert le
 * (type 1) or their running sum (type 0). One block, one thread per (local expert, source rank) pair.
 */
struct IdsOfRanks {
    const int32_t *p[ZBALHIP_MAX_REDUCE_PEERS];
};

__global__ void __launch_bounds__(ZB_MAX_EXPERTS)
ll_counts_kernel(IdsOfRanks ids, int ranks, int me, int tokens, int topk, int experts, int token_nums_type,
                 int32_t *__restrict__ all_counts, int32_t *__restrict__ ep_recv_counts,
                 int64_t *__restrict__ expert_token_nums)
{
    __shared__ int32_t hist[ZB_MAX_EXPERTS];
    __shared__ int32_t mine[ZB_MAX_EXPERTS];
    __shared__ int32_t wsum[ZB_MAX_EXPERTS / 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nwaves = blockDim.x >> 6;
    const int n = tokens * topk, e_loc = experts / ranks;
    for (int s = 0; s < ranks; ++s) {
        for (int e = tid; e < experts; e += blockDim.x) hist[e] = 0;
        __syncthreads();
        for (int i = tid; i < n; i += blockDim.x) {
            const int e = ids.p[s][i];
            if (e >= 0 && e < experts) atomicAdd(&hist[e], 1);
        }
        __syncthreads();
        for (int e = tid; e < experts; e += blockDim.x) all_counts[s * experts + e] = hist[e];
        __syncthreads();
    }
    for (int r = 0; r < ranks; ++r) {
        const int le = tid / ranks, s = tid - le * ranks;
        const int32_t c = tid < experts ? all_counts[s * experts + r * e_loc + le] : 0;
        int32_t incl = c;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int32_t o = __shfl_up(incl, off, 64);
            if (lane >= off) incl += o;
        }
        if (lane == 63) wsum[wave] = incl;
        __syncthreads();
        for (int w = 0; w < wave && w < nwaves; ++w) incl += wsum[w];
        if (tid < experts) {
            ep_recv_counts[r * experts + tid] = incl;
            if (r == me) mine[tid] = incl;
        }
        __syncthreads();
    }
    for (int le = tid; le < e_loc; le += blockDim.x) {
        const int32_t hi = mine[(le + 1) * ranks - 1], lo = le ? mine[le * ranks - 1] : 0;
        expert_token_nums[le] = token_nums_type == 0 ? (int64_t)hi : (int64_t)(hi - lo);
    }
}

/* ---- router ----------------------------------------------------------------- */

/*
 * One wave per token; lane l holds logits l, l + 64, ... (PER_LANE of them: the launcher picks the smallest
 * instantiation that covers `experts`, the arithmetic and its order are the same in all of them).
 */
/*
 * Up to 64 experts: one logit per lane, and no serial rounds of wave arg-max. A lane's pick position is its rank:
 * the number of logits that are larger, or equal with a lower index (the order K rounds of arg-max with ties to
 * the lower index produce). Ranks come from one pass over the experts with the logit of expert m read from lane m
 * as a scalar; maximum and sums run on the DPP path. Same formulas as the general kernel below
 * (p = exp(l - max) / sum; weight = p / sum of the picked p), sums taken in a different order.
 */
__global__ void __launch_bounds__(256)
topk_route_small_kernel(const float *__restrict__ logits, int tokens, int experts, int topk, void *__restrict__ topk_idx,
                        int idx_is_i64, float *__restrict__ topk_w)
{
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (t >= tokens) return; /* whole waves leave together */
    const bool mine = lane < experts;
    const float v = mine ? logits[(int64_t)t * experts + lane] : -__builtin_inff();
    const float mx = zb_wave_reduce_dpp<true>(v);
    const float ex = mine ? zb_expf(v - mx) : 0.0f;
    const float sum = zb_wave_reduce_dpp<false>(ex);
    int rank = 0;
    for (int m = 0; m < experts; ++m) {
        const float s = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), m));
        rank += (s > v || (s == v && m < lane)) ? 1 : 0;
    }
    const bool picked = mine && rank < topk;
    const float p = ex / sum;
    const float wsum = zb_wave_reduce_dpp<false>(picked ? p : 0.0f);
    if (picked) {
        if (idx_is_i64) static_cast<int64_t *>(topk_idx)[(int64_t)t * topk + rank] = lane;
        else static_cast<int32_t *>(topk_idx)[(int64_t)t * topk + rank] = lane;
        topk_w[(int64_t)t * topk + rank] = p / wsum;
    }
}

template <int PER_LANE>
__global__ void __launch_bounds__(256)
topk_route_kernel(const float *__restrict__ logits, int tokens, int experts, int topk, void *__restrict__ topk_idx,
                  int idx_is_i64, float *__restrict__ topk_w)
{
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (t >= tokens) return; /* whole waves leave together */
    const float *l = logits + (int64_t)t * experts;
    float v[PER_LANE];
    float mx = -__builtin_inff();
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
        const int e = j * 64 + lane;
        v[j] = (e < experts) ? l[e] : -__builtin_inff();
        mx = fmaxf(mx, v[j]);
    }
    mx = zb_wave_reduce_dpp<true>(mx);
    float part = 0.0f;
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
        const int e = j * 64 + lane;
        if (e < experts) part += zb_expf(v[j] - mx);
    }
    const float sum = zb_wave_reduce_dpp<false>(part);

    /*
     * K rounds of arg-max, each without an LDS round trip: the largest remaining logit by a DPP reduction of the
     * lanes' own best, then its owner by one ballot per logit slot, lowest slot and lowest lane first (the lowest
     * expert index among equal logits, as a sequential scan would pick).
     */
    uint32_t used = 0; /* bit j: this lane's j-th logit was picked */
    float wsum = 0.0f;
    float myw = 0.0f;  /* lane k keeps the k-th weight (topk <= 32) */
    int myidx = 0;
    for (int k = 0; k < topk; ++k) {
        float best = -__builtin_inff();
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j) {
            const int e = j * 64 + lane;
            if (e < experts && !((used >> j) & 1u)) best = fmaxf(best, v[j]);
        }
        best = zb_wave_reduce_dpp<true>(best);
        int bidx = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j) {
            const int e = j * 64 + lane;
            const uint64_t owners = __ballot(e < experts && !((used >> j) & 1u) && v[j] == best);
            if (bidx == 0x7fffffff && owners) bidx = j * 64 + (__ffsll((long long)owners) - 1);
        }
        if ((bidx & 63) == lane) used |= 1u << (bidx >> 6);
        const float p = zb_expf(best - mx) / sum;
        wsum += p;
        if (lane == k) { myw = p; myidx = bidx; }
    }
    if (lane < topk) {
        if (idx_is_i64) static_cast<int64_t *>(topk_idx)[(int64_t)t * topk + lane] = myidx;
        else static_cast<int32_t *>(topk_idx)[(int64_t)t * topk + lane] = myidx;
        topk_w[(int64_t)t * topk + lane] = myw / wsum;
    }
}

__global__ void fill_i32_kernel(int32_t *p, int64_t n, int32_t v)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = v;
}

inline int ceil_log2(int64_t v)
{
    int b = 0;
    while ((1ll << b) < v) ++b;
    return b;
}

} // namespace

/* Used by the other translation units of the library (fused path, low-latency dispatch). */
int32_t zbalhip_layout_internal(const void *idx, int32_t idx_is_i64, int64_t tokens, int64_t experts, int64_t topk,
                                int32_t ranks, int32_t *tokens_per_rank, int32_t *send_token_idx, int32_t *scratch,
                                int max_blocks, int *nblk_out, hipStream_t st)
{
    const LayoutPlan p = plan_layout(tokens, topk, max_blocks);
    const int nbits = ceil_log2(experts);
    if (idx_is_i64) {
        layout_hist_kernel<int64_t><<<p.nblk, ZB_LAYOUT_THREADS, 0, st>>>(
            (const int64_t *)idx, (int)tokens, (int)topk, (int)experts, ranks, p.tokens_per_block, scratch,
            tokens_per_rank);
        layout_rank_kernel<int64_t><<<p.nblk, ZB_LAYOUT_THREADS, 0, st>>>(
            (const int64_t *)idx, (int)tokens, (int)topk, (int)experts, ranks, p.tokens_per_block, nbits, scratch,
            send_token_idx, tokens_per_rank);
    } else {
        layout_hist_kernel<int32_t><<<p.nblk, ZB_LAYOUT_THREADS, 0, st>>>(
            (const int32_t *)idx, (int)tokens, (int)topk, (int)experts, ranks, p.tokens_per_block, scratch,
            tokens_per_rank);
        layout_rank_kernel<int32_t><<<p.nblk, ZB_LAYOUT_THREADS, 0, st>>>(
            (const int32_t *)idx, (int)tokens, (int)topk, (int)experts, ranks, p.tokens_per_block, nbits, scratch,
            send_token_idx, tokens_per_rank);
    }
    *nblk_out = p.nblk;
    return zbalhip_check_launch();
}

/* ranks + offsets in one launch (no per-rank counts, no scratch) */
int32_t zbalhip_layout_fused_internal(const int32_t *idx, int64_t tokens, int64_t experts, int64_t topk,
                                      int32_t token_nums_type, const uint8_t *active_mask, int32_t *send_token_idx,
                                      int32_t *incl_i32, int32_t *row_off, int64_t *counts_i64, int64_t *nums_typed,
                                      hipStream_t st)
{
    const LayoutPlan p = plan_layout(tokens, topk, 64);
    layout_fused_kernel<int32_t><<<p.nblk, ZB_FUSED_THREADS, 0, st>>>(idx, (int)tokens, (int)topk, (int)experts,
                                                                    p.tokens_per_block, ceil_log2(experts), token_nums_type,
                                                                    active_mask, send_token_idx, incl_i32, row_off,
                                                                    counts_i64, nums_typed);
    return zbalhip_check_launch();
}

/* ranks within token ranges + one histogram per range, for the permute kernel's table mode; returns the ranges' size */
int32_t zbalhip_layout_ranges_internal(const int32_t *idx, int64_t tokens, int64_t experts, int64_t topk,
                                       const uint8_t *active_mask, int32_t *send_token_idx, int32_t *hist, int nblk,
                                       int tokens_per_block, hipStream_t st)
{
    /*
     * Ranking costs a block about 0.2 + 0.017 x experts microseconds per 1024 picks (32 experts: 5.0 us for 5248
     * picks; 128 experts: 21 us for 8192): slices of so many picks that a block is through in about five.
     */
    int64_t slice_picks = 1024 * (int64_t)(5.0 / (0.2 + 0.017 * (double)experts));
    if (slice_picks < 1024) slice_picks = 1024;
    int64_t subs = ((int64_t)tokens_per_block * topk + slice_picks - 1) / slice_picks;
    subs = subs < 1 ? 1 : (subs > 8 ? 8 : subs);
    if (subs > tokens_per_block) subs = tokens_per_block;
    if (subs == 1)
        layout_ranges_kernel<int32_t, false><<<(unsigned)nblk, ZB_FUSED_THREADS, 0, st>>>(
            idx, (int)tokens, (int)topk, (int)experts, tokens_per_block, 1, ceil_log2(experts), active_mask, send_token_idx, hist);
    else
        layout_ranges_kernel<int32_t, true><<<(unsigned)(nblk * subs), ZB_FUSED_THREADS, 0, st>>>(
            idx, (int)tokens, (int)topk, (int)experts, tokens_per_block, (int)subs, ceil_log2(experts), active_mask,
            send_token_idx, hist);
    return zbalhip_check_launch();
}

int32_t zbalhip_ll_counts_internal(const int32_t *const *ids, int ranks, int me, int64_t tokens, int64_t topk,
                                   int64_t experts, int32_t token_nums_type, int32_t *all_counts, int32_t *ep_recv_counts,
                                   int64_t *expert_token_nums, hipStream_t st)
{
    IdsOfRanks all = {};
    for (int r = 0; r < ranks; ++r) all.p[r] = ids[r];
    const int threads = (int)((experts + 63) / 64 * 64);
    ll_counts_kernel<<<1, threads, 0, st>>>(all, ranks, me, (int)tokens, (int)topk, (int)experts, token_nums_type, all_counts,
                                            ep_recv_counts, expert_token_nums);
    return zbalhip_check_launch();
}

int32_t zbalhip_scan_internal(const int32_t *hist, int nblk, int64_t experts, int64_t topk, int32_t token_nums_type,
                              int32_t *counts_i32, int32_t *excl_i32, int32_t *incl_i32, int32_t *row_off,
                              int64_t *counts_i64, int64_t *nums_typed, int32_t *total, int32_t *balance,
                              hipStream_t st)
{
    int threads = (int)((experts + 63) / 64 * 64);
    layout_scan_kernel<<<1, threads, 0, st>>>(hist, nblk, (int)experts, (int)topk, token_nums_type, counts_i32,
                                              excl_i32, incl_i32, row_off, counts_i64, nums_typed, total, balance);
    return zbalhip_check_launch();
}

static bool layout_args_ok(int64_t tokens, int64_t experts, int64_t topk)
{
    return tokens >= 0 && tokens <= 0x7fffffff / (topk > 0 ? topk : 1) && experts > 0 && experts <= ZB_MAX_EXPERTS &&
           topk > 0;
}

extern "C" int32_t zbalhip_fill_i32(int32_t *p, int64_t n, int32_t value, void *stream)
{
    if (n < 0 || (n > 0 && !p)) return ZBALHIP_INVALID;
    if (n == 0) return ZBALHIP_OK;
    int64_t blocks = (n + 255) / 256;
    if (blocks > 1024) blocks = 1024;
    fill_i32_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(p, n, value);
    return zbalhip_check_launch();
}

extern "C" int32_t zbalhip_topk_route(const float *logits, int64_t tokens, int64_t experts, int64_t topk,
                                      void *topk_idx, int32_t idx_is_i64, float *topk_w, void *stream)
{
    if (!logits || !topk_idx || !topk_w || tokens < 0 || experts <= 0 || experts > ZB_MAX_EXPERTS || topk <= 0 ||
        topk > 32 || topk > experts)
        return ZBALHIP_INVALID;
    if (tokens == 0) return ZBALHIP_OK;
    const int wpb = 4;
    const int64_t blocks = (tokens + wpb - 1) / wpb;
    const dim3 grid((unsigned)blocks), block(wpb * 64);
    hipStream_t st = (hipStream_t)stream;
    if (experts <= 64) topk_route_small_kernel<<<grid, block, 0, st>>>(logits, (int)tokens, (int)experts, (int)topk, topk_idx, idx_is_i64, topk_w);
    else if (experts <= 128) topk_route_kernel<2><<<grid, block, 0, st>>>(logits, (int)tokens, (int)experts, (int)topk, topk_idx, idx_is_i64, topk_w);
    else if (experts <= 256) topk_route_kernel<4><<<grid, block, 0, st>>>(logits, (int)tokens, (int)experts, (int)topk, topk_idx, idx_is_i64, topk_w);
    else topk_route_kernel<ZB_MAX_EXPERTS / 64><<<grid, block, 0, st>>>(logits, (int)tokens, (int)experts, (int)topk, topk_idx, idx_is_i64, topk_w);
    return zbalhip_check_launch();
}

extern "C" int32_t zbalhip_dispatch_layout(const void *topk_idx, int32_t idx_is_i64, int64_t tokens, int64_t experts,
                                           int64_t topk, int32_t ranks, int32_t *tokens_per_rank,
                                           int32_t *tokens_per_expert, int32_t *send_token_idx, int32_t *scratch,
                                           void *stream)
{
    if (!topk_idx || !tokens_per_rank || !tokens_per_expert || !send_token_idx || !scratch) return ZBALHIP_INVALID;
    if (!layout_args_ok(tokens, experts, topk) || ranks <= 0 || ranks > experts || experts % ranks != 0)
        return ZBALHIP_INVALID;
    int nblk = 0;
    int32_t rc = zbalhip_layout_internal(topk_idx, idx_is_i64, tokens, experts, topk, ranks, tokens_per_rank,
                                         send_token_idx, scratch, ZBALHIP_LAYOUT_MAX_BLOCKS, &nblk,
                                         (hipStream_t)stream);
    if (rc != ZBALHIP_OK) return rc;
    return zbalhip_scan_internal(scratch, nblk, experts, topk, 1, tokens_per_expert, nullptr, nullptr, nullptr, nullptr,
                                 nullptr, nullptr, nullptr, (hipStream_t)stream);
}

extern "C" int32_t zbalhip_dispatch_layout_static(const void *topk_idx, int32_t idx_is_i64, int64_t tokens, int64_t experts,
                                                  int64_t topk, int32_t ranks, int32_t *tokens_per_rank,
                                                  int32_t *tokens_per_expert, int32_t *send_token_idx, void *stream)
{
    if (!topk_idx || !tokens_per_rank || !tokens_per_expert || !send_token_idx) return ZBALHIP_INVALID;
    if (experts > ZBALHIP_LAYOUT_STATIC_MAX_EXPERTS) {
        zbalhip_set_last_error("zbalhip_dispatch_layout_static: more experts than the static scratch holds (1024)");
        return ZBALHIP_INVALID;
    }
    if (!layout_args_ok(tokens, experts, topk) || ranks <= 0 || ranks > experts || experts % ranks != 0)
        return ZBALHIP_INVALID;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= ZB_MAX_DEVICES) return ZBALHIP_RT_ERROR;
    StaticScratch *ss = static_scratch_of(dev);
    if (ss == nullptr) return ZBALHIP_RT_ERROR;
    hipStream_t st = (hipStream_t)stream;
    /*
     * Under stream capture the order of the array's users is the captured graph's own business (an event recorded
     * outside of the capture cannot be waited for inside it); everywhere else this call queues behind the last one.
     */
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    const bool capturing = st != nullptr && hipStreamIsCapturing(st, &capture) == hipSuccess && capture != hipStreamCaptureStatusNone;
    std::lock_guard<std::mutex> guard(ss->mu);
    if (!capturing && hipStreamWaitEvent(st, ss->last_use, 0) != hipSuccess) return ZBALHIP_RT_ERROR;
    /* the histogram kernel writes every row that the rank and scan kernels read: nothing has to start at zero */
    int nblk = 0;
    int32_t rc = zbalhip_layout_internal(topk_idx, idx_is_i64, tokens, experts, topk, ranks, tokens_per_rank,
                                         send_token_idx, ss->addr, ZBALHIP_LAYOUT_MAX_BLOCKS, &nblk, st);
    if (rc == ZBALHIP_OK)
        rc = zbalhip_scan_internal(ss->addr, nblk, experts, topk, 1, tokens_per_expert, nullptr, nullptr, nullptr, nullptr,
                                   nullptr, nullptr, nullptr, st);
    if (!capturing && hipEventRecord(ss->last_use, st) != hipSuccess && rc == ZBALHIP_OK) rc = ZBALHIP_RT_ERROR;
    return rc;
}

extern "C" int32_t zbalhip_dispatch_notify(const int32_t *const *tokens_per_expert, int32_t ranks, int32_t my_rank,
                                           int64_t experts, int64_t topk, int32_t *recv_data, int32_t *put_offset,
                                           int32_t *total_recv, int64_t *recv_tokens_per_expert, int32_t *balance_matrix,
                                           void *stream)
{
    if (!tokens_per_expert || !recv_data || !put_offset || !total_recv || !recv_tokens_per_expert || !balance_matrix)
        return ZBALHIP_INVALID;
    if (experts <= 0 || experts > ZB_MAX_EXPERTS || topk <= 0) return ZBALHIP_INVALID;
    if (ranks <= 0 || ranks > ZBALHIP_MAX_REDUCE_PEERS || my_rank < 0 || my_rank >= ranks || experts % ranks != 0)
        return ZBALHIP_INVALID;
    for (int r = 0; r < ranks; ++r)
        if (!tokens_per_expert[r]) return ZBALHIP_INVALID;
    if (ranks == 1)
        return zbalhip_scan_internal(tokens_per_expert[0], 0, experts, topk, 1, recv_data, put_offset, nullptr, nullptr,
                                     recv_tokens_per_expert, nullptr, total_recv, balance_matrix, (hipStream_t)stream);
    CountsOfRanks counts = {};
    for (int r = 0; r < ranks; ++r) counts.p[r] = tokens_per_expert[r];
    const int threads = (int)((experts + 63) / 64 * 64);
    notify_ranks_kernel<<<1, threads, 0, (hipStream_t)stream>>>(counts, ranks, my_rank, (int)experts, (int)topk, recv_data,
                                                                put_offset, total_recv, recv_tokens_per_expert,
                                                                balance_matrix);
    return zbalhip_check_launch();
}
