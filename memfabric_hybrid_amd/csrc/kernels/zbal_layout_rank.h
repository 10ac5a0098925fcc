/*
 * Stable ranking of a block's picks, shared by the layout kernels and by the permute kernel that carries the layout
 * of large batches along (dispatch.hip).
 */
#ifndef ZBAL_LAYOUT_RANK_H_
#define ZBAL_LAYOUT_RANK_H_

#include "zbal_device.h"

/*
 * Stable ranks of the picks [p0, p1) of one block: `run[e]` holds the number of earlier picks of expert e on entry
 * and the number up to p1 on return. Picks are taken 64 per wave at a time; lanes holding the same expert find
 * each other by intersecting one ballot per index bit. The waves do not take turns: each leaves the size of its
 * groups in `cnt` (one byte per wave and expert, a group has at most 64 members) and a pick's rank is the running
 * count plus the groups of the waves before its own. Ends on a barrier.
 */
template <typename IdxT>
__device__ __forceinline__ void rank_picks(const IdxT *__restrict__ idx, int64_t p0, int64_t p1, int experts, int nbits,
                                           int32_t *run, uint8_t *cnt /* [waves][experts rounded up to 4] */,
                                           int32_t *__restrict__ send_token_idx)
{
    const int np = (int)(p1 - p0);
    const int threads = blockDim.x, nwaves = threads >> 6;
    const int iters = (np + threads - 1) / threads;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    const int pad = (experts + 3) & ~3;

    for (int it = 0; it < iters; ++it) {
        const int64_t i = p0 + (int64_t)it * threads + threadIdx.x;
        int64_t e64 = (i < p1) ? (int64_t)idx[i] : -1;
        for (int j = threadIdx.x; j < nwaves * pad / 4; j += threads) reinterpret_cast<uint32_t *>(cnt)[j] = 0u;
        const bool valid = (e64 >= 0 && e64 < experts);
        const int e = valid ? (int)e64 : 0;
        uint64_t peers = __ballot(valid);
        for (int bit = 0; bit < nbits; ++bit) {
            const bool one = (e >> bit) & 1;
            const uint64_t bal = __ballot(valid && one);
            peers &= one ? bal : ~bal;
        }
        const int before = __popcll(peers & lt_mask);
        const int group = __popcll(peers);
        const bool last = valid && ((peers >> lane) >> 1) == 0; /* highest lane of its group */
        __syncthreads();
        if (last) cnt[wave * pad + e] = (uint8_t)group;
        __syncthreads();
        if (valid) {
            int32_t basev = run[e];
            for (int w = 0; w < wave; ++w) basev += cnt[w * pad + e];
            send_token_idx[i] = basev + before;
        } else if (i < p1) {
            send_token_idx[i] = -1;
        }
        __syncthreads();
        for (int e2 = threadIdx.x; e2 < experts; e2 += threads) {
            int32_t sum = 0;
            for (int w = 0; w < nwaves; ++w) sum += cnt[w * pad + e2];
            run[e2] += sum;
        }
        __syncthreads();
    }
}

#endif /* ZBAL_LAYOUT_RANK_H_ */
