/*
 * Inner C ABI: the HIP kernel launchers the zbal operator layer sits on.
 *
 * This is the seam the reference calls "zbal_kernel": its host launchers
 * ZBALOp* (app/zbal/src/csrc/operators/npu/zbal_npu_operators.h:18-97) take
 * tensor descriptors and a CommGroupInfo; the functions below take the same
 * information as plain device pointers and sizes so that C, ctypes, cgo or
 * JNI callers can drive the kernels without the communicator layer.
 *
 * Conventions: every pointer is a device pointer unless stated; `stream` is
 * a hipStream_t passed as void* (NULL = null stream); launches are
 * asynchronous; the return value is 0 or a negative ZResult (-2 invalid
 * parameter, -11 HIP runtime error). Unless a function takes `ranks`, one
 * rank owns all `experts`; rows of the permuted activation matrix are
 * expert-major in flat (t,k) pick order. dtype arguments are zbal_datatype_t
 * values.
 */
#ifndef ZBAL_HIP_KERNELS_H_
#define ZBAL_HIP_KERNELS_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* exported even when the library is built with hidden default visibility */
#define ZBALHIP_API __attribute__((visibility("default")))

#define ZBALHIP_MAX_REDUCE_PEERS 16
#define ZBALHIP_LAYOUT_MAX_BLOCKS 50 /* scratch rows, reference dispatch_layout.h:33 (MAX_BLOCK) */

/*
 * Router (no reference counterpart). logits [T,E] fp32 -> topk_idx [T,K]
 * int64 (idx_is_i64 != 0, the type the layout operator takes) or int32 (the
 * type the dispatch and fused operators take), topk_w [T,K] fp32.
 * E <= 1024, K <= 32, K <= E.
 */
ZBALHIP_API int32_t zbalhip_topk_route(const float *logits, int64_t tokens, int64_t experts, int64_t topk, void *topk_idx,
                           int32_t idx_is_i64, float *topk_w, void *stream);

/*
 * Replaces ZBALOpDispatchLayout (zbal_npu_operators.h:47-50; kernel
 * dispatch_layout.h:97-183). idx_is_i64 selects int64 or int32 indices.
 * Outputs: tokens_per_rank [ranks] i32, tokens_per_expert [experts] i32,
 * send_token_idx [T,K] i32 (-1 for picks outside [0,experts)).
 * scratch: [ZBALHIP_LAYOUT_MAX_BLOCKS * experts] i32, contents undefined after.
 */
ZBALHIP_API int32_t zbalhip_dispatch_layout(const void *topk_idx, int32_t idx_is_i64, int64_t tokens, int64_t experts, int64_t topk,
                                int32_t ranks, int32_t *tokens_per_rank, int32_t *tokens_per_expert,
                                int32_t *send_token_idx, int32_t *scratch, void *stream);

/*
 * zbalhip_dispatch_layout for callers that cannot allocate device memory
 * (code under HIP graph capture, serving loops and harnesses that forbid
 * hipMalloc). No counterpart in the reference. Same arguments, outputs and
 * results as zbalhip_dispatch_layout, minus `scratch`: the per-block
 * histograms live in a file-scope device array of the library
 * (ZBALHIP_LAYOUT_MAX_BLOCKS * ZBALHIP_LAYOUT_STATIC_MAX_EXPERTS int32 =
 * 200 KiB on every GPU the library runs on, held until the process ends).
 * The call allocates and frees nothing. experts above
 * ZBALHIP_LAYOUT_STATIC_MAX_EXPERTS is refused with -2 and a last-error text.
 * All calls on one GPU share that array: calls that overlap on one GPU
 * (different streams, different threads) race; order them on one stream.
 * The first call on a GPU looks up the array's device address
 * (hipGetSymbolAddress): make it before a graph capture starts.
 */
#define ZBALHIP_LAYOUT_STATIC_MAX_EXPERTS 1024
ZBALHIP_API int32_t zbalhip_dispatch_layout_static(const void *topk_idx, int32_t idx_is_i64, int64_t tokens, int64_t experts,
                                       int64_t topk, int32_t ranks, int32_t *tokens_per_rank,
                                       int32_t *tokens_per_expert, int32_t *send_token_idx, void *stream);

/*
 * Replaces ZBALOpNotifyDispatch (zbal_npu_operators.h:52-56; kernel
 * notify_dispatch.h:356-596) from the point of view of rank `my_rank` of
 * `ranks`. tokens_per_expert is a HOST array of `ranks` device pointers:
 * entry s is rank s's per-expert counts [experts], read where they lie in that
 * rank's window (one GPU: local allocations). Outputs: recv_data
 * [ranks, experts] = the counts; put_offset [ranks * experts]: for every
 * destination rank r, put_offset[r * experts + le * ranks + s] = exclusive
 * running sum of counts[s][r * E_loc + le] in (local expert, source rank)
 * order; total_recv [1] and recv_tokens_per_expert [experts / ranks] i64 for
 * this rank; balance_matrix [ranks, 2 * ranks] = -1 except {0, tokens_i - 1}
 * at [i, 2i], [i, 2i + 1] (no re-balancing). ranks == 1: put_offset is the
 * exclusive cumsum of the counts and balance_matrix {0, tokens - 1}.
 */
ZBALHIP_API int32_t zbalhip_dispatch_notify(const int32_t *const *tokens_per_expert, int32_t ranks, int32_t my_rank,
                                int64_t experts, int64_t topk, int32_t *recv_data, int32_t *put_offset,
                                int32_t *total_recv, int64_t *recv_tokens_per_expert, int32_t *balance_matrix,
                                void *stream);

/*
 * Replaces ZBALOpDispatchNormal (zbal_npu_operators.h:58-62; kernel
 * dispatch_normal.h:479-563). quant_mode: 0 copy, 1 int8 per token with
 * s = 127/(amax+1e-12), 2 e4m3 with 1x128 scales (dest_scale [rows, H/128]).
 * x_dtype: BFP16 or FP16. hidden % 16 == 0 (mode 2: % 128 == 0).
 * dest / dest_scale are HOST arrays of `ranks` device pointers: the receive
 * windows of the ranks (one GPU: local allocations; dest_scale may be null
 * for mode 0). The row of a pick of global expert e goes to window
 * e / (experts / ranks), row put_offset[e * ranks + my_rank] +
 * send_token_idx (dispatch_normal.h:528-533). dest_rows = rows every window
 * holds: a pick that would land past it is dropped, never written out of
 * bounds.
 */
ZBALHIP_API int32_t zbalhip_dispatch_normal(const void *x, int32_t x_dtype, const int32_t *topk_idx, const int32_t *send_token_idx,
                                const int32_t *put_offset, int64_t tokens, int64_t hidden, int64_t topk,
                                int64_t experts, int32_t quant_mode, void *const *dest, float *const *dest_scale,
                                int32_t ranks, int32_t my_rank, int64_t dest_rows, void *stream);

/*
 * Replaces ZBALOpCombineNormal (zbal_npu_operators.h:64-68; kernel
 * combine_normal.h:398-494): out[t] = round(sum_k fp32(row) * w), multiply
 * and add rounded separately, k ascending, invalid ids skipped; a token with
 * send_token_idx = -2 on any pick (or a valid id with a negative
 * send_token_idx) is not written at all: that is how the fused operator's
 * layout marks the tokens past the active ones. y is a HOST array
 * of `ranks` device pointers (the windows the rows were dispatched to, y_rows
 * rows each; a row past that is skipped); the row of a pick of expert e is
 * row base[e * ranks + my_rank] + send_token_idx of window e / (experts /
 * ranks). base_is_inclusive = 1 reads `base` as the low-latency kernels'
 * inclusive running counts (combine_low_latency.h:504-506): the rows of index
 * i = e * ranks + my_rank start at base[i - 1], at 0 where i is a multiple
 * of `experts` (every rank's block of counts starts anew).
 */
ZBALHIP_API int32_t zbalhip_combine(const void *const *y, int32_t ranks, int32_t my_rank, int64_t y_rows, int32_t dtype,
                        const int32_t *base, int32_t base_is_inclusive, const float *w, const int32_t *topk_idx,
                        const int32_t *send_token_idx, int64_t tokens, int64_t hidden, int64_t topk, int64_t experts,
                        void *out, void *stream);

/*
 * Replaces ZBALOpDispatchLowLatency (zbal_npu_operators.h:70-77; kernel
 * dispatch_low_latency.h:528-844) for one rank: layout, counts and the
 * quantising permute in one call. quant_mode 1 uses s = 127/amax (an
 * all-zero row gives q = 0, scale = 0). ep_recv_counts [E] = inclusive
 * running sum; expert_token_nums [E] i64 = counts (type 1) or the running
 * sum (type 0). scratch (scratch_blocks * experts i32, scratch_blocks >= 1)
 * mirrors the reference's putOffset operand; the layout is computed in one
 * launch that does not touch it.
 */
ZBALHIP_API int32_t zbalhip_dispatch_low_latency(const void *x, int32_t x_dtype, const int32_t *expert_ids, int64_t tokens,
                                     int64_t hidden, int64_t topk, int64_t experts, int32_t quant_mode,
                                     int32_t token_nums_type, void *expand_x, float *dynamic_scales,
                                     int32_t *expand_idx, int64_t *expert_token_nums, int32_t *ep_recv_counts,
                                     int32_t *scratch, int32_t scratch_blocks, void *stream);

/*
 * The same for a group of `ranks` modelled ranks (kernel
 * dispatch_low_latency.h: counts of all ranks :344-345, 641-713, rows sent to
 * the rank that owns the expert :760-844). expert_ids, expand_x and
 * dynamic_scales are HOST arrays of `ranks` device pointers: every rank's
 * [tokens, topk] ids (the reference's ranks push their counts to each other
 * and wait; here the other ranks' ids are read where they lie, all ranks
 * with the same tokens and topk) and every rank's receive window (dest_rows
 * rows each; a row past that is dropped). all_counts [ranks * experts] =
 * picks of expert e by rank s at s * experts + e (the reference's putOffset
 * operand); ep_recv_counts [ranks * experts] = inclusive running sums at
 * r * experts + le * ranks + s, starting anew for every destination rank r;
 * expert_token_nums [experts / ranks] = what this rank receives per local
 * expert (type 1) or the running sum (type 0); expand_idx [tokens, topk] =
 * rank of each of this rank's picks among its own earlier picks of the same
 * expert. A pick of expert e lands in window e / (experts / ranks) at row
 * start(e * ranks + my_rank) + expand_idx.
 */
ZBALHIP_API int32_t zbalhip_dispatch_low_latency_ranks(const void *x, int32_t x_dtype, const int32_t *const *expert_ids,
                                           int64_t tokens, int64_t hidden, int64_t topk, int64_t experts,
                                           int32_t quant_mode, int32_t token_nums_type, void *const *expand_x,
                                           float *const *dynamic_scales, int32_t ranks, int32_t my_rank,
                                           int64_t dest_rows, int32_t *expand_idx, int64_t *expert_token_nums,
                                           int32_t *ep_recv_counts, int32_t *all_counts, void *stream);

/*
 * Device trace ring (reference aicore/common/zbal_kernel_trace.h:22-62, layout
 * constants zbal_comm_host_device_struct.h:22-25). The ring is host memory the
 * GPU can write: ZBALHIP_TRACE_UNITS blocks of `points` 64-bit words; word
 * [ZBALHIP_TRACE_IDX_OFF] of a block is the index of its newest record and
 * records start at [ZBALHIP_TRACE_REC_OFF]. A record is
 * frame << 56 | end << 62 | timestamp, the timestamp in ticks of the GPU's
 * constant 100 MHz clock. Workgroup b < ZBALHIP_TRACE_UNITS of a traced kernel
 * writes to block b (one lane, begin and end of each frame); a block that is
 * full drops further records.
 *   zbalhip_trace_alloc: pinned, zeroed host memory and its device address;
 *     the owner (a communicator) passes that address to the launches it wants
 *     traced, so every communicator has a ring of its own.
 *   zbalhip_trace_sync: waits until the device is idle, so that the ring holds
 *     every record of the kernels launched so far.
 *   zbalhip_trace_free: waits for the device, then releases the memory.
 */
#define ZBALHIP_TRACE_UNITS 64
#define ZBALHIP_TRACE_IDX_OFF 8
#define ZBALHIP_TRACE_REC_OFF 16
#define ZBALHIP_TRACE_FRAME_SHIFT 56
#define ZBALHIP_TRACE_BE_SHIFT 62
ZBALHIP_API int32_t zbalhip_trace_alloc(int64_t points, uint64_t **host_ring, uint64_t **device_ring);
ZBALHIP_API int32_t zbalhip_trace_sync(void);
ZBALHIP_API int32_t zbalhip_trace_free(uint64_t *host_ring);

/*
 * The local reduction under ZBALOpReduceScatter / ZBALOpAllReduce
 * (zbal_npu_operators.h:21-25; kernels reducescatter.cpp:94-151,
 * allreduce.cpp:206-260): out[j] = op over p = 0..n_in-1 of in[p][j].
 * `in` is a HOST array of n_in <= ZBALHIP_MAX_REDUCE_PEERS device pointers.
 * Float types accumulate in fp32 in order p = 0..n_in-1 and round once.
 * Every pointer must hold whole elements. 16-byte vectors are used when all
 * pointers sit at the same offset from a 16-byte boundary (aligned buffers,
 * or equal slices of equal windows written to a slice of the same kind; a few
 * leading elements are then handled one by one); pointers at different
 * offsets are reduced element by element, several times slower.
 * op is a zbal_reduce_op_t value; PROD is a true product. trace_frame != 0
 * (a zbal_profiling_name_t value of the reference,
 * zbal_comm_host_device_struct.h:27-70) records that frame around each traced
 * workgroup's work in `trace_ring` (device address from zbalhip_trace_alloc,
 * `trace_points` words per block; null = not traced).
 */
ZBALHIP_API int32_t zbalhip_reduce(const void *const *in, int32_t n_in, int64_t count, int32_t dtype, int32_t op, void *out,
                       int32_t trace_frame, uint64_t *trace_ring, int64_t trace_points, void *stream);

/* p[0..n) = value, as a kernel (safe to record into a HIP graph, unlike a memset node) */
ZBALHIP_API int32_t zbalhip_fill_i32(int32_t *p, int64_t n, int32_t value, void *stream);

/*
 * Weight pre-pack of [E,K,N] (N contiguous). One byte per element:
 * [E][N/128][K/128] blocks of 128 channels x 128 K-bytes, block row r at
 * +128*r with 16-byte chunk c in slot c ^ (r & 7) ^ ((r >> 3) & 1); k and n
 * multiples of 128, pointers 16-byte aligned. Block row r holds channel
 * (r & ~31) | ((r & 15) >> 2) << 3 | ((r >> 4) & 1) << 2 | (r & 3) of the
 * block: a lane of the GEMM then ends up with eight consecutive channels.
 * to_int4 != 0 packs int8 values in [-8,7] two per byte into
 * [E][N/128][K/128] blocks of 8 KiB (block row r, the same channel as above,
 * at +64*r, 16-byte chunk c of 32 k in slot c ^ ((r >> 2) & 3), byte b of
 * dword j = k[8j+b] | k[8j+4+b] << 4). The grouped GEMMs below take `w1` /
 * `w2` in this form.
 */
ZBALHIP_API int32_t zbalhip_weight_prepack(const void *src, int64_t experts, int64_t k, int64_t n, int32_t to_int4, void *dst,
                               void *stream);

/*
 * Permute + quantise stage of the fused operator (QuantToken /
 * LocalQuantFunc, FDM/gemm/kernel/…swiglu_quant_multistage_workspace.h:
 * 952-995, 1859-2058). mode 1: int8, s = 127/amax, optional smooth [E,H]
 * fp32 multiplied in first; mode 2: e4m3 1x128. Outputs q1 [rows,H], xs
 * ([rows] or [rows,H/128]), expand_idx [T,K], counts [E] i64 and the
 * exclusive row offsets row_off [E+1] i32. The launch also sets clear_count
 * 32-bit words at clear_words to zero (0 / null for none): the row maxima that
 * the int modes' first GEMM accumulates into, so that it needs no fill launch
 * of its own (ZBALHIP_ROWMAX_CLEARED). With at most 4096 picks (tokens x topk)
 * the permute kernel works the layout out itself and the stage is one launch.
 * Larger batches: when `scratch` holds scratch_blocks x experts int32
 * (scratch_blocks >= 1; up to one block per 1024 picks ranks faster) and there
 * are at most 256 experts, the layout launch in front of the permute launch
 * only ranks the picks within token ranges and leaves one histogram per range
 * there; the permute workgroups derive offsets from those themselves while
 * their rows are in flight. Otherwise (scratch_blocks = 0) the layout launch
 * does all of it.
 * active_mask (optional, one byte per token): only the first
 * sum(mask) tokens are routed, as in the reference's TokenActiveMaskCal
 * (…swiglu_quant_multistage_workspace.h:836-863); the picks of the others get
 * expand_idx = -2, which zbalhip_combine reads as "leave this token's output
 * row alone" (-1 is a pick with an invalid expert id: it contributes nothing,
 * but its token's row is still written).
 */
ZBALHIP_API int32_t zbalhip_fused_permute_quant(const void *x, int32_t x_dtype, const int32_t *expert_ids, const float *smooth,
                                    const uint8_t *active_mask,
                                    int64_t tokens, int64_t hidden, int64_t topk, int64_t experts, int32_t mode,
                                    void *q1, float *xs, int32_t *expand_idx, int64_t *counts, int32_t *row_off,
                                    uint32_t *clear_words, int64_t clear_count, int32_t *scratch, int32_t scratch_blocks,
                                    void *stream);

/*
 * OR-ed into `mode` of the two grouped GEMMs: `w1`/`w2` and their scales are
 * not one stacked tensor each but device arrays of `experts` 64-bit addresses,
 * entry e = expert e's pre-packed weights / its scales (16-byte aligned;
 * the reference's EXEC_FLAG_TENSOR_LIST,
 * …swiglu_quant_multistage_workspace.h:669-673, 755-757, 1531-1558).
 */
#define ZBALHIP_WEIGHTS_AS_LISTS 0x100
/*
 * OR-ed into `mode` of zbalhip_gmm1_swiglu_quant (int modes): the row maxima
 * behind the SwiGLU values in sgl_ws (max_rows words at sgl_ws + max_rows *
 * N1/2) are already zero - the permute launch cleared them - so the GEMM
 * launches no fill kernel of its own.
 */
#define ZBALHIP_ROWMAX_CLEARED 0x200

/*
 * Grouped GEMM 1 with dequant + SwiGLU + requant epilogue (AIC loop
 * …swiglu_quant_multistage_workspace.h:603-833, epilogue
 * block_epilogue_per_token_dequant_swiglu.h:171-298, BlockQuant
 * …workspace.h:87-316). a [rows,K] expert-major; w1 pre-packed [E,N1,K];
 * row_off [E+1] exclusive offsets (device). mode 1 (W8A8): w1scale fp32
 * [E,N1]; q2 int8 [rows,N1/2], scale2 [rows]; sgl_ws is scratch of
 * max_rows * (N1/2 + 1) * 4 bytes (fp32 SwiGLU values, then one row maximum
 * each). mode 2 (fp8): a_scale [rows,K/128], w1scale fp32
 * [E,K/128,N1/128]; q2 e4m3, scale2 [rows,N1/256]; sgl_ws unused.
 * mode 3 (W4A8): w1 pre-packed int4x2 (N1*K/2 bytes per expert), w1scale fp16 [E,K/128,N1];
 * outputs as mode 1. max_rows bounds the launch (>= total rows). a, w1,
 * w1scale, q2 and sgl_ws must be 16-byte aligned (here and for GMM 2: a, w2,
 * wscale, y), else ZBALHIP_INVALID.
 */
ZBALHIP_API int32_t zbalhip_gmm1_swiglu_quant(const void *a, const float *a_scale, const void *w1, const void *w1scale,
                                  const int32_t *row_off, int64_t experts, int64_t max_rows, int64_t k, int64_t n1,
                                  int32_t mode, void *q2, float *scale2, float *sgl_ws, void *stream);

/*
 * Grouped GEMM 2 with dequant epilogue (kernel
 * grouped_matmul_slice_m_per_token_dequant_multistage_workspace.h:166-548,
 * epilogue block_epilogue_per_token_dequant.hpp:265-397):
 * y[m,n] = round((float(C) * wscale[g,n]) * a_scale[m]) for mode 1
 * (wscale_dtype FP32 or BFP16, [E,N]); block-scaled for mode 2
 * (wscale fp32 [E,K/128,N/128], a_scale [rows,K/128]); group-scaled for
 * mode 3 (wscale fp16 [E,K/128,N]). w2 pre-packed [E,N,K]. y dtype BFP16/FP16.
 */
ZBALHIP_API int32_t zbalhip_gmm2_dequant(const void *a, const float *a_scale, const void *w2, const void *wscale,
                             int32_t wscale_dtype, const int32_t *row_off, int64_t experts, int64_t max_rows,
                             int64_t k, int64_t n, int32_t mode, int32_t out_dtype, void *y, void *stream);

/*
 * One-time set-up of every grouped-GEMM kernel on the current GPU (each raises its dynamic-LDS limit before its
 * first launch, which cannot be recorded into a graph). No counterpart in the reference. Optional: a launch whose
 * kernel is still unprepared does it itself, and refuses with an error if its stream is being captured. The host
 * layer calls it when a communicator is created.
 */
ZBALHIP_API int32_t zbalhip_gemm_prepare(void);

#ifdef __cplusplus
}
#endif

#endif /* ZBAL_HIP_KERNELS_H_ */
