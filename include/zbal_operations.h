/*
 * Operator entry points of the zbal API, MI355X build (outer C ABI).
 *
 * Each prototype is the one a client of the reference binds
 * (app/zbal/src/include/zbal_operations.h, line cited per function). The
 * semantics implemented are the one-GPU share of each operator: every "peer"
 * of a communicator is a local HBM allocation registered with
 * zbal_comm_register_peer_window(); there is no cross-device transport.
 *
 * Error convention (reference zbal_operations.cpp): 0 on success, a negative
 * ZResult otherwise (-2 = invalid parameter); text via
 * zbal_get_last_error_msg(). Launches are asynchronous on `stream`.
 */
#ifndef ZBAL_OPERATIONS_H_
#define ZBAL_OPERATIONS_H_

#include "zbal_def.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- communicator lifecycle: reference zbal_operations.h:28-68 ---- */
int32_t zbal_comm_create(zbal_comm_options_t *options, zbal_comm_t *comm);
int32_t zbal_comm_get_property(zbal_comm_t comm, zbal_comm_property_t *property);
zbal_comm_t zbal_comm_get_global();
zbal_comm_t zbal_comm_get_by_name(const char *name);
int32_t zbal_comm_destroy(zbal_comm_t comm, uint32_t flags);
void zbal_comm_destroy_all(uint32_t flags);

/*
 * extension: declare the HBM window that stands for group rank `rank` of
 * `comm`. A buffer address handed to a collective is translated to the same
 * offset inside every other rank's window, which is what the reference's
 * symmetric address arithmetic does (zbal_kernel_base.h:35-42).
 */
int32_t zbal_comm_register_peer_window(zbal_comm_t comm, uint16_t rank, void *base, uint64_t size);

/*
 * extension: write the communicator's device trace now (the reference does it
 * when the communicator is destroyed and on SIGUSR1, Communicator::
 * DumpProfilingTrace zbal_communicator.h:114, zbal_npu_communicator_base.cpp:
 * 215-276; both still happen here at destruction). Tracing is switched on
 * with the reference's environment variables, read when a communicator is
 * created: ZBAL_PROF_ENABLE=1, ZBAL_PROF_MAX_TRACING_COUNT, ZBAL_PROF_DIR.
 * The file is trace_view_<rank>_<group index>_<date>.json in ZBAL_PROF_DIR, a
 * trace-viewer (chrome://tracing) array of begin / end events, one "thread"
 * per traced workgroup. Returns 0, also when tracing is off.
 */
int32_t zbal_comm_dump_profiling_trace(zbal_comm_t comm);

/*
 * reference zbal_operations.h:82-83. One-GPU share: recv[j] = reduce over
 * ranks p = 0..R-1 of peer_p(send)[j] for all `count` elements (the
 * reduce-scatter phase of every slice followed by the all-gather, which on
 * one device is the identity). `buffer` is validated and unused.
 * Floating types accumulate in fp32 in rank order and round once.
 */
int32_t zbal_all_reduce(const void *send_buff, void *recv_buff, void *buffer, size_t count,
                        zbal_datatype_t data_type, zbal_reduce_op_t op, zbal_comm_t comm, aclrtStream stream);

/*
 * reference zbal_operations.h:97-98. recv[j] = reduce over p of
 * peer_p(send)[me * recv_count + j], j < recv_count.
 */
int32_t zbal_reduce_scatter(const void *sendBuff, void *recvBuff, size_t recv_count, zbal_datatype_t dataType,
                            zbal_reduce_op_t op, zbal_comm_t comm, aclrtStream stream);

/*
 * reference zbal_operations.h:111-209. The data-movement collectives need a transport between devices, which
 * is not part of this build: they are exported so that a client of the reference links unchanged, validate
 * nothing, set the last-error text and return Z_INVALID_PARAM.
 */
int32_t zbal_all_gather(const void *sendBuff, void *recvBuff, size_t send_count, zbal_datatype_t dataType,
                        zbal_comm_t comm, aclrtStream stream);
int32_t zbal_all_to_all_v(const void *sendBuff, void *recvBuff, void *sendCumSum, void *recvSplitCounts, void *elements,
                          zbal_datatype_t dataType, zbal_comm_t comm, aclrtStream stream);
int32_t zbal_broadcast(const void *buf, uint64_t data_count, zbal_datatype_t dataType, uint16_t root, zbal_comm_t comm,
                       aclrtStream stream);
int32_t zbal_scatter(const void *sendBuff, void *recvBuff, uint64_t data_count, zbal_datatype_t dataType, uint16_t root,
                     zbal_comm_t comm, aclrtStream stream);
int32_t zbal_gather(const void *sendBuff, void *recvBuff, uint64_t data_count, zbal_datatype_t dataType, uint16_t root,
                    zbal_comm_t comm, aclrtStream stream);
int32_t zbal_barrier(zbal_comm_t comm, aclrtStream stream);
int32_t zbal_send(const void *sendBuff, zbal_datatype_t dataType, uint32_t peer, zbal_comm_t comm, aclrtStream stream);
int32_t zbal_recv(const void *recvBuff, size_t recvCount, zbal_datatype_t dataType, uint32_t peer, zbal_comm_t comm,
                  aclrtStream stream);

/* reference zbal_operations.h:227-231 */
int32_t zbal_dispatch_normal_notify(const zbal_tensor_info_t *sendTokensPerExpert, int64_t sendCount, int64_t topKNum,
                                    const zbal_tensor_info_t *recvBuff, const zbal_tensor_info_t *totalRecvTokens,
                                    const zbal_tensor_info_t *recvTokensPerExpert,
                                    const zbal_tensor_info_t *pushTargetOffset, const zbal_tensor_info_t *balanceMatrix,
                                    zbal_comm_t comm, aclrtStream stream, int64_t flags);

/* reference zbal_operations.h:249-253 */
int32_t zbal_dispatch_normal_layout(const zbal_tensor_info_t *topkIndex, int64_t tokens, int64_t expertNum,
                                    int64_t topkNum, const zbal_tensor_info_t *tokensPerRank,
                                    const zbal_tensor_info_t *tokensPerExpert,
                                    const zbal_tensor_info_t *sendTokensIndex, const zbal_tensor_info_t *notifySendData,
                                    zbal_comm_t comm, aclrtStream stream, int64_t flags);

/* reference zbal_operations.h:272-276 */
int32_t zbal_dispatch_normal(const zbal_tensor_info_t *srcTokens, const zbal_tensor_info_t *topkIndex,
                             const zbal_tensor_info_t *sendTokensIndex, const zbal_tensor_info_t *pushTargetOffset,
                             const zbal_tensor_info_t *balanceMatrix, int64_t expertNum, zbal_quant_mode_t quantMode,
                             const zbal_tensor_info_t *destTokens, const zbal_tensor_info_t *destScale,
                             zbal_comm_t comm, aclrtStream stream, int64_t flags);

/* reference zbal_operations.h:294-298 */
int32_t zbal_combine_normal(const zbal_tensor_info_t *srcTokens, const zbal_tensor_info_t *srcTokensPerEp,
                            const zbal_tensor_info_t *topKWeight, const zbal_tensor_info_t *topkIndex,
                            const zbal_tensor_info_t *sendTokensIndex, const zbal_tensor_info_t *balanceMatrix,
                            uint16_t expertNum, const zbal_tensor_info_t *destTokens, zbal_comm_t comm,
                            aclrtStream stream, int64_t flags);

/* reference zbal_operations.h:300-307 */
int32_t zbal_dispatch_low_latency(const zbal_tensor_info_t *x, const zbal_tensor_info_t *expertIds,
                                  int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum,
                                  int64_t quantMode, int64_t globalBs, int64_t magicVal, int64_t expertTokenNumsType,
                                  const zbal_tensor_info_t *expandXOut, const zbal_tensor_info_t *dynamicScalesOut,
                                  const zbal_tensor_info_t *expandIdxOut, const zbal_tensor_info_t *expertTokenNumsOut,
                                  const zbal_tensor_info_t *epRecvCountsOut, const zbal_tensor_info_t *putOffset,
                                  const zbal_tensor_info_t *putOffsetStatus, zbal_comm_t comm, aclrtStream stream,
                                  int64_t flags);

/* reference zbal_operations.h:309-312 */
int32_t zbal_combine_low_latency(const zbal_tensor_info_t *expandX, const zbal_tensor_info_t *expertIds,
                                 const zbal_tensor_info_t *expertIdx, const zbal_tensor_info_t *epSendCounts,
                                 const zbal_tensor_info_t *expertScales, const zbal_tensor_info_t *xOut,
                                 int64_t moeExpertNum, zbal_comm_t comm, aclrtStream stream, int64_t flags);

/*
 * reference zbal_operations.h:343-354. quantMode 0 and 1 run the reference's
 * W8A8 pipeline (its kernel ignores the value); 2 = fp8 e4m3 with 1x128
 * activation scales and 128x128 weight scales; 3 = int8 activations with
 * int4 group-128 weights. Weights must be in ZBAL_WEIGHT_FORMAT_PREPACKED.
 * The shared expert (EXEC_FLAG_SHARED_EXPERT in the reference kernel,
 * zbal_kernel_fused_deep_moe.h:470-472) is one more expert applied to every
 * token: shareGmm1Weight [H, shareGmm1HLen] and shareGmm2Weight
 * [shareGmm1HLen/2, H] pre-packed like the others, scales shaped as one
 * expert's, optional shareSmoothScales [H]; its result goes to shareOutput
 * [tokens, H] and is not added to output. Pass all of them or none.
 * xActiveMask [tokens] (one byte per token): only the first sum(mask)
 * tokens are routed and written, as in the reference. isTensorList != 0
 * (EXEC_FLAG_TENSOR_LIST in the reference kernel): `data` of gmm1Weight,
 * gmm1Scale, gmm2Weight and gmm2Scale is a device array of moeExpertNum
 * 64-bit addresses, entry e = expert e's own pre-packed weight / scale tensor
 * (16-byte aligned); dataType, shape and format still describe the stacked
 * tensor. The shared expert's operands are always plain tensors.
 */
int32_t zbal_fused_deep_moe(const zbal_tensor_info_t *x, const zbal_tensor_info_t *expertIds,
                            const zbal_tensor_info_t *gmm1Weight, const zbal_tensor_info_t *gmm1Scale,
                            const zbal_tensor_info_t *gmm2Weight, const zbal_tensor_info_t *gmm2Scale,
                            const zbal_tensor_info_t *expertScales, const zbal_tensor_info_t *expertSmoothScales,
                            const zbal_tensor_info_t *shareGmm1Weight, const zbal_tensor_info_t *shareGmm1Scale,
                            const zbal_tensor_info_t *shareGmm2Weight, const zbal_tensor_info_t *shareGmm2Scale,
                            const zbal_tensor_info_t *shareSmoothScales, const zbal_tensor_info_t *xActiveMask,
                            const zbal_tensor_info_t *output, const zbal_tensor_info_t *shareOutput,
                            const zbal_tensor_info_t *expertTokenNums, const zbal_tensor_info_t *workspace,
                            int64_t moeExpertNum, int64_t quantMode, int64_t globalBs, int64_t gmm1HLen,
                            int64_t shareGmm1HLen, int64_t isTensorList, zbal_comm_t comm, aclrtStream stream,
                            int64_t flags);

/*
 * extension: bytes of workspace zbal_fused_deep_moe needs for a batch of
 * `tokens` rows. Takes the place of the size computation the reference keeps
 * in its adaptor and host launcher (zbal_deepep.cpp:42-84,
 * zbal_kernel_fused_deep_moe_host.cpp:59-132). shareGmm1HLen is 0 without a
 * shared expert. Returns 0 on invalid input.
 */
uint64_t zbal_fused_deep_moe_workspace_size(int64_t tokens, int64_t hidden, int64_t topk, int64_t moeExpertNum,
                                            int64_t gmm1HLen, int64_t shareGmm1HLen, int64_t quantMode);

/*
 * extension: softmax + top-k router. logits [T, E] fp32 -> topkIndex [T, K]
 * (int64, the type zbal_dispatch_normal_layout takes, or int32, the type
 * the dispatch and fused operators take: the descriptor's dataType says
 * which) and topkWeight [T, K] fp32 (probabilities renormalised over the K
 * picks). Picks are ordered by descending probability, ties to the lower
 * expert index. The reference has no router; its tests build these inputs
 * with torch.topk (test_low_latency.py:68-89).
 */
int32_t zbal_moe_topk_route(const zbal_tensor_info_t *logits, int64_t topkNum, const zbal_tensor_info_t *topkIndex,
                            const zbal_tensor_info_t *topkWeight, zbal_comm_t comm, aclrtStream stream, int64_t flags);

/*
 * extension: convert an expert weight tensor from ZBAL_WEIGHT_FORMAT_ND
 * ([E, K, N], N contiguous, one byte per element) to
 * ZBAL_WEIGHT_FORMAT_PREPACKED (layouts in zbal_def.h; K and N must be
 * multiples of 128). When dst->dataType is INT4X2 the source is INT8 with
 * values in [-8, 7] and the result packs two of them per byte. `dst` must not
 * alias `src` and both must be 16-byte aligned. The
 * stand-in for the reference's format cast of fused-kernel weights
 * (test_fused_deep_moe.py:66-69).
 */
int32_t zbal_moe_weight_prepack(const zbal_tensor_info_t *src, const zbal_tensor_info_t *dst, zbal_comm_t comm,
                                aclrtStream stream, int64_t flags);

#ifdef __cplusplus
}
#endif

#endif /* ZBAL_OPERATIONS_H_ */
