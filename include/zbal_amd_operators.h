/*
 * The kernel-launcher seam of the reference, for MI355X: the functions its
 * communicator layer calls to launch an operator
 * (app/zbal/src/csrc/operators/npu/zbal_npu_operators.h:21-25, 47-97; the
 * reference links them from its kernel library and swaps that library for a
 * stub in unit tests, src/csrc/CMakeLists.txt:48-55). Same names, C++
 * linkage, argument lists and return convention (0, or a negative code with
 * the text in the thread's last error); each checks its descriptors and
 * launches the HIP kernels of include/zbal_hip_kernels.h asynchronously on
 * `stream`. A build of the reference's host layer that links libzbal.so in
 * place of its kernel library runs this hot path on an MI355X.
 *
 * Peer tensors are found through CommGroupInfo as the reference's kernels
 * find them: same offset, (world(r) - world(me)) * localDeviceMemSize bytes
 * away. The low-latency pair and the fused operator take a group of one.
 * enableBalance must be false (token re-balancing is not part of this build);
 * factorHigh / factorLow, tilingDevBuf, groupName, tpGroupInfo and
 * needTilingCopy are accepted and not used.
 */
#ifndef ZBAL_AMD_OPERATORS_H_
#define ZBAL_AMD_OPERATORS_H_

#include <string>

#include "zbal.h"
#include "zbal_comm_group_info.h"

#define ZBAL_KERNEL_API __attribute__((visibility("default")))

/* zbal_npu_operators.h:21-22 */
ZBAL_KERNEL_API int32_t ZBALOpReduceScatter(const void *inp, void *out, size_t recvNumel, zbal_datatype_t dataType,
                                            aclrtStream stream, zbal_reduce_op_t reduceOp, CommGroupInfo &groupInfo);

/* zbal_npu_operators.h:24-25 */
ZBAL_KERNEL_API int32_t ZBALOpAllReduce(const void *inp, void *out, void *buf, size_t numel, zbal_datatype_t dataType,
                                        aclrtStream stream, zbal_reduce_op_t reduceOp, CommGroupInfo &groupInfo);

/* zbal_npu_operators.h:47-50 */
ZBAL_KERNEL_API int32_t ZBALOpDispatchLayout(const zbal_tensor_info_t *topkIndex, int64_t tokens, int64_t expertNum,
                                             int64_t topkNum, const zbal_tensor_info_t *tokensPerRank,
                                             const zbal_tensor_info_t *tokensPerExpert,
                                             const zbal_tensor_info_t *sendTokensIndex,
                                             const zbal_tensor_info_t *notifySendData, aclrtStream stream,
                                             const CommGroupInfo &groupInfo, int64_t flags);

/* zbal_npu_operators.h:52-56 */
ZBAL_KERNEL_API int32_t ZBALOpNotifyDispatch(const zbal_tensor_info_t *sendTokensPerExpert, int64_t sendCount,
                                             int64_t topKNum, const zbal_tensor_info_t *recvBuff,
                                             const zbal_tensor_info_t *totalRecvTokens,
                                             const zbal_tensor_info_t *recvTokensPerExpert,
                                             const zbal_tensor_info_t *pushTargetOffset,
                                             const zbal_tensor_info_t *balanceMatrix, float factorHigh, float factorLow,
                                             aclrtStream stream, const CommGroupInfo &groupInfo, int64_t flags);

/* zbal_npu_operators.h:58-62 */
ZBAL_KERNEL_API int32_t ZBALOpDispatchNormal(const zbal_tensor_info_t *srcTokens, const zbal_tensor_info_t *topkIndex,
                                             const zbal_tensor_info_t *sendTokensIndex,
                                             const zbal_tensor_info_t *pushTargetOffset,
                                             const zbal_tensor_info_t *balanceMatrix, int64_t expertNum,
                                             zbal_quant_mode_t quantMode, const zbal_tensor_info_t *destTokens,
                                             const zbal_tensor_info_t *destScale, bool enableBalance, aclrtStream stream,
                                             const CommGroupInfo &groupInfo, int64_t flags);

/* zbal_npu_operators.h:64-68 */
ZBAL_KERNEL_API int32_t ZBALOpCombineNormal(const zbal_tensor_info_t *srcTokens, const zbal_tensor_info_t *srcTokensPerEp,
                                            const zbal_tensor_info_t *topKWeight, const zbal_tensor_info_t *topkIndex,
                                            const zbal_tensor_info_t *sendTokensIndex,
                                            const zbal_tensor_info_t *balanceMatrix, uint16_t expertNum,
                                            const zbal_tensor_info_t *destTokens, bool enableBalance, aclrtStream stream,
                                            const CommGroupInfo &groupInfo, int64_t flags);

/* zbal_npu_operators.h:70-77 */
ZBAL_KERNEL_API int32_t ZBALOpDispatchLowLatency(const zbal_tensor_info_t *x, const zbal_tensor_info_t *expertIds,
                                                 int64_t moeExpertNum, int64_t sharedExpertNum,
                                                 int64_t sharedExpertRankNum, int64_t quantMode, int64_t globalBs,
                                                 int64_t magicVal, int64_t expertTokenNumsType,
                                                 const zbal_tensor_info_t *expandXOut,
                                                 const zbal_tensor_info_t *dynamicScalesOut,
                                                 const zbal_tensor_info_t *expandIdxOut,
                                                 const zbal_tensor_info_t *expertTokenNumsOut,
                                                 const zbal_tensor_info_t *epRecvCountsOut,
                                                 const zbal_tensor_info_t *putOffset,
                                                 const zbal_tensor_info_t *putOffsetStatus, aclrtStream stream,
                                                 const CommGroupInfo &groupInfo, int64_t flags);

/* zbal_npu_operators.h:79-83 */
ZBAL_KERNEL_API int32_t ZBALOpCombineLowLatency(const zbal_tensor_info_t *expandX, const zbal_tensor_info_t *expertIds,
                                                const zbal_tensor_info_t *expertIdx,
                                                const zbal_tensor_info_t *epSendCounts,
                                                const zbal_tensor_info_t *expertScales, const zbal_tensor_info_t *xOut,
                                                int64_t moeExpertNum, aclrtStream stream, const CommGroupInfo &groupInfo,
                                                int64_t flags);

/* zbal_npu_operators.h:85-97 */
ZBAL_KERNEL_API int32_t ZBALOpFusedDeepMoe(
    const zbal_tensor_info_t *x, const zbal_tensor_info_t *expertIds, const zbal_tensor_info_t *gmm1Weight,
    const zbal_tensor_info_t *gmm1Scale, const zbal_tensor_info_t *gmm2Weight, const zbal_tensor_info_t *gmm2Scale,
    const zbal_tensor_info_t *expertScales, const zbal_tensor_info_t *expertSmoothScales,
    const zbal_tensor_info_t *shareGmm1Weight, const zbal_tensor_info_t *shareGmm1Scale,
    const zbal_tensor_info_t *shareGmm2Weight, const zbal_tensor_info_t *shareGmm2Scale,
    const zbal_tensor_info_t *shareSmoothScales, const zbal_tensor_info_t *xActiveMask, const zbal_tensor_info_t *output,
    const zbal_tensor_info_t *shareOutput, const zbal_tensor_info_t *expertTokenNums, const zbal_tensor_info_t *workspace,
    int64_t moeExpertNum, int64_t quantMode, int64_t globalBs, int64_t gmm1HLen, int64_t shareGmm1HLen, bool isTensorList,
    void *tilingDevBuf, const std::string &groupName, aclrtStream stream, const CommGroupInfo &epGroupInfo,
    const CommGroupInfo &tpGroupInfo, int64_t flags, bool needTilingCopy = true);

#endif /* ZBAL_AMD_OPERATORS_H_ */
