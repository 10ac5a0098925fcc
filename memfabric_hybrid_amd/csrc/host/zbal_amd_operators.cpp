/*
 * The reference's kernel-launcher functions (operators/npu/zbal_npu_operators.h:21-25, 47-97) on top of the HIP
 * backend: each finds (or, the first time a group is seen, builds) the backend object for the group the
 * CommGroupInfo describes and calls the backend's operator, which checks the descriptors and launches the kernels.
 */
#include "zbal_amd_operators.h"

#include <cstring>
#include <mutex>
#include <vector>

#include "zbal_hip_kernels.h"
#include "zbal_host.h"

namespace {

using namespace zbal;

/*
 * The backend objects built so far, by what identifies a group to the kernels: size, own rank, index, the distance
 * between the ranks' memories and the world ranks of the members. A launch on a decode step must not pay for a new
 * object (allocations, the one-time GEMM set-up) every time; a serving process sees a handful of groups.
 */
struct GroupKey {
    uint16_t groupSize, myGroupRank;
    uint32_t groupIndex;
    uint64_t localDeviceMemSize;
    uint16_t worldRank[ZBALHIP_MAX_REDUCE_PEERS];
};
std::mutex gGroupsMutex;
std::vector<std::pair<GroupKey, CommunicatorPtr>> gGroups;

/* the communicator of the group; false (and a last error) when the group cannot be served */
bool GroupOf(const char *op, const CommGroupInfo &g, CommunicatorPtr *out)
{
    ZBAL_VALIDATE_RETURN(g.groupSize >= 1 && g.groupSize <= ZBALHIP_MAX_REDUCE_PEERS,
                         op << " failed as group size " << g.groupSize << " is not in 1.." << ZBALHIP_MAX_REDUCE_PEERS, false);
    ZBAL_VALIDATE_RETURN(g.myGroupRank < g.groupSize, op << " failed as rank " << g.myGroupRank << " is not in the group", false);
    ZBAL_VALIDATE_RETURN(g.groupSize == 1 || g.localDeviceMemSize != 0,
                         op << " failed as localDeviceMemSize is 0 for a group of " << g.groupSize, false);
    GroupKey key;
    std::memset(&key, 0, sizeof(key));
    key.groupSize = (uint16_t)g.groupSize;
    key.myGroupRank = (uint16_t)g.myGroupRank;
    key.groupIndex = (uint32_t)g.groupIndex;
    if (g.groupSize > 1) {
        key.localDeviceMemSize = g.localDeviceMemSize;
        for (uint32_t r = 0; r < g.groupSize; ++r) key.worldRank[r] = (uint16_t)g.peerGroupRank2WorldRank[r];
    }
    std::lock_guard<std::mutex> guard(gGroupsMutex);
    for (const auto &kv : gGroups) {
        if (std::memcmp(&kv.first, &key, sizeof(key)) == 0) {
            *out = kv.second;
            return true;
        }
    }
    GroupInfo info;
    info.name = "kernel-seam";
    info.groupSize = g.groupSize;
    info.myGroupRank = g.myGroupRank;
    info.groupIndex = g.groupIndex;
    info.peers.resize(g.groupSize);
    info.traced = false;
    if (g.groupSize > 1) {
        info.peerStride = g.localDeviceMemSize;
        info.worldRank.assign(g.peerGroupRank2WorldRank, g.peerGroupRank2WorldRank + g.groupSize);
    }
    *out = MakeGpuCommunicator(info);
    if (gGroups.size() >= 256) gGroups.clear(); /* a bound, not a policy: groups are few and long-lived */
    gGroups.emplace_back(key, *out);
    return true;
}

bool Present(const char *op, const char *name, const void *p)
{
    ZBAL_VALIDATE_RETURN(p != nullptr, op << " failed as " << name << " is null", false);
    return true;
}

#define ZB_NEED(op, p)                                     \
    do {                                                   \
        if (!Present(op, #p, p)) return Z_INVALID_PARAM;   \
    } while (0)

} // namespace

int32_t ZBALOpReduceScatter(const void *inp, void *out, size_t recvNumel, zbal_datatype_t dataType, aclrtStream stream,
                            zbal_reduce_op_t reduceOp, CommGroupInfo &groupInfo)
{
    ZB_NEED("ReduceScatter", inp);
    ZB_NEED("ReduceScatter", out);
    CommunicatorPtr c;
    if (!GroupOf("ReduceScatter", groupInfo, &c)) return Z_INVALID_PARAM;
    ++groupInfo.waitSymbol; /* the reference's cross-rank launch counter, zbal_kernel_allreduce.cpp:436 */
    return c->ReduceScatter(inp, out, recvNumel, dataType, reduceOp, stream);
}

int32_t ZBALOpAllReduce(const void *inp, void *out, void *buf, size_t numel, zbal_datatype_t dataType, aclrtStream stream,
                        zbal_reduce_op_t reduceOp, CommGroupInfo &groupInfo)
{
    ZB_NEED("AllReduce", inp);
    ZB_NEED("AllReduce", out);
    CommunicatorPtr c;
    if (!GroupOf("AllReduce", groupInfo, &c)) return Z_INVALID_PARAM;
    ++groupInfo.waitSymbol;
    return c->AllReduce(inp, out, buf, numel, dataType, reduceOp, stream);
}

int32_t ZBALOpDispatchLayout(const zbal_tensor_info_t *topkIndex, int64_t tokens, int64_t expertNum, int64_t topkNum,
                             const zbal_tensor_info_t *tokensPerRank, const zbal_tensor_info_t *tokensPerExpert,
                             const zbal_tensor_info_t *sendTokensIndex, const zbal_tensor_info_t *notifySendData,
                             aclrtStream stream, const CommGroupInfo &groupInfo, int64_t flags)
{
    const char *op = "DispatchLayout";
    ZB_NEED(op, topkIndex); ZB_NEED(op, tokensPerRank); ZB_NEED(op, tokensPerExpert); ZB_NEED(op, sendTokensIndex);
    ZB_NEED(op, notifySendData);
    CommunicatorPtr c;
    if (!GroupOf(op, groupInfo, &c)) return Z_INVALID_PARAM;
    return c->DispatchNormalLayout(topkIndex, tokens, expertNum, topkNum, tokensPerRank, tokensPerExpert, sendTokensIndex,
                                   notifySendData, stream, flags);
}

int32_t ZBALOpNotifyDispatch(const zbal_tensor_info_t *sendTokensPerExpert, int64_t sendCount, int64_t topKNum,
                             const zbal_tensor_info_t *recvBuff, const zbal_tensor_info_t *totalRecvTokens,
                             const zbal_tensor_info_t *recvTokensPerExpert, const zbal_tensor_info_t *pushTargetOffset,
                             const zbal_tensor_info_t *balanceMatrix, float, float, aclrtStream stream,
                             const CommGroupInfo &groupInfo, int64_t flags)
{
    const char *op = "NotifyDispatch";
    ZB_NEED(op, sendTokensPerExpert); ZB_NEED(op, recvBuff); ZB_NEED(op, totalRecvTokens); ZB_NEED(op, recvTokensPerExpert);
    ZB_NEED(op, pushTargetOffset); ZB_NEED(op, balanceMatrix);
    CommunicatorPtr c;
    if (!GroupOf(op, groupInfo, &c)) return Z_INVALID_PARAM;
    return c->DispatchNormalNotify(sendTokensPerExpert, sendCount, topKNum, recvBuff, totalRecvTokens, recvTokensPerExpert,
                                   pushTargetOffset, balanceMatrix, stream, flags);
}

int32_t ZBALOpDispatchNormal(const zbal_tensor_info_t *srcTokens, const zbal_tensor_info_t *topkIndex,
                             const zbal_tensor_info_t *sendTokensIndex, const zbal_tensor_info_t *pushTargetOffset,
                             const zbal_tensor_info_t *balanceMatrix, int64_t expertNum, zbal_quant_mode_t quantMode,
                             const zbal_tensor_info_t *destTokens, const zbal_tensor_info_t *destScale, bool enableBalance,
                             aclrtStream stream, const CommGroupInfo &groupInfo, int64_t flags)
{
    const char *op = "DispatchNormal";
    ZB_NEED(op, srcTokens); ZB_NEED(op, topkIndex); ZB_NEED(op, sendTokensIndex); ZB_NEED(op, pushTargetOffset);
    ZB_NEED(op, destTokens); ZB_NEED(op, destScale);
    ZBAL_VALIDATE_RETURN(!enableBalance, op << " failed as token re-balancing is not part of this build", Z_INVALID_PARAM);
    CommunicatorPtr c;
    if (!GroupOf(op, groupInfo, &c)) return Z_INVALID_PARAM;
    return c->DispatchNormal(srcTokens, topkIndex, sendTokensIndex, pushTargetOffset, balanceMatrix, expertNum, quantMode,
                             destTokens, destScale, stream, flags);
}

int32_t ZBALOpCombineNormal(const zbal_tensor_info_t *srcTokens, const zbal_tensor_info_t *srcTokensPerEp,
                            const zbal_tensor_info_t *topKWeight, const zbal_tensor_info_t *topkIndex,
                            const zbal_tensor_info_t *sendTokensIndex, const zbal_tensor_info_t *balanceMatrix,
                            uint16_t expertNum, const zbal_tensor_info_t *destTokens, bool enableBalance, aclrtStream stream,
                            const CommGroupInfo &groupInfo, int64_t flags)
{
    const char *op = "CombineNormal";
    ZB_NEED(op, srcTokens); ZB_NEED(op, srcTokensPerEp); ZB_NEED(op, topKWeight); ZB_NEED(op, topkIndex);
    ZB_NEED(op, sendTokensIndex); ZB_NEED(op, destTokens);
    ZBAL_VALIDATE_RETURN(!enableBalance, op << " failed as token re-balancing is not part of this build", Z_INVALID_PARAM);
    CommunicatorPtr c;
    if (!GroupOf(op, groupInfo, &c)) return Z_INVALID_PARAM;
    return c->CombineNormal(srcTokens, srcTokensPerEp, topKWeight, topkIndex, sendTokensIndex, balanceMatrix, expertNum,
                            destTokens, stream, flags);
}

int32_t ZBALOpDispatchLowLatency(const zbal_tensor_info_t *x, const zbal_tensor_info_t *expertIds, int64_t moeExpertNum,
                                 int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t quantMode, int64_t globalBs,
                                 int64_t magicVal, int64_t expertTokenNumsType, const zbal_tensor_info_t *expandXOut,
                                 const zbal_tensor_info_t *dynamicScalesOut, const zbal_tensor_info_t *expandIdxOut,
                                 const zbal_tensor_info_t *expertTokenNumsOut, const zbal_tensor_info_t *epRecvCountsOut,
                                 const zbal_tensor_info_t *putOffset, const zbal_tensor_info_t *putOffsetStatus,
                                 aclrtStream stream, const CommGroupInfo &groupInfo, int64_t flags)
{
    const char *op = "DispatchLowlatency";
    ZB_NEED(op, x); ZB_NEED(op, expertIds); ZB_NEED(op, expandXOut); ZB_NEED(op, dynamicScalesOut); ZB_NEED(op, expandIdxOut);
    ZB_NEED(op, expertTokenNumsOut); ZB_NEED(op, epRecvCountsOut); ZB_NEED(op, putOffset);
    CommunicatorPtr c;
    if (!GroupOf(op, groupInfo, &c)) return Z_INVALID_PARAM;
    return c->DispatchLowLatency(x, expertIds, moeExpertNum, sharedExpertNum, sharedExpertRankNum, quantMode, globalBs,
                                 magicVal, expertTokenNumsType, expandXOut, dynamicScalesOut, expandIdxOut,
                                 expertTokenNumsOut, epRecvCountsOut, putOffset, putOffsetStatus, stream, flags);
}

int32_t ZBALOpCombineLowLatency(const zbal_tensor_info_t *expandX, const zbal_tensor_info_t *expertIds,
                                const zbal_tensor_info_t *expertIdx, const zbal_tensor_info_t *epSendCounts,
                                const zbal_tensor_info_t *expertScales, const zbal_tensor_info_t *xOut, int64_t moeExpertNum,
                                aclrtStream stream, const CommGroupInfo &groupInfo, int64_t flags)
{
    const char *op = "CombineLowlatency";
    ZB_NEED(op, expandX); ZB_NEED(op, expertIds); ZB_NEED(op, expertIdx); ZB_NEED(op, epSendCounts); ZB_NEED(op, expertScales);
    ZB_NEED(op, xOut);
    CommunicatorPtr c;
    if (!GroupOf(op, groupInfo, &c)) return Z_INVALID_PARAM;
    return c->CombineLowLatency(expandX, expertIds, expertIdx, epSendCounts, expertScales, xOut, moeExpertNum, stream, flags);
}

int32_t ZBALOpFusedDeepMoe(const zbal_tensor_info_t *x, const zbal_tensor_info_t *expertIds,
                           const zbal_tensor_info_t *gmm1Weight, const zbal_tensor_info_t *gmm1Scale,
                           const zbal_tensor_info_t *gmm2Weight, const zbal_tensor_info_t *gmm2Scale,
                           const zbal_tensor_info_t *expertScales, const zbal_tensor_info_t *expertSmoothScales,
                           const zbal_tensor_info_t *shareGmm1Weight, const zbal_tensor_info_t *shareGmm1Scale,
                           const zbal_tensor_info_t *shareGmm2Weight, const zbal_tensor_info_t *shareGmm2Scale,
                           const zbal_tensor_info_t *shareSmoothScales, const zbal_tensor_info_t *xActiveMask,
                           const zbal_tensor_info_t *output, const zbal_tensor_info_t *shareOutput,
                           const zbal_tensor_info_t *expertTokenNums, const zbal_tensor_info_t *workspace,
                           int64_t moeExpertNum, int64_t quantMode, int64_t globalBs, int64_t gmm1HLen, int64_t shareGmm1HLen,
                           bool isTensorList, void *, const std::string &, aclrtStream stream, const CommGroupInfo &epGroupInfo,
                           const CommGroupInfo &, int64_t flags, bool)
{
    const char *op = "FusedDeepMoe";
    ZB_NEED(op, x); ZB_NEED(op, expertIds); ZB_NEED(op, gmm1Weight); ZB_NEED(op, gmm1Scale); ZB_NEED(op, gmm2Weight);
    ZB_NEED(op, gmm2Scale); ZB_NEED(op, expertScales); ZB_NEED(op, output); ZB_NEED(op, expertTokenNums); ZB_NEED(op, workspace);
    ZBAL_VALIDATE_RETURN(moeExpertNum > 0, op << " failed as moeExpertNum " << moeExpertNum << " is invalid", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(gmm1HLen > 0, op << " failed as gmm1HLen " << gmm1HLen << " is invalid", Z_INVALID_PARAM);
    if (!SharedExpertArgsConsistent(op, shareGmm1Weight, shareGmm1Scale, shareGmm2Weight, shareGmm2Scale, shareSmoothScales,
                                    shareOutput, shareGmm1HLen))
        return Z_INVALID_PARAM;
    CommunicatorPtr c;
    if (!GroupOf(op, epGroupInfo, &c)) return Z_INVALID_PARAM;
    return c->FusedDeepMoe(x, expertIds, gmm1Weight, gmm1Scale, gmm2Weight, gmm2Scale, expertScales, expertSmoothScales,
                           shareGmm1Weight, shareGmm1Scale, shareGmm2Weight, shareGmm2Scale, shareSmoothScales, xActiveMask,
                           output, shareOutput, expertTokenNums, workspace, moeExpertNum, quantMode, globalBs, gmm1HLen,
                           shareGmm1HLen, isTensorList, stream, flags);
}
