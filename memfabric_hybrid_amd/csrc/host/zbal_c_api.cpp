/*
 * Outer C ABI of the operator layer: argument validation, handle lookup and
 * the virtual call into the communicator's backend. Validation order and
 * return codes follow the reference's zbal_operations.cpp (lines cited per
 * function); one deliberate difference: the communicator handle is looked
 * up in the registry before use (the reference casts it blindly and its MoE
 * entry points do not even check it for null, :283-286, :308-311).
 */
#include <cstring>
#include <initializer_list>

#include "zbal_host.h"

using namespace zbal;

#define ZBAL_API extern "C" __attribute__((visibility("default")))

namespace {

struct NamedArg {
    const char *name;
    const void *ptr;
};

/* every listed pointer argument must be non-null; the first missing one is reported */
bool Present(const char *op, std::initializer_list<NamedArg> args)
{
    for (const NamedArg &a : args) {
        if (a.ptr == nullptr) {
            ZBAL_LOG_AND_SET_LAST_ERROR(op << " failed as " << a.name << " is null");
            return false;
        }
    }
    return true;
}

CommunicatorPtr Resolve(const char *op, zbal_comm_t comm)
{
    if (comm == nullptr) {
        ZBAL_LOG_AND_SET_LAST_ERROR(op << " failed as comm is null");
        return nullptr;
    }
    CommunicatorPtr c = registry::Find(comm);
    if (!c) ZBAL_LOG_AND_SET_LAST_ERROR(op << " failed as comm is not a live communicator");
    return c;
}

} // namespace

namespace zbal {
bool SharedExpertArgsConsistent(const char *op, const zbal_tensor_info_t *shareGmm1Weight,
                                const zbal_tensor_info_t *shareGmm1Scale, const zbal_tensor_info_t *shareGmm2Weight,
                                const zbal_tensor_info_t *shareGmm2Scale, const zbal_tensor_info_t *shareSmoothScales,
                                const zbal_tensor_info_t *shareOutput, int64_t shareGmm1HLen)
{
    auto present = [](const zbal_tensor_info_t *t) { return t != nullptr && t->data != nullptr; };
    const bool shared = present(shareGmm1Weight);
    ZBAL_VALIDATE_RETURN(shared == present(shareGmm1Scale) && shared == present(shareGmm2Weight) &&
                             shared == present(shareGmm2Scale) && shared == present(shareOutput) &&
                             shared == (shareGmm1HLen > 0) && (shared || !present(shareSmoothScales)),
                         op << " failed as the shared expert needs both weights, both scales, shareOutput and "
                               "shareGmm1HLen > 0, or none of them",
                         false);
    return true;
}
} // namespace zbal

/* ---- lifecycle: reference zbal_operations.cpp:23-114 ------------------------ */

ZBAL_API int32_t zbal_comm_create(zbal_comm_options_t *options, zbal_comm_t *comm)
{
    ZBAL_VALIDATE_RETURN(options != nullptr, "Create communicator failed as options is null", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(comm != nullptr, "Create communicator failed as comm is null", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(options->name != nullptr, "Create communicator failed as name is null", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(std::strlen(options->name) != 0, "Create communicator failed as name is empty", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(std::strlen(options->name) < ZBAL_COMM_NAME_MAX, "Create communicator failed as name is too long, which should be less than " << ZBAL_COMM_NAME_MAX, Z_INVALID_PARAM);
    const BootState &st = Boot();
    if (!st.bootstrapped) {
        ZBAL_LOG_AND_SET_LAST_ERROR("Create communicator failed as not bootstrapped");
        return Z_NOT_BOOTSTRAPPED;
    }
    if (options->isWorldGroup == 1 && st.worldSize != options->groupSize) {
        ZBAL_LOG_AND_SET_LAST_ERROR("Create communicator failed as world size " << options->groupSize
                                    << " is not equal to bootstrap's world size " << st.worldSize);
        return Z_NOT_BOOTSTRAPPED;
    }
    if (options->isWorldGroup == 0 && st.worldSize < options->groupSize) {
        ZBAL_LOG_AND_SET_LAST_ERROR("Create communicator failed as world size " << options->groupSize
                                    << " is bigger than bootstrap's world size " << st.worldSize);
        return Z_NOT_BOOTSTRAPPED;
    }
    return registry::Create(*options, comm);
}

ZBAL_API int32_t zbal_comm_get_property(zbal_comm_t comm, zbal_comm_property_t *property)
{
    ZBAL_VALIDATE_RETURN(comm != nullptr, "Get property failed as comm is null", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(property != nullptr, "Get property failed as property is null", Z_INVALID_PARAM);
    CommunicatorPtr c = registry::Find(comm);
    if (!c) {
        ZBAL_LOG_AND_SET_LAST_ERROR("Communicator find failed when get property.");
        return Z_COMM_NOT_EXIST_BY_HANDLE;
    }
    const GroupInfo &g = c->Info();
    std::memset(property, 0, sizeof(*property));
    std::strncpy(property->name, g.name.c_str(), ZBAL_COMM_NAME_MAX - 1);
    property->backendType = g.backend;
    property->isWorldGroup = g.isWorldGroup ? 1 : 0;
    property->groupSize = g.groupSize;
    property->groupRankId = g.myGroupRank;
    property->groupIndex = g.groupIndex;
    const PeerWindow &mine = g.peers[g.myGroupRank];
    property->myGVA = mine.base;
    property->localDeviceMemSize = mine.size;
    return Z_OK;
}

ZBAL_API zbal_comm_t zbal_comm_get_global() { return registry::Global(); }

ZBAL_API zbal_comm_t zbal_comm_get_by_name(const char *name)
{
    ZBAL_VALIDATE_RETURN(name != nullptr, "Get communicator failed as name is null", nullptr);
    return registry::ByName(name);
}

ZBAL_API int32_t zbal_comm_destroy(zbal_comm_t comm, uint32_t flags)
{
    (void)flags;
    ZBAL_VALIDATE_RETURN(comm != nullptr, "Destroy communicator failed as comm is null", Z_INVALID_PARAM);
    return registry::Destroy(comm);
}

ZBAL_API void zbal_comm_destroy_all(uint32_t flags)
{
    (void)flags;
    registry::DestroyAll();
}

ZBAL_API int32_t zbal_comm_register_peer_window(zbal_comm_t comm, uint16_t rank, void *base, uint64_t size)
{
    CommunicatorPtr c = Resolve("RegisterPeerWindow", comm);
    if (!c) return Z_INVALID_PARAM;
    ZBAL_VALIDATE_RETURN(rank < c->Info().groupSize, "RegisterPeerWindow failed as rank " << rank << " is out of range", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(base != nullptr && size > 0, "RegisterPeerWindow failed as the window is empty", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN((reinterpret_cast<uintptr_t>(base) & 15u) == 0, "RegisterPeerWindow failed as the window is not 16-byte aligned", Z_INVALID_PARAM);
    c->RegisterPeer(rank, PeerWindow{base, size});
    return Z_OK;
}

ZBAL_API int32_t zbal_comm_dump_profiling_trace(zbal_comm_t comm)
{
    CommunicatorPtr c = Resolve("DumpProfilingTrace", comm);
    if (!c) return Z_INVALID_PARAM;
    c->DumpProfilingTrace();
    return Z_OK;
}

/* ---- reductions: reference zbal_operations.cpp:117-157 ------------------------ */

ZBAL_API int32_t zbal_all_reduce(const void *send_buff, void *recv_buff, void *buffer, size_t count,
                                 zbal_datatype_t data_type, zbal_reduce_op_t op, zbal_comm_t comm, aclrtStream stream)
{
    if (send_buff == nullptr) return Z_OK; /* silent no-op, as in the reference (:120-122) */
    if (!Present("AllReduce", {{"recv_buff", recv_buff}})) return Z_INVALID_PARAM;
    ZBAL_VALIDATE_RETURN(count > 0, "AllReduce failed as count " << count << " is invalid", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(data_type >= 0 && data_type < ZBAL_DATA_TYPE_BUTT, "AllReduce failed as data_type " << data_type << " is invalid", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(op >= 0 && op < ZBAL_REDUCE_BUTT, "AllReduce failed as op " << op << " is invalid", Z_INVALID_PARAM);
    if (!Present("AllReduce", {{"comm", comm}})) return Z_INVALID_PARAM;
    ZBAL_VALIDATE_RETURN(buffer != nullptr, "Allreduce tmp buffer is null", Z_INVALID_PARAM);
    CommunicatorPtr c = Resolve("AllReduce", comm);
    if (!c) return Z_INVALID_PARAM;
    return c->AllReduce(send_buff, recv_buff, buffer, count, data_type, op, stream);
}

ZBAL_API int32_t zbal_reduce_scatter(const void *sendBuff, void *recvBuff, size_t recv_count, zbal_datatype_t dataType,
                                     zbal_reduce_op_t op, zbal_comm_t comm, aclrtStream stream)
{
    if (sendBuff == nullptr) return Z_OK; /* (:141-143) */
    if (!Present("ReduceScatter", {{"recvBuff", recvBuff}})) return Z_INVALID_PARAM;
    ZBAL_VALIDATE_RETURN(recv_count > 0, "ReduceScatter failed as recv_count " << recv_count << " is invalid", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(dataType >= 0 && dataType < ZBAL_DATA_TYPE_BUTT, "ReduceScatter failed as data_type " << dataType << " is invalid", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(op >= 0 && op < ZBAL_REDUCE_BUTT, "ReduceScatter failed as op " << op << " is invalid", Z_INVALID_PARAM);
    if (!Present("ReduceScatter", {{"comm", comm}})) return Z_INVALID_PARAM;
    CommunicatorPtr c = Resolve("ReduceScatter", comm);
    if (!c) return Z_INVALID_PARAM;
    return c->ReduceScatter(sendBuff, recvBuff, recv_count, dataType, op, stream);
}

/* ---- data-movement collectives: exported for link compatibility, refused (no transport between devices here) ---- */

static int32_t NoTransport(const char *op)
{
    ZBAL_LOG_AND_SET_LAST_ERROR(op << " failed as this build has no transport between devices");
    return Z_INVALID_PARAM;
}

ZBAL_API int32_t zbal_all_gather(const void *, void *, size_t, zbal_datatype_t, zbal_comm_t, aclrtStream) { return NoTransport("AllGather"); }
ZBAL_API int32_t zbal_all_to_all_v(const void *, void *, void *, void *, void *, zbal_datatype_t, zbal_comm_t, aclrtStream) { return NoTransport("AllToAllV"); }
ZBAL_API int32_t zbal_broadcast(const void *, uint64_t, zbal_datatype_t, uint16_t, zbal_comm_t, aclrtStream) { return NoTransport("Broadcast"); }
ZBAL_API int32_t zbal_scatter(const void *, void *, uint64_t, zbal_datatype_t, uint16_t, zbal_comm_t, aclrtStream) { return NoTransport("Scatter"); }
ZBAL_API int32_t zbal_gather(const void *, void *, uint64_t, zbal_datatype_t, uint16_t, zbal_comm_t, aclrtStream) { return NoTransport("Gather"); }
ZBAL_API int32_t zbal_barrier(zbal_comm_t, aclrtStream) { return NoTransport("Barrier"); }
ZBAL_API int32_t zbal_send(const void *, zbal_datatype_t, uint32_t, zbal_comm_t, aclrtStream) { return NoTransport("Send"); }
ZBAL_API int32_t zbal_recv(const void *, size_t, zbal_datatype_t, uint32_t, zbal_comm_t, aclrtStream) { return NoTransport("Recv"); }

/* ---- MoE operators: reference zbal_operations.cpp:258-457 ----------------------- */

ZBAL_API int32_t zbal_dispatch_normal_notify(const zbal_tensor_info_t *sendTokensPerExpert, int64_t sendCount,
                                             int64_t topKNum, const zbal_tensor_info_t *recvBuff,
                                             const zbal_tensor_info_t *totalRecvTokens,
                                             const zbal_tensor_info_t *recvTokensPerExpert,
                                             const zbal_tensor_info_t *pushTargetOffset,
                                             const zbal_tensor_info_t *balanceMatrix, zbal_comm_t comm,
                                             aclrtStream stream, int64_t flags)
{
    if (!Present("NotifyDispatch", {{"sendTokensPerExpert", sendTokensPerExpert}})) return Z_INVALID_PARAM;
    ZBAL_VALIDATE_RETURN(sendCount > 0, "NotifyDispatch failed as sendCount " << sendCount << " is invalid", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(topKNum > 0, "NotifyDispatch failed as topKNum " << topKNum << " is invalid", Z_INVALID_PARAM);
    if (!Present("NotifyDispatch", {{"recvBuff", recvBuff}, {"totalRecvTokens", totalRecvTokens}, {"recvTokensPerExpert", recvTokensPerExpert}, {"pushTargetOffset", pushTargetOffset}, {"balanceMatrix", balanceMatrix}})) return Z_INVALID_PARAM;
    CommunicatorPtr c = Resolve("NotifyDispatch", comm);
    if (!c) return Z_INVALID_PARAM;
    return c->DispatchNormalNotify(sendTokensPerExpert, sendCount, topKNum, recvBuff, totalRecvTokens, recvTokensPerExpert,
                                   pushTargetOffset, balanceMatrix, stream, flags);
}

ZBAL_API int32_t zbal_dispatch_normal_layout(const zbal_tensor_info_t *topkIndex, int64_t tokens, int64_t expertNum,
                                             int64_t topkNum, const zbal_tensor_info_t *tokensPerRank,
                                             const zbal_tensor_info_t *tokensPerExpert,
                                             const zbal_tensor_info_t *sendTokensIndex,
                                             const zbal_tensor_info_t *notifySendData, zbal_comm_t comm,
                                             aclrtStream stream, int64_t flags)
{
    if (!Present("DispatchLayout", {{"topkIndex", topkIndex}, {"tokensPerRank", tokensPerRank}, {"tokensPerExpert", tokensPerExpert}, {"sendTokensIndex", sendTokensIndex}, {"notifySendData", notifySendData}})) return Z_INVALID_PARAM;
    ZBAL_VALIDATE_RETURN(tokens >= 0, "DispatchLayout failed as tokens " << tokens << " is invalid", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(expertNum > 0, "DispatchLayout failed as expertNum " << expertNum << " is invalid", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(topkNum > 0, "DispatchLayout failed as topkNum " << topkNum << " is invalid", Z_INVALID_PARAM);
    CommunicatorPtr c = Resolve("DispatchLayout", comm);
    if (!c) return Z_INVALID_PARAM;
    return c->DispatchNormalLayout(topkIndex, tokens, expertNum, topkNum, tokensPerRank, tokensPerExpert, sendTokensIndex,
                                   notifySendData, stream, flags);
}

ZBAL_API int32_t zbal_dispatch_normal(const zbal_tensor_info_t *srcTokens, const zbal_tensor_info_t *topkIndex,
                                      const zbal_tensor_info_t *sendTokensIndex,
                                      const zbal_tensor_info_t *pushTargetOffset,
                                      const zbal_tensor_info_t *balanceMatrix, int64_t expertNum,
                                      zbal_quant_mode_t quantMode, const zbal_tensor_info_t *destTokens,
                                      const zbal_tensor_info_t *destScale, zbal_comm_t comm, aclrtStream stream,
                                      int64_t flags)
{
    if (!Present("DispatchNormal", {{"srcTokens", srcTokens}, {"topkIndex", topkIndex}, {"sendTokensIndex", sendTokensIndex}, {"pushTargetOffset", pushTargetOffset}, {"balanceMatrix", balanceMatrix}, {"destTokens", destTokens}, {"destScale", destScale}})) return Z_INVALID_PARAM;
    ZBAL_VALIDATE_RETURN(expertNum > 0, "DispatchNormal failed as expertNum " << expertNum << " is invalid", Z_INVALID_PARAM);
    CommunicatorPtr c = Resolve("DispatchNormal", comm);
    if (!c) return Z_INVALID_PARAM;
    return c->DispatchNormal(srcTokens, topkIndex, sendTokensIndex, pushTargetOffset, balanceMatrix, expertNum, quantMode,
                             destTokens, destScale, stream, flags);
}

ZBAL_API int32_t zbal_combine_normal(const zbal_tensor_info_t *srcTokens, const zbal_tensor_info_t *srcTokensPerEp,
                                     const zbal_tensor_info_t *topKWeight, const zbal_tensor_info_t *topkIndex,
                                     const zbal_tensor_info_t *sendTokensIndex, const zbal_tensor_info_t *balanceMatrix,
                                     uint16_t expertNum, const zbal_tensor_info_t *destTokens, zbal_comm_t comm,
                                     aclrtStream stream, int64_t flags)
{
    if (!Present("CombineNormal", {{"srcTokens", srcTokens}, {"srcTokensPerEp", srcTokensPerEp}, {"topKWeight", topKWeight}, {"topkIndex", topkIndex}, {"sendTokensIndex", sendTokensIndex}, {"balanceMatrix", balanceMatrix}, {"destTokens", destTokens}})) return Z_INVALID_PARAM;
    ZBAL_VALIDATE_RETURN(expertNum > 0, "CombineNormal failed as expertNum " << expertNum << " is invalid", Z_INVALID_PARAM);
    CommunicatorPtr c = Resolve("CombineNormal", comm);
    if (!c) return Z_INVALID_PARAM;
    return c->CombineNormal(srcTokens, srcTokensPerEp, topKWeight, topkIndex, sendTokensIndex, balanceMatrix, expertNum,
                            destTokens, stream, flags);
}

ZBAL_API int32_t zbal_dispatch_low_latency(
    const zbal_tensor_info_t *x, const zbal_tensor_info_t *expertIds, int64_t moeExpertNum, int64_t sharedExpertNum,
    int64_t sharedExpertRankNum, int64_t quantMode, int64_t globalBs, int64_t magicVal, int64_t expertTokenNumsType,
    const zbal_tensor_info_t *expandXOut, const zbal_tensor_info_t *dynamicScalesOut,
    const zbal_tensor_info_t *expandIdxOut, const zbal_tensor_info_t *expertTokenNumsOut,
    const zbal_tensor_info_t *epRecvCountsOut, const zbal_tensor_info_t *putOffset,
    const zbal_tensor_info_t *putOffsetStatus, zbal_comm_t comm, aclrtStream stream, int64_t flags)
{
    if (!Present("DispatchLowlatency", {{"x", x}, {"expertIds", expertIds}})) return Z_INVALID_PARAM;
    ZBAL_VALIDATE_RETURN(moeExpertNum > 0, "DispatchLowlatency failed as moeExpertNum " << moeExpertNum << " is invalid", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(sharedExpertNum >= 0, "DispatchLowlatency failed as sharedExpertNum " << sharedExpertNum << " is invalid", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(sharedExpertRankNum >= 0, "DispatchLowlatency failed as sharedExpertRankNum " << sharedExpertRankNum << " is invalid", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(globalBs >= 0, "DispatchLowlatency failed as globalBs " << globalBs << " is invalid", Z_INVALID_PARAM);
    if (!Present("DispatchLowlatency", {{"expandXOut", expandXOut}, {"dynamicScalesOut", dynamicScalesOut}, {"expandIdxOut", expandIdxOut}, {"expertTokenNumsOut", expertTokenNumsOut}, {"epRecvCountsOut", epRecvCountsOut}, {"putOffset", putOffset}, {"putOffsetStatus", putOffsetStatus}})) return Z_INVALID_PARAM;
    CommunicatorPtr c = Resolve("DispatchLowlatency", comm);
    if (!c) return Z_INVALID_PARAM;
    return c->DispatchLowLatency(x, expertIds, moeExpertNum, sharedExpertNum, sharedExpertRankNum, quantMode, globalBs,
                                 magicVal, expertTokenNumsType, expandXOut, dynamicScalesOut, expandIdxOut,
                                 expertTokenNumsOut, epRecvCountsOut, putOffset, putOffsetStatus, stream, flags);
}

ZBAL_API int32_t zbal_combine_low_latency(const zbal_tensor_info_t *expandX, const zbal_tensor_info_t *expertIds,
                                          const zbal_tensor_info_t *expertIdx, const zbal_tensor_info_t *epSendCounts,
                                          const zbal_tensor_info_t *expertScales, const zbal_tensor_info_t *xOut,
                                          int64_t moeExpertNum, zbal_comm_t comm, aclrtStream stream, int64_t flags)
{
    if (!Present("CombineLowlatency", {{"expandX", expandX}, {"expertIds", expertIds}, {"expertIdx", expertIdx}, {"epSendCounts", epSendCounts}, {"expertScales", expertScales}, {"xOut", xOut}})) return Z_INVALID_PARAM;
    ZBAL_VALIDATE_RETURN(moeExpertNum > 0, "CombineLowlatency failed as moeExpertNum " << moeExpertNum << " is invalid", Z_INVALID_PARAM);
    CommunicatorPtr c = Resolve("CombineLowlatency", comm);
    if (!c) return Z_INVALID_PARAM;
    return c->CombineLowLatency(expandX, expertIds, expertIdx, epSendCounts, expertScales, xOut, moeExpertNum, stream, flags);
}

ZBAL_API int32_t zbal_fused_deep_moe(
    const zbal_tensor_info_t *x, const zbal_tensor_info_t *expertIds, const zbal_tensor_info_t *gmm1Weight,
    const zbal_tensor_info_t *gmm1Scale, const zbal_tensor_info_t *gmm2Weight, const zbal_tensor_info_t *gmm2Scale,
    const zbal_tensor_info_t *expertScales, const zbal_tensor_info_t *expertSmoothScales,
    const zbal_tensor_info_t *shareGmm1Weight, const zbal_tensor_info_t *shareGmm1Scale,
    const zbal_tensor_info_t *shareGmm2Weight, const zbal_tensor_info_t *shareGmm2Scale,
    const zbal_tensor_info_t *shareSmoothScales, const zbal_tensor_info_t *xActiveMask,
    const zbal_tensor_info_t *output, const zbal_tensor_info_t *shareOutput, const zbal_tensor_info_t *expertTokenNums,
    const zbal_tensor_info_t *workspace, int64_t moeExpertNum, int64_t quantMode, int64_t globalBs, int64_t gmm1HLen,
    int64_t shareGmm1HLen, int64_t isTensorList, zbal_comm_t comm, aclrtStream stream, int64_t flags)
{
    if (!Present("FusedDeepMoe", {{"x", x}, {"expertIds", expertIds}, {"gmm1Weight", gmm1Weight}, {"gmm1Scale", gmm1Scale}, {"gmm2Weight", gmm2Weight}, {"gmm2Scale", gmm2Scale}, {"expertScales", expertScales}, {"output", output}, {"expertTokenNums", expertTokenNums}, {"workspace", workspace}})) return Z_INVALID_PARAM;
    ZBAL_VALIDATE_RETURN(moeExpertNum > 0, "FusedDeepMoe failed as moeExpertNum " << moeExpertNum << " is invalid", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(gmm1HLen > 0, "FusedDeepMoe failed as gmm1HLen " << gmm1HLen << " is invalid", Z_INVALID_PARAM);
    if (!SharedExpertArgsConsistent("FusedDeepMoe", shareGmm1Weight, shareGmm1Scale, shareGmm2Weight, shareGmm2Scale,
                                    shareSmoothScales, shareOutput, shareGmm1HLen))
        return Z_INVALID_PARAM;
    CommunicatorPtr c = Resolve("FusedDeepMoe", comm);
    if (!c) return Z_INVALID_PARAM;
    return c->FusedDeepMoe(x, expertIds, gmm1Weight, gmm1Scale, gmm2Weight, gmm2Scale, expertScales, expertSmoothScales,
                           shareGmm1Weight, shareGmm1Scale, shareGmm2Weight, shareGmm2Scale, shareSmoothScales, xActiveMask,
                           output, shareOutput, expertTokenNums, workspace, moeExpertNum, quantMode, globalBs, gmm1HLen,
                           shareGmm1HLen, isTensorList != 0, stream, flags);
}

/* ---- extensions -------------------------------------------------------------------------- */

ZBAL_API uint64_t zbal_fused_deep_moe_workspace_size(int64_t tokens, int64_t hidden, int64_t topk, int64_t moeExpertNum,
                                                     int64_t gmm1HLen, int64_t shareGmm1HLen, int64_t quantMode)
{
    FusedWorkspace ws;
    if (!PlanFusedWorkspace(tokens, hidden, topk, moeExpertNum, gmm1HLen, shareGmm1HLen, quantMode, &ws)) return 0;
    return ws.total;
}

ZBAL_API int32_t zbal_moe_topk_route(const zbal_tensor_info_t *logits, int64_t topkNum,
                                     const zbal_tensor_info_t *topkIndex, const zbal_tensor_info_t *topkWeight,
                                     zbal_comm_t comm, aclrtStream stream, int64_t flags)
{
    if (!Present("TopkRoute", {{"logits", logits}, {"topkIndex", topkIndex}, {"topkWeight", topkWeight}})) return Z_INVALID_PARAM;
    ZBAL_VALIDATE_RETURN(topkNum > 0, "TopkRoute failed as topkNum " << topkNum << " is invalid", Z_INVALID_PARAM);
    CommunicatorPtr c = Resolve("TopkRoute", comm);
    if (!c) return Z_INVALID_PARAM;
    return c->TopkRoute(logits, topkNum, topkIndex, topkWeight, stream, flags);
}

ZBAL_API int32_t zbal_moe_weight_prepack(const zbal_tensor_info_t *src, const zbal_tensor_info_t *dst, zbal_comm_t comm,
                                         aclrtStream stream, int64_t flags)
{
    if (!Present("WeightPrepack", {{"src", src}, {"dst", dst}})) return Z_INVALID_PARAM;
    CommunicatorPtr c = Resolve("WeightPrepack", comm);
    if (!c) return Z_INVALID_PARAM;
    return c->WeightPrepack(src, dst, stream, flags);
}
