/*
 * Host layer of the zbal MI355X library: result codes, logging / last-error
 * plumbing, the communicator registry and the backend interface the C entry
 * points call into.
 *
 * Mirrors the reference's host structure: result codes
 * (common/zbal_defines.h:24-53), log + last-error macros (common/zbal_logger.h,
 * common/zbal_last_error.h), abstract Communicator with one virtual per
 * operator (operators/zbal_communicator.h), a do-nothing backend for host-only
 * tests (operators/zbal_communicator_dummy.h:23-120) and a device backend
 * that forwards to kernel launchers (operators/npu/zbal_npu_communicator_base.cpp).
 */
#ifndef ZBAL_HOST_H_
#define ZBAL_HOST_H_

#include <cstdint>
#include <memory>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

#include "zbal.h"

namespace zbal {

enum ZResult : int32_t {
    Z_OK = 0,
    Z_ERROR = -1,
    Z_INVALID_PARAM = -2,
    Z_NEW_OBJ_FAILED = -3,
    Z_ERROR_ALLOC = -9,
    Z_NOT_ENOUGH_MEM = -10,
    Z_RT_ERROR = -11,
    Z_INIT_BOOTSTRAP_FAILED = -13,
    Z_CANNOT_UNBOOTSTRAP = -14,
    Z_NOT_BOOTSTRAPPED = -15,
    Z_CREATE_COMM_FAILED = -16,
    Z_COMM_EXEC_FAILED = -18,
    Z_COMM_NOT_EXIST_BY_NAME = -19,
    Z_COMM_NOT_EXIST_BY_HANDLE = -20,
    Z_COMM_NOT_FOUND = -21,
    Z_COMM_DESTROY_GLOBAL_LAST = -25,
};

/* ---- logging and last error ------------------------------------------------ */

enum LogLevel { LOG_DEBUG = 0, LOG_INFO = 1, LOG_WARN = 2, LOG_ERROR = 3 };

void LogWrite(int level, const std::string &text);
bool LogEnabled(int level);
void SetLastError(const std::string &text);

#define ZBAL_LOG(level, expr)                          \
    do {                                               \
        if (::zbal::LogEnabled(level)) {               \
            std::ostringstream zbal_oss__;             \
            zbal_oss__ << expr;                        \
            ::zbal::LogWrite(level, zbal_oss__.str()); \
        }                                              \
    } while (0)

#define ZBAL_LOG_AND_SET_LAST_ERROR(expr)                      \
    do {                                                       \
        std::ostringstream zbal_oss__;                         \
        zbal_oss__ << expr;                                    \
        ::zbal::SetLastError(zbal_oss__.str());                \
        ::zbal::LogWrite(::zbal::LOG_ERROR, zbal_oss__.str()); \
    } while (0)

#define ZBAL_VALIDATE_RETURN(cond, expr, ret) \
    do {                                      \
        if (!(cond)) {                        \
            ZBAL_LOG_AND_SET_LAST_ERROR(expr); \
            return ret;                       \
        }                                     \
    } while (0)

/* ---- bootstrap state ---------------------------------------------------------- */

struct BootState {
    bool bootstrapped = false;
    uint16_t worldSize = 0;
    uint16_t rankId = 0;
    uint16_t deviceId = 0;
    uint64_t deviceMemorySize = 0;
};
BootState &Boot();

/* ---- communicator ---------------------------------------------------------------- */

struct PeerWindow {
    void *base = nullptr;
    uint64_t size = 0;
};

/*
 * Per-group state the kernels need. The reference copies a 2160-byte
 * CommGroupInfo to the device (operators/zbal_comm_host_device_struct.h:133-151);
 * here the only device-visible part is the table of peer windows, which the
 * launchers pass by value.
 */
struct GroupInfo {
    std::string name;
    uint16_t groupSize = 0;
    uint16_t myGroupRank = 0;
    bool isWorldGroup = false;
    uint32_t groupIndex = 0;
    zbal_backend_t backend = ZBAL_AMD_GPU;
    std::vector<PeerWindow> peers; /* one per group rank */
    /*
     * The reference's symmetric address space instead of registered windows: group rank r's copy of a tensor lies
     * (worldRank[r] - worldRank[me]) * peerStride bytes from this rank's (CommGroupInfo::localDeviceMemSize and
     * peerGroupRank2WorldRank). Used when peerStride != 0; the launchers of zbal_amd_operators.h fill it in.
     */
    uint64_t peerStride = 0;
    std::vector<uint16_t> worldRank;
    bool traced = true;            /* false: never owns a trace ring, whatever ZBAL_PROF_ENABLE says */
};

class Communicator {
public:
    explicit Communicator(const GroupInfo &info) : info_(info) {}
    virtual ~Communicator() = default;

    const GroupInfo &Info() const { return info_; }

    /* writes what the device trace ring holds as a trace-viewer file; a no-op when tracing is off
       (reference zbal_communicator.h:114) */
    virtual void DumpProfilingTrace() noexcept {}

    /* peer windows may be registered while another thread runs an operator on the same communicator */
    void RegisterPeer(uint16_t rank, const PeerWindow &w)
    {
        std::lock_guard<std::mutex> guard(peersMutex_);
        info_.peers[rank] = w;
    }
    std::vector<PeerWindow> Peers() const
    {
        std::lock_guard<std::mutex> guard(peersMutex_);
        return info_.peers;
    }

    virtual int32_t AllReduce(const void *send, void *recv, void *buffer, size_t count, zbal_datatype_t dt,
                              zbal_reduce_op_t op, aclrtStream stream) = 0;
    virtual int32_t ReduceScatter(const void *send, void *recv, size_t recvCount, zbal_datatype_t dt,
                                  zbal_reduce_op_t op, aclrtStream stream) = 0;
    virtual int32_t DispatchNormalLayout(const zbal_tensor_info_t *topkIndex, int64_t tokens, int64_t expertNum,
                                         int64_t topkNum, const zbal_tensor_info_t *tokensPerRank,
                                         const zbal_tensor_info_t *tokensPerExpert,
                                         const zbal_tensor_info_t *sendTokensIndex,
                                         const zbal_tensor_info_t *notifySendData, aclrtStream stream,
                                         int64_t flags) = 0;
    virtual int32_t DispatchNormalNotify(const zbal_tensor_info_t *sendTokensPerExpert, int64_t sendCount,
                                         int64_t topKNum, const zbal_tensor_info_t *recvBuff,
                                         const zbal_tensor_info_t *totalRecvTokens,
                                         const zbal_tensor_info_t *recvTokensPerExpert,
                                         const zbal_tensor_info_t *pushTargetOffset,
                                         const zbal_tensor_info_t *balanceMatrix, aclrtStream stream,
                                         int64_t flags) = 0;
    virtual int32_t DispatchNormal(const zbal_tensor_info_t *srcTokens, const zbal_tensor_info_t *topkIndex,
                                   const zbal_tensor_info_t *sendTokensIndex,
                                   const zbal_tensor_info_t *pushTargetOffset, const zbal_tensor_info_t *balanceMatrix,
                                   int64_t expertNum, zbal_quant_mode_t quantMode, const zbal_tensor_info_t *destTokens,
                                   const zbal_tensor_info_t *destScale, aclrtStream stream, int64_t flags) = 0;
    virtual int32_t CombineNormal(const zbal_tensor_info_t *srcTokens, const zbal_tensor_info_t *srcTokensPerEp,
                                  const zbal_tensor_info_t *topKWeight, const zbal_tensor_info_t *topkIndex,
                                  const zbal_tensor_info_t *sendTokensIndex, const zbal_tensor_info_t *balanceMatrix,
                                  uint16_t expertNum, const zbal_tensor_info_t *destTokens, aclrtStream stream,
                                  int64_t flags) = 0;
    virtual int32_t DispatchLowLatency(const zbal_tensor_info_t *x, const zbal_tensor_info_t *expertIds,
                                       int64_t moeExpertNum, int64_t sharedExpertNum, int64_t sharedExpertRankNum,
                                       int64_t quantMode, int64_t globalBs, int64_t magicVal,
                                       int64_t expertTokenNumsType, const zbal_tensor_info_t *expandXOut,
                                       const zbal_tensor_info_t *dynamicScalesOut,
                                       const zbal_tensor_info_t *expandIdxOut,
                                       const zbal_tensor_info_t *expertTokenNumsOut,
                                       const zbal_tensor_info_t *epRecvCountsOut, const zbal_tensor_info_t *putOffset,
                                       const zbal_tensor_info_t *putOffsetStatus, aclrtStream stream,
                                       int64_t flags) = 0;
    virtual int32_t CombineLowLatency(const zbal_tensor_info_t *expandX, const zbal_tensor_info_t *expertIds,
                                      const zbal_tensor_info_t *expertIdx, const zbal_tensor_info_t *epSendCounts,
                                      const zbal_tensor_info_t *expertScales, const zbal_tensor_info_t *xOut,
                                      int64_t moeExpertNum, aclrtStream stream, int64_t flags) = 0;
    virtual int32_t FusedDeepMoe(const zbal_tensor_info_t *x, const zbal_tensor_info_t *expertIds,
                                 const zbal_tensor_info_t *gmm1Weight, const zbal_tensor_info_t *gmm1Scale,
                                 const zbal_tensor_info_t *gmm2Weight, const zbal_tensor_info_t *gmm2Scale,
                                 const zbal_tensor_info_t *expertScales, const zbal_tensor_info_t *expertSmoothScales,
                                 const zbal_tensor_info_t *shareGmm1Weight, const zbal_tensor_info_t *shareGmm1Scale,
                                 const zbal_tensor_info_t *shareGmm2Weight, const zbal_tensor_info_t *shareGmm2Scale,
                                 const zbal_tensor_info_t *shareSmoothScales, const zbal_tensor_info_t *xActiveMask,
                                 const zbal_tensor_info_t *output, const zbal_tensor_info_t *shareOutput,
                                 const zbal_tensor_info_t *expertTokenNums, const zbal_tensor_info_t *workspace,
                                 int64_t moeExpertNum, int64_t quantMode, int64_t globalBs, int64_t gmm1HLen,
                                 int64_t shareGmm1HLen, bool isTensorList, aclrtStream stream, int64_t flags) = 0;
    virtual int32_t TopkRoute(const zbal_tensor_info_t *logits, int64_t topkNum, const zbal_tensor_info_t *topkIndex,
                              const zbal_tensor_info_t *topkWeight, aclrtStream stream, int64_t flags) = 0;
    virtual int32_t WeightPrepack(const zbal_tensor_info_t *src, const zbal_tensor_info_t *dst, aclrtStream stream,
                                  int64_t flags) = 0;

protected:
    GroupInfo info_;
    mutable std::mutex peersMutex_;
};

using CommunicatorPtr = std::shared_ptr<Communicator>;

/* Backends */
CommunicatorPtr MakeGpuCommunicator(const GroupInfo &info);
CommunicatorPtr MakeDummyCommunicator(const GroupInfo &info);

/* Registry (reference operators/zbal_communicator.cpp:36-300) */
namespace registry {
int32_t Create(const zbal_comm_options_t &options, zbal_comm_t *out);
int32_t Destroy(zbal_comm_t comm);
void DestroyAll();
zbal_comm_t Global();
zbal_comm_t ByName(const std::string &name);
/* shared ownership keeps the object alive for the duration of an operator call */
CommunicatorPtr Find(zbal_comm_t comm);
uint32_t Count();
/* every communicator writes its device trace (reference Communicator::DumpAllComm, zbal_communicator.cpp:180-186) */
void DumpAllTraces();
} // namespace registry

/*
 * The shared expert of the fused operator comes as a set: both weights, both scales, shareOutput and a positive
 * shareGmm1HLen, or none of them (smooth scales only with it). One check for the C API and the launcher seam.
 */
bool SharedExpertArgsConsistent(const char *op, const zbal_tensor_info_t *shareGmm1Weight,
                                const zbal_tensor_info_t *shareGmm1Scale, const zbal_tensor_info_t *shareGmm2Weight,
                                const zbal_tensor_info_t *shareGmm2Scale, const zbal_tensor_info_t *shareSmoothScales,
                                const zbal_tensor_info_t *shareOutput, int64_t shareGmm1HLen);

/* Layout of the fused operator's workspace; one function so that sizing and carving cannot diverge. */
struct FusedWorkspace {
    uint64_t q1, xs, expand_idx, counts, row_off, layout_scratch, q2, scale2, sgl, y, total;
};
/* shareN1 = output width of the shared expert's first GEMM, 0 without a shared expert */
bool PlanFusedWorkspace(int64_t tokens, int64_t hidden, int64_t topk, int64_t experts, int64_t n1, int64_t shareN1,
                        int64_t quantMode, FusedWorkspace *ws);

} // namespace zbal

#endif /* ZBAL_HOST_H_ */
