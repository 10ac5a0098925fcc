/*
 * HIP backend of the communicator: checks tensor descriptors against what
 * each kernel assumes (type, rank, extent, alignment), then forwards to the
 * zbalhip_* launchers. The counterpart of the reference's
 * operators/npu/zbal_npu_communicator_base.cpp, which forwards each virtual
 * to a ZBALOp* launcher (:306-369 for the MoE operators, :371-438 for the
 * fused one).
 *
 * Ranks are modelled on one GPU: a group's peer windows are local
 * allocations registered per rank. Normal-mode notify, dispatch and combine
 * and the reductions address the other ranks' buffers through that window
 * table (the same offset in every window); a group of one needs no window.
 * The low-latency and fused operators run for a group of one rank, which
 * owns all experts.
 */
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <fstream>

#include "zbal_hip_kernels.h"
#include "zbal_host.h"

namespace zbal {

static uint64_t Align256(uint64_t v) { return (v + 255u) & ~uint64_t(255); }

namespace {

int64_t Numel(const zbal_tensor_info_t *t)
{
    if (t->dim == 0 || t->dim > ZBAL_MAX_TENSOR_DIM) return 0;
    int64_t n = 1;
    for (int i = 0; i < t->dim; ++i) n *= t->shape[i];
    return n;
}

const char *DtName(int dt)
{
    static const char *names[] = {"int8",  "int16", "int32",  "int64",  "uint64", "fp64",    "fp16",
                                  "fp32",  "bf16",  "uint8",  "uint16", "uint32", "fp8e4m3", "int4x2"};
    return (dt >= 0 && dt < ZBAL_DATA_TYPE_BUTT) ? names[dt] : "?";
}

/* data non-null, one of two allowed types, at least min_elems elements */
bool CheckTensor(const char *op, const char *name, const zbal_tensor_info_t *t, int dt_a, int dt_b, int64_t min_elems)
{
    if (t->data == nullptr) {
        ZBAL_LOG_AND_SET_LAST_ERROR(op << " failed as " << name << " has no data");
        return false;
    }
    if ((int)t->dataType != dt_a && (int)t->dataType != dt_b) {
        ZBAL_LOG_AND_SET_LAST_ERROR(op << " failed as " << name << " has type " << DtName(t->dataType) << ", expected "
                                       << DtName(dt_a) << (dt_b != dt_a ? std::string(" or ") + DtName(dt_b) : ""));
        return false;
    }
    if (Numel(t) < min_elems) {
        ZBAL_LOG_AND_SET_LAST_ERROR(op << " failed as " << name << " holds " << Numel(t) << " elements, needs "
                                       << min_elems);
        return false;
    }
    if ((reinterpret_cast<uintptr_t>(t->data) & 15u) != 0) {
        ZBAL_LOG_AND_SET_LAST_ERROR(op << " failed as " << name << " is not 16-byte aligned");
        return false;
    }
    return true;
}

#define ZB_CHECK(...)                           \
    do {                                        \
        if (!CheckTensor(__VA_ARGS__)) return Z_INVALID_PARAM; \
    } while (0)

int32_t Launched(const char *op, int32_t rc)
{
    if (rc != 0) ZBAL_LOG_AND_SET_LAST_ERROR(op << " launch failed, code " << rc);
    return rc;
}

/* names of the frames the kernels record, by zbal_profiling_name_t value (reference
   zbal_comm_host_device_struct.h:27-70 and g_profName :76-120) */
enum { PROF_RS_KERNEL_ALL = 7, PROF_AR_KERNEL_ALL = 17 };
const char *ProfName(uint64_t frame)
{
    switch (frame) {
        case PROF_RS_KERNEL_ALL: return "RS_KERNEL_ALL";
        case PROF_AR_KERNEL_ALL: return "AR_KERNEL_ALL";
        default: return nullptr;
    }
}

class GpuCommunicator final : public Communicator {
public:
    /*
     * Tracing follows the reference's switches (zbal_env_helper.h:20-22, SetupProfMemory
     * zbal_npu_communicator_base.cpp:145-199): ZBAL_PROF_ENABLE=1 turns it on, ZBAL_PROF_MAX_TRACING_COUNT is the
     * number of 64-bit words per traced workgroup (20480 unless in [20480, 204800)), ZBAL_PROF_DIR the directory
     * of the dump. The ring is pinned host memory the kernels write directly; every communicator created with
     * tracing on owns one and hands it to its own launches.
     */
    explicit GpuCommunicator(const GroupInfo &info) : Communicator(info)
    {
        /*
         * The grouped-GEMM kernels are set up for this GPU now, so that none of them meets its first launch inside a
         * stream capture later. Without a usable GPU (host-only checks of the API) this fails and is left to the launches.
         */
        (void)zbalhip_gemm_prepare();
        const char *sw = std::getenv("ZBAL_PROF_ENABLE");
        if (!info.traced || sw == nullptr || std::atoi(sw) != 1) return;
        int64_t points = 20480;
        if (const char *c = std::getenv("ZBAL_PROF_MAX_TRACING_COUNT")) {
            const long long v = std::atoll(c);
            if (v >= 20480 && v < 204800) points = v;
        }
        if (zbalhip_trace_alloc(points, &traceHost_, &traceDev_) != 0) {
            ZBAL_LOG_AND_SET_LAST_ERROR("Failed to allocate " << points * ZBALHIP_TRACE_UNITS * 8 << " bytes of trace memory");
            traceHost_ = traceDev_ = nullptr;
            return;
        }
        tracePoints_ = points;
    }

    ~GpuCommunicator() override
    {
        if (traceHost_ == nullptr) return;
        DumpProfilingTrace();
        zbalhip_trace_free(traceHost_);
    }

    /*
     * One begin / end event per record, in the format of the reference's trace-viewer writer
     * (zbal_trace_viewer_dumper.h:277-304; DumpProfilingTrace zbal_npu_communicator_base.cpp:215-271): a JSON
     * array that chrome://tracing and Perfetto load. Timestamps are microseconds of the GPU's 100 MHz clock.
     */
    void DumpProfilingTrace() noexcept override
    {
        if (traceHost_ == nullptr) return;
        if (zbalhip_trace_sync() != 0) return;
        const char *dir = std::getenv("ZBAL_PROF_DIR");
        char stamp[64];
        std::time_t now = std::time(nullptr);
        struct tm lt;
        localtime_r(&now, &lt);
        std::strftime(stamp, sizeof(stamp), "%Y_%m_%d_%H_%M_%S", &lt);
        const uint32_t rank = info_.myGroupRank;
        const std::string path = std::string(dir ? dir : "/home/") + "/trace_view_" + std::to_string(rank) + "_" +
                                 std::to_string(info_.groupIndex) + "_" + stamp + ".json";
        std::ofstream f(path);
        if (!f) {
            ZBAL_LOG_AND_SET_LAST_ERROR("rank " << rank << " print profiling, open dump file " << path << " failed");
            return;
        }
        f << "[";
        bool first = true;
        for (uint64_t u = 0; u < ZBALHIP_TRACE_UNITS; ++u) {
            const uint64_t *blk = traceHost_ + u * tracePoints_;
            for (uint64_t j = ZBALHIP_TRACE_REC_OFF; j < (uint64_t)tracePoints_; ++j) {
                const uint64_t rec = blk[j];
                const uint64_t frame = (rec >> ZBALHIP_TRACE_FRAME_SHIFT) & ((1u << (ZBALHIP_TRACE_BE_SHIFT - ZBALHIP_TRACE_FRAME_SHIFT)) - 1);
                if (frame == 0) break; /* the rest of the block is empty */
                const char *name = ProfName(frame);
                if (name == nullptr) break;
                const bool end = (rec >> ZBALHIP_TRACE_BE_SHIFT) & 1;
                const uint64_t ticks = rec & ((1ull << ZBALHIP_TRACE_FRAME_SHIFT) - 1);
                char ts[32];
                std::snprintf(ts, sizeof(ts), "%llu.%02llu", (unsigned long long)(ticks / 100), (unsigned long long)(ticks % 100));
                f << (first ? "\n" : ",\n") << "{\"name\":\"" << name << "\", \"ph\":\"" << (end ? 'E' : 'B')
                  << "\", \"pid\":\"RANK_" << rank << "\", \"tid\":\"wg " << u << "\", \"ts\":" << ts << "}";
                first = false;
            }
        }
        f << "\n]";
        ZBAL_LOG(LOG_INFO, "dump trace " << info_.groupIndex << " on rank " << rank << " finished: " << path);
    }

private:
    uint64_t *traceHost_ = nullptr, *traceDev_ = nullptr;
    int64_t tracePoints_ = 0;

public:

    bool SingleRank(const char *op) const
    {
        if (info_.groupSize == 1) return true;
        ZBAL_LOG_AND_SET_LAST_ERROR(op << " failed as this build runs MoE operators on a group of one rank, group has "
                                       << info_.groupSize);
        return false;
    }

    /* address of `p` (inside my window) in rank r's window */
    bool Translate(const char *op, const void *p, size_t bytes, const void **out) const
    {
        if (info_.peerStride != 0) { /* symmetric address space: the same offset in every rank's slice */
            const int64_t me = info_.worldRank[info_.myGroupRank];
            for (uint16_t r = 0; r < info_.groupSize; ++r)
                out[r] = static_cast<const uint8_t *>(p) + ((int64_t)info_.worldRank[r] - me) * (int64_t)info_.peerStride;
            return true;
        }
        const std::vector<PeerWindow> peers = Peers();
        const PeerWindow &mine = peers[info_.myGroupRank];
        const uintptr_t a = reinterpret_cast<uintptr_t>(p), b = reinterpret_cast<uintptr_t>(mine.base);
        if (mine.base == nullptr || a < b || a + bytes > b + mine.size) {
            ZBAL_LOG_AND_SET_LAST_ERROR(op << " failed as the send buffer is not inside this rank's registered window");
            return false;
        }
        for (uint16_t r = 0; r < info_.groupSize; ++r) {
            const PeerWindow &w = peers[r];
            if (w.base == nullptr || (a - b) + bytes > w.size) {
                ZBAL_LOG_AND_SET_LAST_ERROR(op << " failed as rank " << r << " has no window covering the buffer");
                return false;
            }
            out[r] = static_cast<const uint8_t *>(w.base) + (a - b);
        }
        return true;
    }

    /* the copies of `p` in every rank's window; a group of one needs no window: its only copy is `p` itself */
    bool PeerCopies(const char *op, const void *p, size_t bytes, const void **out) const
    {
        if (info_.groupSize == 1 && info_.peerStride == 0 && Peers()[0].base == nullptr) {
            out[0] = p;
            return true;
        }
        return Translate(op, p, bytes, out);
    }

    static size_t ElemSize(zbal_datatype_t dt)
    {
        switch (dt) {
            case ZBAL_DATA_TYPE_INT8: case ZBAL_DATA_TYPE_UINT8: case ZBAL_DATA_TYPE_FP8_E4M3: case ZBAL_DATA_TYPE_INT4X2: return 1;
            case ZBAL_DATA_TYPE_INT16: case ZBAL_DATA_TYPE_UINT16: case ZBAL_DATA_TYPE_FP16: case ZBAL_DATA_TYPE_BFP16: return 2;
            case ZBAL_DATA_TYPE_INT32: case ZBAL_DATA_TYPE_UINT32: case ZBAL_DATA_TYPE_FP32: return 4;
            case ZBAL_DATA_TYPE_INT64: case ZBAL_DATA_TYPE_UINT64: case ZBAL_DATA_TYPE_FP64: return 8;
            default: return 0;
        }
    }

    int32_t Reduce(const char *opName, int traceFrame, const void *send, size_t sliceOffsetElems, void *recv, size_t count,
                   zbal_datatype_t dt, zbal_reduce_op_t op, aclrtStream stream)
    {
        switch (dt) { /* the types the reference instantiates, zbal_kernel_allreduce.cpp:378-416 */
            case ZBAL_DATA_TYPE_INT8: case ZBAL_DATA_TYPE_INT16: case ZBAL_DATA_TYPE_INT32: case ZBAL_DATA_TYPE_INT64:
            case ZBAL_DATA_TYPE_FP16: case ZBAL_DATA_TYPE_BFP16: case ZBAL_DATA_TYPE_FP32: break;
            default:
                ZBAL_LOG_AND_SET_LAST_ERROR(opName << " failed as data type " << DtName(dt) << " is not supported");
                return Z_INVALID_PARAM;
        }
        if (info_.groupSize > ZBALHIP_MAX_REDUCE_PEERS) {
            ZBAL_LOG_AND_SET_LAST_ERROR(opName << " failed as group size " << info_.groupSize << " exceeds "
                                               << ZBALHIP_MAX_REDUCE_PEERS);
            return Z_INVALID_PARAM;
        }
        const size_t es = ElemSize(dt);
        const void *peer[ZBALHIP_MAX_REDUCE_PEERS];
        if (info_.groupSize == 1 && info_.peerStride == 0 && Peers()[0].base == nullptr) {
            peer[0] = send; /* a group of one needs no window */
        } else if (!Translate(opName, send, (sliceOffsetElems + count) * es, peer)) {
            return Z_INVALID_PARAM;
        }
        for (uint16_t r = 0; r < info_.groupSize; ++r)
            peer[r] = static_cast<const uint8_t *>(peer[r]) + sliceOffsetElems * es;
        return Launched(opName, zbalhip_reduce(peer, info_.groupSize, (int64_t)count, dt, op, recv, traceFrame, traceDev_,
                                               tracePoints_, stream));
    }

    int32_t AllReduce(const void *send, void *recv, void *, size_t count, zbal_datatype_t dt, zbal_reduce_op_t op,
                      aclrtStream stream) override
    {
        return Reduce("AllReduce", PROF_AR_KERNEL_ALL, send, 0, recv, count, dt, op, stream);
    }

    int32_t ReduceScatter(const void *send, void *recv, size_t recvCount, zbal_datatype_t dt, zbal_reduce_op_t op,
                          aclrtStream stream) override
    {
        return Reduce("ReduceScatter", PROF_RS_KERNEL_ALL, send, (size_t)info_.myGroupRank * recvCount, recv, recvCount, dt, op,
                      stream);
    }

    int32_t DispatchNormalLayout(const zbal_tensor_info_t *topkIndex, int64_t tokens, int64_t expertNum,
                                 int64_t topkNum, const zbal_tensor_info_t *tokensPerRank,
                                 const zbal_tensor_info_t *tokensPerExpert, const zbal_tensor_info_t *sendTokensIndex,
                                 const zbal_tensor_info_t *notifySendData, aclrtStream stream, int64_t) override
    {
        const char *op = "DispatchLayout";
        const int64_t R = info_.groupSize;
        ZBAL_VALIDATE_RETURN(expertNum % R == 0, op << " failed as expertNum " << expertNum
                                                    << " is not a multiple of the group size " << R, Z_INVALID_PARAM);
        ZBAL_VALIDATE_RETURN(expertNum <= 1024, op << " failed as expertNum " << expertNum << " exceeds 1024",
                             Z_INVALID_PARAM);
        ZB_CHECK(op, "tokensPerRank", tokensPerRank, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, R);
        ZB_CHECK(op, "tokensPerExpert", tokensPerExpert, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, expertNum);
        ZB_CHECK(op, "notifySendData", notifySendData, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32,
                 (int64_t)ZBALHIP_LAYOUT_MAX_BLOCKS * expertNum);
        if (tokens > 0) {
            ZB_CHECK(op, "topkIndex", topkIndex, ZBAL_DATA_TYPE_INT64, ZBAL_DATA_TYPE_INT32, tokens * topkNum);
            ZB_CHECK(op, "sendTokensIndex", sendTokensIndex, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32,
                     tokens * topkNum);
        }
        return Launched(op, zbalhip_dispatch_layout(topkIndex->data, topkIndex->dataType == ZBAL_DATA_TYPE_INT64,
                                                    tokens, expertNum, topkNum, (int32_t)R,
                                                    (int32_t *)tokensPerRank->data, (int32_t *)tokensPerExpert->data,
                                                    (int32_t *)sendTokensIndex->data, (int32_t *)notifySendData->data,
                                                    stream));
    }

    int32_t DispatchNormalNotify(const zbal_tensor_info_t *sendTokensPerExpert, int64_t sendCount, int64_t topKNum,
                                 const zbal_tensor_info_t *recvBuff, const zbal_tensor_info_t *totalRecvTokens,
                                 const zbal_tensor_info_t *recvTokensPerExpert,
                                 const zbal_tensor_info_t *pushTargetOffset, const zbal_tensor_info_t *balanceMatrix,
                                 aclrtStream stream, int64_t) override
    {
        const char *op = "NotifyDispatch";
        const int64_t R = info_.groupSize, me = info_.myGroupRank;
        const int64_t E = sendCount; /* one count per expert, zbal_deepep.cpp:325-326 */
        ZBAL_VALIDATE_RETURN(E <= 1024, op << " failed as sendCount " << E << " exceeds 1024", Z_INVALID_PARAM);
        ZBAL_VALIDATE_RETURN(R <= ZBALHIP_MAX_REDUCE_PEERS && E % R == 0,
                             op << " failed as " << E << " experts do not split over a group of " << R, Z_INVALID_PARAM);
        ZB_CHECK(op, "sendTokensPerExpert", sendTokensPerExpert, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, E);
        ZB_CHECK(op, "recvBuff", recvBuff, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, R * E);
        ZB_CHECK(op, "totalRecvTokens", totalRecvTokens, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, 1);
        ZB_CHECK(op, "recvTokensPerExpert", recvTokensPerExpert, ZBAL_DATA_TYPE_INT64, ZBAL_DATA_TYPE_INT64, E / R);
        ZB_CHECK(op, "pushTargetOffset", pushTargetOffset, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, R * E);
        ZB_CHECK(op, "balanceMatrix", balanceMatrix, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, R * 2 * R);
        /* the counts of the other ranks are read where they lie: at the same offset in each rank's window */
        const void *counts[ZBALHIP_MAX_REDUCE_PEERS];
        if (!PeerCopies(op, sendTokensPerExpert->data, (size_t)E * 4, counts)) return Z_INVALID_PARAM;
        return Launched(op, zbalhip_dispatch_notify((const int32_t *const *)counts, (int32_t)R, (int32_t)me, E, topKNum,
                                                    (int32_t *)recvBuff->data, (int32_t *)pushTargetOffset->data,
                                                    (int32_t *)totalRecvTokens->data,
                                                    (int64_t *)recvTokensPerExpert->data,
                                                    (int32_t *)balanceMatrix->data, stream));
    }

    static bool TokensShape(const char *op, const zbal_tensor_info_t *x, int64_t *tokens, int64_t *hidden)
    {
        if (x->dim != 2) {
            ZBAL_LOG_AND_SET_LAST_ERROR(op << " failed as the token tensor must be [tokens, hidden]");
            return false;
        }
        *tokens = x->shape[0];
        *hidden = x->shape[1];
        return true;
    }

    int32_t DispatchNormal(const zbal_tensor_info_t *srcTokens, const zbal_tensor_info_t *topkIndex,
                           const zbal_tensor_info_t *sendTokensIndex, const zbal_tensor_info_t *pushTargetOffset,
                           const zbal_tensor_info_t *, int64_t expertNum, zbal_quant_mode_t quantMode,
                           const zbal_tensor_info_t *destTokens, const zbal_tensor_info_t *destScale,
                           aclrtStream stream, int64_t) override
    {
        const char *op = "DispatchNormal";
        const int64_t R = info_.groupSize, me = info_.myGroupRank;
        ZBAL_VALIDATE_RETURN(R <= ZBALHIP_MAX_REDUCE_PEERS && expertNum % R == 0,
                             op << " failed as " << expertNum << " experts do not split over a group of " << R, Z_INVALID_PARAM);
        int64_t T = 0, H = 0;
        if (!TokensShape(op, srcTokens, &T, &H)) return Z_INVALID_PARAM;
        ZBAL_VALIDATE_RETURN(topkIndex->dim == 2 && topkIndex->shape[0] == T, op << " failed as topkIndex must be [tokens, topk]",
                             Z_INVALID_PARAM);
        const int64_t K = topkIndex->shape[1];
        ZBAL_VALIDATE_RETURN(quantMode == NO_QUANT || quantMode == QUANT_BF16_2_INT8 ||
                                 quantMode == QUANT_BF16_2_FP8E4M3_B128,
                             op << " failed as quantMode " << quantMode << " is invalid", Z_INVALID_PARAM);
        /* rows are stored densely; the reference pads row strides to 32 bytes (dispatch_normal.h:215) */
        const int64_t rowBytes = H * (quantMode == NO_QUANT ? 2 : 1);
        ZBAL_VALIDATE_RETURN(rowBytes % 32 == 0, op << " failed as a row of " << rowBytes << " bytes is not a multiple of 32",
                             Z_INVALID_PARAM);
        if (T == 0) return Z_OK;
        ZB_CHECK(op, "srcTokens", srcTokens, ZBAL_DATA_TYPE_BFP16, ZBAL_DATA_TYPE_FP16, T * H);
        ZB_CHECK(op, "topkIndex", topkIndex, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, T * K);
        ZB_CHECK(op, "sendTokensIndex", sendTokensIndex, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, T * K);
        ZB_CHECK(op, "pushTargetOffset", pushTargetOffset, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, expertNum * R);
        int64_t scalesPerRow = 0;
        if (quantMode == NO_QUANT) {
            ZB_CHECK(op, "destTokens", destTokens, srcTokens->dataType, srcTokens->dataType, H);
        } else if (quantMode == QUANT_BF16_2_INT8) {
            ZB_CHECK(op, "destTokens", destTokens, ZBAL_DATA_TYPE_INT8, ZBAL_DATA_TYPE_INT8, H);
            ZB_CHECK(op, "destScale", destScale, ZBAL_DATA_TYPE_FP32, ZBAL_DATA_TYPE_FP32, 1);
            scalesPerRow = 1;
        } else {
            ZB_CHECK(op, "destTokens", destTokens, ZBAL_DATA_TYPE_FP8_E4M3, ZBAL_DATA_TYPE_UINT8, H);
            ZB_CHECK(op, "destScale", destScale, ZBAL_DATA_TYPE_FP32, ZBAL_DATA_TYPE_FP32, H / 128);
            scalesPerRow = H / 128;
        }
        /*
         * The receive tensors may be sized from the received-token total (the reference does, zbal_deepep.cpp:359-375):
         * the kernel gets the number of rows they hold and drops what would land past it instead of writing there.
         */
        int64_t destRows = Numel(destTokens) / H;
        if (scalesPerRow > 0 && Numel(destScale) / scalesPerRow < destRows) destRows = Numel(destScale) / scalesPerRow;
        /* rank r's receive tensors sit at the same offset in rank r's window */
        const void *dest[ZBALHIP_MAX_REDUCE_PEERS], *scale[ZBALHIP_MAX_REDUCE_PEERS] = {};
        if (!PeerCopies(op, destTokens->data, (size_t)destRows * rowBytes, dest)) return Z_INVALID_PARAM;
        if (scalesPerRow > 0 && !PeerCopies(op, destScale->data, (size_t)destRows * scalesPerRow * 4, scale)) return Z_INVALID_PARAM;
        return Launched(op, zbalhip_dispatch_normal(srcTokens->data, srcTokens->dataType, (const int32_t *)topkIndex->data,
                                                    (const int32_t *)sendTokensIndex->data,
                                                    (const int32_t *)pushTargetOffset->data, T, H, K, expertNum,
                                                    (int32_t)quantMode, (void *const *)dest,
                                                    scalesPerRow > 0 ? (float *const *)scale : nullptr, (int32_t)R,
                                                    (int32_t)me, destRows, stream));
    }

    int32_t CombineNormal(const zbal_tensor_info_t *srcTokens, const zbal_tensor_info_t *srcTokensPerEp,
                          const zbal_tensor_info_t *topKWeight, const zbal_tensor_info_t *topkIndex,
                          const zbal_tensor_info_t *sendTokensIndex, const zbal_tensor_info_t *, uint16_t expertNum,
                          const zbal_tensor_info_t *destTokens, aclrtStream stream, int64_t) override
    {
        const char *op = "CombineNormal";
        const int64_t R = info_.groupSize, me = info_.myGroupRank;
        ZBAL_VALIDATE_RETURN(R <= ZBALHIP_MAX_REDUCE_PEERS && expertNum % R == 0,
                             op << " failed as " << expertNum << " experts do not split over a group of " << R, Z_INVALID_PARAM);
        int64_t T = 0, H = 0;
        if (!TokensShape(op, destTokens, &T, &H)) return Z_INVALID_PARAM;
        ZBAL_VALIDATE_RETURN(topkIndex->dim == 2 && topkIndex->shape[0] == T, op << " failed as topkIndex must be [tokens, topk]",
                             Z_INVALID_PARAM);
        const int64_t K = topkIndex->shape[1];
        ZBAL_VALIDATE_RETURN(K <= 32, op << " failed as topk " << K << " exceeds 32", Z_INVALID_PARAM);
        ZBAL_VALIDATE_RETURN((H * 2) % 32 == 0, op << " failed as hidden " << H << " gives rows that are not a multiple of 32 bytes",
                             Z_INVALID_PARAM);
        if (T == 0) return Z_OK;
        ZB_CHECK(op, "srcTokens", srcTokens, ZBAL_DATA_TYPE_BFP16, ZBAL_DATA_TYPE_FP16, H);
        ZBAL_VALIDATE_RETURN(srcTokens->dataType == destTokens->dataType, op << " failed as source and destination types differ",
                             Z_INVALID_PARAM);
        ZB_CHECK(op, "destTokens", destTokens, srcTokens->dataType, srcTokens->dataType, T * H);
        ZB_CHECK(op, "srcTokensPerEp", srcTokensPerEp, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, expertNum * R);
        ZB_CHECK(op, "topKWeight", topKWeight, ZBAL_DATA_TYPE_FP32, ZBAL_DATA_TYPE_FP32, T * K);
        ZB_CHECK(op, "topkIndex", topkIndex, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, T * K);
        ZB_CHECK(op, "sendTokensIndex", sendTokensIndex, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, T * K);
        /* the expert outputs are read from the window of the rank that owns the expert; rows past what they hold are skipped */
        const int64_t srcRows = Numel(srcTokens) / H;
        const void *src[ZBALHIP_MAX_REDUCE_PEERS];
        if (!PeerCopies(op, srcTokens->data, (size_t)srcRows * H * 2, src)) return Z_INVALID_PARAM;
        return Launched(op, zbalhip_combine(src, (int32_t)R, (int32_t)me, srcRows, srcTokens->dataType,
                                            (const int32_t *)srcTokensPerEp->data, 0, (const float *)topKWeight->data,
                                            (const int32_t *)topkIndex->data, (const int32_t *)sendTokensIndex->data, T, H, K,
                                            expertNum, destTokens->data, stream));
    }

    int32_t DispatchLowLatency(const zbal_tensor_info_t *x, const zbal_tensor_info_t *expertIds, int64_t moeExpertNum,
                               int64_t, int64_t sharedExpertRankNum, int64_t quantMode, int64_t, int64_t,
                               int64_t expertTokenNumsType, const zbal_tensor_info_t *expandXOut,
                               const zbal_tensor_info_t *dynamicScalesOut, const zbal_tensor_info_t *expandIdxOut,
                               const zbal_tensor_info_t *expertTokenNumsOut, const zbal_tensor_info_t *epRecvCountsOut,
                               const zbal_tensor_info_t *putOffset, const zbal_tensor_info_t *, aclrtStream stream,
                               int64_t) override
    {
        const char *op = "DispatchLowlatency";
        const int64_t R = info_.groupSize, me = info_.myGroupRank;
        ZBAL_VALIDATE_RETURN(R <= ZBALHIP_MAX_REDUCE_PEERS && moeExpertNum % R == 0,
                             op << " failed as " << moeExpertNum << " experts do not split over a group of " << R, Z_INVALID_PARAM);
        ZBAL_VALIDATE_RETURN(sharedExpertRankNum == 0, op << " failed as shared expert ranks are not supported", Z_INVALID_PARAM);
        ZBAL_VALIDATE_RETURN(expertTokenNumsType == 0 || expertTokenNumsType == 1,
                             op << " failed as expertTokenNumsType " << expertTokenNumsType << " is invalid", Z_INVALID_PARAM);
        ZBAL_VALIDATE_RETURN(quantMode >= 0 && quantMode <= 2, op << " failed as quantMode " << quantMode << " is invalid",
                             Z_INVALID_PARAM);
        ZBAL_VALIDATE_RETURN(moeExpertNum <= 1024, op << " failed as moeExpertNum exceeds 1024", Z_INVALID_PARAM);
        int64_t T = 0, H = 0;
        if (!TokensShape(op, x, &T, &H)) return Z_INVALID_PARAM;
        ZBAL_VALIDATE_RETURN(expertIds->dim == 2 && expertIds->shape[0] == T, op << " failed as expertIds must be [tokens, topk]",
                             Z_INVALID_PARAM);
        const int64_t K = expertIds->shape[1];
        const int64_t rowBytes = H * (quantMode == 0 ? 2 : 1);
        ZBAL_VALIDATE_RETURN(rowBytes % 32 == 0, op << " failed as a row of " << rowBytes << " bytes is not a multiple of 32",
                             Z_INVALID_PARAM);
        const int64_t E = moeExpertNum;
        /* per local expert; one count per (rank, expert) pair (zbal_deepep.cpp:525-534) */
        ZB_CHECK(op, "expertTokenNumsOut", expertTokenNumsOut, ZBAL_DATA_TYPE_INT64, ZBAL_DATA_TYPE_INT64, E / R);
        ZB_CHECK(op, "epRecvCountsOut", epRecvCountsOut, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, E * R);
        ZB_CHECK(op, "putOffset", putOffset, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, E * R);
        /* an empty batch has empty per-token tensors (torch hands out a null pointer for them): only the counts are written */
        if (T > 0) {
            ZB_CHECK(op, "x", x, ZBAL_DATA_TYPE_BFP16, ZBAL_DATA_TYPE_FP16, T * H);
            ZB_CHECK(op, "expertIds", expertIds, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, T * K);
            ZB_CHECK(op, "expandIdxOut", expandIdxOut, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, T * K);
            /* every pick may be valid, so the packed output must hold tokens * topk rows */
            if (quantMode == 0) {
                ZB_CHECK(op, "expandXOut", expandXOut, x->dataType, x->dataType, T * K * H);
            } else {
                ZB_CHECK(op, "expandXOut", expandXOut, quantMode == 1 ? ZBAL_DATA_TYPE_INT8 : ZBAL_DATA_TYPE_FP8_E4M3,
                         quantMode == 1 ? ZBAL_DATA_TYPE_INT8 : ZBAL_DATA_TYPE_UINT8, T * K * H);
                ZB_CHECK(op, "dynamicScalesOut", dynamicScalesOut, ZBAL_DATA_TYPE_FP32, ZBAL_DATA_TYPE_FP32,
                         quantMode == 1 ? T * K : T * K * (H / 128));
            }
        }
        if (R > 1) {
            /*
             * Every rank's expert ids and receive tensors sit at the same offset in that rank's window: the counts are
             * taken from all ranks' ids, the rows go to the window of the rank that owns the expert. The receive
             * tensors may be sized for what the rank receives; rows past them are dropped, not written.
             */
            const int64_t scalesPerRow = quantMode == 0 ? 0 : (quantMode == 1 ? 1 : H / 128);
            int64_t destRows = T > 0 ? Numel(expandXOut) / H : 0;
            if (T > 0 && scalesPerRow > 0 && Numel(dynamicScalesOut) / scalesPerRow < destRows)
                destRows = Numel(dynamicScalesOut) / scalesPerRow;
            const void *ids[ZBALHIP_MAX_REDUCE_PEERS] = {}, *dest[ZBALHIP_MAX_REDUCE_PEERS] = {}, *scale[ZBALHIP_MAX_REDUCE_PEERS] = {};
            if (T > 0) {
                if (!PeerCopies(op, expertIds->data, (size_t)(T * K) * 4, ids)) return Z_INVALID_PARAM;
                if (!PeerCopies(op, expandXOut->data, (size_t)destRows * rowBytes, dest)) return Z_INVALID_PARAM;
                if (scalesPerRow > 0 && !PeerCopies(op, dynamicScalesOut->data, (size_t)destRows * scalesPerRow * 4, scale))
                    return Z_INVALID_PARAM;
            }
            return Launched(op, zbalhip_dispatch_low_latency_ranks(
                                    x->data, x->dataType, (const int32_t *const *)ids, T, H, K, E, (int32_t)quantMode,
                                    (int32_t)expertTokenNumsType, (void *const *)dest, (float *const *)scale, (int32_t)R,
                                    (int32_t)me, destRows, (int32_t *)expandIdxOut->data, (int64_t *)expertTokenNumsOut->data,
                                    (int32_t *)epRecvCountsOut->data, (int32_t *)putOffset->data, stream));
        }
        int64_t blocks = Numel(putOffset) / E;
        if (blocks > ZBALHIP_LAYOUT_MAX_BLOCKS) blocks = ZBALHIP_LAYOUT_MAX_BLOCKS;
        return Launched(op, zbalhip_dispatch_low_latency(x->data, x->dataType, (const int32_t *)expertIds->data, T, H, K, E,
                                                         (int32_t)quantMode, (int32_t)expertTokenNumsType,
                                                         expandXOut->data, (float *)dynamicScalesOut->data,
                                                         (int32_t *)expandIdxOut->data,
                                                         (int64_t *)expertTokenNumsOut->data,
                                                         (int32_t *)epRecvCountsOut->data, (int32_t *)putOffset->data,
                                                         (int32_t)blocks, stream));
    }

    int32_t CombineLowLatency(const zbal_tensor_info_t *expandX, const zbal_tensor_info_t *expertIds,
                              const zbal_tensor_info_t *expertIdx, const zbal_tensor_info_t *epSendCounts,
                              const zbal_tensor_info_t *expertScales, const zbal_tensor_info_t *xOut,
                              int64_t moeExpertNum, aclrtStream stream, int64_t) override
    {
        const char *op = "CombineLowlatency";
        const int64_t R = info_.groupSize, me = info_.myGroupRank;
        ZBAL_VALIDATE_RETURN(R <= ZBALHIP_MAX_REDUCE_PEERS && moeExpertNum % R == 0,
                             op << " failed as " << moeExpertNum << " experts do not split over a group of " << R, Z_INVALID_PARAM);
        int64_t T = 0, H = 0;
        if (!TokensShape(op, xOut, &T, &H)) return Z_INVALID_PARAM;
        ZBAL_VALIDATE_RETURN(expertIds->dim == 2 && expertIds->shape[0] == T, op << " failed as expertIds must be [tokens, topk]",
                             Z_INVALID_PARAM);
        const int64_t K = expertIds->shape[1];
        ZBAL_VALIDATE_RETURN(K <= 32, op << " failed as topk " << K << " exceeds 32", Z_INVALID_PARAM);
        ZBAL_VALIDATE_RETURN((H * 2) % 32 == 0, op << " failed as hidden " << H << " gives rows that are not a multiple of 32 bytes",
                             Z_INVALID_PARAM);
        if (T == 0) return Z_OK;
        ZB_CHECK(op, "expandX", expandX, ZBAL_DATA_TYPE_BFP16, ZBAL_DATA_TYPE_FP16, H);
        ZBAL_VALIDATE_RETURN(expandX->dataType == xOut->dataType, op << " failed as source and destination types differ",
                             Z_INVALID_PARAM);
        ZB_CHECK(op, "xOut", xOut, expandX->dataType, expandX->dataType, T * H);
        ZB_CHECK(op, "expertIds", expertIds, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, T * K);
        ZB_CHECK(op, "expertIdx", expertIdx, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, T * K);
        ZB_CHECK(op, "epSendCounts", epSendCounts, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, moeExpertNum * R);
        ZB_CHECK(op, "expertScales", expertScales, ZBAL_DATA_TYPE_FP32, ZBAL_DATA_TYPE_FP32, T * K);
        /* the expert outputs are read from the window of the rank that owns the expert (combine_low_latency.h:494-531) */
        const int64_t srcRows = Numel(expandX) / H;
        const void *src[ZBALHIP_MAX_REDUCE_PEERS];
        if (!PeerCopies(op, expandX->data, (size_t)srcRows * H * 2, src)) return Z_INVALID_PARAM;
        return Launched(op, zbalhip_combine(src, (int32_t)R, (int32_t)me, srcRows, expandX->dataType,
                                            (const int32_t *)epSendCounts->data, 1, (const float *)expertScales->data,
                                            (const int32_t *)expertIds->data, (const int32_t *)expertIdx->data, T, H, K,
                                            moeExpertNum, xOut->data, stream));
    }

    /* shapes and types of one FFN's weights and scales: `experts` experts of [H, N1] and [N1/2, H] */
    bool CheckFfnWeights(const char *op, const char *who, int mode, int64_t experts, int64_t H, int64_t N1,
                         const zbal_tensor_info_t *w1, const zbal_tensor_info_t *s1, const zbal_tensor_info_t *w2,
                         const zbal_tensor_info_t *s2, int *wscale2Dt)
    {
        const int64_t I = N1 / 2;
        const int wdt = mode == 1 ? ZBAL_DATA_TYPE_INT8 : (mode == 2 ? ZBAL_DATA_TYPE_FP8_E4M3 : ZBAL_DATA_TYPE_INT4X2);
        const int wdt_alt = mode == 2 ? ZBAL_DATA_TYPE_UINT8 : wdt;
        const int64_t wdiv = mode == 3 ? 2 : 1;
        ZBAL_VALIDATE_RETURN(N1 > 0 && N1 % 256 == 0, op << " failed as the " << who << " gmm1 width " << N1
                                                         << " must be a positive multiple of 256", false);
        ZBAL_VALIDATE_RETURN(w1->reserved[0] == ZBAL_WEIGHT_FORMAT_PREPACKED && w2->reserved[0] == ZBAL_WEIGHT_FORMAT_PREPACKED,
                             op << " failed as the " << who << " weights are not pre-packed (zbal_moe_weight_prepack)", false);
        auto check = [&](const char *name, const zbal_tensor_info_t *t, int dtA, int dtB, int64_t minElems) {
            ZBAL_VALIDATE_RETURN(t->data != nullptr, op << " failed as " << who << " " << name << " has no data", false);
            ZBAL_VALIDATE_RETURN(t->dataType == dtA || t->dataType == dtB,
                                 op << " failed as " << who << " " << name << " has data type " << t->dataType, false);
            ZBAL_VALIDATE_RETURN(Numel(t) >= minElems, op << " failed as " << who << " " << name << " holds " << Numel(t)
                                                          << " elements, needs " << minElems, false);
            return true;
        };
        if (!check("gmm1Weight", w1, wdt, wdt_alt, experts * H * N1 / wdiv)) return false;
        if (!check("gmm2Weight", w2, wdt, wdt_alt, experts * I * H / wdiv)) return false;
        *wscale2Dt = ZBAL_DATA_TYPE_FP32;
        if (mode == 1) {
            if (!check("gmm1Scale", s1, ZBAL_DATA_TYPE_FP32, ZBAL_DATA_TYPE_FP32, experts * N1)) return false;
            if (!check("gmm2Scale", s2, ZBAL_DATA_TYPE_BFP16, ZBAL_DATA_TYPE_FP32, experts * H)) return false;
            *wscale2Dt = s2->dataType;
        } else if (mode == 2) {
            if (!check("gmm1Scale", s1, ZBAL_DATA_TYPE_FP32, ZBAL_DATA_TYPE_FP32, experts * (H / 128) * (N1 / 128))) return false;
            if (!check("gmm2Scale", s2, ZBAL_DATA_TYPE_FP32, ZBAL_DATA_TYPE_FP32, experts * (I / 128) * (H / 128))) return false;
        } else {
            if (!check("gmm1Scale", s1, ZBAL_DATA_TYPE_FP16, ZBAL_DATA_TYPE_FP16, experts * (H / 128) * N1)) return false;
            if (!check("gmm2Scale", s2, ZBAL_DATA_TYPE_FP16, ZBAL_DATA_TYPE_FP16, experts * (I / 128) * H)) return false;
            *wscale2Dt = ZBAL_DATA_TYPE_FP16;
        }
        return true;
    }

    int32_t FusedDeepMoe(const zbal_tensor_info_t *x, const zbal_tensor_info_t *expertIds,
                         const zbal_tensor_info_t *gmm1Weight, const zbal_tensor_info_t *gmm1Scale,
                         const zbal_tensor_info_t *gmm2Weight, const zbal_tensor_info_t *gmm2Scale,
                         const zbal_tensor_info_t *expertScales, const zbal_tensor_info_t *expertSmoothScales,
                         const zbal_tensor_info_t *shareGmm1Weight, const zbal_tensor_info_t *shareGmm1Scale,
                         const zbal_tensor_info_t *shareGmm2Weight, const zbal_tensor_info_t *shareGmm2Scale,
                         const zbal_tensor_info_t *shareSmoothScales, const zbal_tensor_info_t *xActiveMask,
                         const zbal_tensor_info_t *output, const zbal_tensor_info_t *shareOutput,
                         const zbal_tensor_info_t *expertTokenNums, const zbal_tensor_info_t *workspace,
                         int64_t moeExpertNum, int64_t quantMode, int64_t, int64_t gmm1HLen, int64_t shareGmm1HLen,
                         bool isTensorList, aclrtStream stream, int64_t) override
    {
        const char *op = "FusedDeepMoe";
        if (!SingleRank(op)) return Z_INVALID_PARAM;
        ZBAL_VALIDATE_RETURN(quantMode >= 0 && quantMode <= 3, op << " failed as quantMode " << quantMode << " is invalid",
                             Z_INVALID_PARAM);
        const int mode = quantMode <= 1 ? 1 : (int)quantMode; /* 0 and 1 both mean W8A8, as in the reference kernel */
        int64_t T = 0, H = 0;
        if (!TokensShape(op, x, &T, &H)) return Z_INVALID_PARAM;
        ZBAL_VALIDATE_RETURN(expertIds->dim == 2 && expertIds->shape[0] == T, op << " failed as expertIds must be [tokens, topk]",
                             Z_INVALID_PARAM);
        const int64_t K = expertIds->shape[1], E = moeExpertNum, N1 = gmm1HLen, I = N1 / 2;
        const bool shared = shareGmm1Weight != nullptr && shareGmm1Weight->data != nullptr;
        const int64_t SN1 = shared ? shareGmm1HLen : 0, SI = SN1 / 2;
        ZBAL_VALIDATE_RETURN(K <= 32, op << " failed as topk " << K << " exceeds 32", Z_INVALID_PARAM);
        ZBAL_VALIDATE_RETURN(E <= 1024, op << " failed as moeExpertNum exceeds 1024", Z_INVALID_PARAM);
        ZBAL_VALIDATE_RETURN(H % 256 == 0, op << " failed as hidden " << H << " must be a multiple of 256", Z_INVALID_PARAM);
        if (T > 0) { /* an empty batch has empty per-token tensors (null data): only expertTokenNums is written */
            ZB_CHECK(op, "x", x, ZBAL_DATA_TYPE_BFP16, ZBAL_DATA_TYPE_FP16, T * H);
            ZB_CHECK(op, "output", output, x->dataType, x->dataType, T * H);
            ZB_CHECK(op, "expertIds", expertIds, ZBAL_DATA_TYPE_INT32, ZBAL_DATA_TYPE_INT32, T * K);
            ZB_CHECK(op, "expertScales", expertScales, ZBAL_DATA_TYPE_FP32, ZBAL_DATA_TYPE_FP32, T * K);
        } else {
            ZBAL_VALIDATE_RETURN(x->dataType == ZBAL_DATA_TYPE_BFP16 || x->dataType == ZBAL_DATA_TYPE_FP16,
                                 op << " failed as x has type " << DtName(x->dataType), Z_INVALID_PARAM);
        }
        ZB_CHECK(op, "expertTokenNums", expertTokenNums, ZBAL_DATA_TYPE_INT64, ZBAL_DATA_TYPE_INT64, E);
        int wscale2Dt = ZBAL_DATA_TYPE_FP32, shareWscale2Dt = ZBAL_DATA_TYPE_FP32;
        if (!CheckFfnWeights(op, "expert", mode, E, H, N1, gmm1Weight, gmm1Scale, gmm2Weight, gmm2Scale, &wscale2Dt))
            return Z_INVALID_PARAM;
        const float *smooth = nullptr, *shareSmooth = nullptr;
        if (expertSmoothScales && expertSmoothScales->data) {
            ZBAL_VALIDATE_RETURN(mode != 2, op << " failed as smooth scales do not apply to the fp8 mode", Z_INVALID_PARAM);
            ZB_CHECK(op, "expertSmoothScales", expertSmoothScales, ZBAL_DATA_TYPE_FP32, ZBAL_DATA_TYPE_FP32, E * H);
            smooth = (const float *)expertSmoothScales->data;
        }
        if (shared) {
            if (!CheckFfnWeights(op, "shared", mode, 1, H, SN1, shareGmm1Weight, shareGmm1Scale, shareGmm2Weight,
                                 shareGmm2Scale, &shareWscale2Dt))
                return Z_INVALID_PARAM;
            if (T > 0) ZB_CHECK(op, "shareOutput", shareOutput, x->dataType, x->dataType, T * H);
            if (shareSmoothScales && shareSmoothScales->data) {
                ZBAL_VALIDATE_RETURN(mode != 2, op << " failed as smooth scales do not apply to the fp8 mode", Z_INVALID_PARAM);
                ZB_CHECK(op, "shareSmoothScales", shareSmoothScales, ZBAL_DATA_TYPE_FP32, ZBAL_DATA_TYPE_FP32, H);
                shareSmooth = (const float *)shareSmoothScales->data;
            }
        }
        const uint8_t *activeMask = nullptr;
        if (xActiveMask && xActiveMask->data) { /* one bool per token; the first sum(mask) tokens are routed */
            if (T > 0) ZB_CHECK(op, "xActiveMask", xActiveMask, ZBAL_DATA_TYPE_UINT8, ZBAL_DATA_TYPE_INT8, T);
            activeMask = (const uint8_t *)xActiveMask->data;
        }
        FusedWorkspace ws;
        ZBAL_VALIDATE_RETURN(PlanFusedWorkspace(T, H, K, E, N1, SN1, quantMode, &ws), op << " failed as the shapes are invalid",
                             Z_INVALID_PARAM);
        ZBAL_VALIDATE_RETURN(workspace->data != nullptr && (reinterpret_cast<uintptr_t>(workspace->data) & 255u) == 0,
                             op << " failed as the workspace is null or not 256-byte aligned", Z_INVALID_PARAM);
        const uint64_t wsBytes = (uint64_t)Numel(workspace) * ElemSize(workspace->dataType);
        if (wsBytes < ws.total) { /* the reference reports this case with a raw -1, host launcher :224-232 */
            ZBAL_LOG_AND_SET_LAST_ERROR(op << " failed as the workspace holds " << wsBytes << " bytes, needs " << ws.total);
            return Z_ERROR;
        }
        uint8_t *base = (uint8_t *)workspace->data;
        const int64_t rows = T * K;
        void *q1 = base + ws.q1;
        float *xs = (float *)(base + ws.xs);
        int32_t *expandIdx = (int32_t *)(base + ws.expand_idx);
        int32_t *rowOff = (int32_t *)(base + ws.row_off);
        int32_t *layoutScratch = (int32_t *)(base + ws.layout_scratch);   /* per-block histograms of the large-batch layout */
        void *q2 = base + ws.q2;
        float *scale2 = (float *)(base + ws.scale2);
        float *sgl = mode == 2 ? nullptr : (float *)(base + ws.sgl);
        void *y = base + ws.y;
        const int qmode = mode == 2 ? 2 : 1;
        /* tensor lists: the four routed-expert descriptors point at device tables of one address per expert */
        const int32_t gemmMode = mode | (isTensorList ? ZBALHIP_WEIGHTS_AS_LISTS : 0);
        /* int modes: the permute launch clears the row maxima the first GEMM accumulates into (no fill launch) */
        const int32_t clearedFlag = sgl ? ZBALHIP_ROWMAX_CLEARED : 0;
        if (T == 0) { /* nothing routed: counts are zero */
            return Launched(op, zbalhip_fused_permute_quant(x->data, x->dataType, (const int32_t *)expertIds->data, smooth,
                                                            nullptr, 0, H, K, E, qmode, q1, xs, expandIdx,
                                                            (int64_t *)expertTokenNums->data, rowOff, nullptr, 0, nullptr, 0,
                                                            stream));
        }
        int32_t rc = 0;
        if (shared) {
            /*
             * The shared expert is the same pipeline with one expert that every token picks once: the rows stay in
             * token order, so the second GEMM writes shareOutput directly. It runs first and borrows the routed
             * pass's workspace regions (sized for the larger of the two); its all-zero expert ids and its one count
             * sit at the start of the y region, which nothing else uses until the routed second GEMM.
             */
            int32_t *zeroIds = (int32_t *)y;
            int64_t *shareCount = (int64_t *)((uint8_t *)y + Align256((uint64_t)T * 4));
            rc = zbalhip_fill_i32(zeroIds, T, 0, stream);
            if (rc != 0) return Launched(op, rc);
            /* with x_active_mask the shared expert, too, sees only the first sum(mask) tokens (TokenActiveMaskCal) */
            rc = zbalhip_fused_permute_quant(x->data, x->dataType, zeroIds, shareSmooth, activeMask, T, H, 1, 1, qmode, q1, xs, expandIdx,
                                             shareCount, rowOff, sgl ? (uint32_t *)(sgl + T * SI) : nullptr, sgl ? T : 0,
                                             layoutScratch, ZBALHIP_LAYOUT_MAX_BLOCKS, stream);
            if (rc != 0) return Launched(op, rc);
            rc = zbalhip_gmm1_swiglu_quant(q1, xs, shareGmm1Weight->data, shareGmm1Scale->data, rowOff, 1, T, H, SN1,
                                           mode | clearedFlag, q2, scale2, sgl, stream);
            if (rc != 0) return Launched(op, rc);
            rc = zbalhip_gmm2_dequant(q2, scale2, shareGmm2Weight->data, shareGmm2Scale->data, shareWscale2Dt, rowOff, 1, T,
                                      SI, H, mode, x->dataType, shareOutput->data, stream);
            if (rc != 0) return Launched(op, rc);
        }
        rc = zbalhip_fused_permute_quant(x->data, x->dataType, (const int32_t *)expertIds->data, smooth, activeMask, T, H, K, E,
                                         qmode, q1, xs, expandIdx, (int64_t *)expertTokenNums->data, rowOff,
                                         sgl ? (uint32_t *)(sgl + rows * I) : nullptr, sgl ? rows : 0, layoutScratch,
                                         ZBALHIP_LAYOUT_MAX_BLOCKS, stream);
        if (rc != 0) return Launched(op, rc);
        rc = zbalhip_gmm1_swiglu_quant(q1, xs, gmm1Weight->data, gmm1Scale->data, rowOff, E, rows, H, N1,
                                       gemmMode | clearedFlag, q2, scale2, sgl, stream);
        if (rc != 0) return Launched(op, rc);
        rc = zbalhip_gmm2_dequant(q2, scale2, gmm2Weight->data, gmm2Scale->data, wscale2Dt, rowOff, E, rows, I, H, gemmMode,
                                  x->dataType, y, stream);
        if (rc != 0) return Launched(op, rc);
        const void *ySrc[1] = {y};
        return Launched(op, zbalhip_combine(ySrc, 1, 0, rows, x->dataType, rowOff, 0, (const float *)expertScales->data,
                                            (const int32_t *)expertIds->data, expandIdx, T, H, K, E, output->data,
                                            stream));
    }

    int32_t TopkRoute(const zbal_tensor_info_t *logits, int64_t topkNum, const zbal_tensor_info_t *topkIndex,
                      const zbal_tensor_info_t *topkWeight, aclrtStream stream, int64_t) override
    {
        const char *op = "TopkRoute";
        ZBAL_VALIDATE_RETURN(logits->dim == 2, op << " failed as logits must be [tokens, experts]", Z_INVALID_PARAM);
        const int64_t T = logits->shape[0], E = logits->shape[1];
        ZBAL_VALIDATE_RETURN(E > 0 && E <= 1024 && topkNum <= 32 && topkNum <= E,
                             op << " failed as experts " << E << " / topk " << topkNum << " are out of range", Z_INVALID_PARAM);
        if (T == 0) return Z_OK;
        ZB_CHECK(op, "logits", logits, ZBAL_DATA_TYPE_FP32, ZBAL_DATA_TYPE_FP32, T * E);
        /* int64 is what the layout operator takes, int32 what the dispatch and fused operators take */
        ZB_CHECK(op, "topkIndex", topkIndex, ZBAL_DATA_TYPE_INT64, ZBAL_DATA_TYPE_INT32, T * topkNum);
        ZB_CHECK(op, "topkWeight", topkWeight, ZBAL_DATA_TYPE_FP32, ZBAL_DATA_TYPE_FP32, T * topkNum);
        return Launched(op, zbalhip_topk_route((const float *)logits->data, T, E, topkNum, topkIndex->data,
                                               topkIndex->dataType == ZBAL_DATA_TYPE_INT64, (float *)topkWeight->data,
                                               stream));
    }

    int32_t WeightPrepack(const zbal_tensor_info_t *src, const zbal_tensor_info_t *dst, aclrtStream stream, int64_t) override
    {
        const char *op = "WeightPrepack";
        ZBAL_VALIDATE_RETURN(src->dim == 3, op << " failed as src must be [experts, K, N]", Z_INVALID_PARAM);
        const int64_t E = src->shape[0], K = src->shape[1], N = src->shape[2];
        const bool int4 = dst->dataType == ZBAL_DATA_TYPE_INT4X2;
        ZBAL_VALIDATE_RETURN(ElemSize(src->dataType) == 1, op << " failed as src must hold one byte per element", Z_INVALID_PARAM);
        ZBAL_VALIDATE_RETURN(!int4 || src->dataType == ZBAL_DATA_TYPE_INT8, op << " failed as int4 packing needs an int8 source",
                             Z_INVALID_PARAM);
        ZBAL_VALIDATE_RETURN(src->data && dst->data && src->data != dst->data, op << " failed as src/dst are null or alias",
                             Z_INVALID_PARAM);
        ZBAL_VALIDATE_RETURN(Numel(dst) * (int4 ? 2 : 1) >= E * K * N, op << " failed as dst is too small", Z_INVALID_PARAM);
        return Launched(op, zbalhip_weight_prepack(src->data, E, K, N, int4 ? 1 : 0, dst->data, stream));
    }
};

} // namespace

CommunicatorPtr MakeGpuCommunicator(const GroupInfo &info) { return std::make_shared<GpuCommunicator>(info); }


bool PlanFusedWorkspace(int64_t tokens, int64_t hidden, int64_t topk, int64_t experts, int64_t n1, int64_t shareN1,
                        int64_t quantMode, FusedWorkspace *ws)
{
    if (tokens < 0 || hidden <= 0 || topk <= 0 || experts <= 0 || n1 <= 0 || shareN1 < 0 || quantMode < 0 || quantMode > 3)
        return false;
    if (hidden % 128 != 0 || n1 % 256 != 0 || shareN1 % 256 != 0) return false;
    const uint64_t rows = (uint64_t)(tokens * topk > 0 ? tokens * topk : 1);
    const uint64_t T = (uint64_t)(tokens > 0 ? tokens : 1);
    const uint64_t H = hidden, I = n1 / 2, SI = shareN1 / 2, E = experts;
    const bool fp8 = quantMode == 2;
    /* the shared expert's pass (T rows, width SI) reuses the regions of the routed pass (rows rows, width I) */
    auto both = [&](uint64_t routed, uint64_t shared) { return SI > 0 && shared > routed ? shared : routed; };
    uint64_t off = 0;
    auto take = [&](uint64_t bytes) { uint64_t o = off; off = Align256(off + bytes); return o; };
    ws->q1 = take(rows * H);
    ws->xs = take(rows * (fp8 ? H / 128 : 1) * 4);
    ws->expand_idx = take(rows * 4);
    ws->counts = take(E * 8);
    ws->row_off = take((E + 1) * 4);
    ws->layout_scratch = take((uint64_t)ZBALHIP_LAYOUT_MAX_BLOCKS * E * 4);
    ws->q2 = take(both(rows * I, T * SI));
    ws->scale2 = take(both(rows * (fp8 ? (I + 127) / 128 : 1), T * (fp8 ? (SI + 127) / 128 : 1)) * 4);
    ws->sgl = fp8 ? off : take(both(rows * (I + 1), T * (SI + 1)) * 4);
    ws->y = take(both(rows * H * 2, Align256(T * 4) + 256));
    ws->total = off;
    return true;
}

} // namespace zbal
