/*
 * Communicator registry and the do-nothing backend.
 *
 * Lifecycle rules follow the reference (operators/zbal_communicator.cpp):
 * names are unique (:191-194); the world group is created first and only
 * once (:226-252); it is destroyed last (:262-268, Z_COMM_DESTROY_GLOBAL_LAST);
 * destroying an unknown handle is not an error (:281-285). Handles are the
 * object addresses, but every use looks the address up first, so a stale or
 * foreign pointer yields an error code instead of a wild dereference.
 */
#include <unordered_map>

#include "zbal_host.h"

namespace zbal {

namespace {

std::mutex gMutex;
CommunicatorPtr gWorld;
std::unordered_map<uintptr_t, CommunicatorPtr> gByHandle; /* non-world groups */
std::unordered_map<std::string, CommunicatorPtr> gByName; /* all groups */
uint32_t gNextIndex = 0;

/*
 * Backend for host-only tests: every operator validates nothing further and
 * reports success, like the reference's CommunicatorDummy.
 */
class DummyCommunicator final : public Communicator {
public:
    using Communicator::Communicator;
    int32_t AllReduce(const void *, void *, void *, size_t, zbal_datatype_t, zbal_reduce_op_t, aclrtStream) override { return Z_OK; }
    int32_t ReduceScatter(const void *, void *, size_t, zbal_datatype_t, zbal_reduce_op_t, aclrtStream) override { return Z_OK; }
    int32_t DispatchNormalLayout(const zbal_tensor_info_t *, int64_t, int64_t, int64_t, const zbal_tensor_info_t *,
                                 const zbal_tensor_info_t *, const zbal_tensor_info_t *, const zbal_tensor_info_t *,
                                 aclrtStream, int64_t) override { return Z_OK; }
    int32_t DispatchNormalNotify(const zbal_tensor_info_t *, int64_t, int64_t, const zbal_tensor_info_t *,
                                 const zbal_tensor_info_t *, const zbal_tensor_info_t *, const zbal_tensor_info_t *,
                                 const zbal_tensor_info_t *, aclrtStream, int64_t) override { return Z_OK; }
    int32_t DispatchNormal(const zbal_tensor_info_t *, const zbal_tensor_info_t *, const zbal_tensor_info_t *,
                           const zbal_tensor_info_t *, const zbal_tensor_info_t *, int64_t, zbal_quant_mode_t,
                           const zbal_tensor_info_t *, const zbal_tensor_info_t *, aclrtStream, int64_t) override { return Z_OK; }
    int32_t CombineNormal(const zbal_tensor_info_t *, const zbal_tensor_info_t *, const zbal_tensor_info_t *,
                          const zbal_tensor_info_t *, const zbal_tensor_info_t *, const zbal_tensor_info_t *, uint16_t,
                          const zbal_tensor_info_t *, aclrtStream, int64_t) override { return Z_OK; }
    int32_t DispatchLowLatency(const zbal_tensor_info_t *, const zbal_tensor_info_t *, int64_t, int64_t, int64_t, int64_t,
                               int64_t, int64_t, int64_t, const zbal_tensor_info_t *, const zbal_tensor_info_t *,
                               const zbal_tensor_info_t *, const zbal_tensor_info_t *, const zbal_tensor_info_t *,
                               const zbal_tensor_info_t *, const zbal_tensor_info_t *, aclrtStream, int64_t) override { return Z_OK; }
    int32_t CombineLowLatency(const zbal_tensor_info_t *, const zbal_tensor_info_t *, const zbal_tensor_info_t *,
                              const zbal_tensor_info_t *, const zbal_tensor_info_t *, const zbal_tensor_info_t *, int64_t,
                              aclrtStream, int64_t) override { return Z_OK; }
    int32_t FusedDeepMoe(const zbal_tensor_info_t *, const zbal_tensor_info_t *, const zbal_tensor_info_t *,
                         const zbal_tensor_info_t *, const zbal_tensor_info_t *, const zbal_tensor_info_t *,
                         const zbal_tensor_info_t *, const zbal_tensor_info_t *, const zbal_tensor_info_t *,
                         const zbal_tensor_info_t *, const zbal_tensor_info_t *, const zbal_tensor_info_t *,
                         const zbal_tensor_info_t *, const zbal_tensor_info_t *, const zbal_tensor_info_t *,
                         const zbal_tensor_info_t *, const zbal_tensor_info_t *, const zbal_tensor_info_t *, int64_t,
                         int64_t, int64_t, int64_t, int64_t, bool, aclrtStream, int64_t) override { return Z_OK; }
    int32_t TopkRoute(const zbal_tensor_info_t *, int64_t, const zbal_tensor_info_t *, const zbal_tensor_info_t *,
                      aclrtStream, int64_t) override { return Z_OK; }
    int32_t WeightPrepack(const zbal_tensor_info_t *, const zbal_tensor_info_t *, aclrtStream, int64_t) override { return Z_OK; }
};

} // namespace

CommunicatorPtr MakeDummyCommunicator(const GroupInfo &info) { return std::make_shared<DummyCommunicator>(info); }

namespace registry {

int32_t Create(const zbal_comm_options_t &options, zbal_comm_t *out)
{
    std::lock_guard<std::mutex> guard(gMutex);
    const std::string name(options.name);
    if (gByName.count(name)) {
        ZBAL_LOG_AND_SET_LAST_ERROR("Create communicator failed as there is already one named " << name);
        return Z_CREATE_COMM_FAILED;
    }
    ZBAL_VALIDATE_RETURN(options.groupSize > 0, "Create communicator failed as groupSize is 0", Z_INVALID_PARAM);
    ZBAL_VALIDATE_RETURN(options.groupRankId < options.groupSize,
                         "Create communicator failed as groupRankId " << options.groupRankId
                                                                      << " is not below groupSize " << options.groupSize,
                         Z_INVALID_PARAM);
    const bool world = options.isWorldGroup == 1;
    if (world && gWorld) {
        ZBAL_LOG_AND_SET_LAST_ERROR("Create communicator failed as world group already created");
        return Z_CREATE_COMM_FAILED;
    }
    if (!world && !gWorld) {
        ZBAL_LOG_AND_SET_LAST_ERROR("Create communicator failed as world group not created");
        return Z_CREATE_COMM_FAILED;
    }
    GroupInfo info;
    info.name = name;
    info.groupSize = options.groupSize;
    info.myGroupRank = options.groupRankId;
    info.isWorldGroup = world;
    info.groupIndex = gNextIndex++;
    info.backend = options.backendType;
    info.peers.resize(options.groupSize);

    CommunicatorPtr comm;
    switch (options.backendType) {
        case ZBAL_AMD_GPU: comm = MakeGpuCommunicator(info); break;
        case ZBAL_BACK_BUTT: comm = MakeDummyCommunicator(info); break;
        default:
            ZBAL_LOG_AND_SET_LAST_ERROR("Created communicator failed as backendType is invalid");
            return Z_CREATE_COMM_FAILED;
    }
    if (!comm) {
        ZBAL_LOG_AND_SET_LAST_ERROR("Create communicator failed, probably out of memory");
        return Z_CREATE_COMM_FAILED;
    }
    if (world) gWorld = comm;
    else gByHandle.emplace(reinterpret_cast<uintptr_t>(comm.get()), comm);
    gByName.emplace(name, comm);
    *out = comm.get();
    ZBAL_LOG(LOG_DEBUG, "Created communicator " << name << ", world: " << world << ", size " << info.groupSize);
    return Z_OK;
}

int32_t Destroy(zbal_comm_t comm)
{
    std::lock_guard<std::mutex> guard(gMutex);
    if (gWorld && comm == gWorld.get()) {
        if (!gByHandle.empty()) {
            ZBAL_LOG_AND_SET_LAST_ERROR("Destroy other non world communicator firstly, then destroy the world one");
            return Z_COMM_DESTROY_GLOBAL_LAST;
        }
        gByName.erase(gWorld->Info().name);
        gWorld.reset();
        return Z_OK;
    }
    auto it = gByHandle.find(reinterpret_cast<uintptr_t>(comm));
    if (it == gByHandle.end()) {
        ZBAL_LOG(LOG_INFO, "Destroy communicator find communicator not existed");
        return Z_OK;
    }
    gByName.erase(it->second->Info().name);
    gByHandle.erase(it);
    return Z_OK;
}

void DestroyAll()
{
    std::lock_guard<std::mutex> guard(gMutex);
    gByHandle.clear();
    gByName.clear();
    gWorld.reset();
}

zbal_comm_t Global()
{
    std::lock_guard<std::mutex> guard(gMutex);
    return gWorld ? gWorld.get() : nullptr;
}

zbal_comm_t ByName(const std::string &name)
{
    std::lock_guard<std::mutex> guard(gMutex);
    auto it = gByName.find(name);
    return it == gByName.end() ? nullptr : it->second.get();
}

CommunicatorPtr Find(zbal_comm_t comm)
{
    std::lock_guard<std::mutex> guard(gMutex);
    if (gWorld && comm == gWorld.get()) return gWorld;
    auto it = gByHandle.find(reinterpret_cast<uintptr_t>(comm));
    return it == gByHandle.end() ? nullptr : it->second;
}

uint32_t Count()
{
    std::lock_guard<std::mutex> guard(gMutex);
    return (uint32_t)gByName.size();
}

void DumpAllTraces()
{
    std::vector<CommunicatorPtr> all;
    {
        std::lock_guard<std::mutex> guard(gMutex);
        for (auto &kv : gByName) all.push_back(kv.second);
    }
    for (auto &c : all) c->DumpProfilingTrace();
}

} // namespace registry
} // namespace zbal
