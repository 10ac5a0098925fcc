/*
 * The per-group record the reference's kernel launchers take
 * (app/zbal/src/csrc/operators/zbal_comm_host_device_struct.h:133-151): plain
 * data, 2160 bytes, copied to the device by the reference and read on the host
 * by the launchers in zbal_amd_operators.h. Field order, types and offsets are
 * the reference's, so a CommGroupInfo filled in by its communicator layer can
 * be handed over as it is.
 *
 * What the launchers here read: groupSize, myGroupRank, peerGroupRank2WorldRank
 * and localDeviceMemSize (a tensor of group rank r lies
 * (world(r) - world(me)) * localDeviceMemSize bytes from this rank's copy: the
 * reference's symmetric address space, aicore/common/zbal_kernel_base.h:35-42;
 * on one GPU the "ranks" are slices of one allocation at that stride),
 * waitSymbol (bumped by the two reductions, as the reference does,
 * zbal_kernel_allreduce.cpp:436) and groupIndex.
 */
#ifndef ZBAL_COMM_GROUP_INFO_H_
#define ZBAL_COMM_GROUP_INFO_H_

#include <stddef.h>
#include <stdint.h>

#define ZBAL_MAX_RANKS 1024

struct CommGroupInfo {
    uint16_t groupSize;                                /* ranks in the group */
    uint16_t myGroupRank;                              /* this rank's id in the group */
    uintptr_t myMetaGva;                               /* not used by this build */
    uintptr_t myParamDataGva;                          /* not used by this build */
    uintptr_t myAddressExchangeGva;                    /* not used by this build */
    uint64_t sizeForCommGroupInfo;
    uint64_t sizeForParam;
    uint64_t sizeForExchangeAddress;
    uint64_t fftsConfig;
    uint16_t peerGroupRank2WorldRank[ZBAL_MAX_RANKS];  /* group rank -> world rank */
    uint64_t localDeviceMemSize;                       /* bytes between the windows of consecutive world ranks */
    uint64_t waitSymbol;                               /* launch counter of the cross-rank operators */
    uintptr_t hostMemoryForProfiling;
    uintptr_t devMemoryForProfiling;
    uint64_t tracePointPerCore;
    uint16_t groupIndex;
    uint32_t dataOpType;
};

#ifdef __cplusplus
static_assert(sizeof(CommGroupInfo) == 2160, "CommGroupInfo must keep the reference's size");
static_assert(offsetof(CommGroupInfo, peerGroupRank2WorldRank) == 64, "CommGroupInfo layout");
static_assert(offsetof(CommGroupInfo, localDeviceMemSize) == 2112, "CommGroupInfo layout");
static_assert(offsetof(CommGroupInfo, groupIndex) == 2152 && offsetof(CommGroupInfo, dataOpType) == 2156, "CommGroupInfo layout");
#endif

#endif /* ZBAL_COMM_GROUP_INFO_H_ */
