/*
 * Public types of the zbal operator API, MI355X build.
 *
 * Binary contract: every enum value, field order and struct size below equals
 * the reference's app/zbal/src/include/zbal_def.h (file:line cited per item),
 * so a client compiled against either header links against this library.
 * Additions made by this build are marked "extension" and use values the
 * reference leaves free.
 */
#ifndef ZBAL_DEF_H_
#define ZBAL_DEF_H_

#include <stddef.h>
#include <stdint.h>
#include <stdio.h>

#ifdef __cplusplus
extern "C" {
#endif

/* reference zbal_def.h:23-25 */
#define ZBAL_COMM_NAME_MAX  128
#define ZBAL_MAX_IPPORT_LEN 64
#define ZBAL_MAX_TENSOR_DIM 12

/* Opaque communicator handle (reference zbal_def.h:27). */
typedef void *zbal_comm_t;

/*
 * The stream argument keeps the reference's type name (zbal_def.h:29) so that
 * signatures stay identical; on this build the pointer carries a hipStream_t
 * unchanged (NULL = the HIP null stream).
 */
typedef void *aclrtStream;

/* Element types, reference zbal_def.h:31-46 (values 0..11 identical). */
typedef enum {
    ZBAL_DATA_TYPE_INT8 = 0,
    ZBAL_DATA_TYPE_INT16 = 1,
    ZBAL_DATA_TYPE_INT32 = 2,
    ZBAL_DATA_TYPE_INT64 = 3,
    ZBAL_DATA_TYPE_UINT64 = 4,
    ZBAL_DATA_TYPE_FP64 = 5,
    ZBAL_DATA_TYPE_FP16 = 6,
    ZBAL_DATA_TYPE_FP32 = 7,
    ZBAL_DATA_TYPE_BFP16 = 8,
    ZBAL_DATA_TYPE_UINT8 = 9,
    ZBAL_DATA_TYPE_UINT16 = 10,
    ZBAL_DATA_TYPE_UINT32 = 11,
    ZBAL_DATA_TYPE_FP8_E4M3 = 12, /* extension: OCP e4m3fn, 1 byte              */
    ZBAL_DATA_TYPE_INT4X2 = 13,   /* extension: two signed 4-bit values per byte */

    ZBAL_DATA_TYPE_BUTT
} zbal_datatype_t;

/* Reduction operators, reference zbal_def.h:48-55. */
typedef enum {
    ZBAL_REDUCE_PROD = 0,
    ZBAL_REDUCE_SUM = 1,
    ZBAL_REDUCE_MAX = 2,
    ZBAL_REDUCE_MIN = 3,

    ZBAL_REDUCE_BUTT
} zbal_reduce_op_t;

/*
 * Backends, reference zbal_def.h:57-61. Value 0 is the production device
 * backend (the HIP backend here); ZBAL_BACK_BUTT selects the do-nothing
 * backend used by host-only tests, as in the reference
 * (zbal_communicator.cpp:202-217).
 */
typedef enum {
    ZBAL_ASCEND_NPU = 0,
    ZBAL_AMD_GPU = 0, /* extension: alias, same backend slot */

    ZBAL_BACK_BUTT
} zbal_backend_t;

/* reference zbal_def.h:63-67 */
typedef enum {
    BOOT_BY_MEMFABRIC = 0,

    BOOT_BY_BUTT
} zbal_bootstrap_type_t;

/* reference zbal_def.h:75-87 */
typedef struct {
    uint32_t flags;
    zbal_bootstrap_type_t btType;
    char ipPort[ZBAL_MAX_IPPORT_LEN];
    uint16_t worldSize;
    uint16_t rankId;
    uint16_t deviceId;
    uint16_t startConfigServer;
    uint64_t deviceMemorySize;
    uint32_t dataOperationType;
    uint16_t commMetaSpaceSize;
    uint16_t commGroupCap;
} zbal_bootstrap_options_t;

/* reference zbal_def.h:89-98 */
typedef struct {
    void *deviceGva;
    uint64_t createdDeviceMemorySpaceSize;
    uint64_t allocatedDeviceMemorySize;
    void *myDeviceGva;
    void *myCommMetaDeviceGva;
    uint64_t metaSizeOfDevice;
    void *mySMAGva;
    uint64_t smaSizeOfDevice;
} zbal_bootstrap_output_t;

/* reference zbal_def.h:106-114 */
typedef struct {
    char *name;
    zbal_backend_t backendType;
    uint32_t flags;
    uint16_t isWorldGroup;
    uint16_t groupSize;
    uint16_t groupRankId;
    uint16_t symmetricMetaGva;
} zbal_comm_options_t;

/* reference zbal_def.h:116-136 */
typedef struct {
    char name[ZBAL_COMM_NAME_MAX];
    zbal_backend_t backendType;
    uint32_t flags;
    uint16_t isWorldGroup;
    uint16_t groupSize;
    uint16_t groupRankId;
    uint16_t symmetricMetaGva;
    void *myGVA;
    void *myMetaGVA;
    void *myMetaGVAForOpParam;
    void *myMetaGVAForOpExchange;
    void *hostMemoryForProfiling;
    void *devMemoryForProfiling;
    uint64_t sizeOfMetaArea;
    uint64_t sizeOfMetaForOpParam;
    uint64_t sizeOfMetaForAddressExchange;
    uint64_t tracePointPerCore;
    uint64_t localDeviceMemSize;
    uint32_t groupIndex;
} zbal_comm_property_t;

/*
 * Tensor descriptor, reference zbal_def.h:141-147. Tensors are dense
 * row-major (there is no stride field). The struct occupies 72 bytes with
 * the usual x86-64 / gcc layout: data 0, dataType 8, dim 12, shape 16,
 * reserved 64.
 *
 * extension: for the weight operands of zbal_fused_deep_moe, reserved[0]
 * carries the storage format (ZBAL_WEIGHT_FORMAT_*). Every other operand
 * must leave it 0.
 */
typedef struct {
    void *data;
    zbal_datatype_t dataType;
    uint16_t dim;
    uint32_t shape[ZBAL_MAX_TENSOR_DIM];
    uint16_t reserved[1];
} zbal_tensor_info_t;

/*
 * Weight storage formats (extension). The reference's fused kernel takes its
 * weights in a hardware-private fractal layout made by a format-cast step
 * (test_fused_deep_moe.py:66-69); the equivalent step here is
 * zbal_moe_weight_prepack(), which turns the logical [E, K, N] row-major
 * tensor into ZBAL_WEIGHT_FORMAT_PREPACKED, the order in which the grouped
 * GEMM streams it (same number of bytes; K and N multiples of 128):
 *   one byte per element: [E][N/128][K/128] blocks of 16 KiB; a block holds
 *     128 channels x 128 K-bytes, block row r at +128*r, and within a row
 *     the 16-byte chunk c of its K-bytes at slot c ^ (r & 7) ^ ((r >> 3) & 1);
 *     block row r holds the block's channel
 *     (r & ~31) | ((r & 15) >> 2) << 3 | ((r >> 4) & 1) << 2 | (r & 3);
 *   INT4X2: the same block and row order with 8 KiB blocks (128 channels x
 *     128 k, two values per byte); block row r at +64*r, and within a row the
 *     16-byte chunk c (k in [32c, 32c+32)) at slot c ^ ((r >> 2) & 3); in a
 *     chunk, byte b of dword j holds k[8j+b] in the low and k[8j+4+b] in the
 *     high nibble.
 */
#define ZBAL_WEIGHT_FORMAT_ND      0 /* logical [E, K, N], N contiguous */
#define ZBAL_WEIGHT_FORMAT_PREPACKED 1 /* made by zbal_moe_weight_prepack */

/*
 * Activation quantisation modes, reference zbal_def.h:149-155 (0 and 1
 * identical). Mode 2 and 3 are extensions of the same operator API.
 */
typedef enum {
    NO_QUANT = 0,
    QUANT_BF16_2_INT8 = 1,          /* per-token symmetric int8, one fp32 scale per row      */
    QUANT_BF16_2_FP8E4M3_B128 = 2,  /* extension: e4m3, one fp32 scale per 1x128 block       */
    QUANT_W4A8_G128 = 3,            /* extension (fused op only): int8 rows x int4 g128 weights */

    QUANT_BUTT
} zbal_quant_mode_t;

#ifdef __cplusplus
}
#endif

#endif /* ZBAL_DEF_H_ */
