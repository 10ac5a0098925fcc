/*
 * Weight pre-pack: the logical [E, K, N] byte matrix (N contiguous) is put
 * into the order in which the grouped GEMM streams it. A one-time step per
 * weight tensor.
 *
 * 8-bit weights: [E][N/128][K/128] blocks of 16 KiB. A block holds 128
 * channels x 128 K-bytes exactly as the GEMM wants them in LDS: block row r
 * at +128*r, and within it the 16-byte chunk c of the K-bytes in slot
 * c ^ f(r), f(r) = (r & 7) ^ ((r >> 3) & 1). A workgroup's weight stream is
 * then two runs of consecutive addresses, and each LDS-DMA instruction copies
 * 1 KiB of consecutive bytes.
 *
 * Block row r holds channel zb_block_row_channel(r) of the block, a
 * permutation within each group of 32 rows: rows 16t .. 16t+15 are one MFMA
 * operand of the GEMM, whose output leaves a lane with rows 4q .. 4q+3 of it
 * (q = lane / 16). With channels 8q .. 8q+3 in those rows of the even
 * operand t and channels 8q+4 .. 8q+7 in those of the odd operand t+1, the
 * lane ends up with 8 consecutive channels and stores them with one
 * instruction.
 *
 * int4 weights: the same block order with 8 KiB blocks, two values per
 * byte (details at the kernel).
 */
#include "zbal_device.h"
#include "zbal_hip_kernels.h"

namespace {

__global__ void __launch_bounds__(256)
tile_swizzle_bytes_kernel(const uint8_t *__restrict__ src, int64_t K, int64_t N, uint8_t *__restrict__ dst)
{
    __shared__ uint8_t tile[128][128 + 16];          /* [k][n] */
    const int64_t e = blockIdx.z;
    const int64_t k0 = (int64_t)blockIdx.y * 128, n0 = (int64_t)blockIdx.x * 128;
    const uint8_t *s = src + e * K * N;
    for (int i = threadIdx.x; i < 128 * 8; i += blockDim.x) {
        const int kk = i >> 3, c = i & 7;
        *reinterpret_cast<u32x4 *>(&tile[kk][c * 16]) = *reinterpret_cast<const u32x4 *>(s + (k0 + kk) * N + n0 + c * 16);
    }
    __syncthreads();
    uint8_t *d = dst + ((e * (N / 128) + blockIdx.x) * (K / 128) + blockIdx.y) * 16384;
    for (int i = threadIdx.x; i < 1024; i += blockDim.x) {      /* one 16-byte slot per iteration */
        const int r = i >> 3, slot = i & 7;
        const int c = slot ^ ((r & 7) ^ ((r >> 3) & 1));
        const int ch = zb_block_row_channel(r);
        uint32_t w[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
            w[q] = (uint32_t)tile[c * 16 + 4 * q][ch] | ((uint32_t)tile[c * 16 + 4 * q + 1][ch] << 8) |
                   ((uint32_t)tile[c * 16 + 4 * q + 2][ch] << 16) | ((uint32_t)tile[c * 16 + 4 * q + 3][ch] << 24);
        *reinterpret_cast<u32x4 *>(d + i * 16) = u32x4{w[0], w[1], w[2], w[3]};
    }
}

/*
 * int8 values in [-8,7], [E,K,N] -> [E][N/128][K/128] blocks of 8 KiB, two values per byte. A block holds 128
 * channels x 128 k as the GEMM wants them in LDS: block row r (channel zb_block_row_channel(r), as for 8-bit
 * weights) at +64*r, and within it the 16-byte chunk c (k in [32c, 32c+32)) in slot c ^ ((r >> 2) & 3), so that
 * the 64 lanes of a fragment read (16 rows x 4 chunks) touch 64 distinct slots. Within a chunk, byte b of dword j holds k[8j+b] in its low nibble and k[8j+4+b] in
 * its high nibble: the GEMM unpacks a dword into two dwords of four consecutive k with one shift and two masks.
 */
__global__ void __launch_bounds__(256)
tile_pack_int4_kernel(const int8_t *__restrict__ src, int64_t K, int64_t N, uint8_t *__restrict__ dst)
{
    __shared__ int8_t tile[128][128 + 16];           /* [k][n] */
    const int64_t e = blockIdx.z;
    const int64_t k0 = (int64_t)blockIdx.y * 128, n0 = (int64_t)blockIdx.x * 128;
    const int8_t *s = src + e * K * N;
    for (int i = threadIdx.x; i < 128 * 8; i += blockDim.x) {
        const int kk = i >> 3, c = i & 7;
        *reinterpret_cast<u32x4 *>(&tile[kk][c * 16]) = *reinterpret_cast<const u32x4 *>(s + (k0 + kk) * N + n0 + c * 16);
    }
    __syncthreads();
    uint8_t *d = dst + ((e * (N / 128) + blockIdx.x) * (K / 128) + blockIdx.y) * 8192;
    for (int i = threadIdx.x; i < 512; i += blockDim.x) {       /* one 16-byte chunk per iteration */
        const int r = i >> 2, c = i & 3;
        const int ch = zb_block_row_channel(r);
        uint32_t w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            w[j] = 0;
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) {
                const uint32_t lo = (uint32_t)tile[32 * c + 8 * j + bb][ch] & 0xfu;
                const uint32_t hi = (uint32_t)tile[32 * c + 8 * j + 4 + bb][ch] & 0xfu;
                w[j] |= (lo | (hi << 4)) << (8 * bb);
            }
        }
        const int slot = c ^ (((r & 15) >> 2) & 3);
        *reinterpret_cast<u32x4 *>(d + (r >> 4) * 1024 + (r & 15) * 64 + slot * 16) = u32x4{w[0], w[1], w[2], w[3]};
    }
}

} // namespace

extern "C" int32_t zbalhip_weight_prepack(const void *src, int64_t experts, int64_t k, int64_t n, int32_t to_int4,
                                          void *dst, void *stream)
{
    if (!src || !dst || src == dst || experts <= 0 || k <= 0 || n <= 0) return ZBALHIP_INVALID;
    if (experts > 65535) return ZBALHIP_INVALID;
    if ((k % 128) != 0 || (n % 128) != 0 || k / 128 > 65535) return ZBALHIP_INVALID;
    if (((uintptr_t)src & 15) != 0 || ((uintptr_t)dst & 15) != 0) return ZBALHIP_INVALID;
    dim3 grid((unsigned)(n / 128), (unsigned)(k / 128), (unsigned)experts);
    if (to_int4) tile_pack_int4_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const int8_t *)src, k, n, (uint8_t *)dst);
    else tile_swizzle_bytes_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const uint8_t *)src, k, n, (uint8_t *)dst);
    return zbalhip_check_launch();
}
