/*
 * Grouped (per-expert, ragged-M) quantised GEMM with fused epilogues for gfx950.
 *
 * Operands: activations A [rows, K] one byte per element (int8 or e4m3),
 * expert-major rows delimited by row_off[E+1]; weights W pre-packed
 * [E, N, K] with K contiguous (int4: [E, N, K/2]). Both operands are
 * K-contiguous, so either can feed either MFMA input; the kernel feeds the
 * WEIGHT fragment as the matrix-A input and the ACTIVATION fragment as the
 * matrix-B input, i.e. it computes C^T. With the 16x16 MFMA output layout
 * (lane l holds output column l%16, rows 4*(l/16)+i) every lane then owns ONE
 * token row and FOUR consecutive output channels per instruction, and with
 * the pre-pack's order of the weight rows EIGHT consecutive channels per pair
 * of instructions: per-token scales are one value per lane, per-channel
 * scales 16-byte vectors, gate/up pairs of the SwiGLU sit in the same lane,
 * and results leave as 8-element vectors.
 *
 * Workgroup tile: 256 (or 128) token rows x 256 output channels x 128 K-bytes
 * per step, eight (four) waves, each wave 64 rows x 128 channels = 4x8 MFMA
 * tiles (128 accumulator registers). For GMM1 the 256 channels are 128 gate
 * columns j and the matching 128 up columns I+j, so the SwiGLU product and,
 * in the fp8 mode, the complete 1x128 requantisation happen in registers.
 * K slabs go from HBM to LDS by DMA, in a swizzled order that the weights are
 * pre-packed in, one persistent workgroup per CU; the details stand at the
 * kernel below.
 *
 * Tile schedule: workgroup ids are dealt round-robin to the 8 XCDs by the
 * hardware; XCD x takes a contiguous run of the logical tile order and its
 * workgroups take consecutive tiles of it. Logical tiles walk an expert in
 * groups of (all its row tiles) x (8 channel tiles), row tile fastest, so
 * the workgroups resident on an XCD share both their A and their W slabs in
 * that XCD's L2.
 */
#include <atomic>
#include <mutex>
#include <type_traits>

#include "zbal_device.h"
#include "zbal_hip_kernels.h"

namespace {

constexpr int BN = 256;          /* output channels per workgroup tile */
constexpr int BKB = 128;         /* K bytes of an activation row per slab (128 int8/e4m3 elements) */
constexpr int GROUP_N = 8;       /* channel tiles per schedule group, at most */

enum { MODE_W8A8 = 1, MODE_FP8 = 2, MODE_W4A8 = 3 };

struct GemmParams {
    const uint8_t *a;        /* [rows, K] */
    const float *a_scale;    /* [rows] or [rows, K/128] */
    const uint8_t *w;        /* pre-packed blocks, [E][N/128][K/128] x 16 KiB (8-bit) or 8 KiB (int4) */
    const void *wscale;
    const int32_t *row_off;  /* [E+1] */
    int experts;
    int max_rows;            /* rows the A / output buffers hold */
    int K;
    int N;                   /* weight rows per expert (N1 for GMM1) */
    int wscale_is_bf16;
    int w_is_list;           /* `w` and `wscale` are device tables of `experts` addresses, one expert's tensor each */
    void *out;               /* GMM1: q2 bytes; GMM2: y */
    float *out_scale;        /* GMM1: scale2 (fp8 mode) */
    float *sgl_ws;           /* GMM1 int8 modes: fp32 SwiGLU values [rows, N/2] */
    uint32_t *rowmax;        /* GMM1 int8 modes: per-row absmax bits */
};

/*
 * First element of expert e's weights or scales: base + e * stride, or entry e of the address table. The table is
 * read through the constant address space: a scalar load, which does not queue behind the slabs in flight.
 */
template <typename T>
__device__ __forceinline__ const T *expert_base(const void *base, int is_list, int expert, int64_t stride_elems)
{
    if (is_list) {
        typedef const uint64_t __attribute__((address_space(4))) *table_t;
        return (const T *)(uintptr_t)((table_t)(uintptr_t)base)[expert];
    }
    return (const T *)base + (int64_t)expert * stride_elems;
}

struct TileCoord {
    int expert, m_tile, n_tile;
};

__device__ __forceinline__ f32x4 mfma_fp8_16x16x128(const i32x8 &wfrag, const i32x8 &afrag)
{
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    /* cbsz = blgp = 0 selects e4m3 for both inputs; scale exponents 0 leave the product unscaled */
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wfrag, afrag, zero, 0, 0, 0, 0, 0, 0);
}

/* four consecutive bytes -> one dword store helpers */
__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d)
{
    return zb_cvt_pk_e4m3(a, b) | (zb_cvt_pk_e4m3(c, d) << 16);
}

/*
 * Shared epilogue. The calling wave holds, for sub-tile (mt, nt), block rows nt*16 + 4*(lane/16) + i of its weight
 * rows, for token row (RG*mt + wm)*16 + lane%16 of the tile (RG = row groups of waves; a wave's 16-row sub-tiles
 * are dealt round-robin over the row groups, so a tile that is not full leaves every SIMD the same share). The pre-pack put channels 32*(nt/2) + 8*(lane/16) + 4*(nt%2) + i in
 * those rows (zb_block_row_channel), so the sub-tiles nt = 2s and 2s+1 together are eight consecutive channels.
 * `lds_rowmax` is [2][tile_rows] floats of scratch for the row maxima of the two channel halves (GMM1 only).
 */
template <int MODE, bool GMM1, int OUT_DT, int RG, int MTM>
__device__ __forceinline__ void epilogue(const GemmParams &p, const TileCoord &tc, f32x4 (&accf)[MTM][8],
                                         i32x4 (&acci)[MTM][8], int row_begin, int row_end, int wm, int wn, int lane,
                                         float *lds_rowmax, int tile_rows, const float *es)
{
    /*
     * W8A8: `es` is this tile's scales in LDS, brought there by DMA while the tile was multiplied: [0, 256) the
     * channel scales of the tile's 256 weight rows (fp32, or 256 bf16 in the first 512 bytes), [256, 256 +
     * tile_rows) the per-token scales of its rows. A global load here is waited for with a count that also waits
     * for the next tile's slabs, which are already in flight (decode: 5-6 % of both GEMMs). The W4A8 mode, whose
     * channel scales travel with the slabs, still loads its per-token scale here: its kernel has no registers to
     * spare, and a spill costs more than the wait.
     */
    const float *es_row = es + 256;
    const int frag_row = lane & 15;
    const int I = p.N / 2;
    const int q8 = (lane >> 4) * 8;
    if constexpr (!GMM1) {
        uint16_t *y = (uint16_t *)p.out;
#pragma unroll
        for (int mt = 0; mt < MTM; ++mt) {
            const int row = row_begin + (RG * mt + wm) * 16 + frag_row;
            if (row >= row_end) continue;
            float xs = 1.0f;
            if (MODE == MODE_W8A8) xs = es_row[(RG * mt + wm) * 16 + frag_row];
            else if (MODE == MODE_W4A8) xs = p.a_scale[row];
#pragma unroll
            for (int s = 0; s < 4; ++s) {         /* sub-tiles 2s and 2s+1: eight consecutive channels from n */
                const int nl = wn * 128 + s * 32 + q8;       /* within the tile */
                const int n = tc.n_tile * BN + nl;
                float ws[8];
                if constexpr (MODE == MODE_W8A8) {
                    if (p.wscale_is_bf16) {
                        const u32x4 v = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const uint16_t *>(es) + nl);
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            ws[2 * i] = zb_bf16_to_f32(v[i] & 0xffffu);
                            ws[2 * i + 1] = zb_bf16_to_f32(v[i] >> 16);
                        }
                    } else {
                        const float *wsp = es + nl;
                        const f32x4 v0 = *reinterpret_cast<const f32x4 *>(wsp), v1 = *reinterpret_cast<const f32x4 *>(wsp + 4);
#pragma unroll
                        for (int i = 0; i < 4; ++i) { ws[i] = v0[i]; ws[4 + i] = v1[i]; }
                    }
                }
                float d[8];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int nt = 2 * s + h;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if constexpr (MODE == MODE_W8A8) d[4 * h + i] = ((float)acci[mt][nt][i] * ws[4 * h + i]) * xs;
                        else if constexpr (MODE == MODE_FP8) d[4 * h + i] = accf[mt][nt][i];
                        else d[4 * h + i] = accf[mt][nt][i] * xs;
                    }
                }
                *reinterpret_cast<u32x4 *>(y + (int64_t)row * p.N + n) =
                    u32x4{zb_pack2_half<OUT_DT>(d[0], d[1]), zb_pack2_half<OUT_DT>(d[2], d[3]),
                          zb_pack2_half<OUT_DT>(d[4], d[5]), zb_pack2_half<OUT_DT>(d[6], d[7])};
            }
        }
    } else {
        /* SwiGLU on gate sub-tile nt and up sub-tile nt+4: columns j = n_tile*128 + wn*64 + 32*(nt/2) + q8 + 4*(nt%2) + i */
        float sg[MTM][4][4];
        float rmax[MTM];
#pragma unroll
        for (int mt = 0; mt < MTM; ++mt) {
            /*
             * A 16-row sub-tile past the tile's end holds nothing (the K loop left it out as well): its SwiGLU, which is
             * most of this epilogue's arithmetic (an exact exp and a division per value in the int modes), is skipped.
             * Wave-uniform. Few-row tiles spent 10 us here per tile before, one seventh of the decode kernel.
             */
            if ((RG * mt + wm) * 16 >= row_end - row_begin) continue;
            const int row = row_begin + (RG * mt + wm) * 16 + frag_row;
            float xs = 1.0f;
            if (MODE == MODE_W8A8) xs = es_row[(RG * mt + wm) * 16 + frag_row];
            else if (MODE == MODE_W4A8) xs = p.a_scale[row < p.max_rows ? row : p.max_rows - 1];
            rmax[mt] = 0.0f;
#pragma unroll
            for (int nt = 0; nt < 4; ++nt) {
                const int jl = wn * 64 + (nt >> 1) * 32 + q8 + (nt & 1) * 4;       /* within the tile's 128 SwiGLU columns */
                float g[4], u[4];
                if constexpr (MODE == MODE_W8A8) {
                    const f32x4 wg = *reinterpret_cast<const f32x4 *>(es + jl);             /* gate scales, then up scales */
                    const f32x4 wu = *reinterpret_cast<const f32x4 *>(es + 128 + jl);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        g[i] = ((float)acci[mt][nt][i] * wg[i]) * xs;
                        u[i] = ((float)acci[mt][nt + 4][i] * wu[i]) * xs;
                    }
                } else if constexpr (MODE == MODE_FP8) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) { g[i] = accf[mt][nt][i]; u[i] = accf[mt][nt + 4][i]; }
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) { g[i] = accf[mt][nt][i] * xs; u[i] = accf[mt][nt + 4][i] * xs; }
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float left;
                    if constexpr (MODE == MODE_FP8) {
                        /* e4m3 keeps 3 mantissa bits: the hardware exp2 / reciprocal approximations (1 ulp) are ample */
                        left = g[i] * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g[i] * -1.44269504088896341f));
                    } else {
                        left = g[i] / (1.0f + zb_expf(-g[i]));
                    }
                    const float s = left * u[i];
                    sg[mt][nt][i] = s;
                    rmax[mt] = fmaxf(rmax[mt], fabsf(s));
                }
            }
            /* the four lane groups (lane/16) hold different columns of the same row */
            rmax[mt] = fmaxf(rmax[mt], __shfl_xor(rmax[mt], 16, 64));
            rmax[mt] = fmaxf(rmax[mt], __shfl_xor(rmax[mt], 32, 64));
            if (lane < 16) lds_rowmax[wn * tile_rows + (RG * mt + wm) * 16 + lane] = rmax[mt];
        }
        __syncthreads();
#pragma unroll
        for (int mt = 0; mt < MTM; ++mt) {
            const int lr = (RG * mt + wm) * 16 + frag_row;
            const int row = row_begin + lr;
            const float amax_tile = fmaxf(lds_rowmax[lr], lds_rowmax[tile_rows + lr]);
            if (row >= row_end) continue;
            if constexpr (MODE == MODE_FP8) {
                const float amax = fmaxf(amax_tile, 1e-4f);
                const float mult = 448.0f / amax;
                uint8_t *q2 = (uint8_t *)p.out;
#pragma unroll
                for (int s = 0; s < 2; ++s) {         /* sub-tiles 2s and 2s+1: eight consecutive columns */
                    const int j = tc.n_tile * 128 + wn * 64 + s * 32 + q8;
                    u32x2 v;
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                        v[h] = pack4_e4m3(sg[mt][2 * s + h][0] * mult, sg[mt][2 * s + h][1] * mult, sg[mt][2 * s + h][2] * mult,
                                          sg[mt][2 * s + h][3] * mult);
                    *reinterpret_cast<u32x2 *>(q2 + (int64_t)row * I + j) = v;
                }
                if (wn == 0 && lane < 16) p.out_scale[(int64_t)row * (I / 128) + tc.n_tile] = amax * (1.0f / 448.0f);
            } else {
#pragma unroll
                for (int nt = 0; nt < 4; ++nt) {
                    const int j = tc.n_tile * 128 + wn * 64 + (nt >> 1) * 32 + q8 + (nt & 1) * 4;
                    const f32x4 v = f32x4{sg[mt][nt][0], sg[mt][nt][1], sg[mt][nt][2], sg[mt][nt][3]};
                    *reinterpret_cast<f32x4 *>(p.sgl_ws + (int64_t)row * I + j) = v;
                }
                if (wn == 0 && lane < 16) atomicMax(&p.rowmax[row], __float_as_uint(amax_tile));
            }
        }
    }
}

/* ------------------------------------------------------------------------------------------------------
 * The grouped GEMM kernel (W8A8, fp8, W4A8): TM token rows x 256 channels x 128 K elements per workgroup,
 * eight waves (four row groups x two 128-channel halves; a wave's rows are the 16-row sub-tiles s with
 * s % 4 = its row group), one workgroup per CU.
 *
 * K slabs go from HBM to LDS without passing through registers: every wave issues
 * global_load_lds_dwordx4, which deposits the 64 lanes' 16-byte chunks in 1 KiB of consecutive LDS
 * (lane l at +16*l). A block of 1 KiB holds 8 tile rows of 128 bytes; which global chunk a lane fetches is
 * free, so the chunk stored in slot s of row r is logical chunk s ^ f(r), f(r) = (r & 7) ^ ((r >> 3) & 1).
 * A fragment read touches 16 consecutive rows at the same logical chunk (128-byte pitch); with f every
 * aligned run of 8 rows lands in 8 distinct 16-byte slots and the 16 rows in 16 distinct (row parity, slot)
 * pairs, so the read is free of bank conflicts whether the LDS serves 8 or 16 lanes per pass; plain
 * row-major storage would put all 16 rows on the same slot.
 *
 * Three shapes are built. TM = 256 and TM = 320 with two stages of 64 / 72 KiB (the slab for step k+1 is in
 * flight while step k is multiplied) have the arithmetic intensity that many-row experts need; the 320-row
 * shape gives every wave a fifth sub-tile. TM = 128 with three stages of 48 KiB is for
 * few-row experts, where the job is to stream every weight byte once at HBM speed: it keeps two weight slabs
 * (64 KiB) in flight per CU, two sub-tiles per wave, and skips the MFMAs of sub-tiles past the expert's end.
 * Either way there is one barrier per step.
 *
 * W4A8: the weight slab stays packed in LDS (64 bytes per channel; block layout and nibble order as written by
 * the pre-pack) and is unpacked to int8 * 16 in registers, a shift and two masks per packed dword; the factor 16
 * is divided out of the accumulators, exactly, before the epilogue. Each 128-deep slab is one scale group:
 * its 256 fp16 group scales ride along by DMA and `acc = fma(float(partial), gs, acc)` promotes the int32 partial.
 * ------------------------------------------------------------------------------------------------------ */
constexpr int D_MAX_KB = 256;                 /* K up to 32768 */
constexpr int D_MAX_EXPERTS = 1024;

/* WRB = bytes of one weight row per slab: 128 (8-bit) or 64 (packed int4) */
template <int TM, int NSTAGE, int WRB>
struct DmaShape {
    static constexpr int ROW_GROUPS = 4;                   /* row groups of two waves each: eight waves, two per SIMD */
    static constexpr int MTM = (TM / 16 + ROW_GROUPS - 1) / ROW_GROUPS;   /* 16-row sub-tiles per wave, at most: 2, 4, or 5 in the 320-row shape */
    static constexpr int NW = ROW_GROUPS * 2;
    static constexpr int THREADS = NW * 64;
    static constexpr int A_BYTES = TM * BKB;
    static constexpr int W_BYTES = BN * WRB;
    static constexpr int STAGE_BYTES = A_BYTES + W_BYTES;
    static constexpr int HALF_BLOCKS = 128 * WRB / 1024;   /* 1 KiB blocks per 128-channel half: 16 or 8 */
    static constexpr int MAX_EXPERTS = TM > 256 ? 512 : D_MAX_EXPERTS;   /* what the lookup tables hold: the 320-row shape has 160 KiB of LDS less 144 KiB of stages for everything else */
    static constexpr int A_PARTS = (A_BYTES / 1024 + NW - 1) / NW;   /* 1 KiB blocks of the A tile per wave: 2, 4 or 5 */
    static constexpr int W_PARTS = W_BYTES / 1024 / NW;    /* 1 KiB blocks of the W tile per wave (2, 4 or 8) */
    static constexpr int PARTS = W_PARTS > A_PARTS ? W_PARTS : A_PARTS;
    static constexpr bool TWO_PHASE = TM == 256;            /* the tiles of short experts run after all the others (see the kernel) */
    /* two buffers of per-tile scales, floats each: fp8 2 x D_MAX_KB weight block scales; W8A8 256 channel + TM token scales */
    static constexpr int SW_STRIDE = TM > 256 ? 576 : 2 * D_MAX_KB;
    static constexpr int SW_BYTES = 2 * SW_STRIDE * 4;
    static_assert(SW_STRIDE >= 2 * D_MAX_KB && SW_STRIDE >= 256 + TM, "scale buffer too small");
    static constexpr int LDS_BYTES = NSTAGE * STAGE_BYTES + NSTAGE * TM * 4 + 2 * TM * 4 + SW_BYTES +
                                     2 * (MAX_EXPERTS + 1) * 4 + (WRB == 64 ? NSTAGE * BN * 2 : 0) +
                                     (TWO_PHASE ? MAX_EXPERTS * 2 + (MAX_EXPERTS + 1) * 4 : 0);
    static_assert(PARTS >= 2 && (PARTS % 4 == 0 || PARTS == 2 || (NSTAGE == 2 && PARTS == 5)),
                  "the issue schedule hands out parts q * PARTS / 4 .. (q + 1) * PARTS / 4 - 1 of a slab with quarter q of a step");
    static_assert(NW <= HALF_BLOCKS && HALF_BLOCKS % NW == 0, "a wave's W blocks must not straddle a weight half");
    static_assert(LDS_BYTES <= 160 * 1024, "tile does not fit the LDS");
};

/* the pointer as scalar registers; a no-op where the compiler already knows it is wave-uniform */
template <typename T>
__device__ __forceinline__ const T *uniform_ptr(const T *p)
{
    const uint64_t v = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const T *)(((uint64_t)hi << 32) | lo);
}

/*
 * One LDS-DMA transfer with the address split the way the instruction wants it: a wave-uniform 64-bit base in
 * scalar registers plus a 32-bit offset per lane, and the wave's LDS destination in M0. Spelled out because
 * the compiler otherwise keeps a 64-bit vector address per transfer alive across the whole K loop.
 *
 * The base often reaches the asm through v_readfirstlane. A scalar register written by a vector instruction must not
 * be read by a vector-memory instruction within five wait states, and the compiler, which inserts such waits for its
 * own instructions, does not look inside the asm text. So the text brings them along: the move to M0 is one,
 * `s_nop 3` the other four. (With no wait state at all the load used the register's old contents and the kernel
 * faulted; the two states of an `s_nop 0` ran clean, but the documented figure is five.)
 */
__device__ __forceinline__ void dma16_sv(const uint8_t *uniform_base, uint32_t lane_off, uint32_t lds_wave_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_wave_addr), "v"(lane_off), "s"(uniform_ptr(uniform_base))
                 : "memory", "m0");
}

/*
 * The same with the streaming hint, for weight slabs that no other workgroup asks for again (experts with a single
 * row tile: each slab is read once). Measured on the few-row shape: the decode layer 5 % faster, the weight stream of
 * a 128-token fp8 layer 5.3 -> 5.9 TB/s; on slabs that several row tiles share it costs 3-9 %, and decided tile by
 * tile inside the kernel it cost registers, so the launcher decides per launch (WSTREAM).
 */
__device__ __forceinline__ void dma16_sv_nt(const uint8_t *uniform_base, uint32_t lane_off, uint32_t lds_wave_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %1, %2 nt"
                 :
                 : "s"(lds_wave_addr), "v"(lane_off), "s"(uniform_ptr(uniform_base))
                 : "memory", "m0");
}

__device__ __forceinline__ void dma4_sv(const float *uniform_base, uint32_t lane_off_bytes, uint32_t lds_wave_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tglobal_load_lds_dword %1, %2"
                 :
                 : "s"(lds_wave_addr), "v"(lane_off_bytes), "s"(uniform_ptr(uniform_base))
                 : "memory", "m0");
}

__device__ __forceinline__ uint32_t lds_addr(const void *p)
{
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p;
}


/* wait until at most N of this wave's vector-memory operations are outstanding (they complete in order) */
template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

/* what a workgroup needs to know about one tile; every member is wave-uniform and lives in scalar registers */
struct DmaTile {
    bool valid;
    int expert, n_tile, row_begin, row_end, last_rel;
    const uint8_t *a_base;            /* first K-byte of the tile's first activation row */
    const float *sa_base;             /* its fp8 block scales */
    const uint8_t *w_half[2];         /* K slab 0 of the tile's two 128-channel weight block rows */
    const uint16_t *gs_mine;          /* W4A8: fp16 group scales, slab 0, of the weight half this wave brings in (wave % 2) */
};

template <int MODE, bool GMM1, int OUT_DT, int TM, int NSTAGE, bool WSTREAM>
/*
 * Eight waves, two per SIMD (256 registers each), in every shape. The 128-row shape used to run four waves with the
 * wave tile of the 256-row shape (64 x 128), one per SIMD with nobody to cover its waits; as eight waves of 32 x 128
 * it is faster wherever it is used: decode layer (128 tokens, W8A8) 0.295 -> 0.288 ms, fp8 with 96 rows per expert
 * on 32 experts 0.404 -> 0.342 ms, W4A8 with 32-96 rows per expert first GEMM 9-12 % and second 7-8 % faster.
 */
__global__ void __launch_bounds__(512, 2)
grouped_gemm_dma_kernel(GemmParams p)
{
    static_assert(MODE == MODE_W8A8 || MODE == MODE_FP8 || MODE == MODE_W4A8, "unknown mode");
    static_assert(NSTAGE == 2 || NSTAGE == 3, "two or three stages");
    constexpr int WRB = MODE == MODE_W4A8 ? 64 : 128;
    using S = DmaShape<TM, NSTAGE, WRB>;
    constexpr int NW = S::NW, STAGE_BYTES = S::STAGE_BYTES, A_BYTES = S::A_BYTES, W_PARTS = S::W_PARTS, PARTS = S::PARTS;
    constexpr int HALF_BLOCKS = S::HALF_BLOCKS, W_BLOCK_BYTES = 128 * WRB;     /* one 128-channel block of one slab */
    constexpr int RG = S::ROW_GROUPS;                /* row groups of waves; 16-row sub-tile s of a tile belongs to group s % RG */
    using Tile = DmaTile;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    float *lds_sa = reinterpret_cast<float *>(smem + NSTAGE * STAGE_BYTES);   /* [NSTAGE][TM] */
    float *lds_rowmax = lds_sa + NSTAGE * TM;                                 /* [2][TM] */
    constexpr int SW_STRIDE = S::SW_STRIDE;
    float *lds_sw = lds_rowmax + 2 * TM;                                      /* [2 tiles][SW_STRIDE]: fp8 [2][D_MAX_KB] weight block scales */
    int *lds_mtp = reinterpret_cast<int *>(lds_sw + 2 * SW_STRIDE);            /* [experts + 1] tiles of TM rows before expert e */
    int *lds_roff = lds_mtp + (S::MAX_EXPERTS + 1);                            /* [experts + 1] copy of row_off */
    uint16_t *lds_gs = reinterpret_cast<uint16_t *>(lds_roff + (S::MAX_EXPERTS + 1));   /* [NSTAGE][BN] W4A8 group scales (fp16) */
    uint16_t *lds_short = lds_gs + (WRB == 64 ? NSTAGE * BN : 0);                       /* [experts] the short experts, second phase */
    int *lds_cost = reinterpret_cast<int *>(lds_short + S::MAX_EXPERTS);                 /* [experts + 1] 16-row sub-tiles of the main tiles before expert e */
    constexpr bool TWO_PHASE = S::TWO_PHASE;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int wm = wave_u >> 1, wn = wave_u & 1;      /* wave-uniform, so everything derived from them lives in scalar registers */
    const int n_tiles = GMM1 ? (p.N / 2) / 128 : p.N / BN;
    const int K = p.K;
    const int KB = K / 128;
    const int I = p.N / 2;
    const int E = p.experts;

    /*
     * The workgroup is persistent: it walks a fixed sequence of tiles, and the DMA runs NSTAGE-1 slabs ahead of the
     * MFMAs across tile boundaries, so a tile's epilogue and the next tile's first loads overlap. The tile lookup
     * tables are built once, in LDS, so that finding the next tile costs no vector-memory traffic (whose waits would
     * also wait for the slabs in flight).
     */
    /*
     * Tile order. A tile with a few rows keeps most waves idle and runs at the pace of its own loads; in the middle
     * of the sequence it drifts away from the workgroups it shares slabs with, and the L2 stops serving them
     * together (measured on 4096 tokens over 32 experts with 42-row tail tiles in the sequence: 3.6 GB of HBM reads
     * per launch for 1.25 GB of operands, against 1.45 GB when every expert has exactly 1024 rows). Rows are
     * therefore cut into even tiles (fill_tile below), and the experts whose rows fill at most half a tile are kept
     * out of the main sequence and run after it, the longer class first: tiles that run side by side take about the
     * same time.
     */
    int n_short = 0;
    if (wave == 0) {
        int run = 0, run_c = 0;
        for (int base = 0; base < E; base += 64) {
            const int e = base + lane;
            int mt = 0, rows_e = 0;
            if (e < E) {
                const int lo = p.row_off[e];
                rows_e = p.row_off[e + 1] - lo;
                mt = (rows_e + TM - 1) / TM;
                if (TWO_PHASE && rows_e <= TM / 2) mt = 0;      /* a short expert's only tile is not a main tile */
                lds_roff[e] = lo;
            }
            /* what the expert's main tiles cost: their number times their height in 16-row sub-tiles (fill_tile cuts them evenly) */
            const int cost = mt > 0 ? mt * ((((rows_e + mt - 1) / mt) + 15) >> 4) : 0;
            int incl = mt, incl_c = cost;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const int o = __shfl_up(incl, off, 64), oc = __shfl_up(incl_c, off, 64);
                if (lane >= off) { incl += o; incl_c += oc; }
            }
            if (e < E) {
                lds_mtp[e] = run + incl - mt;
                if (TWO_PHASE) lds_cost[e] = run_c + incl_c - cost;
            }
            run += __shfl(incl, 63, 64);
            run_c += __shfl(incl_c, 63, 64);
        }
        if (lane == 0) {
            lds_mtp[E] = run;
            lds_roff[E] = p.row_off[E];
            if (TWO_PHASE) lds_cost[E] = run_c;
        }
        if (TWO_PHASE) {
            for (int cls = 2; cls >= 1; --cls) {          /* experts of TM/4+1 .. TM/2 rows, then those of 1 .. TM/4 */
                for (int base = 0; base < E; base += 64) {
                    const int e = base + lane;
                    bool mine = false;
                    if (e < E) {
                        const int rows = p.row_off[e + 1] - p.row_off[e];
                        mine = rows > 0 && rows <= TM / 2 && (rows > TM / 4) == (cls == 2);
                    }
                    const uint64_t bal = __ballot(mine);
                    if (mine) lds_short[n_short + __popcll(bal & ((1ull << lane) - 1))] = (uint16_t)e;
                    n_short += __popcll(bal);
                }
            }
            if (lane == 0) lds_rowmax[0] = __int_as_float(n_short);    /* for the other waves; the epilogues use this later */
        }
    }
    __syncthreads();
    if (TWO_PHASE) {
        n_short = __builtin_amdgcn_readfirstlane(__float_as_int(lds_rowmax[0]));
        __syncthreads();
    }
    /*
     * XCD x (workgroups x, x+8, ...) owns a contiguous range of the logical tile order. Where tiles differ in height
     * the ranges are cut at equal cost (16-row sub-tiles), not at equal tile counts: the kernel lasts as long as its
     * slowest XCD.
     */
    const int total = __builtin_amdgcn_readfirstlane(lds_mtp[E]) * n_tiles;
    const int chunk = (total + 7) / 8;
    const int xcd = blockIdx.x & 7, slots = gridDim.x >> 3;
    auto first_id_of = [&](int x) __attribute__((always_inline)) -> int {
        if (!TWO_PHASE) return x * chunk < total ? x * chunk : total;
        if (x >= 8) return total;
        /* the tile at which the cost before it reaches x/8 of the whole: expert by search, tile within it by division */
        const int64_t target = (int64_t)lds_cost[E] * n_tiles * x / 8;
        int id = total;
        for (int base = 0; base < E; base += 64) {
            const int e = base + lane;
            int64_t lo = INT64_MAX, hi = INT64_MAX;
            if (e < E) { lo = (int64_t)lds_cost[e] * n_tiles; hi = (int64_t)lds_cost[e + 1] * n_tiles; }
            const uint64_t bal = __ballot(lo <= target && target < hi);
            if (bal) {
                const int src = __ffsll((long long)bal) - 1;
                const int ex = base + src;
                const int mt_e = lds_mtp[ex + 1] - lds_mtp[ex];
                const int height = (lds_cost[ex + 1] - lds_cost[ex]) / mt_e;      /* sub-tiles per tile of this expert */
                id = lds_mtp[ex] * n_tiles + (int)((target - (int64_t)lds_cost[ex] * n_tiles) / height);
                break;
            }
        }
        return __builtin_amdgcn_readfirstlane(id);
    };
    const int lid_begin = first_id_of(xcd);
    const int lid_end = first_id_of(xcd + 1);
    /* the short experts' tiles follow as ids total, total + 1, ...: n_short * n_tiles of them, split evenly over the XCDs */
    const int total_b = n_short * n_tiles;
    const int chunk_b = (total_b + 7) / 8;
    const int bid_begin = total + xcd * chunk_b + (blockIdx.x >> 3);
    const int bid_end = total + ((xcd + 1) * chunk_b < total_b ? (xcd + 1) * chunk_b : total_b);
    int lid = lid_begin + (blockIdx.x >> 3);
    if (lid >= lid_end) lid = bid_begin;
    /* the id after `id` in this workgroup's sequence */
    auto next_id = [&](int id) __attribute__((always_inline)) {
        const int n = id + slots;
        return (id < total && n >= lid_end) ? bid_begin : n;
    };

    auto fill_tile = [&](Tile &t, int expert, int n_tile, int m_tile) __attribute__((always_inline)) {
        t.expert = expert;
        t.n_tile = n_tile;
        /*
         * An expert's rows are cut into its ceil(rows / TM) tiles evenly, in multiples of 16: 1066 rows are five tiles
         * of 224, 224, 224, 224 and 170 rows rather than four of 256 and one of 42. The tiles cost what their 16-row
         * sub-tiles cost (the K loop leaves out the absent ones), so this is no more work, and no tile is so short
         * that it runs ahead of the tiles it shares slabs with.
         */
        const int first_row = __builtin_amdgcn_readfirstlane(lds_roff[expert]);
        const int end_row = __builtin_amdgcn_readfirstlane(lds_roff[expert + 1]);
        const int n_row_tiles = (end_row - first_row + TM - 1) / TM;
        const int height = (((end_row - first_row + n_row_tiles - 1) / n_row_tiles) + 15) & ~15;
        t.row_begin = first_row + m_tile * height;
        t.row_end = t.row_begin + height < end_row ? t.row_begin + height : end_row;
        t.last_rel = t.row_end - 1 - t.row_begin;   /* rows past the tile's end re-read its last row: in bounds, and one line */
        t.a_base = p.a + (int64_t)t.row_begin * K;
        t.sa_base = p.a_scale + (int64_t)t.row_begin * KB;
        /* weights come pre-packed as 16 KiB blocks of 128 channels x 128 K-bytes in LDS order ([E][N/128][K/128]) */
        const int col0 = GMM1 ? t.n_tile : t.n_tile * 2, col1 = GMM1 ? I / 128 + t.n_tile : t.n_tile * 2 + 1;
        const uint8_t *wb = expert_base<uint8_t>(p.w, p.w_is_list, expert, (int64_t)(p.N / 128) * KB * W_BLOCK_BYTES);
        t.w_half[0] = wb + ((int64_t)col0 * KB) * W_BLOCK_BYTES;
        t.w_half[1] = wb + ((int64_t)col1 * KB) * W_BLOCK_BYTES;
        if (MODE == MODE_W4A8) {      /* fp16 group scales [E][K/128][N]: the slab's 128 scales of each half are 256 bytes */
            const uint16_t *gs = expert_base<uint16_t>(p.wscale, p.w_is_list, expert, (int64_t)KB * p.N);
            t.gs_mine = gs + ((wave_u & 1) ? col1 : col0) * 128;
        }
    };
    auto load_tile = [&](int id, Tile &t) __attribute__((always_inline)) {
        t.valid = id < total ? id < lid_end : id < bid_end;
        if (!t.valid) return;
        if (TWO_PHASE && id >= total) {              /* short expert number (id - total) / n_tiles, channel tile the remainder */
            const int j = (id - total) / n_tiles;
            const int expert = __builtin_amdgcn_readfirstlane((int)lds_short[j]);
            fill_tile(t, expert, id - total - j * n_tiles, 0);
            return;
        }
        const int q = id / n_tiles;                  /* index among all TM-row tiles: expert e has [mtp[e], mtp[e+1]) */
        int expert = 0, first = 0, next = 0;
        for (int base = 0; base < E; base += 64) {
            const int e = base + lane;
            int lo = 0x7fffffff, hi = 0x7fffffff;
            if (e < E) { lo = lds_mtp[e]; hi = lds_mtp[e + 1]; }
            const uint64_t bal = __ballot(lo <= q && q < hi);
            if (bal) {
                const int src = __ffsll((long long)bal) - 1;
                expert = base + src;
                first = __shfl(lo, src, 64);
                next = __shfl(hi, src, 64);
                break;
            }
        }
        expert = __builtin_amdgcn_readfirstlane(expert);
        first = __builtin_amdgcn_readfirstlane(first);
        const int mt_e = __builtin_amdgcn_readfirstlane(next) - first;
        /*
         * Within the expert: groups of (all its row tiles) x (a few channel tiles), row tile fastest, so that concurrent
         * tiles share slabs: as many channel tiles as make the group fit the workgroups of one XCD, GROUP_N at most.
         */
        const int l = id - first * n_tiles;
        int group_n = slots / mt_e;
        group_n = group_n < 1 ? 1 : (group_n > GROUP_N ? GROUP_N : group_n);
        const int per_group = mt_e * group_n;
        const int ng = l / per_group;
        const int r = l - ng * per_group;
        fill_tile(t, expert, ng * group_n + r / mt_e, r % mt_e);
    };

    /*
     * DMA: this wave fills 1 KiB blocks wave + NW*j of the A tile (j < A_PARTS) and of the W tile (j < W_PARTS). An A block is
     * tile rows 8*NW*j + r0 with r0 = 8*wave + lane/8, one swizzled 16-byte chunk per lane; rows past the expert's end
     * are clamped onto its last row. 1 KiB block number b = wave + NW*j of the W tile is block b % HALF_BLOCKS of
     * the weight half b / HALF_BLOCKS, a straight copy. Addresses are a wave-uniform base plus a 32-bit lane offset.
     */
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane(lds_addr(smem) + wave * 1024);     /* this wave's block 0 of stage 0 */
    constexpr int SA_WAVES = (TM + 63) / 64;          /* waves that bring in 64 activation block scales each */
    const uint32_t lds_sa0 = __builtin_amdgcn_readfirstlane(lds_addr(lds_sa) + (wave % SA_WAVES) * 256);
    const bool sa_wave = MODE == MODE_FP8 && wave < SA_WAVES;
    const bool gs_wave = MODE == MODE_W4A8 && wave < 2;            /* wave h brings the group scales of weight half h */
    const uint32_t lds_gs0 = __builtin_amdgcn_readfirstlane(lds_addr(lds_gs) + (wave & 1) * 256);
    /*
     * The 320-row shape has no register to spare for the transfers' lane offsets across a K step: there they are worked
     * out afresh for every transfer from a copy of the lane number that the K loop makes opaque once per step (kept
     * across the loop they were spilled, and a reload waits for the slabs in flight).
     */
    int lane_dma = lane;
    /* part j of a slab: the wave's j-th block of the W tile (j < W_PARTS), of the A tile (j < A_PARTS) and, with part 0, the scales */
    auto issue_part = [&](const Tile &t, int kb, int stage, int j) __attribute__((always_inline)) {
        const int lane_x = TM > 256 ? lane_dma : lane;
        const int r0 = 8 * wave_u + (lane_x >> 3);
        const uint32_t a_chunk = ((lane_x & 7) ^ ((r0 & 7) ^ ((r0 >> 3) & 1))) * 16;
        const uint32_t w_off = wave_u * 1024 + lane_x * 16;
        const uint32_t dst = lds0 + stage * STAGE_BYTES + j * (NW * 1024);
        if (j < W_PARTS) {
            const uint8_t *wsrc = t.w_half[(NW * j) / HALF_BLOCKS] + ((int64_t)kb * W_BLOCK_BYTES + ((NW * j) % HALF_BLOCKS) * 1024);
            if (WSTREAM) dma16_sv_nt(wsrc, w_off, dst + A_BYTES);
            else dma16_sv(wsrc, w_off, dst + A_BYTES);
        }
        if (j < S::A_PARTS && (TM % (8 * NW) == 0 || 8 * NW * j + 8 * wave_u < TM)) {
            /*
             * An 8-row block past the expert's end moves 16 bytes instead of 1 KiB (one lane): the transfer still
             * counts as one operation of this wave, which keeps the outstanding-operation arithmetic the same for
             * every wave and tile. (The two-stage shapes wait for all of their transfers every step, so there a block
             * past the tile's end is simply not issued.)
             */
            const bool present = 8 * NW * j + 8 * wave_u <= t.last_rel;
            int rel = 8 * NW * j + r0;
            if (rel > t.last_rel) rel = t.last_rel;
            if ((present || lane == 0) && (present || NSTAGE != 2)) dma16_sv(t.a_base + (int64_t)kb * BKB, (uint32_t)rel * (uint32_t)K + a_chunk, dst);
        }
        if (j == 0 && sa_wave) {
            int rel = wave_u * 64 + lane_x;
            const bool in_tile = TM % 64 == 0 || rel < TM;          /* the ring holds TM scales per stage: lanes past that stay out */
            if (rel > t.last_rel) rel = t.last_rel;
            if (in_tile) dma4_sv(t.sa_base + kb, (uint32_t)rel * (uint32_t)KB * 4u, lds_sa0 + stage * TM * 4);
        }
        if (j == 0 && gs_wave)      /* 128 fp16 scales = 64 dwords, one per lane */
            dma4_sv((const float *)(t.gs_mine + (int64_t)kb * p.N), lane_x * 4u, lds_gs0 + stage * (BN * 2));
    };
    auto issue = [&](const Tile &t, int kb, int stage) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < PARTS; ++j) issue_part(t, kb, stage, j);
    };
    /* the two weight block scales of every K slab of a tile go to LDS by DMA as well: lane = K slab */
    auto issue_sw = [&](const Tile &t, int buf) __attribute__((always_inline)) {
        if (MODE != MODE_FP8) return;
        const int sw_stride = p.N / 128;
        const float *base = expert_base<float>(p.wscale, p.w_is_list, t.expert, (int64_t)KB * sw_stride);
        const int c0 = GMM1 ? t.n_tile : t.n_tile * 2, c1 = GMM1 ? I / 128 + t.n_tile : t.n_tile * 2 + 1;
        for (int b = wave_u * 64; b < KB; b += NW * 64) {
            if (b + lane < KB) {
                const uint32_t off = (uint32_t)(b + lane) * (uint32_t)sw_stride * 4u;
                const uint32_t dst = lds_addr(lds_sw) + (buf * SW_STRIDE + b) * 4;
                dma4_sv(base + c0, off, __builtin_amdgcn_readfirstlane(dst));
                dma4_sv(base + c1, off, __builtin_amdgcn_readfirstlane(dst) + D_MAX_KB * 4);
            }
        }
    };
    /*
     * W8A8: the scales a tile's epilogue needs go to LDS by DMA as well (layout: see the epilogue), into the
     * buffer of the tile's parity, which the fp8 mode uses for its weight block scales. Rows past the tile's end
     * repeat its last row. Issued where the block scales are: older than every slab that follows.
     */
    auto issue_es = [&](const Tile &t, int buf) __attribute__((always_inline)) {
        if (MODE != MODE_W8A8) return;
        const uint32_t dst0 = lds_addr(lds_sw) + buf * SW_STRIDE * 4;
        if (wave_u < (TM + 63) / 64) {
            int rel = wave_u * 64 + lane;
            if (rel > t.last_rel) rel = t.last_rel;
            dma4_sv(p.a_scale + t.row_begin, (uint32_t)rel * 4u, __builtin_amdgcn_readfirstlane(dst0 + 1024 + wave_u * 256));
        }
        if (wave_u < 4) {
            if (GMM1) {
                const float *wsb = expert_base<float>(p.wscale, p.w_is_list, t.expert, p.N);
                const float *src = wave_u < 2 ? wsb + t.n_tile * 128 + wave_u * 64 : wsb + I + t.n_tile * 128 + (wave_u - 2) * 64;
                dma4_sv(src, lane * 4u, __builtin_amdgcn_readfirstlane(dst0 + wave_u * 256));
            } else if (!p.wscale_is_bf16) {
                const float *wsb = expert_base<float>(p.wscale, p.w_is_list, t.expert, p.N);
                dma4_sv(wsb + t.n_tile * BN + wave_u * 64, lane * 4u, __builtin_amdgcn_readfirstlane(dst0 + wave_u * 256));
            } else if (wave_u < 2) {
                const uint16_t *wsb = expert_base<uint16_t>(p.wscale, p.w_is_list, t.expert, p.N);
                dma4_sv(reinterpret_cast<const float *>(wsb + t.n_tile * BN + wave_u * 128), lane * 4u,
                        __builtin_amdgcn_readfirstlane(dst0 + wave_u * 256));
            }
        }
    };
    /* this wave's vector-memory operations per slab: what may stay outstanding while an older slab is awaited */
    constexpr int OPS = W_PARTS + S::A_PARTS;
    const bool extra_op_wave = sa_wave || gs_wave;                  /* one more operation per slab: the scales */

    /* fragment reads: row lane%16 of a 16-row sub-tile, logical chunks 2*(lane/16) and 2*(lane/16)+1 */
    const int frag_row = lane & 15;
    const int key = (lane & 7) ^ ((lane >> 3) & 1), g2 = (lane >> 4) * 2;
    const int off_lo = frag_row * BKB + ((g2 ^ key) * 16), off_hi = frag_row * BKB + (((g2 + 1) ^ key) * 16);
    /* int4: one 16-byte chunk per lane, chunk lane/16 of channel lane%16 of the 16-channel block, at its swizzled slot */
    const int w4_off = frag_row * 64 + (((lane >> 4) ^ ((frag_row >> 2) & 3)) * 16);
    int w_sub[8], w_ch[8];
#pragma unroll
    for (int nt = 0; nt < 8; ++nt) {
        int r;
        if (GMM1) r = (nt < 4) ? wn * 64 + nt * 16 : 128 + wn * 64 + (nt - 4) * 16;
        else r = wn * 128 + nt * 16;
        w_sub[nt] = A_BYTES + r * WRB;
        w_ch[nt] = zb_block_row_channel(r);       /* tile-local channel held by the sub-tile's first block row */
    }
    const int lane_ch = (lane >> 4) * 8;          /* block rows 4q .. 4q+3 of a sub-tile hold channels 8q .. 8q+3 past that */

    Tile cur, nxt;
    load_tile(lid, cur);
    if (!cur.valid) return;
    int sw_buf = 0;
    issue_sw(cur, sw_buf);
    issue_es(cur, sw_buf);
#pragma unroll
    for (int s = 0; s < NSTAGE - 1; ++s) issue(cur, s, s);        /* the host guarantees KB >= NSTAGE - 1 */
    int stage = 0;
    while (true) {
        lid = next_id(lid);
        load_tile(lid, nxt);

        constexpr int MTM = S::MTM;
        f32x4 accf[MTM][8];
        i32x4 acci[MTM][8];
#pragma unroll
        for (int mt = 0; mt < MTM; ++mt)
#pragma unroll
            for (int nt = 0; nt < 8; ++nt) {
                accf[mt][nt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                acci[mt][nt] = i32x4{0, 0, 0, 0};
            }
        /*
         * The wave's 16-row sub-tiles are rows (RG*mt + wm)*16 .. +15 of the tile, mt = 0 .. MTM-1. Only the first `mt_act` of
         * them hold rows of this tile; a wave with none still moves data and meets the barriers, but skips the math.
         */
        const int tile_subs = (cur.row_end - cur.row_begin + 15) >> 4;
        int mt_act = (tile_subs - wm + RG - 1) / RG;
        mt_act = mt_act < 0 ? 0 : (mt_act > MTM ? MTM : mt_act);
        const float *sw_cur = lds_sw + sw_buf * SW_STRIDE;

        /* the K loop over the wave's first MT row sub-tiles; MT is a compile-time constant so that the loops unroll */
        auto k_loop = [&](auto mt_tag) __attribute__((always_inline)) {
        constexpr int MT = decltype(mt_tag)::value;
        for (int kb = 0; kb < KB; ++kb) {
            /* the slab after this one exists if the tile or the sequence goes on; its loads may stay in flight */
            const bool later = kb + 1 < KB || nxt.valid;
            if (NSTAGE == 3 && later) {
                if (extra_op_wave) wait_vmcnt<OPS + 1>();
                else wait_vmcnt<OPS>();
            } else {
                wait_vmcnt<0>();
            }
            __syncthreads();                /* slab kb has landed for everybody; the stage read in the step before is free */
            if constexpr (TM > 256) asm volatile("" : "+v"(lane_dma));
            /*
             * The next tile's weight block scales go into the buffer the tile before this one used. Every wave is
             * past this tile's first barrier now, so none of them still reads that buffer; the transfers are older
             * than every slab issued from here on, so the slab waits cover them.
             */
            if (kb == 0 && nxt.valid) {
                issue_sw(nxt, sw_buf ^ 1);
                issue_es(nxt, sw_buf ^ 1);
            }
            /*
             * That stage takes the slab NSTAGE-1 steps ahead, which may belong to the next tile. It is issued in parts,
             * spread over the first half of this step's MFMAs: a wave that pushes all of its loads at once sits in the
             * memory pipeline's queue while the matrix unit idles.
             */
            const bool ahead_in_tile = kb + NSTAGE - 1 < KB;
            const Tile &ft = ahead_in_tile ? cur : nxt;
            const int fill_kb = ahead_in_tile ? kb + NSTAGE - 1 : kb + NSTAGE - 1 - KB;
            const bool more = ahead_in_tile || nxt.valid;
            const int fill_stage = stage == 0 ? NSTAGE - 1 : stage - 1;
            const uint8_t *sb = smem + stage * STAGE_BYTES;
            const int cur_stage = stage;
            stage = stage + 1 == NSTAGE ? 0 : stage + 1;
            if constexpr (MT == 0) {
                if (more) issue(ft, fill_kb, fill_stage);
                continue;
            }
            auto issue_quarter = [&](int q) __attribute__((always_inline)) {
#pragma unroll
                for (int j = q * PARTS / 4; j < (q + 1) * PARTS / 4; ++j) issue_part(ft, fill_kb, fill_stage, j);
            };
            auto load_w = [&](int nt) -> i32x8 {
                const u32x4 lo = *reinterpret_cast<const u32x4 *>(sb + w_sub[nt] + off_lo);
                const u32x4 hi = *reinterpret_cast<const u32x4 *>(sb + w_sub[nt] + off_hi);
                return i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
            };

            if constexpr (MT > 0) {
                /* five row sub-tiles in the fp8 mode: two passes over the weight fragments, see below */
                constexpr bool TWO_PASS = MODE == MODE_FP8 && MT == 5;
                constexpr bool AF_PER_PASS = TWO_PASS && GMM1;
                constexpr int AFN = AF_PER_PASS ? 3 : MT;
                i32x8 af[AFN];
                i32x8 wf_first = {};
#pragma unroll
                for (int mt = 0; mt < AFN; ++mt) {
                    const uint8_t *ab = sb + ((RG * mt + wm) * 16) * BKB;
                    const u32x4 lo = *reinterpret_cast<const u32x4 *>(ab + off_lo);
                    const u32x4 hi = *reinterpret_cast<const u32x4 *>(ab + off_hi);
                    af[mt] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
                    if (mt == 0 && MODE != MODE_W4A8) {
                        /*
                         * All waves start their fragment reads together after the barrier and the LDS serves them in the
                         * order asked, so the two fragments of the first MFMA are asked for before the rest (measured,
                         * alternating with the unordered build on one GPU: 1 % of the kernel; forcing the order of all of
                         * them is slower).
                         */
                        wf_first = load_w(0);
                        asm volatile("" ::: "memory");
                    }
                }

                if constexpr (MODE == MODE_FP8) {
                    /*
                     * Software pipeline over the 8 x MT (channel sub-tile, row sub-tile) pairs: the MFMA of pair p+1 is
                     * issued before the four scale-and-accumulate FMAs of pair p, so the vector ALU works under the
                     * matrix unit.
                     */
                    const float sw0 = sw_cur[kb], sw1 = sw_cur[D_MAX_KB + kb];
                    if constexpr (MT == 5) {
                        /*
                         * Five row sub-tiles: 160 accumulators leave no room for five activation fragments beside the
                         * weight fragment fetched ahead and the block-scale products. The step goes over the eight
                         * weight fragments twice, first for row sub-tiles 0-2, then for 3-4, whose activation
                         * fragments take the registers of the first three (the weight fragments are read again: LDS
                         * reads are cheap here, registers are not). Each pass is the pipeline of the loop below.
                         */
                        auto pass = [&](auto lo_tag, auto n_tag) __attribute__((always_inline)) {
                            constexpr int M0 = decltype(lo_tag)::value, MN = decltype(n_tag)::value;
                            constexpr int A0 = AF_PER_PASS ? 0 : M0;       /* where the pass's fragments sit in af */
                            if constexpr (!AF_PER_PASS) {
                                /*
                                 * Second GEMM: a wave's channels share one weight block scale, so one product per row
                                 * sub-tile does; that leaves room for all five activation fragments from the start, and
                                 * the weight fragment is read where it is used (measured against the form below on one
                                 * GPU, 4096 tokens over 32 experts: 0.563 against 0.590 ms; the first GEMM the other way
                                 * round, 1.16 against 1.00 ms).
                                 */
                                const float swx = wn == 1 ? sw1 : sw0;
                                float sc[MN];
#pragma unroll
                                for (int m = 0; m < MN; ++m)
                                    sc[m] = lds_sa[cur_stage * TM + (RG * (M0 + m) + wm) * 16 + frag_row] * swx;
#pragma unroll
                                for (int nt = 0; nt < 8; ++nt) {
                                    const i32x8 wfj = (M0 == 0 && nt == 0) ? wf_first : load_w(nt);
                                    if (M0 == 0 && more && (nt == 0 || nt == 2)) { issue_quarter(nt); issue_quarter(nt + 1); }
                                    f32x4 part = mfma_fp8_16x16x128(wfj, af[A0]);
#pragma unroll
                                    for (int m = 0; m < MN; ++m) {
                                        f32x4 nxt_part = part;
                                        if (m + 1 < MN) nxt_part = mfma_fp8_16x16x128(wfj, af[A0 + m + 1]);
#pragma unroll
                                        for (int i = 0; i < 4; ++i) accf[M0 + m][nt][i] = __builtin_fmaf(part[i], sc[m], accf[M0 + m][nt][i]);
                                        part = nxt_part;
                                    }
                                }
                                return;
                            }
                            i32x8 wf = wf_first;
                            if (M0 != 0) {
                                asm volatile("" ::: "memory");        /* not before the first pass is through with af */
#pragma unroll
                                for (int m = 0; m < MN; ++m) {
                                    const uint8_t *ab = sb + ((RG * (M0 + m) + wm) * 16) * BKB;
                                    const u32x4 lo = *reinterpret_cast<const u32x4 *>(ab + off_lo);
                                    const u32x4 hi = *reinterpret_cast<const u32x4 *>(ab + off_hi);
                                    af[m] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
                                    if (m == 0) wf = load_w(0);
                                }
                            }
                            float s0[MN], s1[MN];
#pragma unroll
                            for (int m = 0; m < MN; ++m) {
                                const float sa = lds_sa[cur_stage * TM + (RG * (M0 + m) + wm) * 16 + frag_row];
                                s0[m] = sa * sw0;
                                s1[m] = sa * sw1;
                            }
                            f32x4 part = mfma_fp8_16x16x128(wf, af[0]);
#pragma unroll
                            for (int nt = 0; nt < 8; ++nt) {
                                i32x8 wf_n = wf;
                                if (nt + 1 < 8) wf_n = load_w(nt + 1);
                                if (M0 == 0 && more && (nt == 0 || nt == 2)) { issue_quarter(nt); issue_quarter(nt + 1); }
                                const bool second = GMM1 ? (nt >= 4) : (wn == 1);
#pragma unroll
                                for (int m = 0; m < MN; ++m) {
                                    f32x4 nxt_part = part;
                                    if (m + 1 < MN) nxt_part = mfma_fp8_16x16x128(wf, af[m + 1]);
                                    else if (nt + 1 < 8) nxt_part = mfma_fp8_16x16x128(wf_n, af[0]);
                                    const float sc = second ? s1[m] : s0[m];
#pragma unroll
                                    for (int i = 0; i < 4; ++i) accf[M0 + m][nt][i] = __builtin_fmaf(part[i], sc, accf[M0 + m][nt][i]);
                                    part = nxt_part;
                                }
                                wf = wf_n;
                            }
                        };
                        pass(std::integral_constant<int, 0>{}, std::integral_constant<int, 3>{});
                        pass(std::integral_constant<int, 3>{}, std::integral_constant<int, 2>{});
                    } else {

                        float s0[MT], s1[MT];
    #pragma unroll
                        for (int mt = 0; mt < MT; ++mt) {
                            const float sa = lds_sa[cur_stage * TM + (RG * mt + wm) * 16 + frag_row];
                            s0[mt] = sa * sw0;
                            s1[mt] = sa * sw1;
                        }
                        i32x8 wf = wf_first;
                        f32x4 part = mfma_fp8_16x16x128(wf, af[0]);
    #pragma unroll
                        for (int nt = 0; nt < 8; ++nt) {
                            i32x8 wf_n = wf;
                            if (nt + 1 < 8) wf_n = load_w(nt + 1);
                            /* the 256-row fp8 loop hands the slab out in two halves (0.6 % faster, measured against quarters on one GPU; the other loops are slower that way) */
                            if (TM == 256) {
                                if (more && (nt == 0 || nt == 2)) { issue_quarter(nt); issue_quarter(nt + 1); }
                            } else if (nt < 4 && more) {
                                issue_quarter(nt);
                            }
                            const bool second = GMM1 ? (nt >= 4) : (wn == 1);
    #pragma unroll
                            for (int mt = 0; mt < MT; ++mt) {
                                f32x4 nxt_part = part;
                                if (mt + 1 < MT) nxt_part = mfma_fp8_16x16x128(wf, af[mt + 1]);
                                else if (nt + 1 < 8) nxt_part = mfma_fp8_16x16x128(wf_n, af[0]);
                                const float sc = second ? s1[mt] : s0[mt];
    #pragma unroll
                                for (int i = 0; i < 4; ++i) accf[mt][nt][i] = __builtin_fmaf(part[i], sc, accf[mt][nt][i]);
                                part = nxt_part;
                            }
                            wf = wf_n;
                        }
                    }
                } else if constexpr (MODE == MODE_W4A8) {
                    /*
                     * The lane's 16 packed bytes are its 32 K values of this slab: dwords 0-1 unpack into the operand of
                     * the first 64-deep MFMA, dwords 2-3 into the second (times 16: the nibble moves to the top of its
                     * byte, which keeps the sign). The pair's int32 sum is promoted with the slab's group scales, and as
                     * in the fp8 mode the MFMAs of pair p+1 are issued before the conversions and FMAs of pair p.
                     */
                    const uint16_t *gsb = lds_gs + cur_stage * BN;
                    auto load_pk = [&](int nt) -> u32x4 { return *reinterpret_cast<const u32x4 *>(sb + w_sub[nt] + w4_off); };
                    auto load_gs = [&](int nt) -> u32x2 { return *reinterpret_cast<const u32x2 *>(gsb + lane_ch + w_ch[nt]); };
                    auto lo4 = [](uint32_t v) -> int { return (int)((v << 4) & 0xf0f0f0f0u); };
                    auto hi4 = [](uint32_t v) -> int { return (int)(v & 0xf0f0f0f0u); };
                    auto mfma_pair = [&](const u32x4 &pk, const i32x8 &a) -> i32x4 {
                        const i32x4 w0 = i32x4{lo4(pk[0]), hi4(pk[0]), lo4(pk[1]), hi4(pk[1])};
                        const i32x4 w1 = i32x4{lo4(pk[2]), hi4(pk[2]), lo4(pk[3]), hi4(pk[3])};
                        i32x4 part = __builtin_amdgcn_mfma_i32_16x16x64_i8(w0, i32x4{a[0], a[1], a[2], a[3]}, i32x4{0, 0, 0, 0}, 0, 0, 0);
                        return __builtin_amdgcn_mfma_i32_16x16x64_i8(w1, i32x4{a[4], a[5], a[6], a[7]}, part, 0, 0, 0);
                    };
                    /* the packed chunk and the raw fp16 scales of the next channel sub-tile are fetched one sub-tile ahead */
                    u32x4 pk = load_pk(0);
                    u32x2 gsr = load_gs(0);
                    i32x4 part = mfma_pair(pk, af[0]);
#pragma unroll
                    for (int nt = 0; nt < 8; ++nt) {
                        u32x4 pkn = pk;
                        u32x2 gsn = gsr;
                        if (nt + 1 < 8) {
                            pkn = load_pk(nt + 1);
                            gsn = load_gs(nt + 1);
                        }
                        if (nt < 4 && more) issue_quarter(nt);
                        const float gs[4] = {zb_fp16_to_f32(gsr[0] & 0xffffu), zb_fp16_to_f32(gsr[0] >> 16),
                                             zb_fp16_to_f32(gsr[1] & 0xffffu), zb_fp16_to_f32(gsr[1] >> 16)};
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt) {
                            i32x4 nxt_part = part;
                            if (mt + 1 < MT) nxt_part = mfma_pair(pk, af[mt + 1]);
                            else if (nt + 1 < 8) nxt_part = mfma_pair(pkn, af[0]);
#pragma unroll
                            for (int i = 0; i < 4; ++i) accf[mt][nt][i] = __builtin_fmaf((float)part[i], gs[i], accf[mt][nt][i]);
                            part = nxt_part;
                        }
                        pk = pkn;
                        gsr = gsn;
                    }
                } else {
                    /*
                     * int8: lane's 32 K bytes feed two 64-deep MFMAs; the two updates of one accumulator are kept apart.
                     * (Asking for the next weight fragment before the MFMAs of this one was 0.5 % slower here: the
                     * SIMD's other wave covers the read.)
                     */
#pragma unroll
                    for (int nt = 0; nt < 8; ++nt) {
                        const i32x8 wf = nt == 0 ? wf_first : load_w(nt);
                        if (nt < 4 && more) issue_quarter(nt);
                        const i32x4 wf0 = i32x4{wf[0], wf[1], wf[2], wf[3]}, wf1 = i32x4{wf[4], wf[5], wf[6], wf[7]};
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt)
                            acci[mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(
                                wf0, i32x4{af[mt][0], af[mt][1], af[mt][2], af[mt][3]}, acci[mt][nt], 0, 0, 0);
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt)
                            acci[mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(
                                wf1, i32x4{af[mt][4], af[mt][5], af[mt][6], af[mt][7]}, acci[mt][nt], 0, 0, 0);
                    }
                }
            }
        }
        };
        if (MTM >= 5 && mt_act == 5) k_loop(std::integral_constant<int, MTM >= 5 ? 5 : MTM>{});
        else if (MTM >= 4 && mt_act == 4) k_loop(std::integral_constant<int, MTM >= 4 ? 4 : MTM>{});
        else if (MTM >= 3 && mt_act == 3) k_loop(std::integral_constant<int, MTM >= 3 ? 3 : MTM>{});
        else if (MTM >= 2 && mt_act == 2) k_loop(std::integral_constant<int, MTM >= 2 ? 2 : MTM>{});
        else if (mt_act == 1) k_loop(std::integral_constant<int, 1>{});
        else k_loop(std::integral_constant<int, 0>{});
        if constexpr (MODE == MODE_W4A8) {      /* the unpacked weights were 16 x their value; a power of two divides out exactly */
#pragma unroll
            for (int mt = 0; mt < MTM; ++mt)
#pragma unroll
                for (int nt = 0; nt < 8; ++nt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) accf[mt][nt][i] *= 0.0625f;
        }
        TileCoord tc;
        tc.expert = cur.expert;
        tc.m_tile = 0;
        tc.n_tile = cur.n_tile;
        /*
         * The epilogue's lane-derived offsets are worked out afresh per tile from an opaque copy of the lane number:
         * hoisted out of the tile loop they stay live across the K loop, spill, and every reload of a spilled
         * register is a vector-memory operation whose wait also waits for the next tile's slab in flight.
         */
        int lane_e = lane;
        asm volatile("" : "+v"(lane_e));
        epilogue<MODE, GMM1, OUT_DT, RG, S::MTM>(p, tc, accf, acci, cur.row_begin, cur.row_end, wm, wn, lane_e, lds_rowmax, TM,
                                         lds_sw + sw_buf * SW_STRIDE);
        if (!nxt.valid) break;
        cur = nxt;
        sw_buf ^= 1;
    }
}

/*
 * Second pass of the int8 GMM1 epilogue: whole-row requantisation from the fp32 SwiGLU values. A row is a few KiB, so
 * one wave takes one row at a time and every lane asks for its (up to eight) 16-byte pieces of the row before it
 * converts the first. Measured on 131 072 rows of 1536 values (read 805 MB, write 201 MB): 256 threads with one piece
 * in flight per lane 200 us (5.0 TB/s), two waves with four pieces 182 us, one wave with eight 166 us (6.1 TB/s).
 */
constexpr int kRequantThreads = 64, kRequantPieces = 8;

__global__ void __launch_bounds__(kRequantThreads)
requant_rows_kernel(const float *__restrict__ sgl, const uint32_t *__restrict__ rowmax, const int32_t *__restrict__ row_off,
                    int experts, int I, int8_t *__restrict__ q2, float *__restrict__ scale2)
{
    const int total = row_off[experts];
    const int vecs = I / 4;
    for (int row = blockIdx.x; row < total; row += gridDim.x) {
        const float mx = __uint_as_float(rowmax[row]);
        const float inv = mx == 0.0f ? 0.0f : 1.0f / mx;
        if (threadIdx.x == 0) scale2[row] = mx * (1.0f / 127.0f);
        const f32x4 *src = reinterpret_cast<const f32x4 *>(sgl + (int64_t)row * I);
        uint32_t *dst = reinterpret_cast<uint32_t *>(q2 + (int64_t)row * I);
        for (int c0 = 0; c0 < vecs; c0 += kRequantThreads * kRequantPieces) {
            f32x4 v[kRequantPieces];
#pragma unroll
            for (int u = 0; u < kRequantPieces; ++u) {
                const int c = c0 + u * kRequantThreads + (int)threadIdx.x;
                v[u] = c < vecs ? __builtin_nontemporal_load(src + c) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
#pragma unroll
            for (int u = 0; u < kRequantPieces; ++u) {
                const int c = c0 + u * kRequantThreads + (int)threadIdx.x;
                uint32_t w = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) w |= ((uint32_t)zb_rint_i8((v[u][i] * 127.0f) * inv) & 0xffu) << (8 * i);
                if (c < vecs) dst[c] = w;
            }
        }
    }
}

__global__ void fill_u32_kernel(uint32_t *p, int64_t n, uint32_t v)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = v;
}

/* rows, weight blocks and channel scales move as 16-byte vectors (with tensor lists: the tables; their entries are the caller's) */
inline bool misaligned16(const void *p) { return ((uintptr_t)p & 15) != 0; }

inline unsigned grid_for(int64_t max_rows, int64_t experts, int n_tiles, int tile_m)
{
    int64_t m_tiles = (max_rows + tile_m - 1) / tile_m + experts;   /* each expert adds at most one partial tile */
    int64_t g = m_tiles * n_tiles;
    return (unsigned)((g + 7) / 8 * 8);
}

/*
 * The kernels need more dynamic LDS than the default limit: raised once per kernel instantiation and device, which
 * cannot be recorded into a graph. zbalhip_gemm_prepare does it for every instantiation ahead of time (the host layer
 * calls it when a communicator is created), so that no first launch falls into a stream capture; a launch that still
 * finds its kernel unprepared does it itself, and fails with a clear error if the stream is capturing.
 * Returns the device's CU count through n_cus.
 */
template <int MODE, bool GMM1, int OUT_DT, int TM, int NSTAGE, bool WSTREAM>
int32_t prepare_shape(hipStream_t st, int *n_cus)
{
    using S = DmaShape<TM, NSTAGE, MODE == MODE_W4A8 ? 64 : 128>;
    static std::mutex mu;          /* one per kernel instantiation: guards its per-device set-up below */
    static int cus[64] = {};
    const void *kern = reinterpret_cast<const void *>(&grouped_gemm_dma_kernel<MODE, GMM1, OUT_DT, TM, NSTAGE, WSTREAM>);
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return ZBALHIP_RT_ERROR;
    std::lock_guard<std::mutex> guard(mu);
    if (cus[dev] == 0) {
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        if (st != nullptr && hipStreamIsCapturing(st, &capture) == hipSuccess && capture != hipStreamCaptureStatusNone) {
            zbalhip_set_last_error("grouped GEMM: the first launch on a device must happen outside of a stream capture");
            return ZBALHIP_RT_ERROR;
        }
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return ZBALHIP_RT_ERROR;
        if (hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, S::LDS_BYTES) != hipSuccess)
            return ZBALHIP_RT_ERROR;
        cus[dev] = n;
    }
    *n_cus = cus[dev];
    return ZBALHIP_OK;
}

/* launched with one persistent workgroup per CU, or fewer when there are not that many tiles */
template <int MODE, bool GMM1, int OUT_DT, int TM, int NSTAGE, bool WSTREAM = false>
int32_t launch_dma_shape(const GemmParams &p, int n_tiles, hipStream_t st)
{
    using S = DmaShape<TM, NSTAGE, MODE == MODE_W4A8 ? 64 : 128>;
    int n_cus = 0;
    const int32_t rc = prepare_shape<MODE, GMM1, OUT_DT, TM, NSTAGE, WSTREAM>(st, &n_cus);
    if (rc != ZBALHIP_OK) return rc;
    unsigned grid = grid_for(p.max_rows, p.experts, n_tiles, TM);
    const unsigned resident = (unsigned)(n_cus + 7) / 8 * 8;
    if (grid > resident) grid = resident;
    grouped_gemm_dma_kernel<MODE, GMM1, OUT_DT, TM, NSTAGE, WSTREAM><<<grid, S::THREADS, S::LDS_BYTES, st>>>(p);
    return zbalhip_check_launch();
}

/* every shape a launch of (MODE, GMM1, OUT_DT) can take */
template <int MODE, bool GMM1, int OUT_DT>
int32_t prepare_mode()
{
    int n = 0;
    int32_t rc = prepare_shape<MODE, GMM1, OUT_DT, 256, 2, false>(nullptr, &n);
    if constexpr (MODE != MODE_W4A8)
        if (rc == ZBALHIP_OK) rc = prepare_shape<MODE, GMM1, OUT_DT, 320, 2, false>(nullptr, &n);
    if (rc == ZBALHIP_OK) rc = prepare_shape<MODE, GMM1, OUT_DT, 128, 3, false>(nullptr, &n);
    if constexpr (MODE != MODE_W4A8)
        if (rc == ZBALHIP_OK) rc = prepare_shape<MODE, GMM1, OUT_DT, 128, 3, true>(nullptr, &n);
    return rc;
}

/*
 * Shape choice from what the host knows (the row counts themselves live on the device). With few rows per expert the
 * GEMM is a weight-streaming job and takes the three-stage 128-row shape (which needs two K slabs to fill its
 * pipeline); with many it needs the arithmetic intensity of a two-stage shape, 320 or 256 rows high. The shapes were
 * timed against each other on 7168 x 4096 / 2048 x 7168 experts (W4A8: 4096 x 3072 / 1536 x 4096, 128 experts) with 32
 * and with 256 experts, random routing; rows per expert on average, first / second GEMM, 128-row against tall
 * (W4A8: 256-row) shape in ms:
 *   - fp8, 32 experts: 128 rows 0.247 / 0.136 against 0.256 / 0.145; 192 rows 0.298 / 0.160 against 0.278 / 0.166;
 *     256 rows 0.369 / 0.194 against 0.306 / 0.188. 256 experts: 128 rows 1.889 / 0.961 against 1.877 / 1.088;
 *     192 rows 2.314 / 1.204 against 2.108 / 1.148;
 *   - W8A8, 32 experts: 128 rows 0.243 / 0.129 against 0.254 / 0.138; 192 rows 0.289 / 0.146 against 0.275 / 0.150;
 *     256 rows 0.342 / 0.174 against 0.303 / 0.163. 256 experts: 128 rows 1.788 / 0.892 against 1.799 / 0.931;
 *     192 rows 2.197 / 1.093 against 2.016 / 1.106;
 *   - W4A8: 96 rows 0.358 / 0.171 against 0.366 / 0.178; 128 rows 0.503 / 0.237 against 0.457 / 0.216.
 */
template <int MODE, bool GMM1>
inline int64_t few_rows_limit(const GemmParams &p, int n_tiles)
{
    if (MODE == MODE_W4A8) return 96;
    if (GMM1) return 128;
    const bool few_tiles = (int64_t)p.experts * n_tiles <= 1024;
    return (MODE == MODE_FP8 && !few_tiles) ? 128 : 192;
}

/*
 * Two thirds of a two-stage tile's time does not depend on its rows (weight fragments, barrier, slab transfers), so
 * the fewer row tiles an expert has the better, and an expert whose rows just miss a multiple of 256 pays for a whole
 * tile more. The tall shape (five sub-tiles per wave; first built 288 rows high, then 320, which is the same loop and
 * 1.5 % faster even on the same tiles) cuts an expert into ceil(rows / 320) even tiles: where that is as many as
 * ceil(rows / 256) they are the same tiles as the 256-row shape's (and cost 1-4 % more in this kernel), where it is
 * fewer the expert is a tile's fixed cost shorter. Measured against the 256-row shape on 32 experts of 7168 x 4096 /
 * 2048 x 7168, random routing, first / second GEMM, rows per expert on average:
 *   - fp8: 256 rows -29 % / -15 %, 512 rows -16 % / -9 %, 1024 rows -8 % / -5 % (the 288-row build; 320 rows another
 *     -2 % / 0 %), 1500 rows 0 / +3 %, 2048 rows +2 % / +2 %, 3072 rows +2 % / +4 %, 4096 rows +2 % / +3 %: its
 *     five-sub-tile loop goes over the weight fragments twice and gives back what the saved tiles bring, hence the limit;
 *   - W8A8: 256 rows -26 % / -17 %, 1024 rows -9 % / -5 %, 1500 rows -5 % / -5 %, 2048 rows -4.5 % / -8 %, 3072 rows
 *     -3 % / -6 %, 4096 rows -5 % / -9 %: no limit;
 *   - with exactly 1024 rows for every expert fp8 +3 % / +4.6 % (the 288-row build).
 * W4A8 has no such shape (its loop has no registers for a fifth row sub-tile). The tall shape's LDS leaves room for
 * lookup tables of 512 experts; launches with more take the 256-row shape.
 */
constexpr int64_t kTallRowsLimitFp8 = 1536;

template <int MODE, bool GMM1, int OUT_DT>
int32_t launch_dma(const GemmParams &p, int n_tiles, hipStream_t st)
{
    if ((int64_t)p.max_rows <= few_rows_limit<MODE, GMM1>(p, n_tiles) * (int64_t)p.experts && p.K >= 256) {
        /*
         * With few rows per expert nearly every expert has a single row tile and its weight slabs are read once: they
         * are requested with the streaming hint. Measured on 32 experts of 7168 x 4096 / 2048 x 7168, first / second
         * GEMM: at 32 rows per expert on average fp8 11 % / 2 % and W8A8 7 % / 6 % faster (decode layer, Zipf routing:
         * 0.304 -> 0.288 ms); at 64 rows W8A8 4.5 % / 2 % faster, fp8 equal; at 96 rows W8A8 3 % / 0 % faster, fp8
         * 4 % / 1 % slower; at 128 rows, where row tiles share slabs through the L2, both 5-9 % slower. W4A8's few-row
         * kernel is bound by its unpack and promote instructions: 1-2 % with the hint at 32-96 rows, left as it is.
         */
        if constexpr (MODE != MODE_W4A8) {
            const int64_t stream_limit = MODE == MODE_W8A8 ? 96 : 32;
            if ((int64_t)p.max_rows <= stream_limit * (int64_t)p.experts) return launch_dma_shape<MODE, GMM1, OUT_DT, 128, 3, true>(p, n_tiles, st);
        }
        return launch_dma_shape<MODE, GMM1, OUT_DT, 128, 3>(p, n_tiles, st);
    }
    if constexpr (MODE != MODE_W4A8) {
        using Tall = DmaShape<320, 2, 128>;
        const bool tall_pays = MODE == MODE_W8A8 || (int64_t)p.max_rows <= kTallRowsLimitFp8 * (int64_t)p.experts;
        if (tall_pays && p.experts <= Tall::MAX_EXPERTS) return launch_dma_shape<MODE, GMM1, OUT_DT, 320, 2>(p, n_tiles, st);
    }
    return launch_dma_shape<MODE, GMM1, OUT_DT, 256, 2>(p, n_tiles, st);
}

} // namespace

extern "C" int32_t zbalhip_gmm1_swiglu_quant(const void *a, const float *a_scale, const void *w1, const void *w1scale,
                                             const int32_t *row_off, int64_t experts, int64_t max_rows, int64_t k,
                                             int64_t n1, int32_t mode, void *q2, float *scale2, float *sgl_ws,
                                             void *stream)
{
    const int w_is_list = (mode & ZBALHIP_WEIGHTS_AS_LISTS) != 0;
    const bool rowmax_cleared = (mode & ZBALHIP_ROWMAX_CLEARED) != 0;
    mode &= ~(ZBALHIP_WEIGHTS_AS_LISTS | ZBALHIP_ROWMAX_CLEARED);
    if (!a || !a_scale || !w1 || !w1scale || !row_off || !q2 || !scale2) return ZBALHIP_INVALID;
    if (mode < MODE_W8A8 || mode > MODE_W4A8) return ZBALHIP_INVALID;
    if (misaligned16(a) || misaligned16(w1) || misaligned16(w1scale) || misaligned16(q2) || misaligned16(sgl_ws)) return ZBALHIP_INVALID;
    if (experts <= 0 || experts > 1024 || max_rows < 0 || k <= 0 || k % 128 != 0 || k > 128 * 256 || n1 <= 0 || n1 % 256 != 0)
        return ZBALHIP_INVALID;
    if (max_rows == 0) return ZBALHIP_OK;
    hipStream_t st = (hipStream_t)stream;
    GemmParams p = {};
    p.a = (const uint8_t *)a; p.a_scale = a_scale; p.w = (const uint8_t *)w1; p.wscale = w1scale; p.row_off = row_off;
    p.experts = (int)experts; p.max_rows = (int)max_rows; p.K = (int)k; p.N = (int)n1;
    p.out = q2; p.out_scale = scale2; p.sgl_ws = sgl_ws; p.w_is_list = w_is_list;
    const int n_tiles = (int)(n1 / 2 / 128);
    if (mode == MODE_FP8) return launch_dma<MODE_FP8, true, ZDT_BF16>(p, n_tiles, st);
    if (!sgl_ws) return ZBALHIP_INVALID;
    /* the row maxima live behind the SwiGLU values in the same scratch allocation */
    p.rowmax = (uint32_t *)(sgl_ws + max_rows * (n1 / 2));
    if (!rowmax_cleared) fill_u32_kernel<<<(unsigned)((max_rows + 255) / 256), 256, 0, st>>>(p.rowmax, max_rows, 0u);
    if (mode == MODE_W8A8) {
        const int32_t rc = launch_dma<MODE_W8A8, true, ZDT_BF16>(p, n_tiles, st);
        if (rc != ZBALHIP_OK) return rc;
    } else {
        const int32_t rc = launch_dma<MODE_W4A8, true, ZDT_BF16>(p, n_tiles, st);
        if (rc != ZBALHIP_OK) return rc;
    }
    int64_t rb = max_rows < 16384 ? max_rows : 16384;
    requant_rows_kernel<<<(unsigned)rb, kRequantThreads, 0, st>>>(sgl_ws, p.rowmax, row_off, (int)experts, (int)(n1 / 2),
                                                    (int8_t *)q2, scale2);
    return zbalhip_check_launch();
}

extern "C" int32_t zbalhip_gmm2_dequant(const void *a, const float *a_scale, const void *w2, const void *wscale,
                                        int32_t wscale_dtype, const int32_t *row_off, int64_t experts,
                                        int64_t max_rows, int64_t k, int64_t n, int32_t mode, int32_t out_dtype,
                                        void *y, void *stream)
{
    const int w_is_list = (mode & ZBALHIP_WEIGHTS_AS_LISTS) != 0;
    mode &= ~ZBALHIP_WEIGHTS_AS_LISTS;
    if (!a || !a_scale || !w2 || !wscale || !row_off || !y) return ZBALHIP_INVALID;
    if (mode < MODE_W8A8 || mode > MODE_W4A8) return ZBALHIP_INVALID;
    if (misaligned16(a) || misaligned16(w2) || misaligned16(wscale) || misaligned16(y)) return ZBALHIP_INVALID;
    if (out_dtype != ZDT_BF16 && out_dtype != ZDT_FP16) return ZBALHIP_INVALID;
    if (experts <= 0 || experts > 1024 || max_rows < 0 || k <= 0 || k % 128 != 0 || k > 128 * 256 || n <= 0 || n % BN != 0)
        return ZBALHIP_INVALID;
    if (mode == MODE_W8A8 && wscale_dtype != ZDT_FP32 && wscale_dtype != ZDT_BF16) return ZBALHIP_INVALID;
    if (max_rows == 0) return ZBALHIP_OK;
    hipStream_t st = (hipStream_t)stream;
    GemmParams p = {};
    p.a = (const uint8_t *)a; p.a_scale = a_scale; p.w = (const uint8_t *)w2; p.wscale = wscale; p.row_off = row_off;
    p.experts = (int)experts; p.max_rows = (int)max_rows; p.K = (int)k; p.N = (int)n;
    p.wscale_is_bf16 = (wscale_dtype == ZDT_BF16);
    p.w_is_list = w_is_list;
    p.out = y;
    const int n_tiles = (int)(n / BN);
    const bool bf = out_dtype == ZDT_BF16;
    if (mode == MODE_W8A8)
        return bf ? launch_dma<MODE_W8A8, false, ZDT_BF16>(p, n_tiles, st) : launch_dma<MODE_W8A8, false, ZDT_FP16>(p, n_tiles, st);
    if (mode == MODE_FP8)
        return bf ? launch_dma<MODE_FP8, false, ZDT_BF16>(p, n_tiles, st) : launch_dma<MODE_FP8, false, ZDT_FP16>(p, n_tiles, st);
    return bf ? launch_dma<MODE_W4A8, false, ZDT_BF16>(p, n_tiles, st) : launch_dma<MODE_W4A8, false, ZDT_FP16>(p, n_tiles, st);
}

extern "C" int32_t zbalhip_gemm_prepare(void)
{
    /* once per device and process: later calls (every communicator that is created makes one) cost one device query */
    static std::atomic<bool> prepared[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return ZBALHIP_RT_ERROR;
    if (prepared[dev].load(std::memory_order_acquire)) return ZBALHIP_OK;
    int32_t rc = prepare_mode<MODE_W8A8, true, ZDT_BF16>();
    if (rc == ZBALHIP_OK) rc = prepare_mode<MODE_FP8, true, ZDT_BF16>();
    if (rc == ZBALHIP_OK) rc = prepare_mode<MODE_W4A8, true, ZDT_BF16>();
    if (rc == ZBALHIP_OK) rc = prepare_mode<MODE_W8A8, false, ZDT_BF16>();
    if (rc == ZBALHIP_OK) rc = prepare_mode<MODE_W8A8, false, ZDT_FP16>();
    if (rc == ZBALHIP_OK) rc = prepare_mode<MODE_FP8, false, ZDT_BF16>();
    if (rc == ZBALHIP_OK) rc = prepare_mode<MODE_FP8, false, ZDT_FP16>();
    if (rc == ZBALHIP_OK) rc = prepare_mode<MODE_W4A8, false, ZDT_BF16>();
    if (rc == ZBALHIP_OK) rc = prepare_mode<MODE_W4A8, false, ZDT_FP16>();
    if (rc == ZBALHIP_OK) prepared[dev].store(true, std::memory_order_release);
    return rc;
}
