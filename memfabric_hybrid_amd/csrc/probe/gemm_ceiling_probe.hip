/*
 * Ceilings of the block-scaled fp8 grouped GEMM's main loop on gfx950, one piece at a time.
 *
 * The GEMM's K step is 32 MFMAs of 16x16x128 per wave, each followed by four scale-and-accumulate FMAs (the 1x128 /
 * 128x128 block scales), fed by 24 16-byte LDS fragment reads, with one barrier and one 64-KiB slab of DMA per
 * workgroup. This program runs that loop shape with the pieces switched on one after the other, on every CU
 * (one workgroup of eight waves per CU, two waves per SIMD, as the GEMM), and prints for each variant the rate and
 * the core clock the GPU sustained while it ran (core-clock ticks over constant 100-MHz ticks, read inside the
 * kernel). Operands are random e4m3 codes unless the line says zeros: the sustained clock depends on the data.
 *
 *   ./gemm_ceiling_probe            all variants
 *   ./gemm_ceiling_probe 5          one variant (for a profiler pass)
 *   ./gemm_ceiling_probe -1 128     all variants on 128 workgroups (16 of the 32 CUs of every XCD)
 *
 * The same instruction shapes with 32x32x64 MFMAs (two chained per 128-deep block, sixteen FMAs per pair) are
 * measured beside the 16x16x128 ones.
 */
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

#define CK(x)                                                                         \
    do {                                                                              \
        hipError_t e_ = (x);                                                          \
        if (e_ != hipSuccess) {                                                       \
            std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
            std::exit(1);                                                             \
        }                                                                             \
    } while (0)

namespace {

constexpr int THREADS = 512;
constexpr int STAGE = 65536;
constexpr int LDS_BYTES = 2 * STAGE + 4096;

__device__ __forceinline__ v4f mfma16(v8i a, v8i b, v4f c)
{
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}
__device__ __forceinline__ v16f mfma32(v8i a, v8i b, v16f c)
{
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}
/* tells the compiler that the operand may have changed (no instruction): identical MFMAs would otherwise be merged */
__device__ __forceinline__ void touch(v8i &a)
{
    int x = a[0];
    asm volatile("" : "+v"(x));
    a[0] = x;
}
__device__ __forceinline__ void dma16(const uint8_t *g, uint8_t *l)
{
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)g,
                                     (__attribute__((address_space(3))) void *)l, 16, 0, 0);
}

/* random e4m3 codes without the NaN patterns (0x7f / 0xff) */
__device__ __forceinline__ unsigned rnd_codes(unsigned &h)
{
    h = h * 1664525u + 1013904223u;
    return (h >> 3) & 0xF7F7F7F7u;
}

struct Clocks {
    long long core, wall;
};

enum Piece { MFMA16_CHAIN, MFMA32_CHAIN, MFMA16_PROMOTE, MFMA32_PROMOTE, MFMA16_LDS, MFMA32_LDS, LOOP16_DMA, DMA_ONLY };

/*
 * ZEROS: operands all zero. DMA_MODE (LOOP16_DMA only): 1 = every workgroup re-reads one 64-KiB slab (stays in
 * L2); N >= 2: N/2 workgroups of an XCD in a row stream the same region, slab after slab (2 = every workgroup its
 * own region: HBM bandwidth; 8 or 16 = each slab comes from HBM once and serves 4 or 8 workgroups, the sharing the
 * GEMM's schedule aims at).
 */
template <int PIECE, bool ZEROS, int DMA_MODE, int PREFETCH = 0>
__global__ void __launch_bounds__(THREADS, 2)
probe_kernel(const uint8_t *src, size_t region, float *out, int steps, float s, Clocks *clk)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    unsigned h = tid * 2654435761u + blockIdx.x * 40503u + 12345u;
    for (int i = tid; i < 2 * STAGE / 4; i += THREADS) ((unsigned *)smem)[i] = ZEROS ? 0u : rnd_codes(h);
    __syncthreads();
    const long long c0 = clock64(), w0 = wall_clock64();
    float r = 0.0f;

    if constexpr (PIECE == MFMA16_CHAIN || PIECE == MFMA16_PROMOTE) {
        v8i a, b;
        for (int i = 0; i < 8; ++i) { a[i] = ZEROS ? 0 : (int)rnd_codes(h); b[i] = ZEROS ? 0 : (int)rnd_codes(h); }
        v4f acc[32], part = {0, 0, 0, 0};
        for (int t = 0; t < 32; ++t) acc[t] = v4f{0, 0, 0, 0};
        for (int it = 0; it < steps; ++it) {
            a[it & 7] ^= 0x08080808;          /* the operands change, or the zero-C MFMAs would leave the loop */
#pragma unroll
            for (int t = 0; t < 32; ++t) {
                if (PIECE == MFMA16_CHAIN) {
                    acc[t] = mfma16(a, b, acc[t]);
                } else {               /* the MFMA of pair t is issued before the four FMAs of pair t-1 */
                    touch(a);
                    const v4f p = mfma16(a, b, v4f{0, 0, 0, 0});
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[(t + 31) & 31][j] = __builtin_fmaf(part[j], s, acc[(t + 31) & 31][j]);
                    part = p;
                }
            }
        }
        for (int t = 0; t < 32; ++t) for (int j = 0; j < 4; ++j) r += acc[t][j];
        r += part[0];
    } else if constexpr (PIECE == MFMA32_CHAIN || PIECE == MFMA32_PROMOTE) {
        v8i a, b;
        for (int i = 0; i < 8; ++i) { a[i] = ZEROS ? 0 : (int)rnd_codes(h); b[i] = ZEROS ? 0 : (int)rnd_codes(h); }
        v16f acc[8], part0, part1, zero;
        for (int t = 0; t < 8; ++t) for (int j = 0; j < 16; ++j) acc[t][j] = 0.0f;
        for (int j = 0; j < 16; ++j) { part0[j] = 0.0f; part1[j] = 0.0f; zero[j] = 0.0f; }
        for (int it = 0; it < steps; ++it) {
            a[it & 7] ^= 0x08080808;
            if (PIECE == MFMA32_CHAIN) {
#pragma unroll
                for (int t = 0; t < 8; ++t) acc[t] = mfma32(a, b, acc[t]);
#pragma unroll
                for (int t = 0; t < 8; ++t) acc[t] = mfma32(b, a, acc[t]);
            } else {
                /*
                 * Two chained 64-deep MFMAs make one 128-deep block; two tiles are in flight so that no MFMA waits
                 * for the one it depends on, and the sixteen FMAs of each earlier tile sit between them.
                 */
#pragma unroll
                for (int t = 0; t < 8; t += 2) {
                    const int u0 = (t + 6) & 7, u1 = (t + 7) & 7;
                    touch(a);
                    v16f q0 = mfma32(a, b, zero);
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc[u0][j] = __builtin_fmaf(part0[j], s, acc[u0][j]);
                    touch(a);
                    v16f q1 = mfma32(a, b, zero);
#pragma unroll
                    for (int j = 8; j < 16; ++j) acc[u0][j] = __builtin_fmaf(part0[j], s, acc[u0][j]);
                    q0 = mfma32(b, a, q0);
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc[u1][j] = __builtin_fmaf(part1[j], s, acc[u1][j]);
                    q1 = mfma32(b, a, q1);
#pragma unroll
                    for (int j = 8; j < 16; ++j) acc[u1][j] = __builtin_fmaf(part1[j], s, acc[u1][j]);
                    part0 = q0;
                    part1 = q1;
                }
            }
        }
        for (int t = 0; t < 8; ++t) for (int j = 0; j < 16; ++j) r += acc[t][j];
        r += part0[0] + part1[0];
    } else if constexpr (PIECE == MFMA32_LDS) {
        /* 64 x 128 wave tile as 2 x 4 tiles of 32 x 32: six fragments of 2 KiB per 64-deep half, 24 b128 per step */
        v16f acc[2][4], part0, part1, zero;
        for (int m = 0; m < 2; ++m) for (int n = 0; n < 4; ++n) for (int j = 0; j < 16; ++j) acc[m][n][j] = 0.0f;
        for (int j = 0; j < 16; ++j) { part0[j] = 0.0f; part1[j] = 0.0f; zero[j] = 0.0f; }
        const int row = lane & 31, kh = lane >> 5;
        const int key = (row & 7) ^ ((row >> 3) & 1);
        auto ld = [&](const uint8_t *p, int half) -> v8i {     /* 32 K-bytes of row `row`: chunks 2*(2*half+kh), +1 */
            const int c = 2 * (2 * half + kh);
            const v4u lo = *reinterpret_cast<const v4u *>(p + row * 128 + ((c ^ key) * 16));
            const v4u hi = *reinterpret_cast<const v4u *>(p + row * 128 + (((c + 1) ^ key) * 16));
            return v8i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
        };
        for (int it = 0; it < steps; ++it) {
            const uint8_t *sb = smem + (it & 1) * STAGE;
            __syncthreads();
            v8i af[2][2];
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int hf = 0; hf < 2; ++hf) af[m][hf] = ld(sb + (wm * 64 + m * 32) * 128, hf);
#pragma unroll
            for (int n = 0; n < 4; ++n) {
                const v8i w0 = ld(sb + 32768 + (wn * 128 + n * 32) * 128, 0);
                const v8i w1 = ld(sb + 32768 + (wn * 128 + n * 32) * 128, 1);
                const int pn = (n + 3) & 3;            /* the pair of tiles whose partial sums are promoted meanwhile */
                v16f q0 = mfma32(w0, af[0][0], zero);
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[0][pn][j] = __builtin_fmaf(part0[j], s, acc[0][pn][j]);
                v16f q1 = mfma32(w0, af[1][0], zero);
#pragma unroll
                for (int j = 8; j < 16; ++j) acc[0][pn][j] = __builtin_fmaf(part0[j], s, acc[0][pn][j]);
                q0 = mfma32(w1, af[0][1], q0);
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[1][pn][j] = __builtin_fmaf(part1[j], s, acc[1][pn][j]);
                q1 = mfma32(w1, af[1][1], q1);
#pragma unroll
                for (int j = 8; j < 16; ++j) acc[1][pn][j] = __builtin_fmaf(part1[j], s, acc[1][pn][j]);
                part0 = q0;
                part1 = q1;
            }
        }
        for (int m = 0; m < 2; ++m) for (int n = 0; n < 4; ++n) for (int j = 0; j < 16; ++j) r += acc[m][n][j];
        r += part0[0] + part1[0];
    } else {
        /* MFMA16_LDS and LOOP16_DMA: the GEMM's step. 64 x 128 wave tile as 4 x 8 tiles of 16 x 16 */
        constexpr bool DMA = PIECE == LOOP16_DMA || PIECE == DMA_ONLY;
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        const uint8_t *base = src + (DMA_MODE >= 2 ? (size_t)(xcd + 8 * (slot / (DMA_MODE / 2))) * region : (size_t)xcd * STAGE);
        const size_t kwrap = DMA_MODE >= 2 ? region / STAGE : 1;
        auto issue_part = [&](int kb, int stage, int q) {      /* a quarter of the slab: two 1-KiB blocks of this wave */
            const uint8_t *g = base + (size_t)(kb % kwrap) * STAGE;
#pragma unroll
            for (int i = 2 * q; i < 2 * q + 2; ++i) dma16(g + (wave + 8 * i) * 1024 + lane * 16, smem + stage * STAGE + (wave + 8 * i) * 1024);
        };
        v4f acc[4][8];
        for (int m = 0; m < 4; ++m) for (int n = 0; n < 8; ++n) acc[m][n] = v4f{0, 0, 0, 0};
        const int frag_row = lane & 15, key = (lane & 7) ^ ((lane >> 3) & 1), g2 = (lane >> 4) * 2;
        const int off_lo = frag_row * 128 + ((g2 ^ key) * 16), off_hi = frag_row * 128 + (((g2 + 1) ^ key) * 16);
        auto ld = [&](const uint8_t *p) -> v8i {
            const v4u lo = *reinterpret_cast<const v4u *>(p + off_lo);
            const v4u hi = *reinterpret_cast<const v4u *>(p + off_hi);
            return v8i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
        };
        if (DMA) { for (int q = 0; q < 4; ++q) issue_part(0, 0, q); }
        int dump = 0;
        for (int kb = 0; kb < steps; ++kb) {
            const int stage = kb & 1;
            if (DMA) __builtin_amdgcn_s_waitcnt(0x0F70);
            asm volatile("" : : "v"(dump));          /* the touch load of the step before has written its register by now */
            __syncthreads();
            if (PREFETCH >= 10 && kb + PREFETCH - 10 < steps) {
                /* the sharers of a slab split its 512 lines: this workgroup touches its share, PREFETCH - 10 steps ahead */
                constexpr int SH = DMA_MODE >= 2 ? DMA_MODE / 2 : 1, MINE = 512 / SH;   /* lines per workgroup */
                const int me = slot % SH;
                if (wave * 64 < MINE && lane < MINE) {
                    const uint8_t *g = base + (size_t)((kb + PREFETCH - 10) % kwrap) * STAGE + (me * MINE + wave * 64 + lane) * 128;
                    asm volatile("global_load_dword %0, %1, off" : "=v"(dump) : "v"(g) : "memory");
                }
            } else if (PREFETCH > 0 && kb + PREFETCH < steps) {
                /* one dword of each 128-byte line of the slab PREFETCH steps ahead: 512 lines, 64 per wave */
                const uint8_t *g = base + (size_t)((kb + PREFETCH) % kwrap) * STAGE + (wave * 64 + lane) * 128;
                asm volatile("global_load_dword %0, %1, off" : "=v"(dump) : "v"(g) : "memory");
            }
            const uint8_t *sb = smem + stage * STAGE;
            if (PIECE == DMA_ONLY) {              /* no arithmetic: what the slab transfers alone take */
                if (kb + 1 < steps) for (int q = 0; q < 4; ++q) issue_part(kb + 1, stage ^ 1, q);
                continue;
            }
            v8i af[4];
#pragma unroll
            for (int mt = 0; mt < 4; ++mt) af[mt] = ld(sb + ((4 * mt + wm) * 16) * 128);
            v8i wf = ld(sb + 32768 + (wn * 128) * 128);
            v4f part = mfma16(wf, af[0], v4f{0, 0, 0, 0});
#pragma unroll
            for (int nt = 0; nt < 8; ++nt) {
                v8i wf_n = wf;
                if (nt + 1 < 8) wf_n = ld(sb + 32768 + (wn * 128 + (nt + 1) * 16) * 128);
                if (DMA && kb + 1 < steps) {
                    if (PREFETCH == -1) { if (nt == 0) for (int q = 0; q < 4; ++q) issue_part(kb + 1, stage ^ 1, q); }
                    else if (PREFETCH == -2) { if (nt < 2) for (int q = 2 * nt; q < 2 * nt + 2; ++q) issue_part(kb + 1, stage ^ 1, q); }
                    else if (nt < 4) issue_part(kb + 1, stage ^ 1, nt);
                }
#pragma unroll
                for (int mt = 0; mt < 4; ++mt) {
                    v4f nxt = part;
                    if (mt < 3) nxt = mfma16(wf, af[mt + 1], v4f{0, 0, 0, 0});
                    else if (nt + 1 < 8) nxt = mfma16(wf_n, af[0], v4f{0, 0, 0, 0});
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[mt][nt][i] = __builtin_fmaf(part[i], s, acc[mt][nt][i]);
                    part = nxt;
                }
                wf = wf_n;
            }
        }
        for (int m = 0; m < 4; ++m) for (int n = 0; n < 8; ++n) for (int i = 0; i < 4; ++i) r += acc[m][n][i];
    }
    out[(size_t)blockIdx.x * THREADS + tid] = r;
    if (tid == 0 && blockIdx.x == 17) {
        clk->core = clock64() - c0;
        clk->wall = wall_clock64() - w0;
    }
}

struct Variant {
    const char *name;
    void (*launch)(const uint8_t *, size_t, float *, int, Clocks *, int);
    int steps;
    int slabs;        /* slabs per streamed region (0: the default, one tile's worth) */
};

template <int PIECE, bool ZEROS, int DMA_MODE, int PREFETCH = 0>
void launch(const uint8_t *src, size_t region, float *out, int steps, Clocks *clk, int blocks)
{
    auto fn = probe_kernel<PIECE, ZEROS, DMA_MODE, PREFETCH>;
    static bool set = false;
    if (!set) { CK(hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES)); set = true; }
    hipLaunchKernelGGL(fn, dim3(blocks), dim3(THREADS), LDS_BYTES, 0, src, region, out, steps, 1.0001f, clk);
}

} // namespace

int main(int argc, char **argv)
{
    const int only = argc > 1 ? std::atoi(argv[1]) : -1;
    int dev = 0, cus = 0;
    CK(hipGetDevice(&dev));
    CK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int blocks = argc > 2 ? std::atoi(argv[2]) : cus;       /* fewer workgroups than CUs: what a shared resource costs */
    const size_t region = (size_t)56 * STAGE;                 /* one tile's worth of slabs per workgroup */
    uint8_t *src;
    CK(hipMalloc(&src, region * blocks));
    {
        std::vector<uint32_t> hbuf(region * blocks / 4);
        uint32_t h = 99;
        for (auto &v : hbuf) { h = h * 1664525u + 1013904223u; v = (h >> 3) & 0xF7F7F7F7u; }
        CK(hipMemcpy(src, hbuf.data(), region * blocks, hipMemcpyHostToDevice));
    }
    float *out;
    CK(hipMalloc(&out, (size_t)blocks * THREADS * 4));
    Clocks *clk;
    CK(hipHostMalloc(&clk, sizeof(Clocks)));

    const Variant variants[] = {
        {"0 mfma 16x16x128 chain, zeros", launch<MFMA16_CHAIN, true, 0>, 2000},
        {"1 mfma 16x16x128 chain", launch<MFMA16_CHAIN, false, 0>, 2000},
        {"2 mfma 32x32x64 chain", launch<MFMA32_CHAIN, false, 0>, 2000},
        {"3 mfma 16x16x128 + 4 fma (block scales)", launch<MFMA16_PROMOTE, false, 0>, 2000},
        {"4 2 x mfma 32x32x64 + 16 fma", launch<MFMA32_PROMOTE, false, 0>, 2000},
        {"5 as 3 + lds fragments + barrier", launch<MFMA16_LDS, false, 0>, 2000},
        {"6 as 4 + lds fragments + barrier", launch<MFMA32_LDS, false, 0>, 2000},
        {"7 as 5 + dma of an L2-resident slab", launch<LOOP16_DMA, false, 1>, 2000},
        {"8 as 5 + dma streaming from HBM", launch<LOOP16_DMA, false, 2>, 56 * 8},
        {"9 as 5, zeros", launch<MFMA16_LDS, true, 0>, 2000},
        {"10 as 5 + dma from HBM, 4 workgroups a slab", launch<LOOP16_DMA, false, 8>, 56 * 8},
        {"11 as 5 + dma from HBM, 8 workgroups a slab", launch<LOOP16_DMA, false, 16>, 56 * 8},
        {"12 as 10 + line touches 2 steps ahead", launch<LOOP16_DMA, false, 8, 2>, 56 * 8},
        {"13 as 10 + line touches 3 steps ahead", launch<LOOP16_DMA, false, 8, 3>, 56 * 8},
        {"14 as 10 + line touches 5 steps ahead", launch<LOOP16_DMA, false, 8, 5>, 56 * 8},
        {"15 as 8 + line touches 3 steps ahead", launch<LOOP16_DMA, false, 2, 3>, 56 * 8},
        {"19 as 10 + each sharer touches 1/4, 2 ahead", launch<LOOP16_DMA, false, 8, 12>, 56 * 8},
        {"20 as 10 + each sharer touches 1/4, 3 ahead", launch<LOOP16_DMA, false, 8, 13>, 56 * 8},
        {"21 as 11 + each sharer touches 1/8, 2 ahead", launch<LOOP16_DMA, false, 16, 12>, 56 * 8},
        {"22 as 11 + each sharer touches 1/8, 4 ahead", launch<LOOP16_DMA, false, 16, 14>, 56 * 8},
        {"23 as 10, regions of 2 slabs (1 MiB an XCD)", launch<LOOP16_DMA, false, 8>, 2000, 2},
        {"25 as 10, regions of 4 slabs (2 MiB an XCD)", launch<LOOP16_DMA, false, 8>, 2000, 4},
        {"26 as 11, regions of 4 slabs (1 MiB an XCD)", launch<LOOP16_DMA, false, 16>, 2000, 4},
        {"24 as 10, regions of 32 slabs (L2 + MALL)", launch<LOOP16_DMA, false, 8>, 2000, 32},
        {"27 dma alone, the same slab again and again", launch<DMA_ONLY, false, 1>, 2000},
        {"28 dma alone, L2-resident regions of 4 slabs", launch<DMA_ONLY, false, 8>, 2000, 4},
        {"29 dma alone, from HBM, 4 workgroups a slab", launch<DMA_ONLY, false, 8>, 56 * 8},
        {"30 dma alone, from HBM, every workgroup own", launch<DMA_ONLY, false, 2>, 56 * 8},
        {"31 as 25, whole slab issued at once", launch<LOOP16_DMA, false, 8, -1>, 2000, 4},
        {"32 as 25, slab issued in two halves", launch<LOOP16_DMA, false, 8, -2>, 2000, 4},
        {"16 as 10, whole slab issued at once", launch<LOOP16_DMA, false, 8, -1>, 56 * 8},
        {"17 as 10, slab issued in two halves", launch<LOOP16_DMA, false, 8, -2>, 56 * 8},
        {"18 as 7, whole slab issued at once", launch<LOOP16_DMA, false, 1, -1>, 2000},
    };
    std::printf("%d CUs, one workgroup of 8 waves each; a step = 32 MFMA-equivalents of 65536 FLOP per wave\n", cus);
    std::printf("%-44s %9s %10s %9s %12s\n", "variant", "ms", "PFLOP/s", "clock GHz", "ns per step");
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    int idx = 0;
    for (const Variant &v : variants) {
        if (only >= 0 && only != idx++) continue;
        float ms = 0.0f;
        for (int rep = 0; rep < 3; ++rep) {       /* the last of three runs is reported */
            CK(hipEventRecord(e0));
            v.launch(src, v.slabs ? (size_t)v.slabs * STAGE : region, out, v.steps, clk, blocks);
            CK(hipEventRecord(e1));
            CK(hipEventSynchronize(e1));
            CK(hipEventElapsedTime(&ms, e0, e1));
        }
        const double flop = 2.0 * 16 * 16 * 128 * 32.0 * v.steps * (THREADS / 64) * blocks;
        std::printf("%-44s %9.3f %10.3f %9.3f %12.1f\n", v.name, ms, flop / ms / 1e12, clk->core / (clk->wall * 10.0),
                    ms * 1e6 / v.steps);
    }
    CK(hipFree(src));
    CK(hipFree(out));
    return 0;
}
