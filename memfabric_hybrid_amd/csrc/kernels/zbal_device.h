/*
 * Device-side helpers shared by the gfx950 kernels: scalar format
 * conversions, the fixed expf used by the SwiGLU epilogue, wave64 reductions
 * and the launch-error plumbing of the C ABI.
 *
 * The kernels are compiled with -ffp-contract=off: a product followed by a
 * sum rounds twice unless written as __builtin_fmaf().
 */
#ifndef ZBAL_DEVICE_H_
#define ZBAL_DEVICE_H_

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#define ZBALHIP_OK 0
#define ZBALHIP_INVALID (-2)
#define ZBALHIP_RT_ERROR (-11)

/* zbal_datatype_t values used by the kernels */
#define ZDT_INT8 0
#define ZDT_INT16 1
#define ZDT_INT32 2
#define ZDT_INT64 3
#define ZDT_FP16 6
#define ZDT_FP32 7
#define ZDT_BF16 8

#define ZBAL_WAVE 64

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
typedef int32_t i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

/* thread-local last-error text of the library (zbal_get_last_error_msg), for launchers that refuse a call */
void zbalhip_set_last_error(const char *text);

static inline int32_t zbalhip_check_launch()
{
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? ZBALHIP_OK : ZBALHIP_RT_ERROR;
}

/* ---- scalar formats ------------------------------------------------------ */

__device__ __forceinline__ float zb_bf16_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

/* two floats -> two bf16 in one dword: v_cvt_pk_bf16_f32, round to nearest even, NaN stays a quiet NaN */
__device__ __forceinline__ uint32_t zb_pack2_bf16(float lo, float hi)
{
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}

__device__ __forceinline__ uint32_t zb_f32_to_bf16(float f) { return zb_pack2_bf16(f, 0.0f) & 0xffffu; }

__device__ __forceinline__ float zb_fp16_to_f32(uint32_t h)
{
    _Float16 v;
    uint16_t s = (uint16_t)h;
    __builtin_memcpy(&v, &s, 2);
    return (float)v;
}

__device__ __forceinline__ uint32_t zb_f32_to_fp16(float f)
{
    /*
     * The empty asm keeps the compiler from folding a preceding fp32 multiply into v_fma_mixlo_f16, which
     * rounds the exact product straight to fp16; the result must be the fp32-rounded product rounded again.
     */
    asm volatile("" : "+v"(f));
    _Float16 v = (_Float16)f; /* v_cvt_f16_f32: round to nearest even */
    uint16_t s;
    __builtin_memcpy(&s, &v, 2);
    return s;
}

template <int DT> __device__ __forceinline__ float zb_half_to_f32(uint32_t h)
{
    if constexpr (DT == ZDT_FP16) return zb_fp16_to_f32(h);
    else return zb_bf16_to_f32(h);
}

template <int DT> __device__ __forceinline__ uint32_t zb_f32_to_half(float f)
{
    if constexpr (DT == ZDT_FP16) return zb_f32_to_fp16(f);
    else return zb_f32_to_bf16(f);
}

/* two values rounded to DT, `lo` in the low half of the dword */
template <int DT> __device__ __forceinline__ uint32_t zb_pack2_half(float lo, float hi)
{
    if constexpr (DT == ZDT_FP16) return zb_f32_to_fp16(lo) | (zb_f32_to_fp16(hi) << 16);
    else return zb_pack2_bf16(lo, hi);
}

/* two floats -> two e4m3 codes in the low 16 bits (v_cvt_pk_fp8_f32, OCP format on gfx950); inputs pre-clamped */
__device__ __forceinline__ uint32_t zb_cvt_pk_e4m3(float a, float b)
{
    a = fminf(fmaxf(a, -448.0f), 448.0f);
    b = fminf(fmaxf(b, -448.0f), 448.0f);
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xffffu;
}

/* round-half-even to int, clamped to int8 */
__device__ __forceinline__ int32_t zb_rint_i8(float v)
{
    float r = __builtin_rintf(v);
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    return (int32_t)r;
}

/*
 * exp() of the SwiGLU epilogue: Cody-Waite reduction by ln2, a degree-6
 * polynomial in fmaf form and scaling by two exact powers of two. The same
 * operation sequence is what the CPU checker evaluates, so both sides agree
 * bit for bit (the hardware v_exp_f32 is an approximation and would not).
 */
__device__ __forceinline__ float zb_expf(float x)
{
    if (!(x == x)) return x;
    if (x > 88.72284f) return __builtin_inff();
    if (x < -103.97208f) return 0.0f;
    float n = __builtin_rintf(x * 1.44269504088896341f);
    float r = __builtin_fmaf(n, -0.693145751953125f, x);
    r = __builtin_fmaf(n, -1.42860682030941723e-06f, r);
    float p = 1.3888889e-03f;
    p = __builtin_fmaf(p, r, 8.3333333e-03f);
    p = __builtin_fmaf(p, r, 4.1666668e-02f);
    p = __builtin_fmaf(p, r, 1.6666667e-01f);
    p = __builtin_fmaf(p, r, 0.5f);
    p = __builtin_fmaf(p, r, 1.0f);
    p = __builtin_fmaf(p, r, 1.0f);
    int ni = (int)n;
    int n1 = ni / 2, n2 = ni - n1;
    float s1 = __uint_as_float((uint32_t)(n1 + 127) << 23);
    float s2 = __uint_as_float((uint32_t)(n2 + 127) << 23);
    return (p * s1) * s2;
}

/* ---- wave64 reductions ------------------------------------------------------ */

__device__ __forceinline__ float zb_wave_max(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, ZBAL_WAVE));
    return v;
}

/*
 * Wave-wide reductions on the data-parallel-primitive path (no LDS round trips: six dependent vector instructions
 * instead of six ds_bpermute latencies). Lanes swap within quads, mirror within 8 and 16, then rows 1 and 3 take
 * the totals of rows 0 and 2 and the upper half takes lane 31's; lane 63 ends with the result, which is broadcast.
 */
template <bool IS_MAX> __device__ __forceinline__ float zb_wave_reduce_dpp(float x)
{
    const int ident = IS_MAX ? (int)0xff800000u : 0;       /* -inf or +0 for the lanes a step does not write */
    auto step = [&](auto ctrl_tag, auto mask_tag) __attribute__((always_inline)) {
        constexpr int CTRL = decltype(ctrl_tag)::value, MASK = decltype(mask_tag)::value;
        const float o = __int_as_float(__builtin_amdgcn_update_dpp(ident, __float_as_int(x), CTRL, MASK, 0xf, false));
        x = IS_MAX ? fmaxf(x, o) : x + o;
    };
    step(std::integral_constant<int, 0xB1>{}, std::integral_constant<int, 0xf>{});     /* quad_perm [1,0,3,2] */
    step(std::integral_constant<int, 0x4E>{}, std::integral_constant<int, 0xf>{});     /* quad_perm [2,3,0,1] */
    step(std::integral_constant<int, 0x141>{}, std::integral_constant<int, 0xf>{});    /* row_half_mirror */
    step(std::integral_constant<int, 0x140>{}, std::integral_constant<int, 0xf>{});    /* row_mirror */
    step(std::integral_constant<int, 0x142>{}, std::integral_constant<int, 0xa>{});    /* row_bcast:15 into rows 1 and 3 */
    step(std::integral_constant<int, 0x143>{}, std::integral_constant<int, 0xc>{});    /* row_bcast:31 into rows 2 and 3 */
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), 63));
}

/* max over groups of 2^LOG2 consecutive lanes */
template <int LOG2> __device__ __forceinline__ float zb_group_max(float v)
{
#pragma unroll
    for (int off = (1 << LOG2) >> 1; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, ZBAL_WAVE));
    return v;
}

/* block-wide max through LDS; `red` holds one float per wave; all threads receive the result */
__device__ __forceinline__ float zb_block_max(float v, float *red)
{
    v = zb_wave_max(v);
    const int lane = threadIdx.x & (ZBAL_WAVE - 1), wave = threadIdx.x / ZBAL_WAVE;
    const int nwaves = (blockDim.x + ZBAL_WAVE - 1) / ZBAL_WAVE;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float r = red[0];
    for (int i = 1; i < nwaves; ++i) r = fmaxf(r, red[i]);
    return r;
}

/*
 * Pre-packed weight blocks: which channel of a 128-channel block sits in block row r. Rows 16t .. 16t+15 feed one
 * MFMA of the grouped GEMM and rows 4q .. 4q+3 of it come out in the lanes 16q .. 16q+15; the permutation (within
 * groups of 32 rows) gives those lanes channels 8q .. 8q+3 of the group from the even operand t and 8q+4 .. 8q+7
 * from the odd one, eight consecutive channels per lane.
 */
__host__ __device__ __forceinline__ constexpr int zb_block_row_channel(int r)
{
    return (r & ~31) | (((r & 15) >> 2) << 3) | (((r >> 4) & 1) << 2) | (r & 3);
}

#endif /* ZBAL_DEVICE_H_ */
