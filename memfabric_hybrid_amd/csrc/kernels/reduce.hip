/*
 * N-buffer reduction: out[j] = op over p of in[p][j], the local compute under
 * reduce-scatter / all-reduce. A single pass: every lane streams one 16-byte
 * vector from each of the N inputs (N independent loads in flight), folds
 * them in buffer order (floating types in fp32) and writes one 16-byte
 * vector, so HBM traffic is (N + 1) x the slice size — the reference's
 * copy-then-atomic-accumulate scheme re-reads and re-writes the output slice
 * once per peer.
 */
#include <string.h>

#include "zbal_device.h"
#include "zbal_hip_kernels.h"

namespace {

struct ReducePtrs {
    const void *p[ZBALHIP_MAX_REDUCE_PEERS];
    unsigned long long *trace;      /* device trace ring or null */
    uint32_t trace_points;
    uint32_t trace_frame;
};

/*
 * One record into this workgroup's block of the ring (reference ZBAL_PROF_RECORD, zbal_kernel_trace.h:22-42):
 * bump the block's index word, then write the record there. Called by one lane of workgroups below
 * ZBALHIP_TRACE_UNITS; the ring is host memory, so the stores are made visible to the host with a system fence.
 */
__device__ __forceinline__ void trace_record(const ReducePtrs &in, bool end)
{
    if (in.trace == nullptr || in.trace_frame == 0 || blockIdx.x >= ZBALHIP_TRACE_UNITS || threadIdx.x != 0) return;
    unsigned long long *blk = in.trace + (uint64_t)blockIdx.x * in.trace_points;
    unsigned long long idx = blk[ZBALHIP_TRACE_IDX_OFF] + 1;
    if (idx <= ZBALHIP_TRACE_REC_OFF) idx = ZBALHIP_TRACE_REC_OFF;
    if (idx >= in.trace_points) return;
    const unsigned long long ts = (unsigned long long)wall_clock64() & ((1ull << ZBALHIP_TRACE_FRAME_SHIFT) - 1);
    blk[idx] = ((unsigned long long)in.trace_frame << ZBALHIP_TRACE_FRAME_SHIFT) | ((end ? 1ull : 0ull) << ZBALHIP_TRACE_BE_SHIFT) | ts;
    blk[ZBALHIP_TRACE_IDX_OFF] = idx;
    __threadfence_system();
}

enum { OP_PROD = 0, OP_SUM = 1, OP_MAX = 2, OP_MIN = 3 };

template <int OP, typename A> __device__ __forceinline__ A fold(A a, A b)
{
    if constexpr (OP == OP_PROD) return a * b;
    else if constexpr (OP == OP_SUM) return a + b;
    else if constexpr (OP == OP_MAX) return a > b ? a : b;
    else return a < b ? a : b;
}

/* Element traits: how many per 16 bytes, and how to unpack to / pack from the accumulation type. */
template <int DT> struct Elem;
template <> struct Elem<ZDT_FP32> { typedef float acc_t; static constexpr int per = 4; };
template <> struct Elem<ZDT_BF16> { typedef float acc_t; static constexpr int per = 8; };
template <> struct Elem<ZDT_FP16> { typedef float acc_t; static constexpr int per = 8; };
template <> struct Elem<ZDT_INT32> { typedef uint32_t acc_t; static constexpr int per = 4; };
template <> struct Elem<ZDT_INT16> { typedef int32_t acc_t; static constexpr int per = 8; };
template <> struct Elem<ZDT_INT8> { typedef int32_t acc_t; static constexpr int per = 16; };
template <> struct Elem<ZDT_INT64> { typedef int64_t acc_t; static constexpr int per = 2; };

template <int DT> __device__ __forceinline__ void unpack(const u32x4 &v, typename Elem<DT>::acc_t *o)
{
    if constexpr (DT == ZDT_FP32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = __uint_as_float(v[i]);
    } else if constexpr (DT == ZDT_BF16 || DT == ZDT_FP16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[2 * i] = zb_half_to_f32<DT>(v[i] & 0xffffu);
            o[2 * i + 1] = zb_half_to_f32<DT>(v[i] >> 16);
        }
    } else if constexpr (DT == ZDT_INT32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = v[i];
    } else if constexpr (DT == ZDT_INT16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[2 * i] = (int32_t)(int16_t)(v[i] & 0xffffu);
            o[2 * i + 1] = (int32_t)(int16_t)(v[i] >> 16);
        }
    } else if constexpr (DT == ZDT_INT8) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) o[4 * i + j] = (int32_t)(int8_t)((v[i] >> (8 * j)) & 0xffu);
    } else {
        o[0] = (int64_t)(((uint64_t)v[1] << 32) | v[0]);
        o[1] = (int64_t)(((uint64_t)v[3] << 32) | v[2]);
    }
}

template <int DT> __device__ __forceinline__ u32x4 pack(const typename Elem<DT>::acc_t *a)
{
    u32x4 v;
    if constexpr (DT == ZDT_FP32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = __float_as_uint(a[i]);
    } else if constexpr (DT == ZDT_BF16 || DT == ZDT_FP16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = zb_pack2_half<DT>(a[2 * i], a[2 * i + 1]);
    } else if constexpr (DT == ZDT_INT32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = a[i];
    } else if constexpr (DT == ZDT_INT16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = ((uint32_t)a[2 * i] & 0xffffu) | ((uint32_t)a[2 * i + 1] << 16);
    } else if constexpr (DT == ZDT_INT8) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t w = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) w |= ((uint32_t)a[4 * i + j] & 0xffu) << (8 * j);
            v[i] = w;
        }
    } else {
        v[0] = (uint32_t)(uint64_t)a[0]; v[1] = (uint32_t)((uint64_t)a[0] >> 32);
        v[2] = (uint32_t)(uint64_t)a[1]; v[3] = (uint32_t)((uint64_t)a[1] >> 32);
    }
    return v;
}

/* integer sum / product wrap modulo 2^bits; done in unsigned arithmetic */
template <int DT, int OP>
__device__ __forceinline__ typename Elem<DT>::acc_t fold_elem(typename Elem<DT>::acc_t a, typename Elem<DT>::acc_t b)
{
    typedef typename Elem<DT>::acc_t A;
    if constexpr (DT == ZDT_INT64 && (OP == OP_SUM || OP == OP_PROD)) {
        return (A)fold<OP, uint64_t>((uint64_t)a, (uint64_t)b);
    } else if constexpr (DT == ZDT_INT32 && (OP == OP_MAX || OP == OP_MIN)) {
        return (A)fold<OP, int32_t>((int32_t)a, (int32_t)b);
    } else if constexpr ((DT == ZDT_INT16 || DT == ZDT_INT8) && (OP == OP_SUM || OP == OP_PROD)) {
        /* keep intermediate values inside the element width so that wrapping matches the element type */
        const uint32_t r = fold<OP, uint32_t>((uint32_t)a, (uint32_t)b);
        return DT == ZDT_INT16 ? (A)(int16_t)r : (A)(int8_t)r;
    } else {
        return fold<OP, A>(a, b);
    }
}

template <int DT, int OP, int N>
__global__ void __launch_bounds__(256)
reduce_kernel(ReducePtrs in, int n_in, int64_t nvec, u32x4 *__restrict__ out)
{
    typedef typename Elem<DT>::acc_t A;
    constexpr int PER = Elem<DT>::per;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    trace_record(in, false);
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride) {
        u32x4 v[N];
#pragma unroll
        for (int p = 0; p < N; ++p)
            if (N != ZBALHIP_MAX_REDUCE_PEERS || p < n_in)
                v[p] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(in.p[p]) + i);
        A acc[PER], cur[PER];
        unpack<DT>(v[0], acc);
#pragma unroll
        for (int p = 1; p < N; ++p) {
            if (N != ZBALHIP_MAX_REDUCE_PEERS || p < n_in) {
                unpack<DT>(v[p], cur);
#pragma unroll
                for (int e = 0; e < PER; ++e) acc[e] = fold_elem<DT, OP>(acc[e], cur[e]);
            }
        }
        out[i] = pack<DT>(acc);      /* inputs are streamed (non-temporal loads); the plain store measured 5% faster than a non-temporal one */
    }
    trace_record(in, true);
}

/* elements past the last whole 16-byte vector */
template <int DT, int OP>
__global__ void reduce_tail_kernel(ReducePtrs in, int n_in, int64_t first, int64_t count, void *out)
{
    typedef typename Elem<DT>::acc_t A;
    constexpr int ESZ = 16 / Elem<DT>::per;
    const int64_t j = first + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= count) return;
    auto load = [&](const void *p) -> A {
        if constexpr (ESZ == 4 && DT == ZDT_FP32) return ((const float *)p)[j];
        else if constexpr (ESZ == 4) return (A)((const uint32_t *)p)[j];
        else if constexpr (ESZ == 8) return ((const int64_t *)p)[j];
        else if constexpr (DT == ZDT_INT8) return (A)((const int8_t *)p)[j];
        else if constexpr (DT == ZDT_INT16) return (A)((const int16_t *)p)[j];
        else return zb_half_to_f32<DT>(((const uint16_t *)p)[j]);
    };
    A acc = load(in.p[0]);
    for (int p = 1; p < n_in; ++p) acc = fold_elem<DT, OP>(acc, load(in.p[p]));
    if constexpr (ESZ == 4 && DT == ZDT_FP32) ((float *)out)[j] = acc;
    else if constexpr (ESZ == 4) ((uint32_t *)out)[j] = (uint32_t)acc;
    else if constexpr (ESZ == 8) ((int64_t *)out)[j] = acc;
    else if constexpr (DT == ZDT_INT8) ((int8_t *)out)[j] = (int8_t)acc;
    else if constexpr (DT == ZDT_INT16) ((int16_t *)out)[j] = (int16_t)acc;
    else ((uint16_t *)out)[j] = (uint16_t)zb_f32_to_half<DT>(acc);
}

/* element by element over [first, count): the tail of the vector path, and the whole job when the bases disagree about their alignment */
template <int DT, int OP>
void launch_scalar(const ReducePtrs &ptrs, int n_in, int64_t first, int64_t count, void *out, hipStream_t st)
{
    const int64_t n = count - first;
    if (n <= 0) return;
    if (n <= 64) reduce_tail_kernel<DT, OP><<<1, 64, 0, st>>>(ptrs, n_in, first, count, out);
    else reduce_tail_kernel<DT, OP><<<(unsigned)((n + 255) / 256), 256, 0, st>>>(ptrs, n_in, first, count, out);
}

/*
 * `head` = elements in front of the first 16-byte boundary, the same for every base (0 when they are aligned), or
 * -1 when the bases sit at different offsets from a boundary: then no vector of one lines up with a vector of the
 * others, and the job runs element by element (correct, several times slower; reduce-scatter slices of odd length are
 * the case it is for).
 */
template <int DT, int OP>
int32_t launch_reduce(ReducePtrs ptrs, int n_in, int64_t count, void *out, int head, hipStream_t st)
{
    constexpr int PER = Elem<DT>::per;
    constexpr int ESZ = 16 / PER;
    if (head < 0) {
        launch_scalar<DT, OP>(ptrs, n_in, 0, count, out, st);
        return zbalhip_check_launch();
    }
    if (head > 0) {
        if (head > count) head = (int)count;
        launch_scalar<DT, OP>(ptrs, n_in, 0, head, out, st);
        for (int p = 0; p < n_in; ++p) ptrs.p[p] = (const char *)ptrs.p[p] + (size_t)head * ESZ;
        out = (char *)out + (size_t)head * ESZ;
        count -= head;
        if (count == 0) return zbalhip_check_launch();
    }
    const int64_t nvec = count / PER;
    if (nvec > 0) {
        /* one 16-byte vector per thread: measured on MI355X, short-lived workgroups stream faster (6.2 TB/s for
           8 x 256 MiB) than a capped grid with a grid-stride loop (5.3 TB/s); the loop only serves huge counts */
        int64_t blocks = (nvec + 255) / 256;
        const int64_t cap = 1 << 22;
        if (blocks > cap) blocks = cap;
        u32x4 *o = (u32x4 *)out;
        switch (n_in) {
            case 1: reduce_kernel<DT, OP, 1><<<(unsigned)blocks, 256, 0, st>>>(ptrs, n_in, nvec, o); break;
            case 2: reduce_kernel<DT, OP, 2><<<(unsigned)blocks, 256, 0, st>>>(ptrs, n_in, nvec, o); break;
            case 4: reduce_kernel<DT, OP, 4><<<(unsigned)blocks, 256, 0, st>>>(ptrs, n_in, nvec, o); break;
            case 8: reduce_kernel<DT, OP, 8><<<(unsigned)blocks, 256, 0, st>>>(ptrs, n_in, nvec, o); break;
            default:
                reduce_kernel<DT, OP, ZBALHIP_MAX_REDUCE_PEERS><<<(unsigned)blocks, 256, 0, st>>>(ptrs, n_in, nvec, o);
        }
    }
    launch_scalar<DT, OP>(ptrs, n_in, nvec * PER, count, out, st);
    return zbalhip_check_launch();
}

template <int DT> int32_t dispatch_op(const ReducePtrs &ptrs, int n_in, int64_t count, int op, void *out, hipStream_t st)
{
    /* every base must hold whole elements; where it sits relative to a 16-byte boundary picks the path */
    constexpr int ESZ = 16 / Elem<DT>::per;
    const unsigned mis = (unsigned)((uintptr_t)out & 15u);
    if (mis % ESZ) return ZBALHIP_INVALID;
    bool same = true;
    for (int p = 0; p < n_in; ++p) {
        const unsigned m = (unsigned)((uintptr_t)ptrs.p[p] & 15u);
        if (m % ESZ) return ZBALHIP_INVALID;
        same = same && m == mis;
    }
    const int head = !same ? -1 : (mis ? (int)((16 - mis) / ESZ) : 0);
    switch (op) {
        case OP_PROD: return launch_reduce<DT, OP_PROD>(ptrs, n_in, count, out, head, st);
        case OP_SUM: return launch_reduce<DT, OP_SUM>(ptrs, n_in, count, out, head, st);
        case OP_MAX: return launch_reduce<DT, OP_MAX>(ptrs, n_in, count, out, head, st);
        case OP_MIN: return launch_reduce<DT, OP_MIN>(ptrs, n_in, count, out, head, st);
        default: return ZBALHIP_INVALID;
    }
}

} // namespace

extern "C" int32_t zbalhip_trace_alloc(int64_t points, uint64_t **host_ring, uint64_t **device_ring)
{
    if (points <= ZBALHIP_TRACE_REC_OFF || points > (1 << 24) || !host_ring || !device_ring) return ZBALHIP_INVALID;
    const size_t bytes = (size_t)points * ZBALHIP_TRACE_UNITS * sizeof(uint64_t);
    void *h = nullptr, *d = nullptr;
    if (hipHostMalloc(&h, bytes, hipHostMallocMapped) != hipSuccess) return ZBALHIP_RT_ERROR;
    memset(h, 0, bytes);
    if (hipHostGetDevicePointer(&d, h, 0) != hipSuccess) {
        (void)hipHostFree(h);
        return ZBALHIP_RT_ERROR;
    }
    *host_ring = (uint64_t *)h;
    *device_ring = (uint64_t *)d;
    return ZBALHIP_OK;
}

extern "C" int32_t zbalhip_trace_sync(void) { return hipDeviceSynchronize() == hipSuccess ? ZBALHIP_OK : ZBALHIP_RT_ERROR; }

extern "C" int32_t zbalhip_trace_free(uint64_t *host_ring)
{
    if (!host_ring) return ZBALHIP_INVALID;
    if (hipDeviceSynchronize() != hipSuccess) return ZBALHIP_RT_ERROR;
    return hipHostFree(host_ring) == hipSuccess ? ZBALHIP_OK : ZBALHIP_RT_ERROR;
}

extern "C" int32_t zbalhip_reduce(const void *const *in, int32_t n_in, int64_t count, int32_t dtype, int32_t op,
                                  void *out, int32_t trace_frame, uint64_t *trace_ring, int64_t trace_points, void *stream)
{
    if (!in || !out || n_in <= 0 || n_in > ZBALHIP_MAX_REDUCE_PEERS || count <= 0) return ZBALHIP_INVALID;
    if (trace_frame < 0 || trace_frame >= (1 << (ZBALHIP_TRACE_BE_SHIFT - ZBALHIP_TRACE_FRAME_SHIFT))) return ZBALHIP_INVALID;
    if (trace_ring != nullptr && (trace_points <= ZBALHIP_TRACE_REC_OFF || trace_points > (1 << 24))) return ZBALHIP_INVALID;
    ReducePtrs ptrs;
    for (int p = 0; p < ZBALHIP_MAX_REDUCE_PEERS; ++p) ptrs.p[p] = p < n_in ? in[p] : nullptr;
    ptrs.trace = trace_frame ? (unsigned long long *)trace_ring : nullptr;
    ptrs.trace_points = trace_ring ? (uint32_t)trace_points : 0;
    ptrs.trace_frame = (uint32_t)trace_frame;
    for (int p = 0; p < n_in; ++p)
        if (!in[p]) return ZBALHIP_INVALID;
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case ZDT_INT8: return dispatch_op<ZDT_INT8>(ptrs, n_in, count, op, out, st);
        case ZDT_INT16: return dispatch_op<ZDT_INT16>(ptrs, n_in, count, op, out, st);
        case ZDT_INT32: return dispatch_op<ZDT_INT32>(ptrs, n_in, count, op, out, st);
        case ZDT_INT64: return dispatch_op<ZDT_INT64>(ptrs, n_in, count, op, out, st);
        case ZDT_FP16: return dispatch_op<ZDT_FP16>(ptrs, n_in, count, op, out, st);
        case ZDT_BF16: return dispatch_op<ZDT_BF16>(ptrs, n_in, count, op, out, st);
        case ZDT_FP32: return dispatch_op<ZDT_FP32>(ptrs, n_in, count, op, out, st);
        default: return ZBALHIP_INVALID;
    }
}
