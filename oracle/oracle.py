"""TEST INFRASTRUCTURE: numpy-facing wrapper of the CPU oracle (oracle/zbal_oracle.cpp).

Only tests, the smoke test and the benchmark's cpu_baseline leg import this
module; the shipped package never does. bf16 / fp16 values travel as uint16
bit patterns, e4m3 values as uint8 codes.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# ZBAL_ORACLE_LIB: another build of the same source (the sanitizer build, `make -C oracle asan`)
_LIB_PATH = os.environ.get("ZBAL_ORACLE_LIB") or os.path.join(_HERE, "_build", "libzbal_oracle.so")

DT_INT8, DT_INT16, DT_INT32, DT_INT64 = 0, 1, 2, 3
DT_FP16, DT_FP32, DT_BF16 = 6, 7, 8


def build(force=False):
    """Compile the oracle with its Makefile (gcc only; no GPU toolchain involved)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.zo_num_threads.restype = ctypes.c_int32
        _lib.zo_reduce.restype = ctypes.c_int32
    return _lib


def _p(a):
    if a is None:
        return ctypes.c_void_p(0)
    assert isinstance(a, np.ndarray) and a.flags["C_CONTIGUOUS"], "oracle operands must be C-contiguous numpy arrays"
    return ctypes.c_void_p(a.ctypes.data)


def _i64(v):
    return ctypes.c_int64(int(v))


def _i32(v):
    return ctypes.c_int32(int(v))


def num_threads():
    return int(lib().zo_num_threads())


def set_num_threads(n):
    lib().zo_set_num_threads(_i32(n))


# ---- scalar formats -------------------------------------------------------

def _conv(fn, src, src_dt, dst_dt):
    src = np.ascontiguousarray(src, dtype=src_dt)
    dst = np.empty(src.shape, dtype=dst_dt)
    getattr(lib(), fn)(_p(src), _p(dst), _i64(src.size))
    return dst


def f32_to_bf16(a):
    return _conv("zo_f32_to_bf16", a, np.float32, np.uint16)


def bf16_to_f32(a):
    return _conv("zo_bf16_to_f32", a, np.uint16, np.float32)


def f32_to_fp16(a):
    return _conv("zo_f32_to_fp16", a, np.float32, np.uint16)


def fp16_to_f32(a):
    return _conv("zo_fp16_to_f32", a, np.uint16, np.float32)


def f32_to_e4m3(a):
    return _conv("zo_f32_to_e4m3", a, np.float32, np.uint8)


def e4m3_to_f32(a):
    return _conv("zo_e4m3_to_f32", a, np.uint8, np.float32)


def expf(a):
    return _conv("zo_expf", a, np.float32, np.float32)


# ---- operators ------------------------------------------------------------

def topk_route(logits, K):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    T, E = logits.shape
    idx = np.empty((T, K), dtype=np.int64)
    w = np.empty((T, K), dtype=np.float32)
    lib().zo_topk_route(_p(logits), _i64(T), _i64(E), _i64(K), _p(idx), _p(w))
    return idx, w


def dispatch_layout(topk_idx, E, R=1):
    topk_idx = np.ascontiguousarray(topk_idx, dtype=np.int64)
    T, K = topk_idx.shape
    per_rank = np.zeros(R, dtype=np.int32)
    per_expert = np.zeros(E, dtype=np.int32)
    send_idx = np.zeros((T, K), dtype=np.int32)
    lib().zo_dispatch_layout(_p(topk_idx), _i64(T), _i64(K), _i64(E), _i64(R), _p(per_rank), _p(per_expert),
                             _p(send_idx))
    return per_rank, per_expert, send_idx


def dispatch_notify(counts_all, K, me=0):
    counts_all = np.ascontiguousarray(counts_all, dtype=np.int32)
    R, E = counts_all.shape
    recv = np.empty((R, E), dtype=np.int32)
    put = np.empty((R, E), dtype=np.int32)
    total = np.zeros(1, dtype=np.int32)
    per_exp = np.zeros(E // R, dtype=np.int64)
    bal = np.empty((R, 2 * R), dtype=np.int32)
    lib().zo_dispatch_notify(_p(counts_all), _i64(R), _i64(E), _i64(K), _i64(me), _p(recv), _p(put), _p(total),
                             _p(per_exp), _p(bal))
    return recv, put, total, per_exp, bal


def dispatch_normal(x, x_dtype, topk_idx32, send_idx, put_offset, E, quant_mode, rows, R=1, me=0):
    """x: uint16 [T,H]. Returns (dest, dest_scale); rows never written stay zero."""
    T, H = x.shape
    K = topk_idx32.shape[1]
    if quant_mode == 0:
        dest = np.zeros((rows, H), dtype=np.uint16)
        scale = None
    elif quant_mode == 1:
        dest = np.zeros((rows, H), dtype=np.int8)
        scale = np.zeros(rows, dtype=np.float32)
    else:
        dest = np.zeros((rows, H), dtype=np.uint8)
        scale = np.zeros((rows, H // 128), dtype=np.float32)
    lib().zo_dispatch_normal(_p(x), _i32(x_dtype), _p(np.ascontiguousarray(topk_idx32, dtype=np.int32)),
                             _p(send_idx), _p(put_offset), _i64(T), _i64(H), _i64(K), _i64(E), _i64(R), _i64(me),
                             _i32(quant_mode), _p(dest), _p(scale))
    return dest, scale


def combine(y, dtype, base, w, topk_idx32, send_idx, E, R=1, me=0):
    T, K = topk_idx32.shape
    H = y.shape[1]
    out = np.zeros((T, H), dtype=np.uint16)
    lib().zo_combine(_p(y), _i32(dtype), _p(np.ascontiguousarray(base, dtype=np.int32)),
                     _p(np.ascontiguousarray(w, dtype=np.float32)),
                     _p(np.ascontiguousarray(topk_idx32, dtype=np.int32)), _p(send_idx), _i64(T), _i64(H), _i64(K),
                     _i64(E), _i64(R), _i64(me), _p(out))
    return out


def dispatch_low_latency(x, x_dtype, expert_ids, E, quant_mode, rows, token_nums_type=1):
    T, H = x.shape
    K = expert_ids.shape[1]
    if quant_mode == 0:
        ex = np.zeros((rows, H), dtype=np.uint16)
        sc = np.zeros(rows, dtype=np.float32)
    elif quant_mode == 1:
        ex = np.zeros((rows, H), dtype=np.int8)
        sc = np.zeros(rows, dtype=np.float32)
    else:
        ex = np.zeros((rows, H), dtype=np.uint8)
        sc = np.zeros((rows, H // 128), dtype=np.float32)
    eidx = np.zeros((T, K), dtype=np.int32)
    nums = np.zeros(E, dtype=np.int64)
    counts = np.zeros(E, dtype=np.int32)
    lib().zo_dispatch_low_latency(_p(x), _i32(x_dtype), _p(np.ascontiguousarray(expert_ids, dtype=np.int32)), _i64(T),
                                  _i64(H), _i64(K), _i64(E), _i32(quant_mode), _i32(token_nums_type), _p(ex), _p(sc),
                                  _p(eidx), _p(nums), _p(counts))
    return ex, sc, eidx, nums, counts


def combine_low_latency(expand_x, dtype, expert_ids, expand_idx, ep_send_counts, w, E):
    T, K = expert_ids.shape
    H = expand_x.shape[1]
    out = np.zeros((T, H), dtype=np.uint16)
    lib().zo_combine_low_latency(_p(expand_x), _i32(dtype), _p(np.ascontiguousarray(expert_ids, dtype=np.int32)),
                                 _p(expand_idx), _p(ep_send_counts), _p(np.ascontiguousarray(w, dtype=np.float32)),
                                 _i64(T), _i64(H), _i64(K), _i64(E), _p(out))
    return out


def ll_counts(ids_all, E, me, token_nums_type=1):
    """ids_all [R, T, K] -> (all_counts [R, E], ep_recv_counts [R * E], expert_token_nums [E / R]) as rank `me` sees them."""
    ids = np.ascontiguousarray(ids_all, dtype=np.int32)
    R, T, K = ids.shape
    allc = np.zeros((R, E), dtype=np.int32)
    recv = np.zeros(R * E, dtype=np.int32)
    nums = np.zeros(E // R, dtype=np.int64)
    lib().zo_ll_counts(_p(ids), _i64(R), _i64(me), _i64(T), _i64(K), _i64(E), _i32(token_nums_type), _p(allc), _p(recv), _p(nums))
    return allc, recv, nums


def dispatch_low_latency_ranks(x, x_dtype, expert_ids, E, R, me, quant_mode, ep_recv_counts, windows_x, windows_scale):
    """Rank `me` writes its rows into windows_x [R, rows_cap, H] / windows_scale [R, rows_cap(, H/128)] in place; returns expand_idx."""
    T, H = x.shape
    K = expert_ids.shape[1]
    eidx = np.zeros((T, K), dtype=np.int32)
    lib().zo_dispatch_low_latency_ranks(_p(x), _i32(x_dtype), _p(np.ascontiguousarray(expert_ids, dtype=np.int32)), _i64(T),
                                        _i64(H), _i64(K), _i64(E), _i64(R), _i64(me), _i32(quant_mode),
                                        _p(np.ascontiguousarray(ep_recv_counts, dtype=np.int32)), _i64(windows_x.shape[1]),
                                        _p(windows_x), _p(windows_scale), _p(eidx))
    return eidx


def combine_low_latency_ranks(windows_y, dtype, expert_ids, expand_idx, ep_send_counts, w, E, R, me):
    T, K = expert_ids.shape
    H = windows_y.shape[2]
    out = np.zeros((T, H), dtype=np.uint16)
    lib().zo_combine_low_latency_ranks(_p(windows_y), _i32(dtype), _p(np.ascontiguousarray(expert_ids, dtype=np.int32)),
                                       _p(np.ascontiguousarray(expand_idx, dtype=np.int32)),
                                       _p(np.ascontiguousarray(ep_send_counts, dtype=np.int32)),
                                       _p(np.ascontiguousarray(w, dtype=np.float32)), _i64(T), _i64(H), _i64(K), _i64(E),
                                       _i64(R), _i64(me), _i64(windows_y.shape[1]), _p(out))
    return out


def fused_permute_quant(x, x_dtype, expert_ids, smooth, E, mode):
    T, H = x.shape
    K = expert_ids.shape[1]
    ids = np.ascontiguousarray(expert_ids, dtype=np.int32)
    rows = int(((ids >= 0) & (ids < E)).sum())
    if mode == 2:
        q1 = np.zeros((rows, H), dtype=np.uint8)
        xs = np.zeros((rows, H // 128), dtype=np.float32)
    else:
        q1 = np.zeros((rows, H), dtype=np.int8)
        xs = np.zeros(rows, dtype=np.float32)
    eidx = np.zeros((T, K), dtype=np.int32)
    counts = np.zeros(E, dtype=np.int64)
    lib().zo_fused_permute_quant(_p(x), _i32(x_dtype), _p(ids), _p(smooth), _i64(T), _i64(H), _i64(K), _i64(E),
                                 _i32(mode), _p(q1), _p(xs), _p(eidx), _p(counts))
    return q1, xs, eidx, counts


def grouped_gemm_w8a8_dequant(a, xscale, w, wscale, counts, out_dtype=DT_BF16):
    """a int8 [rows,K]; w int8 [E,K,N] logical; wscale fp32 or uint16(bf16) [E,N]."""
    E, K, N = w.shape
    y = np.zeros((a.shape[0], N), dtype=np.uint16)
    ws_dt = DT_FP32 if wscale.dtype == np.float32 else DT_BF16
    lib().zo_grouped_gemm_w8a8_dequant(_p(a), _p(xscale), _p(w), _p(wscale), _i32(ws_dt),
                                       _p(np.ascontiguousarray(counts, dtype=np.int64)), _i64(E), _i64(K), _i64(N),
                                       _i32(out_dtype), _p(y))
    return y


def gmm1_swiglu_quant_w8a8(a, xs, w1, w1scale, counts, want_sgl=False):
    E, K, N1 = w1.shape
    rows = a.shape[0]
    q2 = np.zeros((rows, N1 // 2), dtype=np.int8)
    s2 = np.zeros(rows, dtype=np.float32)
    sgl = np.zeros((rows, N1 // 2), dtype=np.float32) if want_sgl else None
    lib().zo_gmm1_swiglu_quant_w8a8(_p(a), _p(xs), _p(w1), _p(w1scale), _p(np.ascontiguousarray(counts, dtype=np.int64)),
                                    _i64(E), _i64(K), _i64(N1), _p(q2), _p(s2), _p(sgl))
    return q2, s2, sgl


def gmm1_swiglu_quant_fp8(a, sa, w1, sw1, counts, want_sgl=False):
    E, K, N1 = w1.shape
    rows = a.shape[0]
    q2 = np.zeros((rows, N1 // 2), dtype=np.uint8)
    s2 = np.zeros((rows, N1 // 2 // 128), dtype=np.float32)
    sgl = np.zeros((rows, N1 // 2), dtype=np.float32) if want_sgl else None
    lib().zo_gmm1_swiglu_quant_fp8(_p(a), _p(sa), _p(w1), _p(sw1), _p(np.ascontiguousarray(counts, dtype=np.int64)),
                                   _i64(E), _i64(K), _i64(N1), _p(q2), _p(s2), _p(sgl))
    return q2, s2, sgl


def gmm2_fp8(a, sa, w2, sw2, counts, out_dtype=DT_BF16):
    E, K, N = w2.shape
    y = np.zeros((a.shape[0], N), dtype=np.uint16)
    lib().zo_gmm2_fp8(_p(a), _p(sa), _p(w2), _p(sw2), _p(np.ascontiguousarray(counts, dtype=np.int64)), _i64(E),
                      _i64(K), _i64(N), _i32(out_dtype), _p(y))
    return y


def gmm1_swiglu_quant_w4a8(a, xs, w1, gs1, counts, want_sgl=False):
    E, K, N1 = w1.shape
    rows = a.shape[0]
    q2 = np.zeros((rows, N1 // 2), dtype=np.int8)
    s2 = np.zeros(rows, dtype=np.float32)
    sgl = np.zeros((rows, N1 // 2), dtype=np.float32) if want_sgl else None
    lib().zo_gmm1_swiglu_quant_w4a8(_p(a), _p(xs), _p(w1), _p(gs1), _p(np.ascontiguousarray(counts, dtype=np.int64)),
                                    _i64(E), _i64(K), _i64(N1), _p(q2), _p(s2), _p(sgl))
    return q2, s2, sgl


def gmm2_w4a8(a, xs, w2, gs2, counts, out_dtype=DT_BF16):
    E, K, N = w2.shape
    y = np.zeros((a.shape[0], N), dtype=np.uint16)
    lib().zo_gmm2_w4a8(_p(a), _p(xs), _p(w2), _p(gs2), _p(np.ascontiguousarray(counts, dtype=np.int64)), _i64(E),
                       _i64(K), _i64(N), _i32(out_dtype), _p(y))
    return y


def reduce(buffers, dtype, op):
    """buffers: list of equally shaped numpy arrays (uint16 for bf16/fp16)."""
    n = buffers[0].size
    out = np.empty_like(buffers[0])
    arr = (ctypes.c_void_p * len(buffers))(*[b.ctypes.data for b in buffers])
    rc = lib().zo_reduce(arr, _i64(len(buffers)), _i64(n), _i32(dtype), _i32(op), _p(out))
    if rc != 0:
        raise ValueError("oracle reduce: unsupported dtype %d" % dtype)
    return out


# ---- whole-layer restatements --------------------------------------------

def fused_moe(x, x_dtype, expert_ids, expert_scales, w1, s1, w2, s2, E, mode, smooth=None, stages=False):
    """The fused operator at one rank (FDM/zbal_kernel_fused_deep_moe.h:434-712).

    mode 0/1: W8A8 (w int8, s1 fp32 [E,N1], s2 uint16 bf16 [E,H])
    mode 2:   fp8  (w uint8 codes, s1 fp32 [E,H/128,N1/128], s2 fp32 [E,I/128,H/128])
    mode 3:   W4A8 (w int8 holding int4 values, s1/s2 uint16 fp16 [E,K/128,N])
    Returns (out uint16 [T,H], counts int64 [E]) and, with stages=True, a dict of intermediates.
    """
    ids = np.ascontiguousarray(expert_ids, dtype=np.int32)
    qmode = 2 if mode == 2 else 1
    q1, xs, eidx, counts = fused_permute_quant(x, x_dtype, ids, smooth, E, qmode)
    if mode in (0, 1):
        q2, sc2, sgl = gmm1_swiglu_quant_w8a8(q1, xs, w1, s1, counts, want_sgl=stages)
        y = grouped_gemm_w8a8_dequant(q2, sc2, w2, s2, counts, out_dtype=x_dtype)
    elif mode == 2:
        q2, sc2, sgl = gmm1_swiglu_quant_fp8(q1, xs, w1, s1, counts, want_sgl=stages)
        y = gmm2_fp8(q2, sc2, w2, s2, counts, out_dtype=x_dtype)
    else:
        q2, sc2, sgl = gmm1_swiglu_quant_w4a8(q1, xs, w1, s1, counts, want_sgl=stages)
        y = gmm2_w4a8(q2, sc2, w2, s2, counts, out_dtype=x_dtype)
    base = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.int32)
    out = combine(y, x_dtype, base, expert_scales, ids, eidx, E)
    if stages:
        return out, counts, dict(q1=q1, xs=xs, expand_idx=eidx, q2=q2, scale2=sc2, sgl=sgl, y=y, base=base)
    return out, counts
