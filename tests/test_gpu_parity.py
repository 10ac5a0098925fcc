"""Parity of the HIP path against the CPU oracle, called through the C ABI on identical seeded inputs.
Integer outputs (indices, offsets, permutation, quantised bytes, scales) must match bit for bit; bf16
GEMM / combine outputs within max relative error 2e-2; fp32 reductions within 1e-6."""
import ctypes

import numpy as np
import pytest
import torch

from memfabric_hybrid_amd import capi
from memfabric_hybrid_amd.operators import OperatorBuffer as Buffer
from oracle import oracle as zo
from zbal_testlib import bf16_normal, calc_diff, dev, distinct_topk, host, max_rel_err, rng

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def buf():
    b = Buffer()
    yield b
    torch.cuda.synchronize()
    b.close()


# ---- router ---------------------------------------------------------------------------------

@pytest.mark.parametrize("T,E,K", [(256, 8, 2), (300, 32, 8), (64, 128, 8), (17, 256, 6), (5, 1000, 32), (4096, 32, 8),
                                   (16384, 128, 8), (40, 65, 3), (9, 257, 4), (12, 64, 5)])
def test_router(buf, T, E, K):
    logits = rng(T + E).standard_normal((T, E)).astype(np.float32)
    logits[0, :] = 0.5                       # all tied: lowest indices win
    logits[1, E - 1] = logits[1, 0]          # one tie
    idx, w = buf.topk_route(dev(logits), K)
    ridx, rw = zo.topk_route(logits, K)
    assert np.array_equal(host(idx), ridx)
    assert np.allclose(host(w), rw, rtol=1e-6, atol=0)     # north star: weights within 1e-6 relative


@pytest.mark.parametrize("T,E,K,style", [(1000, 100, 32, "ties"), (1000, 129, 30, "ties"), (3000, 31, 24, "spread"),
                                         (64, 1000, 28, "ties"), (100, 32, 30, "spread")])
def test_router_many_ties_and_wide_spread(buf, T, E, K, style):
    """Small-integer logits (dozens of equal probabilities in every sum) and logits spread over +-100 (weights down to
    subnormal size): indices exact, normal weights within 1e-6 relative, subnormal ones within one subnormal step."""
    g = rng(T + E + K)
    logits = g.integers(-2, 3, (T, E)).astype(np.float32) if style == "ties" else (g.standard_normal((T, E)) * 30).astype(np.float32)
    idx, w = buf.topk_route(dev(logits), K, idx_dtype=torch.int32)
    ridx, rw = zo.topk_route(logits, K)
    assert np.array_equal(host(idx), ridx)
    assert np.allclose(host(w), rw, rtol=1e-6, atol=3e-45)


# ---- layout / notify -------------------------------------------------------------------------

@pytest.mark.parametrize("T,K,E", [(256, 2, 8), (4096, 8, 32), (16384, 8, 128), (1, 1, 1), (7, 3, 5), (1000, 6, 256),
                                    (128, 8, 32)])
def test_layout_and_notify(buf, T, K, E):
    idx = rng(T * 31 + E).integers(-1, E + 1, size=(T, K)).astype(np.int64) if T < 2000 else distinct_topk(T, E, K, 3)
    per_rank, _, per_expert, in_rank, _ = buf.get_dispatch_layout(dev(idx), E)
    r_rank, r_exp, r_send = zo.dispatch_layout(idx, E, 1)
    assert np.array_equal(host(per_expert), r_exp)
    assert np.array_equal(host(per_rank), r_rank)
    assert np.array_equal(host(buf.send_token_idx), r_send)
    x = dev(bf16_normal((T, 64), 1))
    _, _, recv_per_expert, h = buf.dispatch(x, dev(idx), None, per_expert, capi.NO_QUANT)
    r_recv, r_put, r_total, r_per, r_bal = zo.dispatch_notify(r_exp[None, :], K)
    assert np.array_equal(host(h["put_offset"]), r_put)
    assert np.array_equal(host(h["total_recv"]), r_total)
    assert np.array_equal(host(recv_per_expert), r_per)
    assert np.array_equal(host(h["balance_matrix"]), r_bal)


def test_layout_int32_indices_and_empty_batch(buf):
    lib = buf.lib
    E, K = 16, 4
    idx = distinct_topk(50, E, K, 9).astype(np.int32)
    t_idx = dev(idx)
    per_rank = torch.empty(1, dtype=torch.int32, device="cuda")
    per_exp = torch.empty(E, dtype=torch.int32, device="cuda")
    send = torch.empty((50, K), dtype=torch.int32, device="cuda")
    scratch = torch.empty(50 * E, dtype=torch.int32, device="cuda")
    ti = lambda t: ctypes.byref(capi.tensor_info(t))
    assert lib.zbal_dispatch_normal_layout(ti(t_idx), 50, E, K, ti(per_rank), ti(per_exp), ti(send), ti(scratch),
                                           buf.comm, capi.stream_ptr(), 0) == 0
    r_rank, r_exp, r_send = zo.dispatch_layout(idx.astype(np.int64), E, 1)
    assert np.array_equal(host(per_exp), r_exp) and np.array_equal(host(send), r_send)
    # zero tokens: counts are zeroed, nothing else is touched
    assert lib.zbal_dispatch_normal_layout(ti(t_idx), 0, E, K, ti(per_rank), ti(per_exp), ti(send), ti(scratch),
                                           buf.comm, capi.stream_ptr(), 0) == 0
    assert host(per_exp).sum() == 0 and host(per_rank)[0] == 0
    # too small a scratch tensor is refused, not overrun
    small = torch.empty(E, dtype=torch.int32, device="cuda")
    assert lib.zbal_dispatch_normal_layout(ti(t_idx), 50, E, K, ti(per_rank), ti(per_exp), ti(send), ti(small),
                                           buf.comm, capi.stream_ptr(), 0) == capi.Z_INVALID_PARAM


# ---- dispatch (permute + quant) and combine --------------------------------------------------------

def run_dispatch(buf, x16, xdt, idx, E, qmode):
    tdt = torch.bfloat16 if xdt == zo.DT_BF16 else torch.float16
    per_rank, _, per_expert, _, _ = buf.get_dispatch_layout(dev(idx), E)
    recv, scales, _, h = buf.dispatch(dev(x16, tdt), dev(idx), None, per_expert, qmode)
    _, r_exp, r_send = zo.dispatch_layout(idx, E, 1)
    put = np.concatenate([[0], np.cumsum(r_exp)[:-1]]).astype(np.int32)
    rows = int(r_exp.sum())
    r_dest, r_scale = zo.dispatch_normal(x16, xdt, idx.astype(np.int32), r_send, put, E, qmode, rows)
    return recv, scales, h, r_dest, r_scale, rows, put, r_send


@pytest.mark.parametrize("T,H,K,E", [(256, 1024, 2, 8), (128, 7168, 8, 32), (64, 4096, 8, 128), (33, 128, 3, 4),
                                      (9, 16384, 2, 4)])
@pytest.mark.parametrize("qmode", [capi.NO_QUANT, capi.QUANT_INT8, capi.QUANT_FP8_B128])
def test_dispatch_normal_bit_exact(buf, T, H, K, E, qmode):
    x = bf16_normal((T, H), T + H)
    xf = zo.bf16_to_f32(x)
    xf[0, :] = 0.0                  # all-zero token
    xf[1 % T, :] = -2.5             # constant token
    x = zo.f32_to_bf16(xf)
    idx = distinct_topk(T, E, K, 5)
    idx[2 % T, 0] = -1              # an invalid pick
    recv, scales, h, r_dest, r_scale, rows, _, _ = run_dispatch(buf, x, zo.DT_BF16, idx, E, qmode)
    got = host(recv)[:rows]
    assert np.array_equal(got.view(r_dest.dtype), r_dest)
    if qmode != capi.NO_QUANT:
        assert np.array_equal(host(scales)[:rows].view(np.uint32), r_scale.view(np.uint32))


@pytest.mark.parametrize("T,H,K,E,qmode", [(4096, 7168, 8, 32, capi.QUANT_FP8_B128),      # the prefill share
                                           (16384, 4096, 8, 128, capi.QUANT_INT8)])          # the W4A8 layer
def test_dispatch_normal_full_size_bit_exact(buf, T, H, K, E, qmode):
    x = bf16_normal((T, H), 31)
    idx = distinct_topk(T, E, K, 32)
    recv, scales, h, r_dest, r_scale, rows, put, r_send = run_dispatch(buf, x, zo.DT_BF16, idx, E, qmode)
    assert rows == T * K
    assert np.array_equal(host(recv)[:rows].view(r_dest.dtype), r_dest)
    assert np.array_equal(host(scales)[:rows].view(np.uint32), r_scale.view(np.uint32))
    # independent of the oracle: the rows are a permutation of the picks, expert-major and stable within an expert
    dest_row = put[idx] + r_send
    assert np.array_equal(np.sort(dest_row.ravel()), np.arange(rows))
    order = np.argsort(dest_row.ravel(), kind="stable")
    assert np.all(np.diff(idx.ravel()[order]) >= 0)
    assert np.all(np.diff(order)[np.diff(idx.ravel()[order]) == 0] > 0)


def test_combine_normal_full_size_round_trip(buf):
    T, H, K, E = 4096, 7168, 8, 32
    x = bf16_normal((T, H), 33)
    idx = distinct_topk(T, E, K, 34)
    w = rng(35).uniform(0.05, 1.0, (T, K)).astype(np.float32)
    recv, _, h, r_dest, _, rows, put, r_send = run_dispatch(buf, x, zo.DT_BF16, idx, E, capi.NO_QUANT)
    out = buf.combine(recv, h, dev(w))
    assert np.array_equal(host(out), zo.combine(r_dest, zo.DT_BF16, put, w, idx.astype(np.int32), r_send, E))
    assert calc_diff(zo.bf16_to_f32(host(out)), zo.bf16_to_f32(x) * w.sum(1, keepdims=True)) < 5e-5


def test_dispatch_fp16_input(buf):
    T, H, K, E = 40, 512, 4, 16
    x = zo.f32_to_fp16(rng(8).standard_normal((T, H)).astype(np.float32) * 3)
    idx = distinct_topk(T, E, K, 6)
    for qmode in (capi.NO_QUANT, capi.QUANT_INT8, capi.QUANT_FP8_B128):
        recv, scales, h, r_dest, r_scale, rows, _, _ = run_dispatch(buf, x, zo.DT_FP16, idx, E, qmode)
        assert np.array_equal(host(recv)[:rows].view(r_dest.dtype), r_dest)
        if qmode != capi.NO_QUANT:
            assert np.array_equal(host(scales)[:rows], r_scale)


# small batches cut each row into pieces for several workgroups: 7 x 4144 gives four pieces of 130, 130, 130 and 128 chunks
@pytest.mark.parametrize("T,H,K,E", [(256, 2048, 2, 8), (128, 7168, 8, 32), (50, 4096, 8, 128), (3, 64, 1, 2), (7, 4144, 3, 4),
                                     (1, 16384, 8, 16)])
def test_combine_normal_exact_and_round_trip(buf, T, H, K, E):
    x = bf16_normal((T, H), 11)
    idx = distinct_topk(T, E, K, 12)
    if T > 2:
        idx[1, K - 1] = -1
    w = rng(13).uniform(0.05, 1.0, (T, K)).astype(np.float32)
    recv, _, h, r_dest, _, rows, put, r_send = run_dispatch(buf, x, zo.DT_BF16, idx, E, capi.NO_QUANT)
    out = buf.combine(recv, h, dev(w))
    ref = zo.combine(r_dest, zo.DT_BF16, put, w, idx.astype(np.int32), r_send, E)
    assert np.array_equal(host(out), ref)                         # same operation order: bit exact
    # the reference's own check (test_normal.py:225-236): identity experts give x * sum of the valid weights
    wv = np.where((idx >= 0) & (idx < E), w, 0).sum(1, keepdims=True)
    assert calc_diff(zo.bf16_to_f32(host(out)), zo.bf16_to_f32(x) * wv) < 5e-5


def test_combine_fp16(buf):
    T, H, K, E = 20, 256, 4, 8
    x = zo.f32_to_fp16(rng(14).standard_normal((T, H)).astype(np.float32))
    idx = distinct_topk(T, E, K, 15)
    w = rng(16).uniform(0.05, 1.0, (T, K)).astype(np.float32)
    recv, _, h, r_dest, _, rows, put, r_send = run_dispatch(buf, x, zo.DT_FP16, idx, E, capi.NO_QUANT)
    out = buf.combine(recv, h, dev(w))
    assert np.array_equal(host(out), zo.combine(r_dest, zo.DT_FP16, put, w, idx.astype(np.int32), r_send, E))


# ---- low-latency mode ------------------------------------------------------------------------------

@pytest.mark.parametrize("T,H,K,E,zipf", [(128, 7168, 8, 32, 1.2), (1, 7168, 8, 32, None), (80, 4096, 8, 128, None),
                                           (300, 256, 4, 16, None)])
@pytest.mark.parametrize("mode", ["bf16", "int8", "fp8"])
def test_low_latency_dispatch_combine(buf, T, H, K, E, zipf, mode):
    x = bf16_normal((T, H), 21)
    if T > 1:
        x[1, :] = 0                     # all-zero token: q = 0, scale = 0 in this mode
    idx = distinct_topk(T, E, K, 22, zipf=zipf)
    w = rng(23).uniform(0.05, 1.0, (T, K)).astype(np.float32)
    use_fp8, blk, qm = {"bf16": (False, False, 0), "int8": (True, False, 1), "fp8": (True, True, 2)}[mode]
    recv, scales, count, h = buf.low_latency_dispatch(dev(x), dev(idx), T, E, use_fp8=use_fp8, fp8_block_scale=blk)
    rows = T * K
    r_ex, r_sc, r_eidx, r_nums, r_counts = zo.dispatch_low_latency(x, zo.DT_BF16, idx.astype(np.int32), E, qm, rows)
    assert np.array_equal(host(h["expand_idx"])[:rows].reshape(T, K), r_eidx)
    assert np.array_equal(host(count), r_nums) and np.array_equal(host(h["ep_recv_count"]), r_counts)
    assert np.array_equal(host(recv).view(r_ex.dtype), r_ex)
    if qm:
        assert np.array_equal(host(scales).view(np.uint32), r_sc.view(np.uint32))
    if mode == "bf16":
        out = buf.low_latency_combine(recv, dev(w), h)
        ref = zo.combine_low_latency(r_ex, zo.DT_BF16, idx.astype(np.int32), r_eidx, r_counts, w, E)
        assert np.array_equal(host(out), ref)
        assert calc_diff(zo.bf16_to_f32(host(out)), zo.bf16_to_f32(x) * w.sum(1, keepdims=True)) < 1e-5


@pytest.mark.parametrize("T,H,K,E", [
    (512, 256, 8, 32),       # 4096 picks: the largest batch whose layout the permute kernel works out itself
    (513, 256, 8, 32),       # one token more: layout launch + permute launch
    (24, 512, 40, 64),       # more picks per token than the kernel's pick table holds (32)
    (100, 256, 40, 64),      # the same past 4096 picks
    (64, 256, 4, 1024),      # the largest expert count
])
@pytest.mark.parametrize("mode", ["int8", "fp8"])
def test_low_latency_dispatch_at_the_layout_switch(buf, T, H, K, E, mode):
    """Both ways of deriving the layout (inside the permute kernel up to 4096 picks and 32 picks per token, a layout
    launch beyond) against the oracle, with invalid picks among the valid ones."""
    x = bf16_normal((T, H), 31)
    idx = distinct_topk(T, E, K, 32)
    idx[T // 2, 1] = -1
    idx[T - 1, K - 1] = E + 5
    use_fp8, blk, qm = {"int8": (True, False, 1), "fp8": (True, True, 2)}[mode]
    recv, scales, count, h = buf.low_latency_dispatch(dev(x), dev(idx), T, E, use_fp8=use_fp8, fp8_block_scale=blk)
    rows = T * K
    r_ex, r_sc, r_eidx, r_nums, r_counts = zo.dispatch_low_latency(x, zo.DT_BF16, idx.astype(np.int32), E, qm, rows)
    assert np.array_equal(host(h["expand_idx"])[:rows].reshape(T, K), r_eidx)
    assert np.array_equal(host(count), r_nums) and np.array_equal(host(h["ep_recv_count"]), r_counts)
    total = int(r_counts[-1])
    assert np.array_equal(host(recv).view(r_ex.dtype)[:total], r_ex[:total])
    assert np.array_equal(host(scales).view(np.uint32).reshape(rows, -1)[:total], r_sc.view(np.uint32).reshape(rows, -1)[:total])


@pytest.mark.parametrize("T,H,K,E", [
    (512, 256, 8, 32),       # 4096 picks: the permute kernel works the layout out itself
    (513, 256, 8, 32),       # one token more: range-layout launch + table in the permute kernel
    (5000, 128, 8, 32),      # 50 ranges of 100 tokens: the most ranges
    (3000, 128, 6, 256),     # the most experts the table mode takes (8 ranges of 256 entries)
    (3000, 128, 6, 257),     # one more: the one-launch layout in front of the permute
    (200, 128, 32, 64),      # the most picks per token the table mode takes
    (200, 128, 33, 64),      # one more
    (4200, 128, 1, 3),       # top-1 on three experts: 1400 rows per expert from 42 ranges
])
@pytest.mark.parametrize("qmode", [1, 2])
def test_fused_permute_quant_layout_modes(buf, T, H, K, E, qmode):
    """The fused operator's first stage through the kernel ABI, either side of every limit that selects how the layout
    is derived: rows, scales, ranks, counts and offsets against the oracle, bit for bit, with invalid picks and an
    expert without rows."""
    x = bf16_normal((T, H), 71)
    idx = distinct_topk(T, E, K, 72).astype(np.int32)
    if E > 3:
        idx[idx == 1] = 0 if K == 1 else -1           # expert 1 stays empty
    idx[T // 2, 0] = -1
    idx[T - 1, K - 1] = E + 7
    rows = T * K
    q1 = torch.zeros((rows, H), dtype=torch.uint8, device="cuda")
    xs = torch.zeros((rows, H // 128 if qmode == 2 else 1), dtype=torch.float32, device="cuda")
    eidx = torch.full((T, K), -7, dtype=torch.int32, device="cuda")
    counts = torch.full((E,), -7, dtype=torch.int64, device="cuda")
    row_off = torch.full((E + 1,), -7, dtype=torch.int32, device="cuda")
    scratch = torch.zeros((50 * E,), dtype=torch.int32, device="cuda")
    xd, idd = dev(x), dev(idx)
    rc = buf.lib.zbalhip_fused_permute_quant(xd.data_ptr(), capi.DT_BF16, idd.data_ptr(), None, None, T, H, K, E, qmode,
                                             q1.data_ptr(), xs.data_ptr(), eidx.data_ptr(), counts.data_ptr(), row_off.data_ptr(),
                                             None, 0, scratch.data_ptr(), 50, capi.stream_ptr())
    capi.check("fused_permute_quant", rc)
    r_q1, r_xs, r_eidx, r_counts = zo.fused_permute_quant(x, zo.DT_BF16, idx, None, E, qmode)
    total = int(r_counts.sum())
    assert np.array_equal(host(counts), r_counts)
    assert np.array_equal(host(row_off), np.concatenate([[0], np.cumsum(r_counts)]).astype(np.int32))
    assert np.array_equal(host(eidx), r_eidx)
    assert np.array_equal(host(q1)[:total], r_q1.view(np.uint8)[:total])
    assert np.array_equal(host(xs).view(np.uint32).reshape(rows, -1)[:total], r_xs.view(np.uint32).reshape(total, -1))


def test_low_latency_token_nums_type_prefix_sum(buf, monkeypatch):
    monkeypatch.setenv("MOE_EXPERT_TOKEN_NUMS_TYPE", "0")
    T, H, K, E = 64, 256, 4, 16
    idx = distinct_topk(T, E, K, 24)
    _, _, count, _ = buf.low_latency_dispatch(dev(bf16_normal((T, H), 25)), dev(idx), T, E, use_fp8=False)
    assert np.array_equal(host(count), np.cumsum(np.bincount(idx.reshape(-1), minlength=E)))


# ---- N-buffer reduce ----------------------------------------------------------------------------------

NP_DT = {capi.DT_INT8: np.int8, capi.DT_INT16: np.int16, capi.DT_INT32: np.int32, capi.DT_INT64: np.int64,
         capi.DT_FP32: np.float32}


def make_reduce_inputs(dt, n, N, seed):
    if dt in NP_DT and dt != capi.DT_FP32:
        return [rng(seed + p).integers(-100, 100, n).astype(NP_DT[dt]) for p in range(N)]
    f = [rng(seed + p).uniform(0, 10, n).astype(np.float32) - (3 if p % 2 else 0) for p in range(N)]  # reference: uniform(0,10)
    if dt == capi.DT_FP32:
        return f
    return [zo.f32_to_bf16(a) if dt == capi.DT_BF16 else zo.f32_to_fp16(a) for a in f]


@pytest.mark.parametrize("dt", [capi.DT_INT8, capi.DT_INT16, capi.DT_INT32, capi.DT_INT64, capi.DT_FP16, capi.DT_BF16,
                                capi.DT_FP32])
@pytest.mark.parametrize("op", [capi.REDUCE_SUM, capi.REDUCE_MAX, capi.REDUCE_MIN, capi.REDUCE_PROD])
def test_reduce_kernel_all_types(buf, dt, op):
    lib = buf.lib
    for N, n in ((8, 6 * 2 ** 10 + 5), (3, 1000), (1, 77), (16, 4096), (5, 3)):
        ins = make_reduce_inputs(dt, n, N, 100 + N)
        tdt = {capi.DT_BF16: torch.bfloat16, capi.DT_FP16: torch.float16}.get(dt)
        d_in = [dev(a, tdt) for a in ins]
        out = torch.empty_like(d_in[0])
        arr = (ctypes.c_void_p * N)(*[t.data_ptr() for t in d_in])
        assert lib.zbalhip_reduce(arr, N, n, dt, op, out.data_ptr(), 0, None, 0, capi.stream_ptr()) == 0
        ref = zo.reduce(ins, dt, op)
        assert np.array_equal(host(out), ref), (N, n)


@pytest.mark.parametrize("dt", [capi.DT_INT8, capi.DT_BF16, capi.DT_FP32, capi.DT_INT64])
def test_reduce_bases_off_the_16_byte_boundary(buf, dt):
    """Bases that hold whole elements but do not start on a 16-byte boundary: all at the same offset (a scalar head,
    then the vector path), at different offsets (element by element), and half-element offsets (refused). Elements
    in front of and behind the range stay untouched."""
    lib = buf.lib
    tdt = {capi.DT_BF16: torch.bfloat16, capi.DT_FP16: torch.float16}.get(dt)
    for N, n, offs in ((4, 5000, [3] * 5), (3, 70001, [1, 1, 1, 0]), (8, 257, [0, 1, 2, 3, 4, 5, 6, 7, 1]), (2, 1, [1, 1, 1]),
                       (5, 4099, [0] * 5 + [1])):
        pad = 16
        ins = make_reduce_inputs(dt, n + pad, N, 500 + N)
        d_in = [dev(a, tdt) for a in ins]
        es = d_in[0].element_size()
        out = torch.zeros(n + pad, dtype=d_in[0].dtype, device="cuda")
        arr = (ctypes.c_void_p * N)(*[t.data_ptr() + o * es for t, o in zip(d_in, offs)])
        oo = offs[N]
        assert lib.zbalhip_reduce(arr, N, n, dt, capi.REDUCE_SUM, out.data_ptr() + oo * es, 0, None, 0, capi.stream_ptr()) == 0
        ref = zo.reduce([a[o:o + n].copy() for a, o in zip(ins, offs)], dt, capi.REDUCE_SUM)
        got = host(out)
        assert np.array_equal(got[oo:oo + n], ref), (N, n, offs)
        assert not got[:oo].any() and not got[oo + n:].any()
    if dt != capi.DT_INT8:
        a = torch.zeros(64, dtype=torch.uint8, device="cuda")
        arr = (ctypes.c_void_p * 1)(a.data_ptr() + 1)
        assert lib.zbalhip_reduce(arr, 1, 4, dt, capi.REDUCE_SUM, a.data_ptr() + 32, 0, None, 0, capi.stream_ptr()) != 0


def test_reduce_full_size_sampled_windows(buf):
    """8 buffers of 256 MiB in separate allocations, bf16 and fp32 sums: the output is checked on windows sampled at the
    ends and across the range (the reduction is element-wise, so a window needs only the same window of every input)."""
    lib = buf.lib
    N, nbytes = 8, 256 << 20
    g = torch.Generator(device="cuda").manual_seed(5)
    for dt, tdt in ((capi.DT_BF16, torch.bfloat16), (capi.DT_FP32, torch.float32)):
        n = nbytes // (2 if dt == capi.DT_BF16 else 4)
        ins = [torch.randn(n, device="cuda", generator=g).to(tdt) for _ in range(N)]
        out = torch.empty_like(ins[0])
        arr = (ctypes.c_void_p * N)(*[t.data_ptr() for t in ins])
        assert lib.zbalhip_reduce(arr, N, n, dt, capi.REDUCE_SUM, out.data_ptr(), 0, None, 0, capi.stream_ptr()) == 0
        torch.cuda.synchronize()
        w = 1 << 16
        for start in [0, n - w] + [int(v) for v in rng(6).integers(0, n - w, 6)]:
            if dt == capi.DT_BF16:
                parts = [host(t[start:start + w].view(torch.int16)).view(np.uint16) for t in ins]
                got = host(out[start:start + w].view(torch.int16)).view(np.uint16)
            else:
                parts = [host(t[start:start + w]) for t in ins]
                got = host(out[start:start + w])
            assert np.array_equal(got, zo.reduce(parts, dt, capi.REDUCE_SUM)), (dt, start)
        del ins, out


def test_reduce_scatter_and_all_reduce_over_peer_windows(buf):
    """cfg4 shape in miniature: 8 'ranks' as local windows, this rank reduces its slice of every peer's buffer."""
    from memfabric_hybrid_amd.operators import create_group, destroy_group
    lib = buf.lib
    R, me = 8, 5
    comm = create_group("rs8", R, me)
    try:
        # the second slice length puts this rank's slice of every window off the 16-byte boundary
        for dt, tdt, n in ((capi.DT_BF16, torch.bfloat16, 6 * 2 ** 12), (capi.DT_FP32, None, 6 * 2 ** 12),
                           (capi.DT_BF16, torch.bfloat16, 1001), (capi.DT_FP32, None, 333)):
            ins = make_reduce_inputs(dt, R * n, R, 300)
            wins = [dev(a, tdt) for a in ins]
            esz = wins[0].element_size()
            recv = torch.empty(n, dtype=wins[0].dtype, device="cuda")
            if dt == capi.DT_BF16:   # without windows the send buffer cannot be translated
                assert lib.zbal_reduce_scatter(wins[me].data_ptr(), recv.data_ptr(), n, dt, capi.REDUCE_SUM, comm,
                                               capi.stream_ptr()) == capi.Z_INVALID_PARAM
            for r in range(R):
                assert lib.zbal_comm_register_peer_window(comm, r, wins[r].data_ptr(), R * n * esz) == 0
            assert lib.zbal_reduce_scatter(wins[me].data_ptr(), recv.data_ptr(), n, dt, capi.REDUCE_SUM, comm,
                                           capi.stream_ptr()) == 0
            ref = zo.reduce([a[me * n:(me + 1) * n].copy() for a in ins], dt, capi.REDUCE_SUM)
            assert np.array_equal(host(recv), ref)
            full = torch.empty(R * n, dtype=wins[0].dtype, device="cuda")
            tmp = torch.empty(n, dtype=wins[0].dtype, device="cuda")
            assert lib.zbal_all_reduce(wins[me].data_ptr(), full.data_ptr(), tmp.data_ptr(), R * n, dt, capi.REDUCE_SUM,
                                       comm, capi.stream_ptr()) == 0
            assert np.array_equal(host(full), zo.reduce(ins, dt, capi.REDUCE_SUM))
            if dt == capi.DT_FP32:     # north star: fp32 within 1e-6 relative of the exact sum
                exact = np.sum(np.stack(ins).astype(np.float64), 0)
                assert np.allclose(host(full), exact, rtol=1e-6, atol=1e-6)
            # a send buffer outside this rank's window is refused
            assert lib.zbal_reduce_scatter(recv.data_ptr(), recv.data_ptr(), n, dt, capi.REDUCE_SUM, comm,
                                           capi.stream_ptr()) == capi.Z_INVALID_PARAM
            torch.cuda.synchronize()
    finally:
        torch.cuda.synchronize()
        destroy_group(comm)


def test_device_trace_ring_and_trace_viewer_dump(buf, tmp_path, monkeypatch):
    """Tracing as the reference switches it on (ZBAL_PROF_ENABLE / ZBAL_PROF_MAX_TRACING_COUNT / ZBAL_PROF_DIR,
    zbal_env_helper.h:20-22): a communicator created with it records a begin and an end per traced workgroup of each
    reduce launch and writes a trace-viewer JSON array (zbal_trace_viewer_dumper.h:277-304) on request and when it
    is destroyed. Results must not change."""
    import glob
    import json
    from memfabric_hybrid_amd.operators import create_group, destroy_group
    lib = buf.lib
    monkeypatch.setenv("ZBAL_PROF_ENABLE", "1")
    monkeypatch.setenv("ZBAL_PROF_DIR", str(tmp_path))
    R, me, n = 4, 1, 64 * 1024            # 32 workgroups of 256 lanes x 8 bf16: every one of them is traced
    comm = create_group("traced4", R, me)
    try:
        ins = make_reduce_inputs(capi.DT_BF16, R * n, R, 310)
        wins = [dev(a, torch.bfloat16) for a in ins]
        recv = torch.empty(n, dtype=torch.bfloat16, device="cuda")
        for r in range(R):
            assert lib.zbal_comm_register_peer_window(comm, r, wins[r].data_ptr(), R * n * 2) == 0
        launches = 3
        for _ in range(launches):
            assert lib.zbal_reduce_scatter(wins[me].data_ptr(), recv.data_ptr(), n, capi.DT_BF16, capi.REDUCE_SUM, comm,
                                           capi.stream_ptr()) == 0
        full = torch.empty(R * n, dtype=torch.bfloat16, device="cuda")
        tmp = torch.empty(n, dtype=torch.bfloat16, device="cuda")
        assert lib.zbal_all_reduce(wins[me].data_ptr(), full.data_ptr(), tmp.data_ptr(), R * n, capi.DT_BF16,
                                   capi.REDUCE_SUM, comm, capi.stream_ptr()) == 0
        assert lib.zbal_comm_dump_profiling_trace(comm) == 0
        assert np.array_equal(host(recv), zo.reduce([a[me * n:(me + 1) * n].copy() for a in ins], capi.DT_BF16, capi.REDUCE_SUM))
        files = glob.glob(str(tmp_path / "trace_view_1_*.json"))
        assert len(files) == 1
        events = json.load(open(files[0]))
        wgs = n // (256 * 8)
        rs = [e for e in events if e["name"] == "RS_KERNEL_ALL"]
        ar = [e for e in events if e["name"] == "AR_KERNEL_ALL"]
        assert len(rs) == 2 * launches * wgs and len(ar) == 2 * 64          # the all-reduce has 128 workgroups, 64 traced
        assert {e["pid"] for e in events} == {"RANK_1"} and {e["tid"] for e in rs} == {"wg %d" % i for i in range(wgs)}
        for tid in {e["tid"] for e in events}:          # per workgroup: B, E, B, E ... with time going forward
            mine = [e for e in events if e["tid"] == tid]
            assert [e["ph"] for e in mine] == ["B", "E"] * (len(mine) // 2)
            ts = [e["ts"] for e in mine]
            assert all(b <= a for b, a in zip(ts, ts[1:]))
            assert ts[-1] - ts[0] < 5e6                                        # microseconds: the launches took well under 5 s
        # SIGUSR1 dumps every communicator's trace (reference common/zbal_signal_handler.cpp:21-29)
        import os, signal
        for f in files:
            os.remove(f)
        os.kill(os.getpid(), signal.SIGUSR1)
        import time                                       # the handler only wakes the library's helper thread, which writes
        deadline = time.time() + 10
        while not glob.glob(str(tmp_path / "trace_view_1_*.json")) and time.time() < deadline:
            time.sleep(0.02)
        time.sleep(0.2)                                   # let it finish the file
        assert len(glob.glob(str(tmp_path / "trace_view_1_*.json"))) == 1
        # a second traced communicator has a ring of its own: destroying it leaves this one's tracing on
        other = create_group("traced_other", 1, 0)
        destroy_group(other)
        assert lib.zbal_reduce_scatter(wins[me].data_ptr(), recv.data_ptr(), n, capi.DT_BF16, capi.REDUCE_SUM, comm,
                                       capi.stream_ptr()) == 0
        assert lib.zbal_comm_dump_profiling_trace(comm) == 0
        newest = max(glob.glob(str(tmp_path / "trace_view_1_*.json")), key=os.path.getmtime)
        assert len([e for e in json.load(open(newest)) if e["name"] == "RS_KERNEL_ALL"]) == 2 * (launches + 1) * wgs
    finally:
        torch.cuda.synchronize()
        destroy_group(comm)
    assert len(glob.glob(str(tmp_path / "trace_view_1_*.json"))) >= 1         # written again at destruction (same second: same name)
    monkeypatch.delenv("ZBAL_PROF_ENABLE")
    plain = create_group("untraced", 1, 0)                                     # tracing off: nothing is written
    try:
        assert lib.zbal_comm_dump_profiling_trace(plain) == 0
    finally:
        destroy_group(plain)


# ---- weight pre-pack --------------------------------------------------------------------------------------

def test_weight_prepack(buf):
    E, K, N = 3, 256, 384
    w = rng(40).integers(-128, 128, (E, K, N)).astype(np.int8)
    packed = host(buf.prepack_weight(dev(w))).reshape(E, N // 128, K // 128, 128, 8, 16)
    # block [e][nb][kb] holds block row r at +128*r, 16-byte chunk c of its K-bytes in slot c ^ (r & 7) ^ ((r >> 3) & 1);
    # block row r is channel ch[r] of the block (a permutation within groups of 32)
    wt = w.transpose(0, 2, 1).reshape(E, N // 128, 128, K // 128, 8, 16).transpose(0, 1, 3, 2, 4, 5)   # [e][nb][kb][ch][c][16]
    r = np.arange(128)
    ch = (r & ~31) | (((r & 15) >> 2) << 3) | (((r >> 4) & 1) << 2) | (r & 3)
    assert sorted(ch) == list(range(128)) and np.array_equal(ch[:36], [0, 1, 2, 3, 8, 9, 10, 11, 16, 17, 18, 19, 24, 25, 26, 27,
                                                                       4, 5, 6, 7, 12, 13, 14, 15, 20, 21, 22, 23, 28, 29, 30, 31,
                                                                       32, 33, 34, 35])
    f = (r & 7) ^ ((r >> 3) & 1)
    want = np.empty_like(wt)
    for slot in range(8):
        want[:, :, :, r, slot, :] = wt[:, :, :, ch, slot ^ f, :]
    assert np.array_equal(packed, want)
    assert buf.lib.zbalhip_weight_prepack(dev(w).data_ptr(), E, 200, 136, 0, dev(w).data_ptr() + 16, None) != 0
    # int4: 8 KiB blocks of 128 channels x 128 k; block row r (channel ch[r]) at +64*r, the 16-byte chunk c (k in [32c, 32c+32)) in slot
    # c ^ ((r >> 2) & 3) (r taken within its 16-channel group); byte b of dword j = k[8j+b] | k[8j+4+b] << 4
    w4 = rng(41).integers(-8, 8, (E, K, N)).astype(np.int8)
    p4 = host(buf.prepack_weight(dev(w4), int4=True)).reshape(E, N // 128, K // 128, 128, 4, 16)
    wt = w4.transpose(0, 2, 1).reshape(E, N // 128, 128, K // 128, 4, 4, 2, 4)       # [e][nb][r][kb][c][j][half][b]
    nib = ((wt[..., 0, :] & 0xf) | ((wt[..., 1, :] & 0xf) << 4)).astype(np.uint8)     # [e][nb][r][kb][c][j][b]
    nib = nib.reshape(E, N // 128, 128, K // 128, 4, 16).transpose(0, 1, 3, 2, 4, 5)  # [e][nb][kb][r][c][16]
    f4 = ((r & 15) >> 2) & 3
    want4 = np.empty_like(nib)
    for slot in range(4):
        want4[:, :, :, r, slot, :] = nib[:, :, :, ch, slot ^ f4, :]
    assert np.array_equal(p4, want4)
