"""Pins for the CPU oracle itself: every check here is independent of the
oracle's own formulas (library routines, brute force, closed forms, the
invariants the reference's tests assert)."""
import numpy as np
import pytest
import torch

from oracle import oracle as zo


def rng(seed):
    return np.random.default_rng(seed)


# ---- scalar formats --------------------------------------------------------

def test_bf16_matches_torch():
    x = np.concatenate([rng(0).standard_normal(100000).astype(np.float32) * 37.0,
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, 1e-40], dtype=np.float32)])
    got = zo.f32_to_bf16(x)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(zo.bf16_to_f32(got), torch.from_numpy(want.view(np.int16)).view(torch.bfloat16).float().numpy())


def test_fp16_matches_numpy():
    x = np.concatenate([rng(1).standard_normal(100000).astype(np.float32) * 100.0,
                        rng(2).standard_normal(10000).astype(np.float32) * 1e-6,
                        np.array([65504.0, 65519.0, 65520.0, 1e6, 5.96e-8, 2.98e-8, 2.99e-8, 0.0, -0.0], dtype=np.float32)])
    got = zo.f32_to_fp16(x)
    want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)
    allh = np.arange(65536, dtype=np.uint16)
    back = zo.fp16_to_f32(allh)
    ref = allh.view(np.float16).astype(np.float32)
    ok = (back == ref) | (np.isnan(back) & np.isnan(ref))
    assert ok.all()


def test_e4m3_matches_torch_in_range_and_saturates():
    codes = np.arange(256, dtype=np.uint8)
    dec = zo.e4m3_to_f32(codes)
    ref = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    ok = (dec == ref) | (np.isnan(dec) & np.isnan(ref))
    assert ok.all()
    x = np.concatenate([rng(3).uniform(-448, 448, 200000), rng(4).uniform(-0.05, 0.05, 50000),
                        dec[np.isfinite(dec)], (dec[:-1] + dec[1:])[np.isfinite(dec[:-1] + dec[1:])] / 2]).astype(np.float32)
    x = x[np.abs(x) <= 448]
    got = zo.f32_to_e4m3(x)
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(got, want)
    assert list(zo.f32_to_e4m3(np.array([449, 1e9, -500, np.inf], dtype=np.float32))) == [0x7e, 0x7e, 0xfe, 0x7e]


def test_expf_accuracy_and_edges():
    x = np.concatenate([rng(5).uniform(-104, 88.7, 400000), rng(6).uniform(-2, 2, 100000)]).astype(np.float32)
    got = zo.expf(x).astype(np.float64)
    want = np.exp(x.astype(np.float64))
    normal = want > 1.2e-38
    rel = np.abs(got[normal] - want[normal]) / want[normal]
    assert rel.max() < 2.5e-7          # about 2 ulp
    assert np.all(np.abs(got[~normal] - want[~normal]) < 3e-45 + 1e-6 * want[~normal])
    e = zo.expf(np.array([0.0, 89.0, -104.5, np.inf, -np.inf], dtype=np.float32))
    assert e[0] == 1.0 and np.isinf(e[1]) and e[2] == 0.0 and np.isinf(e[3]) and e[4] == 0.0


# ---- router ------------------------------------------------------------------

def test_router_brute_force_and_invariants():
    T, E, K = 256, 8, 2
    logits = rng(0).standard_normal((T, E)).astype(np.float32)
    logits[3, 5] = logits[3, 1]          # a tie: lower index first
    logits[4, :] = 0.25                  # all equal
    idx, w = zo.topk_route(logits, K)
    p = torch.softmax(torch.from_numpy(logits).double(), dim=-1).numpy()
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-logits[t, e], e))[:K]
        assert list(idx[t]) == order
        ref = p[t, order] / p[t, order].sum()
        assert np.allclose(w[t], ref, rtol=1e-6, atol=0)
    assert np.allclose(w.sum(1), 1.0, atol=1e-6)
    assert list(idx[4]) == [0, 1]


# ---- layout / notify -----------------------------------------------------------

def brute_layout(idx, E, R):
    T, K = idx.shape
    flat = idx.reshape(-1)
    send = np.full(T * K, -1, dtype=np.int32)
    for i in range(T * K):
        if 0 <= flat[i] < E:
            send[i] = int(np.sum(flat[:i] == flat[i]))
    per_e = np.array([(flat == e).sum() for e in range(E)], dtype=np.int32)
    eloc = E // R
    per_r = np.zeros(R, dtype=np.int32)
    for t in range(T):
        ranks = {int(e) // eloc for e in idx[t] if 0 <= e < E}
        for r in ranks:
            per_r[r] += 1
    return per_r, per_e, send.reshape(T, K)


@pytest.mark.parametrize("T,K,E,R", [(64, 8, 32, 1), (50, 2, 8, 4), (1, 1, 1, 1), (33, 4, 16, 2)])
def test_layout_brute_force(T, K, E, R):
    idx = rng(T + K).integers(-1, E + 1, size=(T, K)).astype(np.int64)   # includes invalid -1 and E
    got = zo.dispatch_layout(idx, E, R)
    want = brute_layout(idx, E, R)
    for g, w_ in zip(got, want):
        assert np.array_equal(g, w_)


def test_layout_bijection_and_reference_assertions():
    T, K, E = 200, 8, 32
    idx = np.stack([rng(t).permutation(E)[:K] for t in range(T)]).astype(np.int64)
    per_r, per_e, send = zo.dispatch_layout(idx, E, 1)
    # reference test_normal.py:95-98: counts equal a recount
    assert np.array_equal(per_e, np.bincount(idx.reshape(-1), minlength=E))
    assert per_r[0] == T
    _, put, total, per_exp, bal = zo.dispatch_notify(per_e[None, :], K)
    assert np.array_equal(put[0], np.concatenate([[0], np.cumsum(per_e)[:-1]]))
    assert total[0] == T * K and np.array_equal(per_exp, per_e.astype(np.int64))
    assert list(bal[0]) == [0, T - 1]
    rows = put[0][idx] + send
    assert sorted(rows.reshape(-1).tolist()) == list(range(T * K))


def test_notify_multi_rank_closed_form():
    R, E, K = 4, 16, 2
    counts = rng(9).integers(0, 20, size=(R, E)).astype(np.int32)
    counts[:, :] -= counts.sum(1, keepdims=True) % K == 1   # keep it arbitrary; only shapes matter
    counts = np.abs(counts)
    for me in range(R):
        recv, put, total, per_exp, bal = zo.dispatch_notify(counts, K, me)
        eloc = E // R
        assert np.array_equal(recv, counts)
        for r in range(R):
            seq = counts[:, r * eloc:(r + 1) * eloc].T.reshape(-1)          # le-major, src-minor
            assert np.array_equal(put[r].reshape(-1), np.concatenate([[0], np.cumsum(seq)[:-1]]))
        assert total[0] == counts[:, me * eloc:(me + 1) * eloc].sum()
        assert np.array_equal(per_exp, counts[:, me * eloc:(me + 1) * eloc].sum(0))


def test_low_latency_counts_over_ranks_closed_form():
    """zo_ll_counts against numpy: all_counts is a bincount per rank; every destination rank's block of ep_recv_counts
    is the inclusive cumsum of its local experts' counts taken expert by expert and, within one, source rank by
    source rank (starting at 0 for every rank); expert_token_nums are the column sums of the receiving rank's experts
    (type 1) or their running sum (type 0). At R = 1 the block is zo_dispatch_low_latency's ep_recv_counts."""
    R, T, K, E = 4, 37, 3, 16
    ids = rng(70).integers(-1, E + 1, size=(R, T, K)).astype(np.int32)
    e_loc = E // R
    want_all = np.stack([np.bincount(ids[s][(ids[s] >= 0) & (ids[s] < E)], minlength=E) for s in range(R)])
    for me in range(R):
        for typ in (0, 1):
            allc, recv, nums = zo.ll_counts(ids, E, me, typ)
            assert np.array_equal(allc, want_all)
            for r in range(R):
                seq = want_all[:, r * e_loc:(r + 1) * e_loc].T.reshape(-1)          # le-major, src-minor
                assert np.array_equal(recv[r * E:(r + 1) * E], np.cumsum(seq))
            per = want_all[:, me * e_loc:(me + 1) * e_loc].sum(0)
            assert np.array_equal(nums, np.cumsum(per) if typ == 0 else per)
    one = ids[:1]
    x = zo.f32_to_bf16(rng(71).standard_normal((T, 128)).astype(np.float32))
    _, _, eidx1, nums1, counts1 = zo.dispatch_low_latency(x, zo.DT_BF16, one[0], E, 0, T * K)
    allc, recv, nums = zo.ll_counts(one, E, 0, 1)
    assert np.array_equal(recv, counts1) and np.array_equal(nums, nums1)


def test_low_latency_dispatch_and_combine_over_ranks():
    """R ranks dispatch into R windows and combine back: every window ends up densely packed in (local expert,
    source rank, pick order) order with the rows of the tokens that picked the expert -- checked row by row against a
    direct construction --, no row is written twice, and combine(dispatch(x)) = x * sum of the valid picks' weights
    (the reference test's round trip, test_low_latency.py:146-155). At R = 1 both functions equal the one-rank ones."""
    R, T, H, K, E = 3, 29, 128, 4, 12
    e_loc = E // R
    ids = np.stack([np.stack([rng(80 + s * 100 + t).permutation(E + 2)[:K] - 1 for t in range(T)]) for s in range(R)]).astype(np.int32)
    xs = [zo.f32_to_bf16(rng(90 + s).standard_normal((T, H)).astype(np.float32)) for s in range(R)]
    ws = [rng(95 + s).uniform(0, 1, (T, K)).astype(np.float32) for s in range(R)]
    rows_cap = R * T * K
    win = np.zeros((R, rows_cap, H), dtype=np.uint16)
    scale = np.zeros((R, rows_cap), dtype=np.float32)
    _, recv, _ = zo.ll_counts(ids, E, 0)
    eidx = [zo.dispatch_low_latency_ranks(xs[s], zo.DT_BF16, ids[s], E, R, s, 0, recv, win, scale) for s in range(R)]
    for d in range(R):                       # direct construction of window d
        row = 0
        for le in range(e_loc):
            for s in range(R):
                for t in range(T):
                    for k in range(K):
                        if ids[s, t, k] == d * e_loc + le:
                            assert np.array_equal(win[d, row], xs[s][t]), (d, le, s, t, k)
                            row += 1
        assert not win[d, row:].any()
    for s in range(R):
        out = zo.combine_low_latency_ranks(win, zo.DT_BF16, ids[s], eidx[s], recv, ws[s], E, R, s)
        valid = (ids[s] >= 0) & (ids[s] < E)
        want = zo.bf16_to_f32(xs[s]) * (ws[s] * valid).sum(1, keepdims=True)
        got = zo.bf16_to_f32(out)
        for t in range(T):
            assert calc_diff(got[t], want[t]) < 1e-5
    # one rank: the general functions are the one-rank ones
    ex1, _, eidx1, _, counts1 = zo.dispatch_low_latency(xs[0], zo.DT_BF16, ids[0], E, 0, T * K)
    _, recv1, _ = zo.ll_counts(ids[:1], E, 0)
    w1 = np.zeros((1, T * K, H), dtype=np.uint16)
    e1 = zo.dispatch_low_latency_ranks(xs[0], zo.DT_BF16, ids[0], E, 1, 0, 0, recv1, w1, np.zeros((1, T * K), dtype=np.float32))
    assert np.array_equal(w1[0], ex1) and np.array_equal(e1, eidx1) and np.array_equal(recv1, counts1)
    assert np.array_equal(zo.combine_low_latency_ranks(w1, zo.DT_BF16, ids[0], e1, recv1, ws[0], E, 1, 0),
                          zo.combine_low_latency(ex1, zo.DT_BF16, ids[0], eidx1, counts1, ws[0], E))


# ---- quantising dispatch --------------------------------------------------------

def make_dispatch(T, H, K, E, seed):
    x32 = rng(seed).standard_normal((T, H)).astype(np.float32)
    x = zo.f32_to_bf16(x32)
    idx = np.stack([rng(seed * 1000 + t).permutation(E)[:K] for t in range(T)]).astype(np.int64)
    _, per_e, send = zo.dispatch_layout(idx, E, 1)
    _, put, _, _, _ = zo.dispatch_notify(per_e[None, :], K)
    return x, idx.astype(np.int32), send, put.reshape(-1), int(per_e.sum())


def test_dispatch_int8_closed_forms():
    T, H, K, E = 40, 256, 4, 8
    x, idx, send, put, rows = make_dispatch(T, H, K, E, 1)
    xf = zo.bf16_to_f32(x)
    xf[0, :] = 3.0; xf[1, :] = -0.5; xf[2, :] = 0.0
    x = zo.f32_to_bf16(xf)
    dest, scale = zo.dispatch_normal(x, zo.DT_BF16, idx, send, put, E, 1, rows)
    for t in range(T):
        for k in range(K):
            row = put[idx[t, k]] + send[t, k]
            amax = np.abs(xf[t]).max()
            # the permutation invariant: the row is the token's quantised form
            if amax > 0:
                assert np.all(np.abs(dest[row].astype(np.float32) * scale[row] - xf[t]) <= scale[row] * 0.5 + 1e-6 * amax)
                assert np.isclose(scale[row], amax / 127.0, rtol=3e-7)
                assert np.abs(dest[row]).max() == 127
    r0 = put[idx[0, 0]] + send[0, 0]
    assert np.all(dest[r0] == 127)
    r1 = put[idx[1, 0]] + send[1, 0]
    assert np.all(dest[r1] == -127)
    r2 = put[idx[2, 0]] + send[2, 0]
    assert np.all(dest[r2] == 0) and scale[r2] < 1e-13    # the 1e-12 epsilon keeps it finite


def test_dispatch_int8_matches_numpy_float32_formula():
    T, H, K, E = 64, 512, 2, 8
    x, idx, send, put, rows = make_dispatch(T, H, K, E, 2)
    xf = zo.bf16_to_f32(x)
    dest, scale = zo.dispatch_normal(x, zo.DT_BF16, idx, send, put, E, 1, rows)
    amax = np.abs(xf).max(1)
    s = (np.float32(127.0) / (amax + np.float32(1e-12))).astype(np.float32)
    q = np.rint(xf * s[:, None]).astype(np.int8)       # numpy rint is half-to-even, float32 product
    inv = (np.float32(1.0) / s).astype(np.float32)
    for t in range(T):
        for k in range(K):
            row = put[idx[t, k]] + send[t, k]
            assert np.array_equal(dest[row], q[t]) and scale[row] == inv[t]


def test_dispatch_fp8_block_scales_match_torch():
    T, H, K, E = 16, 512, 2, 4
    x, idx, send, put, rows = make_dispatch(T, H, K, E, 3)
    xf = zo.bf16_to_f32(x)
    dest, scale = zo.dispatch_normal(x, zo.DT_BF16, idx, send, put, E, 2, rows)
    xb = xf.reshape(T, H // 128, 128)
    amax = np.maximum(np.abs(xb).max(2), np.float32(1e-4))
    mult = (np.float32(448.0) / amax).astype(np.float32)
    q = torch.from_numpy(np.clip(xb * mult[:, :, None], -448, 448)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    sc = (amax * np.float32(1.0 / 448.0)).astype(np.float32)
    for t in range(T):
        for k in range(K):
            row = put[idx[t, k]] + send[t, k]
            assert np.array_equal(dest[row], q[t].reshape(-1)) and np.array_equal(scale[row], sc[t])
    # the decode the reference's helper performs (utils.py:118-126) recovers x to e4m3 precision
    back = zo.e4m3_to_f32(dest).reshape(rows, H // 128, 128) * scale[:, :, None]
    row = put[idx[5, 1]] + send[5, 1]
    assert np.allclose(back[row].reshape(-1), xf[5], rtol=0.07, atol=1e-3)


def calc_diff(x, y):
    """Reference metric, test/python/deepep/utils.py:129-133."""
    x = x.astype(np.float64) + 1
    y = y.astype(np.float64) + 1
    return 1 - 2 * (x * y).sum() / (x * x + y * y).sum()


def test_combine_round_trip_identity_expert():
    """Reference check test_normal.py:225-236: combine(dispatch(x)) = x * sum_k w."""
    T, H, K, E = 48, 256, 4, 8
    x, idx, send, put, rows = make_dispatch(T, H, K, E, 4)
    w = rng(7).uniform(0.1, 1.0, size=(T, K)).astype(np.float32)
    dest, _ = zo.dispatch_normal(x, zo.DT_BF16, idx, send, put, E, 0, rows)
    out = zo.combine(dest, zo.DT_BF16, put, w, idx, send, E)
    want = zo.bf16_to_f32(x) * w.sum(1, keepdims=True)
    assert calc_diff(zo.bf16_to_f32(out), want) < 5e-5
    # exact value: sequential fp32 multiply-then-add, one rounding
    xf = zo.bf16_to_f32(x)
    acc = np.zeros((T, H), dtype=np.float32)
    for k in range(K):
        acc = acc + (xf * w[:, k:k + 1]).astype(np.float32)
    assert np.array_equal(out, zo.f32_to_bf16(acc))


def test_combine_skips_invalid():
    T, H, K, E = 8, 128, 2, 4
    x, idx, send, put, rows = make_dispatch(T, H, K, E, 5)
    idx2 = idx.copy(); idx2[:, 1] = -1
    _, per_e, send2 = zo.dispatch_layout(idx2.astype(np.int64), E, 1)
    put2 = np.concatenate([[0], np.cumsum(per_e)[:-1]]).astype(np.int32)
    dest, _ = zo.dispatch_normal(x, zo.DT_BF16, idx2, send2, put2, E, 0, int(per_e.sum()))
    w = np.ones((T, K), dtype=np.float32)
    out = zo.combine(dest, zo.DT_BF16, put2, w, idx2, send2, E)
    assert np.array_equal(out, x)


def test_low_latency_dispatch_combine():
    T, H, K, E = 32, 256, 4, 16
    x, idx, send, put, rows = make_dispatch(T, H, K, E, 6)
    ex, sc, eidx, nums, counts = zo.dispatch_low_latency(x, zo.DT_BF16, idx, E, 1, rows, token_nums_type=1)
    per_e = np.bincount(idx.reshape(-1), minlength=E)
    assert np.array_equal(nums, per_e) and np.array_equal(counts, np.cumsum(per_e)) and np.array_equal(eidx, send)
    _, _, _, nums0, _ = zo.dispatch_low_latency(x, zo.DT_BF16, idx, E, 1, rows, token_nums_type=0)
    assert np.array_equal(nums0, np.cumsum(per_e))
    xf = zo.bf16_to_f32(x)
    s = np.float32(127.0) / np.abs(xf).max(1)
    for t in range(T):
        row = put[idx[t, 0]] + send[t, 0]
        assert np.array_equal(ex[row], np.rint(xf[t] * s[t]).astype(np.int8)) and sc[row] == np.float32(1.0) / s[t]
    exb, _, eidx, _, counts = zo.dispatch_low_latency(x, zo.DT_BF16, idx, E, 0, rows)
    w = rng(8).uniform(0.1, 1, size=(T, K)).astype(np.float32)
    out = zo.combine_low_latency(exb, zo.DT_BF16, idx, eidx, counts, w, E)
    assert calc_diff(zo.bf16_to_f32(out), xf * w.sum(1, keepdims=True)) < 1e-5   # test_low_latency.py:146-155


# ---- grouped GEMMs ---------------------------------------------------------------

def ragged_counts(E, rows, seed):
    c = rng(seed).multinomial(rows, np.ones(E) / E).astype(np.int64)
    c[rng(seed + 1).integers(0, E)] += c[0]; c[0] = 0        # one empty expert
    return c


def test_w8a8_gemm_against_numpy_matmul():
    E, K, N, rows = 4, 256, 128, 70
    counts = ragged_counts(E, rows, 10)
    a = rng(11).integers(-127, 128, size=(rows, K)).astype(np.int8)
    w = rng(12).integers(-16, 16, size=(E, K, N)).astype(np.int8)
    xs = rng(13).uniform(0.01, 0.05, rows).astype(np.float32)
    ws = rng(14).uniform(0.0015, 0.0045, (E, N)).astype(np.float32)
    y = zo.grouped_gemm_w8a8_dequant(a, xs, w, ws, counts)
    off = np.concatenate([[0], np.cumsum(counts)])
    for g in range(E):
        sl = slice(off[g], off[g + 1])
        c = a[sl].astype(np.int64) @ w[g].astype(np.int64)
        d = (c.astype(np.float32) * ws[g][None, :]) * xs[sl][:, None]
        assert np.array_equal(y[sl], zo.f32_to_bf16(d))
    ws16 = zo.f32_to_bf16(ws)
    y2 = zo.grouped_gemm_w8a8_dequant(a, xs, w, ws16, counts)
    g = 1; sl = slice(off[g], off[g + 1])
    d = ((a[sl].astype(np.int64) @ w[g].astype(np.int64)).astype(np.float32) * zo.bf16_to_f32(ws16[g])[None, :]) * xs[sl][:, None]
    assert np.array_equal(y2[sl], zo.f32_to_bf16(d))


def test_gmm1_swiglu_quant_w8a8_against_float64():
    E, K, N1, rows = 3, 128, 256, 40
    counts = ragged_counts(E, rows, 20)
    a = rng(21).integers(-127, 128, size=(rows, K)).astype(np.int8)
    w = rng(22).integers(-16, 16, size=(E, K, N1)).astype(np.int8)
    xs = rng(23).uniform(0.01, 0.05, rows).astype(np.float32)
    ws = rng(24).uniform(0.0015, 0.0045, (E, N1)).astype(np.float32)
    q2, s2, sgl = zo.gmm1_swiglu_quant_w8a8(a, xs, w, ws, counts, want_sgl=True)
    off = np.concatenate([[0], np.cumsum(counts)])
    I = N1 // 2
    for g in range(E):
        sl = slice(off[g], off[g + 1])
        d = (a[sl].astype(np.float64) @ w[g].astype(np.float64)) * ws[g][None, :] * xs[sl][:, None]
        ref = d[:, :I] / (1 + np.exp(-d[:, :I])) * d[:, I:]
        assert np.allclose(sgl[sl], ref, rtol=2e-6, atol=1e-30)
        mx = np.abs(sgl[sl]).max(1)
        assert np.allclose(s2[sl], mx / 127, rtol=3e-7)
        assert np.all(np.abs(q2[sl]).max(1) == 127)
        assert np.all(np.abs(q2[sl].astype(np.float64) - ref * 127 / mx[:, None]) <= 0.5 + 1e-3)


def test_fp8_block_gemm_against_float64():
    E, K, N1, rows = 2, 256, 256, 24
    counts = np.array([10, 14], dtype=np.int64)
    a = zo.f32_to_e4m3(rng(31).uniform(-300, 300, (rows, K)).astype(np.float32))
    sa = rng(32).uniform(0.001, 0.01, (rows, K // 128)).astype(np.float32)
    w = zo.f32_to_e4m3(rng(33).uniform(-200, 200, (E, K, N1)).astype(np.float32))
    sw = rng(34).uniform(0.0005, 0.002, (E, K // 128, N1 // 128)).astype(np.float32)
    q2, s2, sgl = zo.gmm1_swiglu_quant_fp8(a, sa, w, sw, counts, want_sgl=True)
    af = zo.e4m3_to_f32(a).astype(np.float64)
    wf = zo.e4m3_to_f32(w).astype(np.float64)
    off = np.concatenate([[0], np.cumsum(counts)])
    I = N1 // 2
    for g in range(E):
        sl = slice(off[g], off[g + 1])
        A = af[sl] * np.repeat(sa[sl], 128, axis=1)
        W = wf[g] * np.repeat(np.repeat(sw[g], 128, axis=0), 128, axis=1)
        d = A @ W
        ref = d[:, :I] / (1 + np.exp(-d[:, :I])) * d[:, I:]
        assert np.allclose(sgl[sl], ref, rtol=1e-4, atol=1e-4 * np.abs(ref).max())
        back = zo.e4m3_to_f32(q2[sl]).reshape(-1, I // 128, 128) * s2[sl][:, :, None]
        assert np.allclose(back.reshape(-1, I), ref, rtol=0.07, atol=np.abs(ref).max() * 2e-3)
    # GMM2 on the same operands (out = bf16 of the block-scaled product)
    y = zo.gmm2_fp8(a, sa, w, sw, counts)
    g = 1; sl = slice(off[g], off[g + 1])
    d = (af[sl] * np.repeat(sa[sl], 128, axis=1)) @ (wf[g] * np.repeat(np.repeat(sw[g], 128, axis=0), 128, axis=1))
    assert np.allclose(zo.bf16_to_f32(y[sl]), d, rtol=1e-2, atol=1e-2 * np.abs(d).max())


def test_w4a8_gemm_against_float64():
    E, K, N1, rows = 2, 256, 256, 20
    counts = np.array([7, 13], dtype=np.int64)
    a = rng(41).integers(-127, 128, size=(rows, K)).astype(np.int8)
    w = rng(42).integers(-8, 8, size=(E, K, N1)).astype(np.int8)
    gs = zo.f32_to_fp16(rng(43).uniform(0.002, 0.01, (E, K // 128, N1)).astype(np.float32))
    xs = rng(44).uniform(0.01, 0.05, rows).astype(np.float32)
    y = zo.gmm2_w4a8(a, xs, w, gs, counts)
    off = np.concatenate([[0], np.cumsum(counts)])
    for g in range(E):
        sl = slice(off[g], off[g + 1])
        W = w[g].astype(np.float64) * np.repeat(zo.fp16_to_f32(gs[g]).astype(np.float64), 128, axis=0)
        d = (a[sl].astype(np.float64) @ W) * xs[sl][:, None]
        assert np.allclose(zo.bf16_to_f32(y[sl]), d, rtol=1e-2, atol=1e-2 * np.abs(d).max())
    q2, s2, sgl = zo.gmm1_swiglu_quant_w4a8(a, xs, w, gs, counts, want_sgl=True)
    g = 0; sl = slice(off[g], off[g + 1]); I = N1 // 2
    W = w[g].astype(np.float64) * np.repeat(zo.fp16_to_f32(gs[g]).astype(np.float64), 128, axis=0)
    d = (a[sl].astype(np.float64) @ W) * xs[sl][:, None]
    ref = d[:, :I] / (1 + np.exp(-d[:, :I])) * d[:, I:]
    assert np.allclose(sgl[sl], ref, rtol=1e-4, atol=1e-5 * np.abs(ref).max())


def test_fused_moe_w8a8_identity_like_properties():
    """Whole layer: counts exact; scaling every routing weight by c scales the output by c (linearity of
    the combine); a token routed twice to the same weights doubles its contribution."""
    T, H, K, E, I = 24, 128, 2, 4, 64
    x = zo.f32_to_bf16(rng(50).uniform(-5, 5, (T, H)).astype(np.float32))
    ids = np.stack([rng(51 + t).permutation(E)[:K] for t in range(T)]).astype(np.int32)
    w1 = rng(52).integers(-16, 16, size=(E, H, 2 * I)).astype(np.int8)
    s1 = rng(53).uniform(0.0015, 0.0045, (E, 2 * I)).astype(np.float32)
    w2 = rng(54).integers(-16, 16, size=(E, I, H)).astype(np.int8)
    s2 = zo.f32_to_bf16(rng(55).uniform(0.0015, 0.0045, (E, H)).astype(np.float32))
    es = rng(56).uniform(0, 1, (T, K)).astype(np.float32)
    out, counts, st = zo.fused_moe(x, zo.DT_BF16, ids, es, w1, s1, w2, s2, E, 0, stages=True)
    assert np.array_equal(counts, np.bincount(ids.reshape(-1), minlength=E))
    out2, _ = zo.fused_moe(x, zo.DT_BF16, ids, es * 2, w1, s1, w2, s2, E, 0)
    assert np.array_equal(zo.bf16_to_f32(out2), zo.bf16_to_f32(out) * 2)          # power-of-two scaling is exact
    # float64 model of the whole layer from the oracle's own quantised stages' inputs
    xf = zo.bf16_to_f32(x).astype(np.float64)
    ref = np.zeros((T, H))
    for t in range(T):
        for k in range(K):
            e = ids[t, k]
            amax = np.abs(xf[t]).max()
            q = np.rint(xf[t] * (127 / amax))
            d = (q @ w1[e].astype(np.float64)) * s1[e] * (amax / 127)
            sg = d[:I] / (1 + np.exp(-d[:I])) * d[I:]
            mx = np.abs(sg).max()
            q2 = np.rint(sg * 127 / mx)
            y = (q2 @ w2[e].astype(np.float64)) * zo.bf16_to_f32(s2[e]) * (mx / 127)
            ref[t] += es[t, k] * y
    assert calc_diff(zo.bf16_to_f32(out), ref) < 1e-4


# ---- reduce ------------------------------------------------------------------------

@pytest.mark.parametrize("op,fn", [(1, np.add), (2, np.maximum), (3, np.minimum), (0, np.multiply)])
def test_reduce_fp32_and_ints(op, fn):
    bufs = [rng(60 + p).uniform(0, 10, 1000).astype(np.float32) for p in range(8)]   # reference generator: uniform(0,10)
    out = zo.reduce(bufs, zo.DT_FP32, op)
    ref = bufs[0].copy()
    for b in bufs[1:]:
        ref = fn(ref, b).astype(np.float32)
    assert np.array_equal(out, ref)
    if op == 1:
        assert np.allclose(out, np.sum(np.stack(bufs).astype(np.float64), 0), rtol=1e-6)
    ib = [rng(70 + p).integers(-50, 50, 1000).astype(np.int32) for p in range(5)]
    out = zo.reduce(ib, zo.DT_INT32, op)
    ref = ib[0].copy()
    for b in ib[1:]:
        ref = fn(ref, b)
    assert np.array_equal(out, ref.astype(np.int32))


def test_reduce_bf16_single_rounding():
    bufs32 = [rng(80 + p).standard_normal(4096).astype(np.float32) for p in range(8)]
    bufs = [zo.f32_to_bf16(b) for b in bufs32]
    out = zo.reduce(bufs, zo.DT_BF16, 1)
    acc = zo.bf16_to_f32(bufs[0])
    for b in bufs[1:]:
        acc = (acc + zo.bf16_to_f32(b)).astype(np.float32)
    assert np.array_equal(out, zo.f32_to_bf16(acc))
    # reference golden rule (test_zbal_allreduce.py:48-58): sum of all ranks' inputs, rtol 1e-4 in its dtype
    tot = np.sum(np.stack([zo.bf16_to_f32(b) for b in bufs]).astype(np.float64), 0)
    assert np.allclose(zo.bf16_to_f32(out), tot, rtol=1e-2, atol=2e-2)
    h = [zo.f32_to_fp16(b) for b in bufs32[:2]]
    o = zo.reduce(h, zo.DT_FP16, 1)
    assert np.array_equal(o, (h[0].view(np.float16).astype(np.float32) + h[1].view(np.float16).astype(np.float32)).astype(np.float16).view(np.uint16))


# ---- branch-level pins: smooth scales, all-zero rows, the fused permute, integer wrap-around, half max/min/prod ----

def _np_quant_int8_noeps(v):
    """numpy float32 restatement of the eps-less per-token quantisation: s = 127/amax, q = rint(v*s), scale = 1/s;
    an all-zero row gives q = 0, scale = 0. Every product is rounded to float32, as separate operations."""
    amax = np.abs(v).max()
    if amax == 0:
        return np.zeros(v.shape, np.int8), np.float32(0)
    s = np.float32(127.0) / amax
    q = np.clip(np.rint((v * s).astype(np.float32)), -128, 127).astype(np.int8)
    return q, np.float32(1.0) / s


def test_fused_permute_quant_rows_smooth_scales_and_zero_rows():
    T, H, K, E = 37, 256, 3, 6
    g = rng(200)
    xf = g.standard_normal((T, H)).astype(np.float32) * 3
    xf[5] = 0.0                                   # an all-zero token: q = 0, scale = 0 (no division by zero)
    x = zo.f32_to_bf16(xf)
    xv = zo.bf16_to_f32(x)
    ids = g.integers(-1, E + 1, size=(T, K)).astype(np.int32)      # some ids invalid
    smooth = g.uniform(0.25, 2.0, (E, H)).astype(np.float32)
    smooth[2, :] = 0.0                            # smoothing can zero a row too
    for sm in (None, smooth):
        q1, xs, eidx, counts = zo.fused_permute_quant(x, zo.DT_BF16, ids, sm, E, 1)
        # permutation: expert-major, flat-pick order inside an expert (numpy stable sort of the valid picks)
        flat = ids.reshape(-1)
        valid = np.flatnonzero((flat >= 0) & (flat < E))
        order = valid[np.argsort(flat[valid], kind="stable")]
        assert np.array_equal(counts, np.bincount(flat[valid], minlength=E))
        assert q1.shape[0] == len(order)
        for row, pick in enumerate(order):
            t, e = pick // K, flat[pick]
            v = xv[t] if sm is None else (xv[t] * sm[e]).astype(np.float32)
            q, sc = _np_quant_int8_noeps(v)
            assert np.array_equal(q1[row], q), (row, t, e)
            assert xs[row].view(np.uint32) == sc.view(np.uint32), (row, t, e)
            assert eidx.reshape(-1)[pick] == np.sum(flat[:pick] == e)
        assert np.all(eidx.reshape(-1)[(flat < 0) | (flat >= E)] == -1)
        zero_rows = [r for r, pick in enumerate(order) if pick // K == 5 or (sm is not None and flat[pick] == 2)]
        assert zero_rows and all(xs[r] == 0 and not q1[r].any() for r in zero_rows)


def test_fused_permute_quant_fp8_rows_match_torch_cast():
    T, H, K, E = 19, 256, 2, 4
    g = rng(201)
    x = zo.f32_to_bf16(g.standard_normal((T, H)).astype(np.float32))
    xv = zo.bf16_to_f32(x)
    ids = g.integers(0, E, size=(T, K)).astype(np.int32)
    q1, xs, _, _ = zo.fused_permute_quant(x, zo.DT_BF16, ids, None, E, 2)
    flat = ids.reshape(-1)
    order = np.argsort(flat, kind="stable")
    for row, pick in enumerate(order):
        v = xv[pick // K].reshape(H // 128, 128)
        amax = np.maximum(np.abs(v).max(1), np.float32(1e-4))
        scaled = (v * (np.float32(448.0) / amax)[:, None]).astype(np.float32)
        want = torch.from_numpy(np.clip(scaled, -448, 448)).to(torch.float8_e4m3fn).view(torch.uint8).numpy().reshape(-1)
        assert np.array_equal(q1[row], want)
        assert np.array_equal(xs[row].view(np.uint32), (amax * np.float32(1.0 / 448.0)).astype(np.float32).view(np.uint32))


@pytest.mark.parametrize("dt,npdt", [(0, np.int8), (1, np.int16), (3, np.int64)])
def test_reduce_integers_wrap_around(dt, npdt):
    info = np.iinfo(npdt)
    g = rng(210 + dt)
    bufs = [g.integers(info.min, info.max, 2000, dtype=npdt, endpoint=True) for _ in range(6)]
    with np.errstate(over="ignore"):
        s = bufs[0].copy()
        p = bufs[0].copy()
        for b in bufs[1:]:
            s = (s + b).astype(npdt)              # numpy integer arithmetic is modular
            p = (p * b).astype(npdt)
    assert np.array_equal(zo.reduce(bufs, dt, 1), s)
    assert np.array_equal(zo.reduce(bufs, dt, 0), p)
    assert np.array_equal(zo.reduce(bufs, dt, 2), np.max(np.stack(bufs), 0))
    assert np.array_equal(zo.reduce(bufs, dt, 3), np.min(np.stack(bufs), 0))
    # the exact sum modulo 2^bits, computed with Python integers
    bits = info.bits
    exact = [(sum(int(b[i]) for b in bufs) + (1 << (bits - 1))) % (1 << bits) - (1 << (bits - 1)) for i in range(50)]
    assert list(zo.reduce(bufs, dt, 1)[:50]) == exact


@pytest.mark.parametrize("dt,to16,from16", [(zo.DT_BF16, zo.f32_to_bf16, zo.bf16_to_f32), (zo.DT_FP16, zo.f32_to_fp16, zo.fp16_to_f32)])
def test_reduce_halves_max_min_prod(dt, to16, from16):
    g = rng(220)
    bufs = [to16(g.uniform(0.5, 1.5, 3000).astype(np.float32) * g.choice([-1.0, 1.0], 3000).astype(np.float32)) for _ in range(5)]
    vals = np.stack([from16(b) for b in bufs])
    assert np.array_equal(zo.reduce(bufs, dt, 2), to16(vals.max(0)))          # max / min of representable values: no rounding
    assert np.array_equal(zo.reduce(bufs, dt, 3), to16(vals.min(0)))
    acc = vals[0].copy()
    for v in vals[1:]:
        acc = (acc * v).astype(np.float32)        # fp32 running product in buffer order, one rounding at the end
    assert np.array_equal(zo.reduce(bufs, dt, 0), to16(acc))
