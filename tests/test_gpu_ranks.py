"""Normal-mode dispatch over a group of R modelled ranks on one GPU: every rank has a window (a local
allocation registered with zbal_comm_register_peer_window) that holds its tensors at the same offsets as every
other rank's, notify reads the peers' counts from their windows, dispatch writes each row into the window of the
rank that owns the expert, and combine reads the rows back from there. Checked against the CPU oracle run with the
same R and rank (bit for bit), through the zbal C ABI and, with the same windows, through the ZBALOp* launcher
functions the reference's communicator layer calls (include/zbal_amd_operators.h), which find the peers through a
CommGroupInfo instead of registered windows."""
import ctypes

import numpy as np
import pytest
import torch

from memfabric_hybrid_amd import capi
from memfabric_hybrid_amd.operators import OperatorBuffer as Buffer, create_group, destroy_group
from oracle import oracle as zo
from zbal_testlib import bf16_normal, host, rng

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def buf():
    b = Buffer()
    yield b
    torch.cuda.synchronize()
    b.close()


class Window:
    """One rank's window: a slice of one allocation (the windows follow each other at a fixed stride, as the ranks'
    memories do in the reference's symmetric address space), carved into named tensors at offsets that are the same
    in every window."""

    @staticmethod
    def make(layout, ranks):
        size = sum((n + 255) // 256 * 256 for _, n, _ in layout)
        whole = torch.zeros(size * ranks, dtype=torch.uint8, device="cuda")
        return [Window(layout, whole[r * size:(r + 1) * size]) for r in range(ranks)]

    def __init__(self, layout, mem):
        self.size = mem.numel()
        self.mem = mem
        self.views = {}
        off = 0
        for name, nbytes, dtype in layout:
            self.views[name] = self.mem[off:off + nbytes].view(dtype)
            off += (nbytes + 255) // 256 * 256

    def __getitem__(self, name):
        return self.views[name]


class OuterAbi:
    """zbal_* entry points on one communicator per modelled rank, the windows registered with each."""

    def __init__(self, lib, wins, tag):
        self.lib, self.R = lib, len(wins)
        self.comms = [create_group("ep%s_%d" % (tag, r), self.R, r) for r in range(self.R)]
        if self.R > 1:
            for c in self.comms:
                for r in range(self.R):
                    assert lib.zbal_comm_register_peer_window(c, r, wins[r].mem.data_ptr(), wins[r].size) == 0

    def close(self):
        for c in self.comms:
            destroy_group(c)

    def layout(self, r, *a):
        return self.lib.zbal_dispatch_normal_layout(*a, self.comms[r], capi.stream_ptr(), 0)

    def notify(self, r, *a):
        return self.lib.zbal_dispatch_normal_notify(*a, self.comms[r], capi.stream_ptr(), 0)

    def dispatch(self, r, *a):
        return self.lib.zbal_dispatch_normal(*a, self.comms[r], capi.stream_ptr(), 0)

    def combine(self, r, *a):
        return self.lib.zbal_combine_normal(*a, self.comms[r], capi.stream_ptr(), 0)

    def ll_dispatch(self, r, *a):
        return self.lib.zbal_dispatch_low_latency(*a, self.comms[r], capi.stream_ptr(), 0)

    def ll_combine(self, r, *a):
        return self.lib.zbal_combine_low_latency(*a, self.comms[r], capi.stream_ptr(), 0)


class KernelSeam:
    """ZBALOp* launchers with a CommGroupInfo per modelled rank: the peers are localDeviceMemSize bytes apart."""

    def __init__(self, lib, wins, tag):
        self.fn = capi.load_cxx()
        self.infos = []
        for r in range(len(wins)):
            g = capi.CommGroupInfo()
            g.groupSize, g.myGroupRank, g.localDeviceMemSize = len(wins), r, wins[0].size
            for i in range(len(wins)):
                g.peerGroupRank2WorldRank[i] = i
            self.infos.append(g)

    def close(self):
        pass

    def layout(self, r, *a):
        return self.fn["ZBALOpDispatchLayout"](*a, capi.stream_ptr(), ctypes.byref(self.infos[r]), 0)

    def notify(self, r, *a):
        return self.fn["ZBALOpNotifyDispatch"](*a, 1.2, 0.8, capi.stream_ptr(), ctypes.byref(self.infos[r]), 0)

    def dispatch(self, r, *a):
        return self.fn["ZBALOpDispatchNormal"](*a, False, capi.stream_ptr(), ctypes.byref(self.infos[r]), 0)

    def combine(self, r, *a):
        return self.fn["ZBALOpCombineNormal"](*a, False, capi.stream_ptr(), ctypes.byref(self.infos[r]), 0)

    def ll_dispatch(self, r, *a):
        return self.fn["ZBALOpDispatchLowLatency"](*a, capi.stream_ptr(), ctypes.byref(self.infos[r]), 0)

    def ll_combine(self, r, *a):
        return self.fn["ZBALOpCombineLowLatency"](*a, capi.stream_ptr(), ctypes.byref(self.infos[r]), 0)


@pytest.mark.parametrize("api_cls", [OuterAbi, KernelSeam])
@pytest.mark.parametrize("R,quant", [(4, capi.NO_QUANT), (4, capi.QUANT_INT8), (2, capi.QUANT_FP8_B128), (1, capi.QUANT_INT8)])
def test_dispatch_and_combine_over_modelled_ranks(buf, R, quant, api_cls):
    run_modelled_ranks(buf, R, quant, api_cls, 96, 4, 16, 256)


@pytest.mark.parametrize("R,quant,T,K,E,H", [(16, capi.QUANT_INT8, 40, 8, 32, 512),       # the most ranks the tables hold
                                             (8, capi.NO_QUANT, 1, 1, 8, 128),            # one token, one expert per rank
                                             (2, capi.QUANT_FP8_B128, 700, 3, 6, 1024),   # more picks than one layout block ranks at once
                                             (3, capi.NO_QUANT, 257, 8, 48, 7168)])       # odd rank count, full hidden size
def test_modelled_ranks_other_shapes(buf, R, quant, T, K, E, H):
    run_modelled_ranks(buf, R, quant, OuterAbi, T, K, E, H)


def run_modelled_ranks(buf, R, quant, api_cls, T, K, E, H):
    lib = buf.lib
    rows_cap = R * T * K                      # what a window's receive tensors hold: every pick of every rank
    ti = capi.tensor_info
    ref = ctypes.byref
    st = capi.stream_ptr()
    qbytes = 2 if quant == capi.NO_QUANT else 1
    scales_per_row = {capi.NO_QUANT: 1, capi.QUANT_INT8: 1, capi.QUANT_FP8_B128: H // 128}[quant]
    layout = [("counts", E * 4, torch.int32), ("recv_x", rows_cap * H * qbytes, torch.uint8),
              ("recv_scale", rows_cap * scales_per_row * 4, torch.float32), ("expert_out", rows_cap * H * 2, torch.bfloat16)]
    wins = Window.make(layout, R)
    api = api_cls(lib, wins, "%d_%d_%d_%d" % (R, quant, T, H))
    try:
        # ---- every rank: layout of its own batch (counts land in its window)
        xs, idx, send_idx, w = [], [], [], []
        for r in range(R):
            x = bf16_normal((T, H), 40 + r)
            ids = rng(50 + r).integers(-1, E + 1, size=(T, K)).astype(np.int64)
            xs.append(x); idx.append(ids); w.append(rng(60 + r).uniform(0, 1, (T, K)).astype(np.float32))
            d_idx = torch.from_numpy(ids).cuda()
            per_rank = torch.empty(R, dtype=torch.int32, device="cuda")
            sidx = torch.empty((T, K), dtype=torch.int32, device="cuda")
            scratch = torch.empty(50 * E, dtype=torch.int32, device="cuda")
            assert api.layout(r, ref(ti(d_idx)), T, E, K, ref(ti(per_rank)), ref(ti(wins[r]["counts"])), ref(ti(sidx)),
                              ref(ti(scratch))) == 0
            r_rank, r_exp, r_send = zo.dispatch_layout(ids, E, R)
            assert np.array_equal(host(per_rank), r_rank) and np.array_equal(host(wins[r]["counts"]), r_exp)
            assert np.array_equal(host(sidx), r_send)
            send_idx.append(sidx)
        counts_all = np.stack([host(wins[r]["counts"]) for r in range(R)])
        # ---- every rank: notify (reads all windows), then dispatch (writes all windows)
        put, want_rows = [], [None] * R
        for r in range(R):
            recv = torch.empty((R, E), dtype=torch.int32, device="cuda")
            total = torch.empty(1, dtype=torch.int32, device="cuda")
            per_exp = torch.empty(E // R, dtype=torch.int64, device="cuda")
            off = torch.empty(R * E, dtype=torch.int32, device="cuda")
            bal = torch.empty((R, 2 * R), dtype=torch.int32, device="cuda")
            assert api.notify(r, ref(ti(wins[r]["counts"])), E, K, ref(ti(recv)), ref(ti(total)), ref(ti(per_exp)), ref(ti(off)),
                              ref(ti(bal))) == 0
            o_recv, o_put, o_total, o_per, o_bal = zo.dispatch_notify(counts_all, K, r)
            assert np.array_equal(host(recv), o_recv) and np.array_equal(host(off), o_put.reshape(-1))
            assert np.array_equal(host(total), o_total) and np.array_equal(host(per_exp), o_per)
            assert np.array_equal(host(bal), o_bal)
            put.append(off)
        for r in range(R):
            ids32 = torch.from_numpy(idx[r].astype(np.int32)).cuda()
            x_d = torch.from_numpy(xs[r]).view(torch.int16).view(torch.bfloat16).cuda()
            recv_dt = {capi.NO_QUANT: capi.DT_BF16, capi.QUANT_INT8: capi.DT_INT8, capi.QUANT_FP8_B128: capi.DT_FP8_E4M3}[quant]
            recv_ti = ti(wins[r]["recv_x"], dtype=recv_dt, shape=(rows_cap, H))
            assert api.dispatch(r, ref(ti(x_d)), ref(ti(ids32)), ref(ti(send_idx[r])), ref(ti(put[r])), ref(ti(put[r])), E, quant,
                                ref(recv_ti), ref(ti(wins[r]["recv_scale"]))) == 0
        torch.cuda.synchronize()
        # ---- the oracle: rank r's picks of the experts that rank d owns land in window d
        e_loc = E // R
        for d in range(R):
            shape = (rows_cap, H)
            want_x = np.zeros(shape, dtype=np.uint16 if quant == capi.NO_QUANT else np.uint8)
            want_s = np.zeros((rows_cap, scales_per_row), dtype=np.float32)
            for r in range(R):
                ids_d = np.where(idx[r] // e_loc == d, idx[r], -1).astype(np.int32)
                o_put = zo.dispatch_notify(counts_all, K, r)[1].reshape(-1)
                gx, gs = zo.dispatch_normal(xs[r], zo.DT_BF16, ids_d, host(send_idx[r]), o_put, E, quant, rows_cap, R, r)
                gx = gx.view(want_x.dtype)
                touched = np.zeros(rows_cap, dtype=bool)
                for t in range(T):
                    for k in range(K):
                        if ids_d[t, k] >= 0 and ids_d[t, k] < E:
                            touched[o_put[ids_d[t, k] * R + r] + host(send_idx[r])[t, k]] = True
                want_x[touched] = gx.reshape(shape)[touched]
                if quant != capi.NO_QUANT:
                    want_s[touched] = gs.reshape(rows_cap, scales_per_row)[touched]
            n_rows = int(counts_all[:, d * e_loc:(d + 1) * e_loc].sum())
            got_x = host(wins[d]["recv_x"]).reshape(rows_cap, H * qbytes)
            got_x = got_x.view(np.uint16) if quant == capi.NO_QUANT else got_x
            assert np.array_equal(got_x[:n_rows], want_x[:n_rows]), "rows in window %d" % d
            if quant != capi.NO_QUANT:
                got_s = host(wins[d]["recv_scale"]).reshape(rows_cap, scales_per_row)
                assert np.array_equal(got_s[:n_rows].view(np.uint32), want_s[:n_rows].view(np.uint32)), "scales in window %d" % d
            want_rows[d] = n_rows
        # ---- combine: identity experts on the un-quantised rows (the reference's round trip, test_normal.py:225-236)
        if quant == capi.NO_QUANT:
            for d in range(R):
                wins[d]["expert_out"][:rows_cap * H].copy_(wins[d]["recv_x"].view(torch.bfloat16))
            for r in range(R):
                ids32 = torch.from_numpy(idx[r].astype(np.int32)).cuda()
                out = torch.empty((T, H), dtype=torch.bfloat16, device="cuda")
                src_ti = ti(wins[r]["expert_out"], shape=(rows_cap, H))
                assert api.combine(r, ref(src_ti), ref(ti(put[r])), ref(ti(torch.from_numpy(w[r]).cuda())), ref(ti(ids32)),
                                   ref(ti(send_idx[r])), ref(ti(put[r])), E, ref(ti(out))) == 0
                valid = (idx[r] >= 0) & (idx[r] < E)
                # every window holds x rows bit for bit, so the oracle's combine of one concatenated buffer is the model
                acc = np.zeros((T, H), dtype=np.float32)
                xf = zo.bf16_to_f32(xs[r])
                for k in range(K):
                    term = (xf * w[r][:, k:k + 1]).astype(np.float32)
                    acc = np.where(valid[:, k:k + 1], (acc + term).astype(np.float32), acc)
                assert np.array_equal(host(out), zo.f32_to_bf16(acc)), "combine of rank %d" % r
    finally:
        torch.cuda.synchronize()
        api.close()


def test_reduce_scatter_and_low_latency_through_the_kernel_seam(buf):
    """ZBALOpReduceScatter over four slices of one allocation (bit-exact against the oracle, waitSymbol bumped) and the
    low-latency pair on a group of one, against the outer ABI's results for the same inputs."""
    fn = capi.load_cxx()
    R, me, n = 4, 2, 3 * 4096
    ins = [zo.f32_to_bf16(rng(70 + r).standard_normal(R * n).astype(np.float32)) for r in range(R)]
    whole = torch.empty(R * R * n, dtype=torch.bfloat16, device="cuda")
    for r in range(R):
        whole[r * R * n:(r + 1) * R * n].copy_(torch.from_numpy(ins[r]).view(torch.int16).view(torch.bfloat16))
    g = capi.CommGroupInfo()
    g.groupSize, g.myGroupRank, g.localDeviceMemSize = R, me, R * n * 2
    for i in range(R):
        g.peerGroupRank2WorldRank[i] = 10 + i            # world ranks need not start at 0
    out = torch.empty(n, dtype=torch.bfloat16, device="cuda")
    mine = whole.data_ptr() + me * R * n * 2
    assert fn["ZBALOpReduceScatter"](mine, out.data_ptr(), n, capi.DT_BF16, capi.stream_ptr(), capi.REDUCE_SUM, ctypes.byref(g)) == 0
    assert g.waitSymbol == 1
    assert np.array_equal(host(out), zo.reduce([a[me * n:(me + 1) * n].copy() for a in ins], capi.DT_BF16, capi.REDUCE_SUM))
    # low-latency dispatch + combine, group of one
    T, K, E, H = 40, 4, 16, 256
    x = torch.from_numpy(bf16_normal((T, H), 80)).view(torch.int16).view(torch.bfloat16).cuda()
    ids = torch.from_numpy(rng(81).integers(0, E, size=(T, K)).astype(np.int32)).cuda()
    w = torch.from_numpy(rng(82).uniform(0, 1, (T, K)).astype(np.float32)).cuda()
    one = capi.CommGroupInfo()
    one.groupSize = 1
    ti, ref = capi.tensor_info, ctypes.byref
    res = []
    for seam in (False, True):
        ex = torch.zeros((T * K, H), dtype=torch.bfloat16, device="cuda")
        sc = torch.zeros((T * K,), dtype=torch.float32, device="cuda")
        eidx = torch.zeros((T, K), dtype=torch.int32, device="cuda")
        nums = torch.zeros((E,), dtype=torch.int64, device="cuda")
        cnt = torch.zeros((E,), dtype=torch.int32, device="cuda")
        put = torch.zeros((E,), dtype=torch.int32, device="cuda")
        back = torch.zeros((T, H), dtype=torch.bfloat16, device="cuda")
        args = (ref(ti(x)), ref(ti(ids)), E, 0, 0, 0, 0, 0, 1, ref(ti(ex)), ref(ti(sc)), ref(ti(eidx)), ref(ti(nums)),
                ref(ti(cnt)), ref(ti(put)), ref(ti(put)))
        cargs = (ref(ti(ex)), ref(ti(ids)), ref(ti(eidx)), ref(ti(cnt)), ref(ti(w)), ref(ti(back)), E)
        if seam:
            assert fn["ZBALOpDispatchLowLatency"](*args, capi.stream_ptr(), ref(one), 0) == 0
            assert fn["ZBALOpCombineLowLatency"](*cargs, capi.stream_ptr(), ref(one), 0) == 0
        else:
            assert buf.lib.zbal_dispatch_low_latency(*args, buf.comm, capi.stream_ptr(), 0) == 0
            assert buf.lib.zbal_combine_low_latency(*cargs, buf.comm, capi.stream_ptr(), 0) == 0
        torch.cuda.synchronize()
        res.append([host(t) for t in (ex, eidx, nums, cnt, back)])
    for a, b in zip(*res):
        assert np.array_equal(a, b)
    # re-balancing is not part of this build: the launchers say so instead of ignoring the flag
    assert fn["ZBALOpDispatchNormal"](ref(ti(x)), ref(ti(ids)), ref(ti(ids)), ref(ti(ids)), ref(ti(ids)), E, 0, ref(ti(x)),
                                      ref(ti(w)), True, capi.stream_ptr(), ref(one), 0) == capi.Z_INVALID_PARAM


def test_dispatch_drops_rows_past_the_receive_tensor(buf):
    """A receive tensor sized below tokens * topk rows (the reference sizes it from the received total): rows that
    fit are written, the others are dropped, nothing is written past the end."""
    T, K, E, H = 64, 4, 8, 128
    ids = rng(7).integers(0, E, size=(T, K)).astype(np.int64)
    x = bf16_normal((T, H), 8)
    per_rank, _, per_expert, _, _ = buf.get_dispatch_layout(torch.from_numpy(ids).cuda(), E)
    recv_full, _, _, h = buf.dispatch(torch.from_numpy(x).view(torch.int16).view(torch.bfloat16).cuda(),
                                      torch.from_numpy(ids).cuda(), None, per_expert, capi.NO_QUANT)
    cap = 100
    guard = torch.full((T * K, H), 7.0, dtype=torch.bfloat16, device="cuda")
    small = capi.tensor_info(guard, shape=(cap, H))
    ti, ref = capi.tensor_info, ctypes.byref
    x_d = torch.from_numpy(x).view(torch.int16).view(torch.bfloat16).cuda()
    assert buf.lib.zbal_dispatch_normal(ref(ti(x_d)), ref(ti(h["expert_ids"])), ref(ti(h["send_token_idx"])),
                                        ref(ti(h["put_offset"])), ref(ti(h["balance_matrix"])), E, capi.NO_QUANT, ref(small),
                                        ref(ti(torch.empty(1, dtype=torch.float32, device="cuda"))), buf.comm,
                                        capi.stream_ptr(), 0) == 0
    torch.cuda.synchronize()
    assert torch.equal(guard[:cap], recv_full[:cap])
    assert bool((guard[cap:] == 7.0).all())


def test_empty_batch_fused_and_low_latency(buf):
    """T = 0: torch hands out null data pointers for the empty per-token tensors; the operators must accept them,
    write all-zero counts and return 0 (the reference's adaptor pads such a batch to one token instead,
    zbal_deepep.cpp:470-490)."""
    lib = buf.lib
    ti, ref = capi.tensor_info, ctypes.byref
    E, H, K, I = 8, 256, 2, 128
    nums = torch.full((E,), 9, dtype=torch.int64, device="cuda")
    x = torch.empty((0, H), dtype=torch.bfloat16, device="cuda")
    ids = torch.empty((0, K), dtype=torch.int32, device="cuda")
    es = torch.empty((0, K), dtype=torch.float32, device="cuda")
    out = torch.empty((0, H), dtype=torch.bfloat16, device="cuda")
    assert x.data_ptr() == 0
    w1 = buf.prepack_weight(torch.zeros((E, H, 2 * I), dtype=torch.int8, device="cuda"))
    w2 = buf.prepack_weight(torch.zeros((E, I, H), dtype=torch.int8, device="cuda"))
    s1 = torch.ones((E, 2 * I), dtype=torch.float32, device="cuda")
    s2 = torch.ones((E, H), dtype=torch.bfloat16, device="cuda")
    ws = torch.empty(buf.fused_workspace_bytes(0, H, K, E, 2 * I, 1), dtype=torch.uint8, device="cuda")
    null = capi.TensorInfo()
    pp = capi.WEIGHT_FORMAT_PREPACKED
    rc = lib.zbal_fused_deep_moe(ref(ti(x)), ref(ti(ids)), ref(ti(w1, weight_format=pp)), ref(ti(s1)), ref(ti(w2, weight_format=pp)),
                                 ref(ti(s2)), ref(ti(es)), ref(null), ref(null), ref(null), ref(null), ref(null), ref(null),
                                 ref(null), ref(ti(out)), ref(null), ref(ti(nums)), ref(ti(ws)), E, 1, 0, 2 * I, 0, 0, buf.comm,
                                 capi.stream_ptr(), 0)
    assert rc == 0, capi.last_error()
    torch.cuda.synchronize()
    assert bool((nums == 0).all())
    # low-latency dispatch
    nums.fill_(9)
    counts = torch.full((E,), 9, dtype=torch.int32, device="cuda")
    put = torch.zeros((E,), dtype=torch.int32, device="cuda")
    ex = torch.empty((0, H), dtype=torch.int8, device="cuda")
    sc = torch.empty((0,), dtype=torch.float32, device="cuda")
    eidx = torch.empty((0, K), dtype=torch.int32, device="cuda")
    rc = lib.zbal_dispatch_low_latency(ref(ti(x)), ref(ti(ids)), E, 0, 0, 1, 0, 0, 1, ref(ti(ex)), ref(ti(sc)), ref(ti(eidx)),
                                       ref(ti(nums)), ref(ti(counts)), ref(ti(put)), ref(ti(put)), buf.comm, capi.stream_ptr(), 0)
    assert rc == 0, capi.last_error()
    torch.cuda.synchronize()
    assert bool((nums == 0).all()) and bool((counts == 0).all())


def test_fused_and_all_reduce_through_the_launcher_seam(buf):
    """ZBALOpFusedDeepMoe and ZBALOpAllReduce, called the way the reference's communicator layer calls them (a
    CommGroupInfo, a std::string group name), give the outer ABI's results bit for bit; a second call on the same
    group reuses the backend object built by the first."""
    lib, fn = buf.lib, capi.load_cxx()
    ti, ref, st = capi.tensor_info, ctypes.byref, capi.stream_ptr()
    T, H, K, E, I = 96, 512, 4, 8, 256
    x = torch.from_numpy(bf16_normal((T, H), 1)).view(torch.int16).view(torch.bfloat16).cuda()
    ids = torch.from_numpy(rng(2).integers(0, E, size=(T, K)).astype(np.int32)).cuda()
    es = torch.from_numpy(rng(3).uniform(0, 1, (T, K)).astype(np.float32)).cuda()
    w1 = buf.prepack_weight(torch.from_numpy(rng(4).integers(-16, 16, (E, H, 2 * I)).astype(np.int8)).cuda())
    s1 = torch.from_numpy(rng(5).uniform(0.0015, 0.0045, (E, 2 * I)).astype(np.float32)).cuda()
    w2 = buf.prepack_weight(torch.from_numpy(rng(6).integers(-16, 16, (E, I, H)).astype(np.int8)).cuda())
    s2 = torch.from_numpy(rng(7).uniform(0.0015, 0.0045, (E, H)).astype(np.float32)).cuda().to(torch.bfloat16)
    want, _, want_nums = buf.fused_deep_moe(x, ids, w1, s1, w2, s2, es, E, quant_mode=0)
    ws = torch.empty(buf.fused_workspace_bytes(T, H, K, E, 2 * I, 0), dtype=torch.uint8, device="cuda")
    g = capi.CommGroupInfo()
    g.groupSize, g.myGroupRank = 1, 0
    name = capi.std_string(b"ep_group")
    null = ref(capi.TensorInfo())
    pre = capi.WEIGHT_FORMAT_PREPACKED
    for _ in range(2):
        out = torch.zeros((T, H), dtype=torch.bfloat16, device="cuda")
        nums = torch.zeros(E, dtype=torch.int64, device="cuda")
        rc = fn["ZBALOpFusedDeepMoe"](ref(ti(x)), ref(ti(ids)), ref(ti(w1, weight_format=pre)), ref(ti(s1)),
                                      ref(ti(w2, weight_format=pre)), ref(ti(s2)), ref(ti(es)), null, null, null, null, null,
                                      null, null, ref(ti(out)), null, ref(ti(nums)), ref(ti(ws)), E, 0, 0, 2 * I, 0, False,
                                      None, ctypes.addressof(name), st, ref(g), ref(g), 0, True)
        assert rc == 0, capi.last_error()
        assert torch.equal(out, want) and torch.equal(nums, want_nums)

    # all-reduce over four windows that lie localDeviceMemSize bytes apart
    R, n = 4, 3000
    stride = (n * 4 + 255) // 256 * 256
    whole = torch.zeros(R * stride, dtype=torch.uint8, device="cuda")
    parts = [whole[r * stride:r * stride + n * 4].view(torch.float32) for r in range(R)]
    for r in range(R):
        parts[r].copy_(torch.from_numpy(rng(20 + r).standard_normal(n).astype(np.float32)))
    ref_sum = parts[0].clone()
    for r in range(1, R):
        ref_sum = ref_sum + parts[r]
    for me in range(R):
        gi = capi.CommGroupInfo()
        gi.groupSize, gi.myGroupRank, gi.localDeviceMemSize = R, me, stride
        for i in range(R):
            gi.peerGroupRank2WorldRank[i] = i
        out = torch.zeros(n, dtype=torch.float32, device="cuda")
        rc = fn["ZBALOpAllReduce"](parts[me].data_ptr(), out.data_ptr(), None, n, capi.DT_FP32, st, capi.REDUCE_SUM, ref(gi))
        assert rc == 0, capi.last_error()
        assert torch.equal(out, ref_sum)
        assert gi.waitSymbol == 1


@pytest.mark.parametrize("api_cls", [OuterAbi, KernelSeam])
@pytest.mark.parametrize("R,quant,T,K,E,H,nums_type", [(1, 1, 48, 4, 16, 256, 1), (2, 0, 48, 4, 16, 256, 0), (4, 1, 33, 8, 32, 512, 1),
                                                        (4, 2, 40, 3, 8, 1024, 0), (2, 1, 700, 8, 64, 256, 1)])
def test_low_latency_pair_over_modelled_ranks(buf, api_cls, R, quant, T, K, E, H, nums_type):
    """Low-latency dispatch and combine over R modelled ranks: counts from every rank's ids, rows into the window of
    the rank that owns the expert at the running-sum offsets ep_recv_counts[r * E + le * R + src], combine reading them
    back from there. Bit for bit against the oracle's R-rank functions, through both ABIs."""
    lib = buf.lib
    ti, ref = capi.tensor_info, ctypes.byref
    rows_cap = R * T * K
    qbytes = 2 if quant == 0 else 1
    spr = {0: 1, 1: 1, 2: H // 128}[quant]
    layout = [("ids", T * K * 4, torch.int32), ("recv_x", rows_cap * H * qbytes, torch.uint8),
              ("recv_scale", rows_cap * spr * 4, torch.float32), ("expert_out", rows_cap * H * 2, torch.bfloat16)]
    wins = Window.make(layout, R)
    api = api_cls(lib, wins, "ll%d_%d_%d_%d" % (R, quant, T, H))
    try:
        ids_all = rng(300 + R).integers(-1, E + 1, size=(R, T, K)).astype(np.int32)
        xs = [bf16_normal((T, H), 310 + r) for r in range(R)]
        w = [rng(320 + r).uniform(0, 1, (T, K)).astype(np.float32) for r in range(R)]
        for r in range(R):
            wins[r]["ids"].copy_(torch.from_numpy(ids_all[r].reshape(-1)))
        recv_dt = {0: capi.DT_BF16, 1: capi.DT_INT8, 2: capi.DT_FP8_E4M3}[quant]
        out = []
        for r in range(R):
            x_d = torch.from_numpy(xs[r]).view(torch.int16).view(torch.bfloat16).cuda()
            eidx = torch.full((T, K), -9, dtype=torch.int32, device="cuda")
            nums = torch.full((E // R,), -9, dtype=torch.int64, device="cuda")
            recv = torch.full((R * E,), -9, dtype=torch.int32, device="cuda")
            put = torch.full((max(R, 2) * E,), -9, dtype=torch.int32, device="cuda")
            status = torch.zeros(R * E, dtype=torch.float32, device="cuda")
            rc = api.ll_dispatch(r, ref(ti(x_d)), ref(ti(wins[r]["ids"], shape=(T, K))), E, 0, 0, quant, 0, 0, nums_type,
                                 ref(ti(wins[r]["recv_x"], dtype=recv_dt, shape=(rows_cap, H))), ref(ti(wins[r]["recv_scale"])),
                                 ref(ti(eidx)), ref(ti(nums)), ref(ti(recv)), ref(ti(put)), ref(ti(status)))
            assert rc == 0, capi.last_error()
            out.append((eidx, nums, recv, put))
        torch.cuda.synchronize()
        np_x = np.zeros((R, rows_cap, H), dtype=np.uint16 if quant == 0 else np.uint8)
        np_s = np.zeros((R, rows_cap, spr) if quant == 2 else (R, rows_cap), dtype=np.float32)
        for r in range(R):
            allc, o_recv, o_nums = zo.ll_counts(ids_all, E, r, nums_type)
            o_eidx = zo.dispatch_low_latency_ranks(xs[r], zo.DT_BF16, ids_all[r], E, R, r, quant, o_recv, np_x, np_s)
            eidx, nums, recv, put = out[r]
            assert np.array_equal(host(eidx), o_eidx) and np.array_equal(host(nums), o_nums)
            assert np.array_equal(host(recv), o_recv)
            if R > 1:
                assert np.array_equal(host(put)[:R * E], allc.reshape(-1))
        e_loc = E // R
        for d in range(R):
            n_rows = int(zo.ll_counts(ids_all, E, d, 1)[2].sum())
            got = host(wins[d]["recv_x"]).reshape(rows_cap, H * qbytes)
            got = got.view(np.uint16) if quant == 0 else got
            assert np.array_equal(got[:n_rows], np_x[d, :n_rows]), "rows in window %d" % d
            if quant != 0:
                assert np.array_equal(host(wins[d]["recv_scale"]).reshape(rows_cap, spr)[:n_rows], np_s[d].reshape(rows_cap, spr)[:n_rows])
        # ---- combine: the expert outputs sit in the windows the rows were dispatched to
        y = np.stack([bf16_normal((rows_cap, H), 330 + d) for d in range(R)])
        for d in range(R):
            wins[d]["expert_out"].copy_(torch.from_numpy(y[d].reshape(-1)).view(torch.int16).view(torch.bfloat16))
        for r in range(R):
            eidx, nums, recv, put = out[r]
            res = torch.zeros((T, H), dtype=torch.bfloat16, device="cuda")
            ids32 = torch.from_numpy(ids_all[r]).cuda()
            rc = api.ll_combine(r, ref(ti(wins[r]["expert_out"], shape=(rows_cap, H))), ref(ti(ids32)), ref(ti(eidx)), ref(ti(recv)),
                                ref(ti(torch.from_numpy(w[r]).cuda())), ref(ti(res)), E)
            assert rc == 0, capi.last_error()
            want = zo.combine_low_latency_ranks(y, zo.DT_BF16, ids_all[r], host(eidx), host(recv), w[r], E, R, r)
            assert np.array_equal(host(res), want), "combine of rank %d" % r
    finally:
        torch.cuda.synchronize()
        api.close()
