"""The layout entry point that allocates nothing (zbalhip_dispatch_layout_static) against the one that takes
the caller's scratch (zbalhip_dispatch_layout): same outputs, bit for bit, on two calls in a row, the second
on a smaller input, so that whatever the first call left in the library's static scratch must not matter.
Both are called through the C ABI (ctypes)."""
import numpy as np
import pytest
import torch

from memfabric_hybrid_amd import capi
from zbal_testlib import rng

pytestmark = pytest.mark.gpu

MAX_BLOCKS = 50          # ZBALHIP_LAYOUT_MAX_BLOCKS


def _layout_pair(lib, idx, experts, ranks):
    """(with caller scratch, with the static scratch): each a tuple of the three outputs as numpy arrays"""
    T, K = idx.shape
    d_idx = torch.from_numpy(idx).cuda()
    is64 = 1 if idx.dtype == np.int64 else 0
    outs = []
    for static in (False, True):
        per_rank = torch.full((ranks,), -7, dtype=torch.int32, device="cuda")
        per_expert = torch.full((experts,), -7, dtype=torch.int32, device="cuda")
        send_idx = torch.full((T, K), -7, dtype=torch.int32, device="cuda")
        if static:
            rc = lib.zbalhip_dispatch_layout_static(d_idx.data_ptr(), is64, T, experts, K, ranks, per_rank.data_ptr(),
                                                    per_expert.data_ptr(), send_idx.data_ptr(), None)
        else:
            scratch = torch.empty((MAX_BLOCKS * experts,), dtype=torch.int32, device="cuda")
            rc = lib.zbalhip_dispatch_layout(d_idx.data_ptr(), is64, T, experts, K, ranks, per_rank.data_ptr(),
                                             per_expert.data_ptr(), send_idx.data_ptr(), scratch.data_ptr(), None)
        assert rc == 0
        torch.cuda.synchronize()
        outs.append((per_rank.cpu().numpy(), per_expert.cpu().numpy(), send_idx.cpu().numpy()))
    return outs


def test_static_layout_matches_scratch_layout_twice():
    lib = capi.load()
    torch.cuda.set_device(0)
    # first call: many blocks and experts, invalid ids mixed in; second call: smaller in every dimension
    for T, K, E, R, dt, seed in ((6000, 8, 256, 8, np.int64, 11), (333, 4, 24, 3, np.int32, 12)):
        idx = rng(seed).integers(-1, E + 1, size=(T, K)).astype(dt)
        want, got = _layout_pair(lib, idx, E, R)
        for w, g, name in zip(want, got, ("tokens_per_rank", "tokens_per_expert", "send_token_idx")):
            assert np.array_equal(w, g), name
        valid = (idx >= 0) & (idx < E)
        assert got[1].sum() == valid.sum()
        assert np.array_equal(got[2][~valid], np.full((~valid).sum(), -1, dtype=np.int32))


def test_static_layout_refuses_what_the_scratch_cannot_hold():
    lib = capi.load()
    torch.cuda.set_device(0)
    idx = torch.zeros((4, 2), dtype=torch.int32, device="cuda")
    out = torch.zeros((2000,), dtype=torch.int32, device="cuda")
    rc = lib.zbalhip_dispatch_layout_static(idx.data_ptr(), 0, 4, 1025, 2, 1, out.data_ptr(), out.data_ptr(),
                                            out.data_ptr(), None)
    assert rc == -2
    assert b"static scratch" in lib.zbal_get_last_error_msg()


def test_static_layout_calls_on_two_streams_take_turns():
    """Calls issued back to back on two streams share the one static scratch: the library queues each behind the
    one before (an event per GPU), so both give the caller-scratch results although their streams are not ordered."""
    lib = capi.load()
    torch.cuda.set_device(0)
    cases = []
    for T, K, E, R, seed in ((5000, 8, 200, 4, 21), (4800, 8, 64, 2, 22), (5200, 6, 256, 8, 23), (300, 4, 16, 1, 24)):
        idx = rng(seed).integers(-1, E + 1, size=(T, K)).astype(np.int32)
        d_idx = torch.from_numpy(idx).cuda()
        scratch = torch.empty((MAX_BLOCKS * E,), dtype=torch.int32, device="cuda")
        want = [torch.empty(R, dtype=torch.int32, device="cuda"), torch.empty(E, dtype=torch.int32, device="cuda"),
                torch.empty((T, K), dtype=torch.int32, device="cuda")]
        assert lib.zbalhip_dispatch_layout(d_idx.data_ptr(), 0, T, E, K, R, want[0].data_ptr(), want[1].data_ptr(),
                                           want[2].data_ptr(), scratch.data_ptr(), None) == 0
        got = [torch.full_like(w, -7) for w in want]
        cases.append((d_idx, T, K, E, R, want, got))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for rep in range(3):
        for i, (d_idx, T, K, E, R, want, got) in enumerate(cases):
            st = streams[i % 2]
            assert lib.zbalhip_dispatch_layout_static(d_idx.data_ptr(), 0, T, E, K, R, got[0].data_ptr(), got[1].data_ptr(),
                                                      got[2].data_ptr(), st.cuda_stream) == 0
    torch.cuda.synchronize()
    for _, _, _, _, _, want, got in cases:
        for w, g in zip(want, got):
            assert torch.equal(w, g)
