"""The DeepEP-compatible `Buffer` driven the way the reference's own tests drive theirs.

Each test restates the assertions of one reference test (app/zbal/test/python/deepep/) on inputs
built by the same recipe, with one rank:
  * test_normal.py:95-98, 137-149  layout counts equal a recount of topk_idx
  * test_normal.py:170-177, 212-213 num_recv_tokens_per_expert_list equals the (all-reduced) counts
  * test_normal.py:225-236         combine(dispatch(x)) = x * sum_k w[t, k], calc_diff < 5e-5
  * test_low_latency.py:146-155    the same round trip in low-latency mode, < 1e-4 (int8) / < 1e-5 (bf16)
  * test_fused_deep_moe.py:284-317 fused layer against the unfused computation (here: the CPU oracle), per token
                                   calc_diff < 1e-2 on at least 95 % of the tokens, expert_token_nums exact
The signatures, defaults and return tuples are checked against zbal_buffer.py on the CPU in
tests/test_capi_host.py.
"""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as zo
from zbal_testlib import calc_diff, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def buffer():
    from memfabric_hybrid_amd.buffer import Buffer
    num_rdma_bytes = Buffer.get_low_latency_rdma_size_hint(128, 7168, 1, 32)
    b = Buffer(None, num_nvl_bytes=0, num_rdma_bytes=num_rdma_bytes, low_latency_mode=True, num_qps_per_rank=32)
    yield b
    b.close()


def per_token_cast_back(q, scales):
    """The reference tests' decode of (rows, scales) (utils.py:118-126) for one fp32 scale per row or per 128 columns."""
    if q.numel() == 0:
        return q.to(torch.bfloat16)
    f = q.to(torch.float32).view(q.size(0), -1, 128)
    s = scales.view(q.size(0), -1, 1)
    return (f * s).view(q.shape).to(torch.bfloat16)


def rotating_topk(num_tokens, num_topk, num_experts):
    """test_normal.py:84-88: token t picks experts (t * topk + k) mod experts."""
    t = torch.arange(num_tokens, device="cuda")[:, None] * num_topk + torch.arange(num_topk, device="cuda")[None, :]
    return (t % num_experts).to(torch.int64).contiguous()


@pytest.mark.parametrize("num_tokens,hidden,num_topk,num_experts", [(1, 1024, 8, 16), (96, 1024, 8, 16), (512, 7168, 8, 32)])
@pytest.mark.parametrize("use_quant", [False, True])
@pytest.mark.parametrize("nums_type", [1, 0])
def test_normal_mode_as_the_reference_test(buffer, monkeypatch, num_tokens, hidden, num_topk, num_experts, use_quant,
                                           nums_type):
    from memfabric_hybrid_amd.buffer import Config
    monkeypatch.setenv("DEEP_NORMAL_MODE_USE_INT8_QUANT", "1" if use_quant else "0")
    monkeypatch.setenv("MOE_EXPERT_TOKEN_NUMS_TYPE", str(nums_type))
    torch.manual_seed(7)
    topk_idx = rotating_topk(num_tokens, num_topk, num_experts)
    if num_tokens > 8:
        topk_idx[3, 1] = -1                     # "-1 means no selections"
        topk_idx[5, :] = -1
    recount = torch.stack([(topk_idx == e).sum() for e in range(num_experts)]).to(torch.int32)
    per_rank_want = (topk_idx >= 0).any(dim=1).sum().to(torch.int32).view(1)

    ref_per_rank, per_rdma, ref_per_expert, ref_in_rank, event = buffer.get_dispatch_layout(topk_idx, num_experts)
    assert per_rdma is None
    assert torch.equal(ref_per_rank, per_rank_want)
    assert torch.equal(ref_per_expert, recount)
    assert ref_in_rank.shape == (num_tokens, 1)

    rank_value = 3.0                            # the reference fills x with its rank; any constant serves
    x = torch.ones((num_tokens, hidden), dtype=torch.bfloat16, device="cuda") * rank_value
    x_pure_rand = torch.randn((num_tokens, hidden), dtype=torch.bfloat16, device="cuda")
    w_const = torch.ones((num_tokens, num_topk), dtype=torch.float32, device="cuda") * rank_value
    w_rand = torch.randn((num_tokens, num_topk), dtype=torch.float32, device="cuda")
    want_list = recount.cumsum(0).tolist() if nums_type == 0 else recount.tolist()
    for current_x, w in ((x, w_const), (x_pure_rand, w_rand)):
        recv_x, recv_topk_idx, recv_topk_weights, recv_list, handle, event = buffer.dispatch(
            x=current_x, num_tokens_per_rank=ref_per_rank, is_token_in_rank=ref_in_rank,
            num_tokens_per_expert=ref_per_expert, config=Config(24, 8, 256, 6, 128), topk_idx=topk_idx, topk_weights=w)
        assert recv_topk_idx is None and recv_topk_weights is None
        assert recv_list == want_list
        assert isinstance(recv_x, tuple) == use_quant
        rows = (recv_x[0] if use_quant else recv_x).size(0)
        assert rows == max(int(recount.sum().item()), 1)          # sized by the received count, one row when empty
        recv = per_token_cast_back(recv_x[0], recv_x[1].view(-1, 1).expand(-1, hidden // 128).contiguous()) \
            if use_quant else recv_x
        assert len(handle) == 5 and handle[1] is topk_idx and handle[2] is w
        combined_x, combined_topk_weights, event = buffer.combine(x=recv, handle=handle, config=None, async_finish=False,
                                                                  topk_weights=handle[2])
        assert combined_topk_weights is None
        ref = current_x.float() * handle[2].masked_fill(topk_idx == -1, 0).sum(dim=1).view(-1, 1)
        diff = calc_diff(host(combined_x.float()), host(ref))
        assert diff < (5e-5 if not use_quant else 2e-4) or math.isnan(diff)


def test_normal_dispatch_without_host_sync(buffer, monkeypatch):
    """num_worst_tokens: recv_x has that many rows, the list is empty, nothing is read back."""
    monkeypatch.setenv("DEEP_NORMAL_MODE_USE_INT8_QUANT", "0")
    T, H, K, E = 64, 1024, 4, 8
    topk_idx = rotating_topk(T, K, E)
    per_rank, _, per_expert, in_rank, _ = buffer.get_dispatch_layout(topk_idx, E)
    x = torch.randn((T, H), dtype=torch.bfloat16, device="cuda")
    w = torch.rand((T, K), dtype=torch.float32, device="cuda")
    recv_x, _, _, lst, handle, ev = buffer.dispatch(x, num_tokens_per_rank=per_rank, is_token_in_rank=in_rank,
                                                    num_tokens_per_expert=per_expert, topk_idx=topk_idx, topk_weights=w,
                                                    num_worst_tokens=T * K, async_finish=True)
    assert lst == [] and recv_x.size(0) == T * K
    ev.current_stream_wait()
    out, _, _ = buffer.combine(recv_x, handle, previous_event=buffer.capture())
    ref = x.float() * w.sum(dim=1, keepdim=True)
    assert calc_diff(host(out.float()), host(ref)) < 5e-5


def test_dispatch_argument_errors(buffer):
    T, H, K, E = 8, 1024, 2, 4
    topk_idx = rotating_topk(T, K, E)
    per_rank, _, per_expert, in_rank, _ = buffer.get_dispatch_layout(topk_idx, E)
    x = torch.zeros((T, H), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(NotImplementedError):
        buffer.dispatch((x, x), num_tokens_per_rank=per_rank, is_token_in_rank=in_rank, num_tokens_per_expert=per_expert,
                        topk_idx=topk_idx)
    with pytest.raises(NotImplementedError):
        buffer.dispatch(x, handle=(1,), num_tokens_per_rank=per_rank, is_token_in_rank=in_rank,
                        num_tokens_per_expert=per_expert, topk_idx=topk_idx)
    with pytest.raises(ValueError):
        buffer.dispatch(x, topk_idx=topk_idx)
    with pytest.raises(ValueError):
        type(buffer).set_num_sms(3)


@pytest.mark.parametrize("num_tokens,hidden,num_topk,num_experts", [(128, 7168, 8, 32), (16, 2048, 4, 8)])
@pytest.mark.parametrize("use_fp8", [True, False])
def test_low_latency_mode_as_the_reference_test(buffer, num_tokens, hidden, num_topk, num_experts, use_fp8):
    torch.manual_seed(11)
    x = torch.ones((num_tokens, hidden), dtype=torch.bfloat16, device="cuda") * 2.0
    scores = torch.randn((num_tokens, num_experts), dtype=torch.float32, device="cuda").abs() + 1
    topk_idx = torch.topk(scores, num_topk, dim=-1, largest=True, sorted=True)[1].int()
    topk_weights = torch.randn((num_tokens, num_topk), dtype=torch.float32, device="cuda").abs()
    topk_weights = topk_weights / topk_weights.sum(dim=-1, keepdim=True)
    stats = torch.zeros((num_experts,), dtype=torch.int, device="cuda")
    for _ in range(3):
        packed_recv_x, packed_recv_count, handle, event, hook = buffer.low_latency_dispatch(
            x, topk_idx, num_tokens, num_experts, use_fp8=use_fp8, round_scale=False, use_ue8m0=False,
            cumulative_local_expert_recv_stats=stats, async_finish=True, return_recv_hook=False)
        hook()
        assert isinstance(packed_recv_x, tuple) == use_fp8
        if use_fp8:
            q, s = packed_recv_x
            simulated_gemm_x = per_token_cast_back(q, s.view(-1, 1).expand(-1, hidden // 128).contiguous())
        else:
            simulated_gemm_x = packed_recv_x
        out = torch.empty((num_tokens, hidden), dtype=torch.bfloat16, device="cuda")
        combined_x, event, hook = buffer.low_latency_combine(simulated_gemm_x, topk_idx, topk_weights, handle,
                                                             async_finish=True, zero_copy=False, return_recv_hook=False,
                                                             out=out)
        assert combined_x is out
    recount = torch.stack([(topk_idx == e).sum() for e in range(num_experts)]).to(torch.int64)
    assert torch.equal(packed_recv_count, recount)
    assert len(handle) == 6 and handle[2] == num_tokens and handle[3] == hidden and handle[4] == num_experts
    ref = x.float() * topk_weights.masked_fill(topk_idx == -1, 0).sum(dim=1).view(-1, 1)
    diff = calc_diff(host(ref), host(combined_x.float()))
    assert torch.isnan(combined_x).sum().item() == 0
    assert diff < (1e-4 if use_fp8 else 1e-5), diff


def test_low_latency_empty_batch_is_padded_like_the_reference(buffer):
    """zbal_deepep.cpp:470-490, 637-644: an empty batch runs as one token of ones that picks experts 0..topk-1; the
    combine hands back the caller's (empty) x."""
    H, K, E = 1024, 4, 8
    x = torch.empty((0, H), dtype=torch.bfloat16, device="cuda")
    topk_idx = torch.empty((0, K), dtype=torch.int32, device="cuda")
    w = torch.empty((0, K), dtype=torch.float32, device="cuda")
    (q, s), count, handle, _, _ = buffer.low_latency_dispatch(x, topk_idx, 16, E)
    assert count.tolist() == [1] * K + [0] * (E - K)
    assert torch.equal(q[:K].to(torch.int32), torch.full((K, H), 127, dtype=torch.int32, device="cuda"))
    y = per_token_cast_back(q, s.view(-1, 1).expand(-1, H // 128).contiguous())
    combined, _, _ = buffer.low_latency_combine(y, topk_idx, w, handle)
    assert combined.shape == (0, H)


@pytest.mark.parametrize("bs,hidden,ffn,num_experts,num_topk", [(64, 1024, 1024, 8, 4), (128, 7168, 4096, 32, 8)])
def test_fused_deep_moe_as_the_reference_test(buffer, bs, hidden, ffn, num_experts, num_topk):
    """Data as test_fused_deep_moe.py:42-70 (seed 42 + rank, x ~ U(-5, 5), weights ~ randint(-16, 16), scales ~
    U(0.0015, 0.0045), expert ids drawn with repetition); weights are passed in the logical layout."""
    torch.manual_seed(42)
    x = (torch.rand((bs, hidden), device="cuda") * 10 - 5).to(torch.bfloat16)
    expert_ids = torch.randint(0, num_experts, (bs, num_topk), dtype=torch.int32, device="cuda") % num_experts
    expert_scales = torch.rand((bs, num_topk), dtype=torch.float32, device="cuda")
    g1_w = torch.randint(-16, 16, (num_experts, hidden, ffn), dtype=torch.int8, device="cuda")
    g1_s = (torch.rand((num_experts, ffn), dtype=torch.float32, device="cuda") * 0.003 + 0.0015).contiguous()
    g2_w = torch.randint(-16, 16, (num_experts, ffn // 2, hidden), dtype=torch.int8, device="cuda")
    g2_s = (torch.rand((num_experts, hidden), dtype=torch.float32, device="cuda") * 0.003 + 0.0015).to(torch.bfloat16)

    for _ in range(2):          # the second call takes the cached pre-packed weights
        fused_out, fused_token_nums = buffer.fused_deep_moe(
            x=x, topk_idx=expert_ids, gmm1_permuted_weight=g1_w, gmm1_permuted_weight_scale=g1_s, gmm2_weight=g2_w,
            gmm2_weight_scale=g2_s, topk_weights=expert_scales, num_experts=num_experts, quant_mode=0,
            num_max_dispatch_tokens_per_rank=0)
    assert fused_out.shape == (bs, hidden) and fused_out.dtype == x.dtype
    assert fused_token_nums.dtype == torch.int64 and fused_token_nums.shape == (num_experts,)

    ref, counts = zo.fused_moe(host(x), zo.DT_BF16, host(expert_ids), host(expert_scales), host(g1_w), host(g1_s),
                               host(g2_w), host(g2_s), num_experts, 0)
    assert np.array_equal(host(fused_token_nums), counts)                       # expert_token_nums: exact
    recount = np.bincount(host(expert_ids).reshape(-1), minlength=num_experts)
    assert np.array_equal(counts, recount)
    got, want = zo.bf16_to_f32(host(fused_out)), zo.bf16_to_f32(ref)
    bad = 0
    for t in range(bs):
        d = calc_diff(got[t], want[t])
        if math.isnan(d) or math.isinf(d) or d >= 1e-2:
            bad += 1
    assert bad <= bs * 0.05
    assert np.array_equal(host(fused_out), ref)                                  # and, in this build, bit-exact


def test_fused_deep_moe_repacks_new_weights_at_a_reused_address(buffer):
    """The Buffer keeps the pre-packed copies of logical weights it has seen. Weights that are freed and replaced by
    others of the same shape usually get the same address back from the allocator: the copy of the old ones must not
    be served for the new ones."""
    bs, hidden, ffn, num_experts, num_topk = 32, 256, 256, 4, 2
    torch.manual_seed(7)
    x = (torch.rand((bs, hidden), device="cuda") * 10 - 5).to(torch.bfloat16)
    ids = torch.randint(0, num_experts, (bs, num_topk), dtype=torch.int32, device="cuda")
    es = torch.rand((bs, num_topk), dtype=torch.float32, device="cuda")
    g1_s = (torch.rand((num_experts, ffn), dtype=torch.float32, device="cuda") * 0.003 + 0.0015).contiguous()
    g2_s = (torch.rand((num_experts, hidden), dtype=torch.float32, device="cuda") * 0.003 + 0.0015).to(torch.bfloat16)
    seen = set()
    for round_ in range(3):
        g1_w = torch.randint(-16, 16, (num_experts, hidden, ffn), dtype=torch.int8, device="cuda")
        g2_w = torch.randint(-16, 16, (num_experts, ffn // 2, hidden), dtype=torch.int8, device="cuda")
        seen.add((g1_w.data_ptr(), g2_w.data_ptr()))
        out, nums = buffer.fused_deep_moe(x=x, topk_idx=ids, gmm1_permuted_weight=g1_w, gmm1_permuted_weight_scale=g1_s,
                                          gmm2_weight=g2_w, gmm2_weight_scale=g2_s, topk_weights=es, num_experts=num_experts)
        ref, _ = zo.fused_moe(host(x), zo.DT_BF16, host(ids), host(es), host(g1_w), host(g1_s), host(g2_w), host(g2_s),
                              num_experts, 0)
        assert np.array_equal(host(out), ref), round_
        del g1_w, g2_w, out
    if len(seen) == 3:            # the allocator never handed an address out again: results were right, but the case went untested
        pytest.skip("the allocator did not re-use an address; the stale-cache case was not exercised")


def test_fused_deep_moe_with_tensor_lists_packs_once(buffer, monkeypatch):
    """Per-expert weight lists through Buffer.fused_deep_moe (32 experts, 64 weight tensors in all): bit-exact against
    the oracle, the whole list pre-packed by one launch per operand, and a second call with the same tensors pre-packs
    nothing."""
    bs, hidden, ffn, num_experts, num_topk = 64, 256, 256, 32, 4
    torch.manual_seed(11)
    x = (torch.rand((bs, hidden), device="cuda") * 10 - 5).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(num_experts, device="cuda")[:num_topk] for _ in range(bs)]).to(torch.int32)
    es = torch.rand((bs, num_topk), dtype=torch.float32, device="cuda")
    g1 = [torch.randint(-16, 16, (hidden, ffn), dtype=torch.int8, device="cuda") for _ in range(num_experts)]
    g2 = [torch.randint(-16, 16, (ffn // 2, hidden), dtype=torch.int8, device="cuda") for _ in range(num_experts)]
    s1 = [(torch.rand(ffn, dtype=torch.float32, device="cuda") * 0.003 + 0.0015) for _ in range(num_experts)]
    s2 = [(torch.rand(hidden, dtype=torch.float32, device="cuda") * 0.003 + 0.0015).to(torch.bfloat16) for _ in range(num_experts)]
    packs = []
    real = buffer.runtime.prepack_weight
    monkeypatch.setattr(buffer.runtime, "prepack_weight", lambda w, int4=False: (packs.append(tuple(w.shape)), real(w, int4=int4))[1])
    ref, counts = zo.fused_moe(host(x), zo.DT_BF16, host(ids), host(es), host(torch.stack(g1)), host(torch.stack(s1)),
                               host(torch.stack(g2)), host(torch.stack(s2)), num_experts, 0)
    for call in range(2):
        out, nums = buffer.fused_deep_moe(x=x, topk_idx=ids, gmm1_permuted_weight=g1, gmm1_permuted_weight_scale=s1,
                                          gmm2_weight=g2, gmm2_weight_scale=s2, topk_weights=es, num_experts=num_experts,
                                          is_tensor_list=True)
        assert np.array_equal(host(nums), counts) and np.array_equal(host(out), ref), call
        assert packs == [(num_experts, hidden, ffn), (num_experts, ffn // 2, hidden)], (call, packs)
