"""DeepEP-compatible `Buffer` for one MI355X: the Python face a caller of the reference switches to.

Method names, positional order, defaults and return tuples follow the reference's
`zbal.Buffer` (app/zbal/src/python/zbal/zbal_buffer.py) and the C++ adaptor under it
(app/zbal/src/csrc/adaptor/deepep/zbal_deepep.cpp); each method cites the lines it
mirrors. The work is done by `operators.OperatorBuffer` (kept as `self.runtime`, the
name the reference gives its C++ object), which calls the zbal C ABI.

What differs, because this build runs one rank on one GPU:
  * `group` may be None (or any object with rank() / size()); a group of more than one
    rank is refused: the cross-rank transport is not part of this build;
  * `fused_deep_moe` takes the weights in the operator's logical layout
    ([experts, hidden, gmm1_h_len] and [experts, gmm1_h_len / 2, hidden]) exactly as the
    reference does before its NZ format cast (test/python/deepep/test_fused_deep_moe.py:66-69)
    and pre-packs them once per weight tensor (cached); already pre-packed tensors from
    `prepack_weight` pass through;
  * `dispatch` honours `num_worst_tokens` (no host synchronisation, empty list), which
    the reference accepts and ignores;
  * events are real: `EventOverlap.current_stream_wait()` waits for the stream position
    captured when the operator returned (the reference's is a no-op).
"""
import os
import weakref
from typing import Callable, List, Optional, Tuple, Union

import torch

from . import capi
from .operators import OperatorBuffer


class Config:
    """Tuning record of the reference (adaptor/deepep/zbal_deepep_config.h:23-49); the kernels here take no tuning."""

    def __init__(self, num_sms: int, num_max_nvl_chunked_send_tokens: int, num_max_nvl_chunked_recv_tokens: int,
                 num_max_rdma_chunked_send_tokens: int, num_max_rdma_chunked_recv_tokens: int) -> None:
        self.num_sms = num_sms
        self.num_max_nvl_chunked_send_tokens = num_max_nvl_chunked_send_tokens
        self.num_max_nvl_chunked_recv_tokens = num_max_nvl_chunked_recv_tokens
        self.num_max_rdma_chunked_send_tokens = num_max_rdma_chunked_send_tokens
        self.num_max_rdma_chunked_recv_tokens = num_max_rdma_chunked_recv_tokens

    def get_nvl_buffer_size_hint(self, hidden_bytes: int, num_ranks: int) -> int:
        return hidden_bytes

    def get_rdma_buffer_size_hint(self, hidden_bytes: int, num_ranks: int) -> int:
        return hidden_bytes


class EventHandle:
    """A position on the current stream (adaptor/deepep/zbal_deep_event.h:22-31, there without content)."""

    def __init__(self) -> None:
        self.event = torch.cuda.Event()
        self.event.record(torch.cuda.current_stream())

    def current_stream_wait(self) -> None:
        torch.cuda.current_stream().wait_event(self.event)


class EventOverlap:
    """python/zbal/zbal_utils.py:8-36: an event plus tensors kept alive until it has passed."""

    def __init__(self, event: Optional[EventHandle] = None, extra_tensors: Optional[Tuple[torch.Tensor]] = None) -> None:
        self.event = event
        self.extra_tensors = extra_tensors

    def current_stream_wait(self) -> None:
        if self.event is not None:
            self.event.current_stream_wait()


def get_low_latency_rdma_size_hint(num_max_dispatch_tokens_per_rank: int, hidden: int, num_ranks: int,
                                   num_experts: int) -> int:
    """adaptor/deepep/zbal_deepep_config.cpp:18-24."""
    return num_max_dispatch_tokens_per_rank


PADDING_SIZE = 1      # an empty batch is padded to this many tokens (zbal_deepep.cpp:85, 470-490)


class Buffer:
    """zbal_buffer.py:12-84. One rank, one GPU: dispatch and combine permute through this GPU's HBM."""

    num_sms: int = 20

    def __init__(self, group=None, num_nvl_bytes: int = 0, num_rdma_bytes: int = 0, low_latency_mode: bool = False,
                 num_qps_per_rank: int = 12, allow_nvlink_for_low_latency_mode: bool = True,
                 allow_mnnvl: bool = False, device=None) -> None:
        self.rank = group.rank() if group is not None else 0
        self.group_size = group.size() if group is not None else 1
        if self.group_size != 1:
            raise NotImplementedError("this build runs the MoE operators on a group of one rank (one GPU)")
        self.num_nvl_bytes = num_nvl_bytes
        self.num_rdma_bytes = num_rdma_bytes
        self.low_latency_mode = low_latency_mode
        self.runtime = OperatorBuffer(device)
        self.device = self.runtime.device
        self._packed = {}          # logical weight tensor -> its pre-packed copy
        self._pad = None           # what low_latency_dispatch padded, for the combine that follows

    def close(self) -> None:
        self.runtime.close()

    # ---- static helpers -------------------------------------------------------------------------------
    @staticmethod
    def get_dispatch_config(num_ranks: int) -> Config:
        """zbal_buffer.py:86-109 (the table's one-rank entry is this build's addition)."""
        table = {1: (24, 256, 6, 128), 2: (24, 256, 6, 128), 4: (6, 256, 6, 128), 8: (6, 256, 6, 128),
                 16: (36, 288, 20, 128), 24: (8, 288, 32, 128), 32: (32, 288, 32, 128), 64: (20, 288, 28, 128),
                 128: (20, 560, 32, 128), 144: (32, 720, 12, 128), 160: (28, 720, 12, 128)}
        return Config(Buffer.num_sms, *table[num_ranks])

    @staticmethod
    def get_combine_config(num_ranks: int) -> Config:
        """zbal_buffer.py:111-135."""
        table = {1: (10, 256, 6, 128), 2: (10, 256, 6, 128), 4: (9, 256, 6, 128), 8: (4, 256, 6, 128),
                 16: (4, 288, 12, 128), 24: (1, 288, 8, 128), 32: (1, 288, 8, 128), 64: (1, 288, 20, 128),
                 128: (1, 560, 12, 128), 144: (2, 720, 8, 128), 160: (2, 720, 8, 128)}
        return Config(Buffer.num_sms, *table[num_ranks])

    @staticmethod
    def set_num_sms(new_num_sms: int) -> None:
        """zbal_buffer.py:137-146."""
        if not new_num_sms % 2 == 0:
            raise ValueError("The SM count must be even")
        Buffer.num_sms = new_num_sms

    @staticmethod
    def capture() -> EventOverlap:
        """zbal_buffer.py:148-155: an event on the current stream."""
        return EventOverlap(EventHandle())

    @staticmethod
    def get_low_latency_rdma_size_hint(num_max_dispatch_tokens_per_rank: int, hidden: int, num_ranks: int,
                                       num_experts: int) -> int:
        """zbal_buffer.py:157-166."""
        return get_low_latency_rdma_size_hint(num_max_dispatch_tokens_per_rank, hidden, num_ranks, num_experts)

    @staticmethod
    def _wait(previous_event: Optional[EventOverlap]) -> None:
        if previous_event is not None:
            previous_event.current_stream_wait()

    @staticmethod
    def _event(async_finish: bool, tensors=None) -> EventOverlap:
        return EventOverlap(EventHandle(), tensors) if async_finish else EventOverlap(None)

    # ---- normal mode ----------------------------------------------------------------------------------
    def get_dispatch_layout(self, topk_idx: torch.Tensor, num_experts: int,
                            previous_event: Optional[EventOverlap] = None, async_finish: bool = False,
                            allocate_on_comm_stream: bool = False
                            ) -> Tuple[torch.Tensor, Optional[torch.Tensor], torch.Tensor, torch.Tensor, EventOverlap]:
        """zbal_buffer.py:168-214, zbal_deepep.cpp:209-257. topk_idx [tokens, topk] int64, -1 = no selection.
        Returns (num_tokens_per_rank, None, num_tokens_per_expert, is_token_in_rank, event)."""
        if topk_idx.dim() != 2 or not topk_idx.is_contiguous():
            raise ValueError("Layout: topk_idx must be a contiguous [num_tokens, num_topk] tensor")
        if num_experts <= 0:
            raise ValueError("Layout: check num_experts failed: %d" % num_experts)
        self._wait(previous_event)
        per_rank, per_rdma, per_expert, in_rank, _ = self.runtime.get_dispatch_layout(topk_idx, num_experts)
        return per_rank, per_rdma, per_expert, in_rank, self._event(async_finish)

    def dispatch(self, x: Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]], handle: Optional[Tuple] = None,
                 num_tokens_per_rank: Optional[torch.Tensor] = None,
                 num_tokens_per_rdma_rank: Optional[torch.Tensor] = None,
                 is_token_in_rank: Optional[torch.Tensor] = None,
                 num_tokens_per_expert: Optional[torch.Tensor] = None, topk_idx: Optional[torch.Tensor] = None,
                 topk_weights: Optional[torch.Tensor] = None, expert_alignment: int = 1, num_worst_tokens: int = 0,
                 config: Optional[Config] = None, previous_event: Optional[EventOverlap] = None,
                 async_finish: bool = False, allocate_on_comm_stream: bool = False,
                 dispatch_wait_recv_cost_stats: Optional[torch.Tensor] = None
                 ) -> Tuple[Union[Tuple[torch.Tensor, torch.Tensor], torch.Tensor], Optional[torch.Tensor],
                            Optional[torch.Tensor], List[int], Tuple, EventOverlap]:
        """zbal_buffer.py:216-348, zbal_deepep.cpp:259-393. Rows arrive expert-major, in flat pick order within an
        expert. With DEEP_NORMAL_MODE_USE_INT8_QUANT=1 the rows are int8 with one fp32 scale each and recv_x is the
        pair. Like the reference this reads the received-row count back (one host synchronisation) to size recv_x
        and to build the Python list, unless num_worst_tokens is given: then recv_x has that many rows, the list is
        empty and nothing waits for the GPU.
        Returns (recv_x, None, None, num_recv_tokens_per_expert_list, handle, event)."""
        config = self.get_dispatch_config(self.group_size) if config is None else config
        if isinstance(x, tuple):
            raise NotImplementedError("Not support fp8")
        use_quant = os.getenv("DEEP_NORMAL_MODE_USE_INT8_QUANT") == "1"
        if handle is not None:
            raise NotImplementedError("Optional communication handle is not supported yet.")
        if not (num_tokens_per_rank is not None and is_token_in_rank is not None and num_tokens_per_expert is not None):
            raise ValueError("num_tokens_per_rank, is_token_in_rank, num_tokens_per_expert must be valid")
        if num_tokens_per_expert.dtype != torch.int32 or num_tokens_per_rank.dtype != torch.int32:
            raise ValueError("num_tokens_per_expert and num_tokens_per_rank must be torch.int")
        if x.dim() != 2 or not x.is_contiguous():
            raise ValueError("x dim not 2 or not contiguous")
        if num_tokens_per_expert.dim() != 1 or num_tokens_per_expert.size(0) % self.group_size != 0:
            raise ValueError("num_tokens_per_expert check failed")
        if num_tokens_per_rank.dim() != 1 or num_tokens_per_rank.size(0) != self.group_size:
            raise ValueError("num_tokens_per_rank check failed")
        if topk_idx is None or topk_idx.dim() != 2 or topk_idx.size(0) != x.size(0) or not topk_idx.is_contiguous():
            raise ValueError("topk_idx check failed")
        token_nums_type = int(os.environ.get("MOE_EXPERT_TOKEN_NUMS_TYPE", "1"))
        if token_nums_type not in (0, 1):
            raise ValueError("expert_token_nums_type is invalid")
        self._wait(previous_event)
        K = topk_idx.size(1)
        note = self.runtime.notify(num_tokens_per_expert, K)
        counts = None
        if num_worst_tokens > 0:
            rows = num_worst_tokens
        else:
            counts = note["recv_per_expert"].cpu()          # the one host synchronisation (zbal_deepep.cpp:359, 379)
            total = int(counts.sum().item())
            rows = 1 if total == 0 else total               # zbal_deepep.cpp:360
        qm = capi.QUANT_INT8 if use_quant else capi.NO_QUANT
        recv_x, recv_x_scales, _, h = self.runtime.dispatch(x, topk_idx, topk_weights, num_tokens_per_expert, qm,
                                                            recv_rows=rows, notified=note)
        num_recv_tokens_per_expert_list: List[int] = []
        if counts is not None:
            run = 0
            for c in counts.tolist():
                run = run + int(c) if token_nums_type == 0 else int(c)
                num_recv_tokens_per_expert_list.append(run)
        handle = (is_token_in_rank, topk_idx, topk_weights, h["put_offset"], h["balance_matrix"])
        return ((recv_x, recv_x_scales) if use_quant else recv_x, None, None, num_recv_tokens_per_expert_list, handle,
                self._event(async_finish))

    def combine(self, x: torch.Tensor, handle: Tuple, topk_weights: Optional[torch.Tensor] = None,
                bias: Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]] = None, config: Optional[Config] = None,
                previous_event: Optional[EventOverlap] = None, async_finish: bool = False,
                allocate_on_comm_stream: bool = False, combine_send_cost_stats: Optional[torch.Tensor] = None
                ) -> Tuple[torch.Tensor, Optional[torch.Tensor], EventOverlap]:
        """zbal_buffer.py:350-411, zbal_deepep.cpp:395-452: out[t] = sum_k w[t, k] * x[row(t, k)] with the weights the
        handle carries (those given to dispatch), as the reference. Returns (combined_x, None, event)."""
        is_token_in_rank, topk_idx, topk_weights_ori, put_offset, balance_matrix = handle
        if x.dim() != 2 or not x.is_contiguous():
            raise ValueError("x dim not 2 or not contiguous")
        if topk_weights_ori is None:
            raise ValueError("topk_weights is empty")
        if topk_weights_ori.dim() != 2 or topk_weights_ori.size(1) != topk_idx.size(1) or \
                topk_weights_ori.dtype != torch.float32:
            raise ValueError("topk_weights check failed")
        self._wait(previous_event)
        h = dict(put_offset=put_offset, balance_matrix=balance_matrix, expert_ids=topk_idx.to(torch.int32),
                 send_token_idx=self.runtime.send_token_idx, num_experts=put_offset.size(1))
        out = self.runtime.combine(x, h, topk_weights_ori)
        return out, None, self._event(async_finish)

    # ---- low-latency mode -----------------------------------------------------------------------------
    def clean_low_latency_buffer(self, num_max_dispatch_tokens_per_rank: int, hidden: int, num_experts: int) -> None:
        """zbal_buffer.py:413-430: nothing to clean (no flags live between calls)."""
        return None

    def low_latency_dispatch(self, x: torch.Tensor, topk_idx: torch.Tensor, num_max_dispatch_tokens_per_rank: int,
                             num_experts: int, cumulative_local_expert_recv_stats: Optional[torch.Tensor] = None,
                             use_fp8: bool = True, round_scale: bool = False, use_ue8m0: bool = False,
                             async_finish: bool = False, return_recv_hook: bool = False
                             ) -> Tuple[Union[Tuple[torch.Tensor, torch.Tensor], torch.Tensor], torch.Tensor, Tuple,
                                        EventOverlap, Callable]:
        """zbal_buffer.py:432-534, zbal_deepep.cpp:454-565. `use_fp8` means int8 rows with one fp32 scale per row, as
        in the reference (zbal_deepep.cpp:514, 525). Rows are packed expert-major; packed_recv_count [experts] int64
        holds counts (MOE_EXPERT_TOKEN_NUMS_TYPE=1, default) or their running sum (0). An empty batch is padded to
        one token of ones that picks experts 0..topk-1, as the reference does.
        Returns (recv_x or (recv_x, scales), packed_recv_count, handle, event, hook)."""
        self._pad = None
        new_x, new_idx = x, topk_idx
        if topk_idx.size(0) < PADDING_SIZE:
            pad = PADDING_SIZE - topk_idx.size(0)
            K = topk_idx.size(1)
            xs = [x] if topk_idx.size(0) != 0 else []
            ts = [topk_idx] if topk_idx.size(0) != 0 else []
            for _ in range(pad):
                xs.append(torch.ones((1, x.size(1)), dtype=x.dtype, device=x.device))
                ts.append(torch.arange(0, K, dtype=topk_idx.dtype, device=topk_idx.device).reshape(1, K))
            new_x, new_idx = torch.cat(xs, 0), torch.cat(ts, 0)
            self._pad = dict(count=pad, ori_x=x.clone(), topk_idx=new_idx)
        recv, scales, packed_recv_count, h = self.runtime.low_latency_dispatch(
            new_x, new_idx, num_max_dispatch_tokens_per_rank, num_experts, use_fp8=use_fp8)
        handle = (h["expand_idx"], h["ep_recv_count"], num_max_dispatch_tokens_per_rank, x.size(1), num_experts,
                  packed_recv_count)
        kept = (x, topk_idx, recv, scales, packed_recv_count, h["expand_idx"], h["ep_recv_count"],
                cumulative_local_expert_recv_stats)
        return ((recv, scales) if use_fp8 else recv, packed_recv_count, handle,
                self._event(async_finish, kept if async_finish else None), (lambda: None))

    def low_latency_combine(self, x: torch.Tensor, topk_idx: torch.Tensor, topk_weights: torch.Tensor, handle: tuple,
                            zero_copy: bool = False, async_finish: bool = False, return_recv_hook: bool = False,
                            out: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, EventOverlap, Callable]:
        """zbal_buffer.py:536-609, zbal_deepep.cpp:567-656. x: the packed expert outputs, bf16.
        Returns (combined_x, event, hook)."""
        src_info, layout_range, num_max_dispatch_tokens_per_rank, hidden, num_experts, packed_recv_count = handle
        if x.dim() != 2 or not x.is_contiguous() or x.dtype != torch.bfloat16:
            raise ValueError("LL combine x check failed")
        new_idx, new_scales = topk_idx, topk_weights
        pad = self._pad
        if pad is not None:
            blocks = [topk_weights] if pad["count"] != PADDING_SIZE else []
            blocks += [torch.zeros((1, topk_weights.size(1)), dtype=topk_weights.dtype, device=topk_weights.device)
                       for _ in range(pad["count"])]
            new_idx, new_scales = pad["topk_idx"], torch.cat(blocks, 0)
        h = dict(expert_ids=new_idx.to(torch.int32), expand_idx=src_info, ep_recv_count=layout_range,
                 num_experts=num_experts)
        combined = self.runtime.low_latency_combine(x, new_scales, h)
        if pad is not None:
            combined = pad["ori_x"] if pad["count"] == PADDING_SIZE else combined[:PADDING_SIZE - pad["count"]]
            self._pad = None
        if out is not None:
            out.copy_(combined)
            combined = out
        kept = (x, topk_idx, topk_weights, src_info, layout_range, combined)
        return combined, self._event(async_finish, kept if async_finish else None), (lambda: None)

    # ---- fused MoE --------------------------------------------------------------------------------------
    def prepack_weight(self, w: torch.Tensor, int4: bool = False) -> torch.Tensor:
        """[experts, K, N] one byte per element -> the library's pre-packed layout (this build's counterpart of the
        reference's NZ format cast). The result is marked, so fused_deep_moe passes it through."""
        p = self.runtime.prepack_weight(w, int4=int4)
        p.zbal_prepacked = True
        return p

    @staticmethod
    def _weight_key(w: torch.Tensor):
        return (w.data_ptr(), tuple(w.shape), w.dtype, w._version)

    def _cache_get(self, key, sources):
        """The cached pre-packed form under `key`, or None. An entry is good only while every tensor it was made
        from is alive: once one is freed the allocator may hand its address to other weights of the same shape, and
        address, shape and version would still match."""
        entry = self._packed.pop(key, None)
        if entry is None or any(r() is None for r in entry[0]):
            return None
        self._packed[key] = entry        # most recently used last
        return entry[1]

    def _cache_put(self, key, sources, packed):
        self._packed[key] = ([weakref.ref(t) for t in sources], packed)
        while len(self._packed) > 16:    # a tensor list is one entry, however many experts it has
            del self._packed[next(iter(self._packed))]
        return packed

    def _packed_weight(self, w: torch.Tensor, int4: bool) -> torch.Tensor:
        if getattr(w, "zbal_prepacked", False):
            return w
        key = self._weight_key(w)
        packed = self._cache_get(key, [w])
        if packed is None:
            w3 = w if w.dim() == 3 else w.unsqueeze(0)
            packed = self._cache_put(key, [w], self.prepack_weight(w3.contiguous(), int4=int4))
        return packed

    def _packed_weight_list(self, ws, int4: bool):
        """A list of per-expert weights -> the list of their pre-packed forms. The whole list is one cache entry and
        one pre-pack launch (the experts stacked); the per-expert results are views of that one tensor."""
        ws = list(ws)
        if all(getattr(t, "zbal_prepacked", False) for t in ws):
            return ws
        key = ("list",) + tuple(self._weight_key(t) for t in ws)
        packed = self._cache_get(key, ws)
        if packed is None:
            stacked = torch.stack([t if t.dim() == 2 else t.squeeze(0) for t in ws], 0)
            whole = self.prepack_weight(stacked, int4=int4)
            views = []
            for e in range(len(ws)):
                v = whole[e:e + 1]
                v.zbal_prepacked = True
                views.append(v)
            packed = self._cache_put(key, ws, views)
        return packed

    def topk_route(self, logits: torch.Tensor, num_topk: int, idx_dtype=torch.int64):
        """Extension: softmax + top-k router; returns (topk_idx, topk_weights)."""
        return self.runtime.topk_route(logits, num_topk, idx_dtype)

    def fused_deep_moe(self, x: torch.Tensor, topk_idx: torch.Tensor, gmm1_permuted_weight: torch.Tensor,
                       gmm1_permuted_weight_scale: torch.Tensor, gmm2_weight: torch.Tensor,
                       gmm2_weight_scale: torch.Tensor, topk_weights: torch.Tensor, num_experts: int,
                       shared_expert_num: int = 0, shared_expert_rank_num: int = 0, quant_mode: int = 0,
                       num_max_dispatch_tokens_per_rank: int = 0, is_tensor_list: bool = False,
                       expert_smooth_scales: Optional[torch.Tensor] = None,
                       share_gmm1_weight: Optional[torch.Tensor] = None,
                       share_gmm1_scale: Optional[torch.Tensor] = None,
                       share_gmm2_weight: Optional[torch.Tensor] = None,
                       share_gmm2_scale: Optional[torch.Tensor] = None,
                       share_smooth_scales: Optional[torch.Tensor] = None,
                       x_active_mask: Optional[torch.Tensor] = None, share_gmm1_h_len: int = 0, fuse_mode: int = 0
                       ) -> Tuple[torch.Tensor, torch.Tensor]:
        """zbal_buffer.py:611-710, zbal_deepep.cpp:658-802: quantise -> permute -> GMM1 -> SwiGLU -> requantise -> GMM2
        -> weighted combine in one call. Weights [experts, hidden, gmm1_h_len] / [experts, gmm1_h_len/2, hidden], one
        byte per element (quant_mode 0 or 1: int8 with per-channel scales, the reference's only mode; 2 = e4m3 with
        128x128 block scales; 3 = int4 values in int8 storage with fp16 group scales), or tensor lists of per-expert
        tensors with is_tensor_list. The shared expert's output is kept in `last_share_output`.
        Returns (output [tokens, hidden], expert_token_nums [experts] int64)."""
        has_share = share_gmm1_weight is not None and share_gmm1_weight.numel() > 0
        if has_share and share_gmm1_h_len <= 0:
            print("[ZBAL WARNING] share_gmm1_weight provided but share_gmm1_h_len is not set (or <=0). "
                  "Please pass share_gmm1_h_len with the correct value to avoid kernel errors.")
        int4 = quant_mode == 3
        if is_tensor_list:
            w1 = self._packed_weight_list(gmm1_permuted_weight, int4)
            w2 = self._packed_weight_list(gmm2_weight, int4)
        else:
            w1, w2 = self._packed_weight(gmm1_permuted_weight, int4), self._packed_weight(gmm2_weight, int4)
        sw1 = self._packed_weight(share_gmm1_weight, int4) if has_share else None
        sw2 = self._packed_weight(share_gmm2_weight, int4) if has_share else None
        out, share_out, nums = self.runtime.fused_deep_moe(
            x, topk_idx.int(), w1, gmm1_permuted_weight_scale, w2, gmm2_weight_scale, topk_weights, num_experts,
            quant_mode=quant_mode, expert_smooth_scales=expert_smooth_scales, share_gmm1_weight=sw1,
            share_gmm1_scale=share_gmm1_scale if has_share else None, share_gmm2_weight=sw2,
            share_gmm2_scale=share_gmm2_scale if has_share else None, share_smooth_scales=share_smooth_scales,
            x_active_mask=x_active_mask, is_tensor_list=is_tensor_list)
        self.last_share_output = share_out
        return out, nums
