"""The operator layer under `memfabric_hybrid_amd.buffer.Buffer`: one method per zbal operator.

`OperatorBuffer` plays the part of adaptor::deep_ep::Buffer (reference
app/zbal/src/csrc/adaptor/deepep/zbal_deepep.cpp), the C++ object the
reference's Python `Buffer` keeps as `self.runtime`: it allocates the
operators' tensors with the reference's shapes and dtypes and makes one or
more calls through the zbal C ABI per method. Nothing here synchronises with
the host; the DeepEP-compatible signatures, handle tuples and Python lists
live in buffer.py. Differences from the reference's adaptor, all deliberate:
  * no host synchronisation between notify and dispatch (the reference reads
    the received-token count back with .item(), zbal_deepep.cpp:359): outputs
    are sized for the worst case tokens * topk rows;
  * one process: MoE operators run on a group of one rank; further "ranks" exist only as HBM windows
    for the reductions;
  * `use_fp8` selects real e4m3 with 1x128 scales when fp8_block_scale=True
    (the reference maps the flag to int8, zbal_deepep.cpp:514,525).
torch is used for device memory and streams only.
"""
import ctypes
import os
import threading

import torch

from . import capi

_LOCK = threading.Lock()
_STATE = {"world": None, "local": None, "users": 0}

# The process models this many "ranks" as local HBM windows; reductions may use groups up to this size.
MODEL_WORLD_SIZE = 16


def _create_comm(lib, name, world, size, rank):
    co = capi.CommOptions(name=name, backendType=capi.BACKEND_GPU, isWorldGroup=world, groupSize=size,
                          groupRankId=rank)
    comm = ctypes.c_void_p()
    capi.check("zbal_comm_create", lib.zbal_comm_create(ctypes.byref(co), ctypes.byref(comm)))
    return comm


def _acquire(device_index):
    """Bootstrap once per process; returns the one-rank group the MoE operators run on."""
    lib = capi.load()
    with _LOCK:
        if _STATE["world"] is None:
            opts = capi.BootstrapOptions()
            capi.check("zbal_bootstrap_options_init", lib.zbal_bootstrap_options_init(ctypes.byref(opts)))
            opts.worldSize, opts.rankId, opts.deviceId = MODEL_WORLD_SIZE, 0, device_index
            capi.check("zbal_bootstrap", lib.zbal_bootstrap(ctypes.byref(opts), None))
            _STATE["world"] = _create_comm(lib, b"world", 1, MODEL_WORLD_SIZE, 0)
            _STATE["local"] = _create_comm(lib, b"local", 0, 1, 0)
        _STATE["users"] += 1
        return _STATE["local"]


def _release():
    lib = capi.load()
    with _LOCK:
        _STATE["users"] -= 1
        if _STATE["users"] == 0 and _STATE["world"] is not None:
            lib.zbal_comm_destroy_all(0)
            lib.zbal_unbootstrap(0)
            _STATE["world"] = _STATE["local"] = None


def create_group(name, size, rank):
    """A sub-group of `size` modelled ranks in which this process is `rank` (needs a live Buffer)."""
    if _STATE["world"] is None:
        raise RuntimeError("create a Buffer first: it bootstraps the library")
    return _create_comm(capi.load(), name.encode(), 0, size, rank)


def destroy_group(comm):
    capi.check("zbal_comm_destroy", capi.load().zbal_comm_destroy(comm, 0))


class OperatorBuffer:
    """One-rank MoE layout / dispatch / combine / fused-MoE operators on worst-case-sized tensors."""

    num_ranks = 1
    rank = 0

    def __init__(self, device=None):
        if not torch.cuda.is_available():
            raise RuntimeError("memfabric_hybrid_amd needs a GPU; there is no CPU path")
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        self.lib = capi.load()
        self.comm = _acquire(self.device.index or 0)
        self.send_token_idx = None       # kept between layout, dispatch and combine (zbal_deepep.cpp:254,305,423)
        self._tables = {}                # device address tables of tensor-list operands
        self._closed = False

    def close(self):
        if not self._closed:
            self._closed = True
            _release()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- helpers ---------------------------------------------------------------------------
    def _empty(self, shape, dtype):
        return torch.empty(shape, dtype=dtype, device=self.device)

    @staticmethod
    def _ti(t, **kw):
        return ctypes.byref(capi.tensor_info(t, **kw))

    def _list_ti(self, seq, num_experts, live, **kw):
        """Descriptor of a tensor list: shape and type of the stacked tensor, `data` = a device table of the
        per-expert addresses (kept in a small cache, so repeated calls with the same tensors copy nothing). The
        descriptor holds the table's raw address only, so the table itself is appended to `live`, which the caller
        keeps until its operator call has been issued: the cache may drop its own reference at any insertion."""
        if len(seq) != num_experts:
            raise ValueError("a tensor list needs one tensor per expert")
        first = seq[0]
        per = tuple(first.shape[1:]) if first.shape[0] == 1 and first.dim() == 3 else tuple(first.shape)
        for t in seq:
            if not t.is_contiguous() or t.dtype != first.dtype or t.numel() != first.numel():
                raise ValueError("tensor-list entries must be contiguous and alike")
        key = tuple(t.data_ptr() for t in seq)
        table = self._tables.pop(key, None)
        if table is None:
            table = torch.tensor(key, dtype=torch.int64).to(self.device)
        self._tables[key] = table        # most recently used last
        while len(self._tables) > 64:
            del self._tables[next(iter(self._tables))]
        live.append(table)
        ti = capi.tensor_info(first, shape=(num_experts,) + per, **kw)
        ti.data = table.data_ptr()
        return ctypes.byref(ti)

    # -- router (extension) ------------------------------------------------------------------
    def topk_route(self, logits, num_topk, idx_dtype=torch.int64):
        """idx_dtype: torch.int64 (what get_dispatch_layout takes) or torch.int32 (what dispatch / fused_deep_moe take)"""
        T = logits.shape[0]
        idx = self._empty((T, num_topk), idx_dtype)
        w = self._empty((T, num_topk), torch.float32)
        capi.check("zbal_moe_topk_route", self.lib.zbal_moe_topk_route(
            self._ti(logits), num_topk, self._ti(idx), self._ti(w), self.comm, capi.stream_ptr(), 0))
        return idx, w

    # -- normal mode -------------------------------------------------------------------------
    def get_dispatch_layout(self, topk_idx, num_experts):
        """zbal_deepep.cpp:209-257. Returns (num_tokens_per_rank, None, num_tokens_per_expert, is_token_in_rank, None)."""
        assert topk_idx.dim() == 2 and topk_idx.is_contiguous() and topk_idx.dtype == torch.int64
        T, K = topk_idx.shape
        per_expert = self._empty((num_experts,), torch.int32)
        per_rank = self._empty((self.num_ranks,), torch.int32)
        send_idx = self._empty((T, K), torch.int32)
        scratch = self._empty((num_experts * 50,), torch.int32)
        capi.check("zbal_dispatch_normal_layout", self.lib.zbal_dispatch_normal_layout(
            self._ti(topk_idx), T, num_experts, K, self._ti(per_rank), self._ti(per_expert), self._ti(send_idx),
            self._ti(scratch), self.comm, capi.stream_ptr(), 0))
        self.send_token_idx = send_idx
        valid = (topk_idx >= 0) & (topk_idx < num_experts)
        is_token_in_rank = valid.any(dim=1, keepdim=True).to(torch.int32)   # the reference leaves this unwritten
        return per_rank, None, per_expert, is_token_in_rank, None

    def notify(self, num_tokens_per_expert, num_topk):
        """zbal_deepep.cpp:318-357: received counts, exclusive put offsets and the balance matrix, left on the device."""
        E = num_tokens_per_expert.shape[0]
        note = dict(recv_data=self._empty((1, E), torch.int32), recv_per_expert=self._empty((E,), torch.int64),
                    put_offset=self._empty((1, E), torch.int32), balance_matrix=self._empty((1, 2), torch.int32),
                    total_recv=self._empty((1,), torch.int32))
        capi.check("zbal_dispatch_normal_notify", self.lib.zbal_dispatch_normal_notify(
            self._ti(num_tokens_per_expert), E, num_topk, self._ti(note["recv_data"]), self._ti(note["total_recv"]),
            self._ti(note["recv_per_expert"]), self._ti(note["put_offset"]), self._ti(note["balance_matrix"]),
            self.comm, capi.stream_ptr(), 0))
        return note

    def dispatch(self, x, topk_idx, topk_weights, num_tokens_per_expert, quant_mode=capi.NO_QUANT, recv_rows=None,
                 notified=None):
        """zbal_deepep.cpp:259-393. Returns (recv_x, recv_x_scales, num_recv_tokens_per_expert (device int64), handle).
        recv_rows: rows of the receive tensors (default: the worst case tokens * topk; rows past a smaller tensor's
        end are dropped); notified: the result of notify() when the caller has already run it."""
        assert self.send_token_idx is not None, "call get_dispatch_layout first"
        T, H = x.shape
        K = topk_idx.shape[1]
        E = num_tokens_per_expert.shape[0]
        expert_ids = topk_idx.to(torch.int32)
        note = self.notify(num_tokens_per_expert, K) if notified is None else notified
        put_offset, balance = note["put_offset"], note["balance_matrix"]
        rows = max(T * K, 1) if recv_rows is None else max(int(recv_rows), 1)
        if quant_mode == capi.NO_QUANT:
            recv_x = self._empty((rows, H), x.dtype)
            scales = self._empty((1,), torch.float32)
        elif quant_mode == capi.QUANT_INT8:
            recv_x = self._empty((rows, H), torch.int8)
            scales = self._empty((rows,), torch.float32)
        else:
            recv_x = self._empty((rows, H), torch.float8_e4m3fn)
            scales = self._empty((rows, H // 128), torch.float32)
        capi.check("zbal_dispatch_normal", self.lib.zbal_dispatch_normal(
            self._ti(x), self._ti(expert_ids), self._ti(self.send_token_idx), self._ti(put_offset), self._ti(balance),
            E, quant_mode, self._ti(recv_x), self._ti(scales), self.comm, capi.stream_ptr(), 0))
        handle = dict(put_offset=put_offset, balance_matrix=balance, expert_ids=expert_ids,
                      send_token_idx=self.send_token_idx, total_recv=note["total_recv"], num_experts=E)
        return recv_x, scales, note["recv_per_expert"], handle

    def combine(self, x, handle, topk_weights):
        """zbal_deepep.cpp:395-452."""
        T, K = handle["expert_ids"].shape
        H = x.shape[1]
        out = self._empty((T, H), x.dtype)
        capi.check("zbal_combine_normal", self.lib.zbal_combine_normal(
            self._ti(x), self._ti(handle["put_offset"]), self._ti(topk_weights), self._ti(handle["expert_ids"]),
            self._ti(handle["send_token_idx"]), self._ti(handle["balance_matrix"]), handle["num_experts"],
            self._ti(out), self.comm, capi.stream_ptr(), 0))
        return out

    # -- low-latency mode ----------------------------------------------------------------------
    def low_latency_dispatch(self, x, topk_idx, num_max_dispatch_tokens_per_rank, num_experts, use_fp8=True,
                             fp8_block_scale=False):
        """zbal_deepep.cpp:454-565. Returns (packed_recv_x, packed_recv_x_scales, packed_recv_count, handle)."""
        T, H = x.shape
        K = topk_idx.shape[1]
        expert_ids = topk_idx.to(torch.int32)
        rows = max(T * K, 1)
        token_nums_type = int(os.environ.get("MOE_EXPERT_TOKEN_NUMS_TYPE", "1"))
        if not use_fp8:
            qm, recv = capi.NO_QUANT, self._empty((rows, H), x.dtype)
            scales = self._empty((rows,), torch.float32)
        elif fp8_block_scale:
            qm, recv = capi.QUANT_FP8_B128, self._empty((rows, H), torch.float8_e4m3fn)
            scales = self._empty((rows, H // 128), torch.float32)
        else:
            qm, recv = capi.QUANT_INT8, self._empty((rows, H), torch.int8)
            scales = self._empty((rows,), torch.float32)
        expand_idx = self._empty((rows,), torch.int32)
        ep_recv_count = self._empty((num_experts,), torch.int32)
        packed_recv_count = self._empty((num_experts,), torch.int64)
        put_offset = self._empty((num_experts,), torch.int32)
        put_offset_status = self._empty((num_experts,), torch.float32)
        capi.check("zbal_dispatch_low_latency", self.lib.zbal_dispatch_low_latency(
            self._ti(x), self._ti(expert_ids), num_experts, 1, 0, qm, max(T, num_max_dispatch_tokens_per_rank), 0,
            token_nums_type, self._ti(recv), self._ti(scales), self._ti(expand_idx), self._ti(packed_recv_count),
            self._ti(ep_recv_count), self._ti(put_offset), self._ti(put_offset_status), self.comm, capi.stream_ptr(),
            0))
        handle = dict(expert_ids=expert_ids, expand_idx=expand_idx, ep_recv_count=ep_recv_count,
                      num_experts=num_experts)
        return recv, scales, packed_recv_count, handle

    def low_latency_combine(self, x, topk_weights, handle):
        """zbal_deepep.cpp:567-656."""
        T, K = handle["expert_ids"].shape
        H = x.shape[1]
        out = self._empty((T, H), x.dtype)
        capi.check("zbal_combine_low_latency", self.lib.zbal_combine_low_latency(
            self._ti(x), self._ti(handle["expert_ids"]), self._ti(handle["expand_idx"], shape=(T, K)),
            self._ti(handle["ep_recv_count"]), self._ti(topk_weights), self._ti(out), handle["num_experts"],
            self.comm, capi.stream_ptr(), 0))
        return out

    # -- fused MoE ------------------------------------------------------------------------------
    def prepack_weight(self, w, int4=False):
        """[E,K,N] one byte per element -> the library's pre-packed layout (the reference's format cast); shape stays [E,N,K]."""
        E, K, N = w.shape
        if int4:
            dst = self._empty((E, N, K // 2), torch.uint8)
            capi.check("zbal_moe_weight_prepack", self.lib.zbal_moe_weight_prepack(
                self._ti(w), self._ti(dst, dtype=capi.DT_INT4X2), self.comm, capi.stream_ptr(), 0))
        else:
            dst = self._empty((E, N, K), w.dtype)
            capi.check("zbal_moe_weight_prepack", self.lib.zbal_moe_weight_prepack(
                self._ti(w), self._ti(dst), self.comm, capi.stream_ptr(), 0))
        return dst

    def fused_workspace_bytes(self, tokens, hidden, topk, num_experts, gmm1_h_len, quant_mode, share_gmm1_h_len=0):
        n = self.lib.zbal_fused_deep_moe_workspace_size(tokens, hidden, topk, num_experts, gmm1_h_len, share_gmm1_h_len,
                                                        quant_mode)
        if n == 0:
            raise ValueError("invalid fused MoE shape")
        return int(n)

    def fused_deep_moe(self, x, topk_idx, gmm1_permuted_weight, gmm1_permuted_weight_scale, gmm2_weight,
                       gmm2_weight_scale, topk_weights, num_experts, quant_mode=0, expert_smooth_scales=None,
                       share_gmm1_weight=None, share_gmm1_scale=None, share_gmm2_weight=None, share_gmm2_scale=None,
                       share_smooth_scales=None, x_active_mask=None, workspace=None, out=None, is_tensor_list=False,
                       share_out=None):
        """zbal_deepep.cpp:658-802. Weights are pre-packed (prepack_weight; shared-expert weights as [1,N,K]).
        Returns (output, share_output, expert_token_nums) like the reference; share_output is None without a shared
        expert. x_active_mask [T] bool: only the first sum(mask) tokens are routed; the other rows of `out` keep
        their contents. is_tensor_list: the four routed-expert operands are sequences of per-expert tensors (each
        pre-packed on its own, [1,N,K] or [N,K]); the library receives one device table of addresses per operand."""
        T, H = x.shape
        K = topk_idx.shape[1]
        n1 = gmm1_permuted_weight[0].shape[-2] if is_tensor_list else gmm1_permuted_weight.shape[1]
        shared = share_gmm1_weight is not None
        sn1 = share_gmm1_weight.shape[-2] if shared else 0
        expert_ids = topk_idx if topk_idx.dtype == torch.int32 else topk_idx.to(torch.int32)
        if workspace is None:
            workspace = self._empty((self.fused_workspace_bytes(T, H, K, num_experts, n1, quant_mode, sn1),), torch.uint8)
        if out is None:
            out = self._empty((T, H), x.dtype)
        if shared and share_out is None:
            share_out = self._empty((T, H), x.dtype)
        if not shared:
            share_out = None
        token_nums = self._empty((num_experts,), torch.int64)
        wdt = {0: None, 1: None, 2: capi.DT_FP8_E4M3, 3: capi.DT_INT4X2}[quant_mode]
        null = ctypes.byref(capi.TensorInfo())
        live = []                        # this call's address tables, referenced until the call has been issued
        if is_tensor_list:
            def wti(t, **kw):
                return self._list_ti(t, num_experts, live, **kw)
        else:
            wti = self._ti
        capi.check("zbal_fused_deep_moe", self.lib.zbal_fused_deep_moe(
            self._ti(x), self._ti(expert_ids),
            wti(gmm1_permuted_weight, dtype=wdt, weight_format=capi.WEIGHT_FORMAT_PREPACKED),
            wti(gmm1_permuted_weight_scale),
            wti(gmm2_weight, dtype=wdt, weight_format=capi.WEIGHT_FORMAT_PREPACKED), wti(gmm2_weight_scale),
            self._ti(topk_weights), self._ti(expert_smooth_scales) if expert_smooth_scales is not None else null,
            self._ti(share_gmm1_weight, dtype=wdt, weight_format=capi.WEIGHT_FORMAT_PREPACKED) if shared else null,
            self._ti(share_gmm1_scale) if shared else null,
            self._ti(share_gmm2_weight, dtype=wdt, weight_format=capi.WEIGHT_FORMAT_PREPACKED) if shared else null,
            self._ti(share_gmm2_scale) if shared else null,
            self._ti(share_smooth_scales) if share_smooth_scales is not None else null,
            self._ti(x_active_mask.view(torch.uint8)) if x_active_mask is not None else null,
            self._ti(out), self._ti(share_out) if shared else null, self._ti(token_nums), self._ti(workspace),
            num_experts, quant_mode, 0, n1, sn1, int(is_tensor_list), self.comm, capi.stream_ptr(), 0))
        return out, share_out, token_nums
