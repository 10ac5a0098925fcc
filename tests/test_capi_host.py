"""Host-side checks that need no GPU: the C ABI library loads and exports every
declared symbol, struct layouts match the reference's, validation and the
communicator lifecycle return the reference's codes (exercised on the
do-nothing backend, as the reference's own unit tests do)."""
import ctypes
import os
import re
import subprocess

import pytest

from memfabric_hybrid_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")


@pytest.fixture(scope="module")
def lib():
    return capi.load()


def declared_symbols():
    names = set()
    for f in os.listdir(INC):
        text = open(os.path.join(INC, f)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(zbal(?:hip)?_\w+)\s*\(", text))
    return names


def test_every_declared_symbol_is_exported_and_bound(lib):
    decl = declared_symbols()
    assert len(decl) >= 38
    for name in decl:
        assert hasattr(lib, name), "library does not export %s" % name
    assert decl == set(capi.SIGNATURES), decl ^ set(capi.SIGNATURES)


def test_headers_compile_as_c_and_cpp_and_struct_sizes(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "zbal.h"\n#include "zbal_hip_kernels.h"\n#include <stdio.h>\n'
                   'int main(void){printf("%zu %zu %zu %zu %zu\\n", sizeof(zbal_tensor_info_t),'
                   'sizeof(zbal_comm_options_t), sizeof(zbal_comm_property_t), sizeof(zbal_bootstrap_options_t),'
                   '__builtin_offsetof(zbal_tensor_info_t, shape));return 0;}\n')
    exe = tmp_path / "t"
    subprocess.check_call(["gcc", "-I", INC, str(src), "-o", str(exe)])
    out = subprocess.check_output([str(exe)]).decode().split()
    # reference zbal_def.h:141-147 measures 72 bytes with gcc on x86-64 (its comment says 64)
    assert int(out[0]) == 72 == ctypes.sizeof(capi.TensorInfo)
    assert int(out[1]) == ctypes.sizeof(capi.CommOptions)
    assert int(out[2]) == ctypes.sizeof(capi.CommProperty)
    assert int(out[3]) == ctypes.sizeof(capi.BootstrapOptions)
    assert int(out[4]) == 16 == capi.TensorInfo.shape.offset
    subprocess.check_call(["g++", "-std=c++17", "-fsyntax-only", "-x", "c++", "-I", INC, os.path.join(INC, "zbal.h")])


def test_enum_values_match_reference():
    assert (capi.DT_INT8, capi.DT_FP16, capi.DT_FP32, capi.DT_BF16, capi.DT_UINT32) == (0, 6, 7, 8, 11)
    assert (capi.REDUCE_PROD, capi.REDUCE_SUM, capi.REDUCE_MAX, capi.REDUCE_MIN) == (0, 1, 2, 3)
    assert (capi.NO_QUANT, capi.QUANT_INT8) == (0, 1)


def test_version_logger_and_last_error(lib):
    assert b"zbal" in lib.zbal_version()
    assert lib.zbal_set_logger_level(7) == capi.Z_INVALID_PARAM
    assert lib.zbal_set_logger_level(3) == 0
    seen = []
    CB = ctypes.CFUNCTYPE(None, ctypes.c_int, ctypes.c_char_p)
    cb = CB(lambda lvl, msg: seen.append((lvl, msg)))
    lib.zbal_set_logger(ctypes.cast(cb, ctypes.c_void_p))
    assert lib.zbal_comm_destroy(None, 0) == capi.Z_INVALID_PARAM
    assert seen and seen[-1][0] == 3 and b"comm is null" in seen[-1][1]
    assert b"comm is null" in lib.zbal_get_last_error_msg()
    assert b"comm is null" in lib.zbal_get_and_clear_last_error_msg()
    assert lib.zbal_get_last_error_msg() == b""
    lib.zbal_set_logger(None)


@pytest.fixture
def host_world(lib):
    """Bootstrap without touching a device (flags bit 0) and tear down afterwards."""
    opts = capi.BootstrapOptions()
    assert lib.zbal_bootstrap_options_init(ctypes.byref(opts)) == 0
    opts.flags = 1
    opts.worldSize = 8
    opts.rankId = 3
    assert lib.zbal_bootstrap(ctypes.byref(opts), None) == 0
    yield lib
    lib.zbal_comm_destroy_all(0)
    assert lib.zbal_unbootstrap(0) == 0


def make_comm(lib, name, world, size, rank, backend=capi.BACKEND_DUMMY):
    co = capi.CommOptions(name=name, backendType=backend, isWorldGroup=world, groupSize=size, groupRankId=rank)
    comm = ctypes.c_void_p()
    rc = lib.zbal_comm_create(ctypes.byref(co), ctypes.byref(comm))
    return rc, comm


def test_create_needs_bootstrap(lib):
    lib.zbal_set_logger_level(3)
    rc, _ = make_comm(lib, b"w", 1, 1, 0)
    assert rc == capi.Z_NOT_BOOTSTRAPPED
    assert lib.zbal_unbootstrap(0) == -14


def test_communicator_lifecycle(host_world):
    lib = host_world
    assert lib.zbal_bootstrap(ctypes.byref(capi.BootstrapOptions(worldSize=1)), None) == -13   # already bootstrapped
    assert lib.zbal_comm_get_global() is None
    rc, _ = make_comm(lib, b"sub", 0, 4, 1)
    assert rc == capi.Z_CREATE_COMM_FAILED              # world group must come first
    rc, _ = make_comm(lib, b"world", 1, 4, 1)
    assert rc == capi.Z_NOT_BOOTSTRAPPED                # size differs from the bootstrap's world size
    rc, world = make_comm(lib, b"world", 1, 8, 3)
    assert rc == 0 and lib.zbal_comm_get_global() == world.value
    rc, _ = make_comm(lib, b"world2", 1, 8, 3)
    assert rc == capi.Z_CREATE_COMM_FAILED              # only one world group
    rc, sub = make_comm(lib, b"sub", 0, 4, 1)
    assert rc == 0
    rc, _ = make_comm(lib, b"sub", 0, 4, 1)
    assert rc == capi.Z_CREATE_COMM_FAILED              # duplicate name
    rc, _ = make_comm(lib, b"big", 0, 16, 1)
    assert rc == capi.Z_NOT_BOOTSTRAPPED                # bigger than the world
    rc, _ = make_comm(lib, b"", 0, 4, 1)
    assert rc == capi.Z_INVALID_PARAM
    rc, _ = make_comm(lib, b"x" * 128, 0, 4, 1)
    assert rc == capi.Z_INVALID_PARAM
    assert lib.zbal_comm_get_by_name(b"sub") == sub.value
    assert lib.zbal_comm_get_by_name(b"nope") is None
    prop = capi.CommProperty()
    assert lib.zbal_comm_get_property(sub, ctypes.byref(prop)) == 0
    assert (prop.groupSize, prop.groupRankId, prop.isWorldGroup, prop.name) == (4, 1, 0, b"sub")
    assert lib.zbal_comm_get_property(ctypes.c_void_p(0x1234), ctypes.byref(prop)) == capi.Z_COMM_NOT_EXIST_BY_HANDLE
    assert lib.zbal_comm_destroy(world, 0) == capi.Z_COMM_DESTROY_GLOBAL_LAST
    assert lib.zbal_comm_destroy(ctypes.c_void_p(0x1234), 0) == 0     # unknown handle: not an error
    assert lib.zbal_comm_destroy(sub, 0) == 0
    assert lib.zbal_comm_get_by_name(b"sub") is None
    assert lib.zbal_comm_destroy(world, 0) == 0
    assert lib.zbal_comm_get_global() is None


def test_operator_validation_codes(host_world):
    """The null / range checks of reference zbal_operations.cpp and test_zbal_operations.cpp:166-213, 408-455."""
    lib = host_world
    rc, world = make_comm(lib, b"world", 1, 8, 3)
    assert rc == 0
    buf = ctypes.create_string_buffer(64)
    p = ctypes.cast(buf, ctypes.c_void_p)
    # null send buffer is a silent success
    assert lib.zbal_all_reduce(None, p, p, 4, capi.DT_FP32, capi.REDUCE_SUM, world, None) == 0
    assert lib.zbal_reduce_scatter(None, p, 4, capi.DT_FP32, capi.REDUCE_SUM, world, None) == 0
    assert lib.zbal_all_reduce(p, None, p, 4, capi.DT_FP32, capi.REDUCE_SUM, world, None) == -2
    assert lib.zbal_all_reduce(p, p, p, 0, capi.DT_FP32, capi.REDUCE_SUM, world, None) == -2
    assert lib.zbal_all_reduce(p, p, p, 4, 99, capi.REDUCE_SUM, world, None) == -2
    assert lib.zbal_all_reduce(p, p, p, 4, capi.DT_FP32, 9, world, None) == -2
    assert lib.zbal_all_reduce(p, p, p, 4, capi.DT_FP32, capi.REDUCE_SUM, None, None) == -2
    assert lib.zbal_all_reduce(p, p, None, 4, capi.DT_FP32, capi.REDUCE_SUM, world, None) == -2
    assert lib.zbal_all_reduce(p, p, p, 4, capi.DT_FP32, capi.REDUCE_SUM, world, None) == 0      # dummy backend
    assert lib.zbal_reduce_scatter(p, p, 0, capi.DT_FP32, capi.REDUCE_SUM, world, None) == -2
    ti = capi.TensorInfo()
    t = ctypes.byref(ti)
    assert lib.zbal_dispatch_normal_layout(None, 4, 8, 2, t, t, t, t, world, None, 0) == -2
    assert lib.zbal_dispatch_normal_layout(t, -1, 8, 2, t, t, t, t, world, None, 0) == -2
    assert lib.zbal_dispatch_normal_layout(t, 4, 0, 2, t, t, t, t, world, None, 0) == -2
    assert lib.zbal_dispatch_normal_layout(t, 4, 8, 0, t, t, t, t, world, None, 0) == -2
    assert lib.zbal_dispatch_normal_layout(t, 4, 8, 2, t, t, t, t, None, None, 0) == -2           # reference dereferences null here
    assert lib.zbal_dispatch_normal_layout(t, 4, 8, 2, t, t, t, t, ctypes.c_void_p(0x40), None, 0) == -2
    assert lib.zbal_dispatch_normal_layout(t, 4, 8, 2, t, t, t, t, world, None, 0) == 0
    assert lib.zbal_dispatch_normal_notify(t, 0, 2, t, t, t, t, t, world, None, 0) == -2
    assert lib.zbal_dispatch_normal_notify(t, 8, 2, t, t, None, t, t, world, None, 0) == -2
    assert lib.zbal_dispatch_normal(t, t, t, t, t, 0, 0, t, t, world, None, 0) == -2
    assert lib.zbal_dispatch_normal(t, t, t, t, t, 8, 0, t, None, world, None, 0) == -2
    assert lib.zbal_combine_normal(t, t, t, t, t, t, 0, t, world, None, 0) == -2
    assert lib.zbal_combine_normal(t, t, None, t, t, t, 8, t, world, None, 0) == -2
    assert lib.zbal_dispatch_low_latency(t, t, 0, 0, 0, 0, 0, 0, 1, t, t, t, t, t, t, t, world, None, 0) == -2
    assert lib.zbal_dispatch_low_latency(t, t, 8, -1, 0, 0, 0, 0, 1, t, t, t, t, t, t, t, world, None, 0) == -2
    assert lib.zbal_dispatch_low_latency(t, t, 8, 0, 0, 0, 0, 0, 1, t, t, t, t, t, t, None, world, None, 0) == -2
    assert lib.zbal_combine_low_latency(t, t, t, t, t, None, 8, world, None, 0) == -2
    assert lib.zbal_combine_low_latency(t, t, t, t, t, t, 0, world, None, 0) == -2
    fused = [t] * 7 + [None] * 7 + [t, None, t, t]
    assert lib.zbal_fused_deep_moe(*fused, 8, 0, 0, 256, 0, 0, world, None, 0) == 0
    assert lib.zbal_fused_deep_moe(*fused, 0, 0, 0, 256, 0, 0, world, None, 0) == -2
    assert lib.zbal_fused_deep_moe(*fused, 8, 0, 0, 0, 0, 0, world, None, 0) == -2
    assert lib.zbal_fused_deep_moe(*fused, 8, 0, 0, 256, 0, 1, world, None, 0) == 0               # tensor list
    half = list(fused); half[8] = ctypes.byref(capi.TensorInfo(data=ctypes.c_void_p(0x1000)))  # shared gmm1 weight alone
    assert lib.zbal_fused_deep_moe(*half, 8, 0, 0, 256, 256, 0, world, None, 0) == -2
    bad = list(fused); bad[17] = None
    assert lib.zbal_fused_deep_moe(*bad, 8, 0, 0, 256, 0, 0, world, None, 0) == -2                # workspace
    assert lib.zbal_comm_register_peer_window(world, 9, p, 64) == -2
    assert lib.zbal_comm_register_peer_window(world, 1, None, 64) == -2
    assert lib.zbal_comm_register_peer_window(world, 1, p, 64) in (0, -2)   # alignment of a host buffer varies


def test_fused_workspace_size_is_monotonic(lib):
    f = lib.zbal_fused_deep_moe_workspace_size
    assert f(0, 7168, 8, 32, 4096, 0, 2) > 0
    a, b = f(128, 7168, 8, 32, 4096, 0, 0), f(256, 7168, 8, 32, 4096, 0, 0)
    assert 0 < a < b
    assert f(128, 7168, 8, 32, 4000, 0, 0) == 0 and f(128, 100, 8, 32, 4096, 0, 0) == 0 and f(128, 7168, 8, 32, 4096, 0, 9) == 0
    # W8A8 keeps an fp32 SwiGLU scratch that the fp8 mode does not need
    assert f(128, 7168, 8, 32, 4096, 0, 2) < f(128, 7168, 8, 32, 4096, 0, 0)
    # a shared expert reuses the routed pass's regions: only one wider than topk routed experts adds bytes
    assert f(128, 7168, 8, 32, 4096, 4096, 0) == a
    assert f(128, 7168, 1, 32, 512, 4096, 0) > f(128, 7168, 1, 32, 512, 0, 0)
    assert f(128, 7168, 8, 32, 4096, 100, 0) == 0


def reference_workspace_bytes(bs, h, gmm1_h_len, share_gmm1_h_len, experts_per_rank, ranks, topk, global_bs, aic_num):
    """The size the reference's adaptor allocates for the fused operator's workspace, restated from
    zbal_deepep.cpp:42-84 (ComputeWorkspaceSize; the host launcher checks against the same sum,
    host/fused_deep_moe/zbal_kernel_fused_deep_moe_host.cpp:59-132): 16 MiB for the system plus regions each rounded
    up to 512 bytes."""
    up = lambda x: (x + 511) // 512 * 512
    max_bs = global_bs // ranks
    max_tokens = max_bs * ranks * min(topk, experts_per_rank)
    gmm2_h, share_gmm2_h = gmm1_h_len // 2, share_gmm1_h_len // 2
    share_tokens = bs if share_gmm1_h_len > 0 else 0
    handled = max_tokens + share_tokens
    x1 = up(handled * h)
    x2 = up(max_tokens * gmm2_h + share_tokens * share_gmm2_h)
    token_scale = up(handled * 4)
    cv_swap = up(aic_num * 32 * 1024 * 4 * 4)
    swiglu = (max_tokens * gmm1_h_len + share_tokens * share_gmm1_h_len) * 4
    gmm2_out = max_tokens * h * 2
    group_list = up(experts_per_rank * 8)
    expand_idx = up(bs * topk * 4)
    send_count = up(ranks * experts_per_rank * 4)
    reserved = up(256 * 1024)
    quant_ws = up(bs * topk * up(h + 4))
    combine_ws = up(experts_per_rank * ranks * max_bs * h * 2)
    return (16 << 20) + max(x1, x2) + token_scale + cv_swap + up(max(swiglu, gmm2_out)) + group_list + expand_idx + \
        send_count + reserved + quant_ws + combine_ws


@pytest.mark.parametrize("tokens,hidden,topk,experts,n1", [(256, 1024, 2, 8, 2048),        # the small CPU-reference layer
                                                           (4096, 7168, 8, 32, 4096),      # prefill share
                                                           (128, 7168, 8, 32, 4096),       # decode share
                                                           (16384, 4096, 8, 128, 3072),    # W4A8 layer
                                                           (1, 7168, 8, 256, 4096), (0, 7168, 8, 32, 4096)])
def test_a_workspace_sized_by_the_reference_is_large_enough(lib, tokens, hidden, topk, experts, n1):
    """A caller that keeps the reference adaptor's own sizing (one rank, global_bs = bs as the adaptor defaults it)
    hands zbal_fused_deep_moe at least what this build asks for: every quant mode, with and without a shared expert.
    The cube-core count enters the reference's sum through a 512 KiB-per-core swap area; the smallest count of any
    Ascend part (20) gives the smallest reference size."""
    for share_n1 in (0, n1):
        want = reference_workspace_bytes(max(tokens, 1), hidden, n1, share_n1, experts, 1, topk, max(tokens, 1), aic_num=20)
        for quant_mode in (0, 1, 2, 3):
            ours = lib.zbal_fused_deep_moe_workspace_size(tokens, hidden, topk, experts, n1, share_n1, quant_mode)
            assert 0 < ours <= want, (share_n1, quant_mode, ours, want)


def test_kernel_seam_types_and_exports():
    """CommGroupInfo keeps the reference's layout (zbal_comm_host_device_struct.h:133-151: 2160 bytes,
    peerGroupRank2WorldRank at 64) and the nine launcher functions of zbal_npu_operators.h are exported with C++
    linkage."""
    import ctypes
    assert ctypes.sizeof(capi.CommGroupInfo) == 2160
    assert capi.CommGroupInfo.peerGroupRank2WorldRank.offset == 64
    assert capi.CommGroupInfo.localDeviceMemSize.offset == 2112
    assert capi.CommGroupInfo.waitSymbol.offset == 2120
    assert capi.CommGroupInfo.groupIndex.offset == 2152
    names = set(capi.cxx_symbols())
    assert names == {"ZBALOpReduceScatter", "ZBALOpAllReduce", "ZBALOpDispatchLayout", "ZBALOpNotifyDispatch",
                     "ZBALOpDispatchNormal", "ZBALOpCombineNormal", "ZBALOpDispatchLowLatency", "ZBALOpCombineLowLatency",
                     "ZBALOpFusedDeepMoe"}
    assert set(capi.CXX_SIGNATURES) <= names


def test_launcher_seam_refuses_an_incomplete_shared_expert(lib):
    """ZBALOpFusedDeepMoe with shared-expert weights but no shareOutput (or no scales) is refused with
    Z_INVALID_PARAM like zbal_fused_deep_moe, before any descriptor is read or a device is touched."""
    fn = capi.load_cxx()["ZBALOpFusedDeepMoe"]
    byte = ctypes.c_char()
    t = capi.TensorInfo()
    t.data = ctypes.addressof(byte)
    r, null = ctypes.byref(t), None
    g = capi.CommGroupInfo()
    g.groupSize, g.myGroupRank = 1, 0
    name = capi.std_string(b"ep")

    def call(share_w1, share_s1, share_w2, share_s2, share_out, share_n1):
        return fn(r, r, r, r, r, r, r, null, share_w1, share_s1, share_w2, share_s2, null, null, r, share_out, r, r,
                  8, 0, 0, 256, share_n1, False, None, ctypes.addressof(name), None, ctypes.byref(g), ctypes.byref(g), 0, True)
    assert call(r, r, r, r, null, 256) == capi.Z_INVALID_PARAM
    assert b"shared expert" in lib.zbal_get_last_error_msg()
    assert call(r, null, r, r, r, 256) == capi.Z_INVALID_PARAM
    assert call(r, r, r, r, r, 0) == capi.Z_INVALID_PARAM
    assert call(null, null, null, null, r, 0) == capi.Z_INVALID_PARAM


def test_sigusr1_is_deferred_chained_and_restored(lib):
    """Bootstrap installs a SIGUSR1 handler that only wakes a helper thread (which writes the traces), passes the
    signal on to the handler that was there before, and unbootstrap puts that one back and joins the thread."""
    import signal
    seen = []
    before = signal.signal(signal.SIGUSR1, lambda *_: seen.append(1))
    try:
        opts = capi.BootstrapOptions()
        assert lib.zbal_bootstrap_options_init(ctypes.byref(opts)) == 0
        opts.flags = 1
        assert lib.zbal_bootstrap(ctypes.byref(opts), None) == 0
        rc, comm = make_comm(lib, b"sig_world", 1, 1, 0)
        assert rc == 0
        os.kill(os.getpid(), signal.SIGUSR1)
        assert seen == [1]                                         # chained to the handler installed before bootstrap
        assert lib.zbal_comm_dump_profiling_trace(comm) == 0       # the library stays usable while the helper thread works
        assert lib.zbal_comm_destroy(comm, 0) == 0
        assert lib.zbal_unbootstrap(0) == 0
        os.kill(os.getpid(), signal.SIGUSR1)
        assert seen == [1, 1]                                      # the old handler is back in place
    finally:
        signal.signal(signal.SIGUSR1, before)


def test_a_process_that_ends_without_unbootstrap_exits_cleanly():
    """The helper thread that bootstrap starts is taken down when the library's statics go: a process that never calls
    zbal_unbootstrap must still end with its own exit code (a joinable std::thread destroyed at exit would abort)."""
    import subprocess
    import sys
    code = ("import ctypes\n"
            "from memfabric_hybrid_amd import capi\n"
            "lib = capi.load()\n"
            "opts = capi.BootstrapOptions()\n"
            "assert lib.zbal_bootstrap_options_init(ctypes.byref(opts)) == 0\n"
            "opts.flags = 1\n"
            "assert lib.zbal_bootstrap(ctypes.byref(opts), None) == 0\n"
            "raise SystemExit(7)\n")
    done = subprocess.run([sys.executable, "-c", code], cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                          capture_output=True, text=True, timeout=120)
    assert done.returncode == 7, (done.returncode, done.stderr[-400:])


def test_deepep_buffer_signatures_follow_the_reference():
    """Parameter names, order and defaults of the DeepEP-compatible Buffer, as the reference's Python face declares
    them (app/zbal/src/python/zbal/zbal_buffer.py:28-37, 168-175, 216-232, 350-360, 432-443, 536-545, 611-634)."""
    import inspect
    from memfabric_hybrid_amd.buffer import Buffer, Config, EventOverlap

    def sig(fn):
        return [(n, p.default if p.default is not inspect.Parameter.empty else "<required>")
                for n, p in inspect.signature(fn).parameters.items() if n != "self"]

    assert sig(Buffer.__init__)[:7] == [
        ("group", None), ("num_nvl_bytes", 0), ("num_rdma_bytes", 0), ("low_latency_mode", False),
        ("num_qps_per_rank", 12), ("allow_nvlink_for_low_latency_mode", True), ("allow_mnnvl", False)]
    assert sig(Buffer.get_dispatch_layout) == [
        ("topk_idx", "<required>"), ("num_experts", "<required>"), ("previous_event", None), ("async_finish", False),
        ("allocate_on_comm_stream", False)]
    assert sig(Buffer.dispatch) == [
        ("x", "<required>"), ("handle", None), ("num_tokens_per_rank", None), ("num_tokens_per_rdma_rank", None),
        ("is_token_in_rank", None), ("num_tokens_per_expert", None), ("topk_idx", None), ("topk_weights", None),
        ("expert_alignment", 1), ("num_worst_tokens", 0), ("config", None), ("previous_event", None),
        ("async_finish", False), ("allocate_on_comm_stream", False), ("dispatch_wait_recv_cost_stats", None)]
    assert sig(Buffer.combine) == [
        ("x", "<required>"), ("handle", "<required>"), ("topk_weights", None), ("bias", None), ("config", None),
        ("previous_event", None), ("async_finish", False), ("allocate_on_comm_stream", False),
        ("combine_send_cost_stats", None)]
    assert sig(Buffer.low_latency_dispatch) == [
        ("x", "<required>"), ("topk_idx", "<required>"), ("num_max_dispatch_tokens_per_rank", "<required>"),
        ("num_experts", "<required>"), ("cumulative_local_expert_recv_stats", None), ("use_fp8", True),
        ("round_scale", False), ("use_ue8m0", False), ("async_finish", False), ("return_recv_hook", False)]
    assert sig(Buffer.low_latency_combine) == [
        ("x", "<required>"), ("topk_idx", "<required>"), ("topk_weights", "<required>"), ("handle", "<required>"),
        ("zero_copy", False), ("async_finish", False), ("return_recv_hook", False), ("out", None)]
    assert sig(Buffer.fused_deep_moe) == [
        ("x", "<required>"), ("topk_idx", "<required>"), ("gmm1_permuted_weight", "<required>"),
        ("gmm1_permuted_weight_scale", "<required>"), ("gmm2_weight", "<required>"), ("gmm2_weight_scale", "<required>"),
        ("topk_weights", "<required>"), ("num_experts", "<required>"), ("shared_expert_num", 0),
        ("shared_expert_rank_num", 0), ("quant_mode", 0), ("num_max_dispatch_tokens_per_rank", 0),
        ("is_tensor_list", False), ("expert_smooth_scales", None), ("share_gmm1_weight", None),
        ("share_gmm1_scale", None), ("share_gmm2_weight", None), ("share_gmm2_scale", None),
        ("share_smooth_scales", None), ("x_active_mask", None), ("share_gmm1_h_len", 0), ("fuse_mode", 0)]
    assert sig(Buffer.clean_low_latency_buffer) == [
        ("num_max_dispatch_tokens_per_rank", "<required>"), ("hidden", "<required>"), ("num_experts", "<required>")]
    c = Buffer.get_dispatch_config(8)
    assert isinstance(c, Config) and (c.num_sms, c.num_max_nvl_chunked_send_tokens, c.num_max_nvl_chunked_recv_tokens,
                                      c.num_max_rdma_chunked_send_tokens, c.num_max_rdma_chunked_recv_tokens) == \
        (Buffer.num_sms, 6, 256, 6, 128)
    c = Buffer.get_combine_config(32)
    assert (c.num_max_nvl_chunked_send_tokens, c.num_max_nvl_chunked_recv_tokens) == (1, 288)
    assert c.get_nvl_buffer_size_hint(14336, 8) == 14336 and c.get_rdma_buffer_size_hint(14336, 8) == 14336
    assert Buffer.get_low_latency_rdma_size_hint(128, 7168, 8, 256) == 128
    assert EventOverlap().current_stream_wait() is None


def test_data_movement_collectives_link_and_refuse(lib):
    """A client of the reference that names these still links; each call says why it cannot run here."""
    assert lib.zbal_barrier(None, None) == capi.Z_INVALID_PARAM
    assert "no transport" in capi.last_error()
    assert lib.zbal_all_gather(None, None, 0, 0, None, None) == capi.Z_INVALID_PARAM
    assert lib.zbal_send(None, 0, 0, None, None) == capi.Z_INVALID_PARAM
