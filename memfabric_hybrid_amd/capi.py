"""ctypes binding of libzbal.so: the zbal C ABI (include/zbal*.h) and the inner
kernel ABI (include/zbal_hip_kernels.h).

The library must have been built (python -m memfabric_hybrid_amd.build); there
is no fallback path: loading raises if the shared object is missing.
PyTorch is used only to own device memory and streams: tensors are handed to
the library as zbal_tensor_info_t descriptors of their data pointers.
"""
import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
# ZBAL_LIB: another build of the library (the host layer under sanitizers, `python -m memfabric_hybrid_amd.build --asan`)
LIB_PATH = os.environ.get("ZBAL_LIB") or os.path.join(_PKG, "lib", "libzbal.so")

ZBAL_MAX_TENSOR_DIM = 12
ZBAL_COMM_NAME_MAX = 128

# zbal_datatype_t
DT_INT8, DT_INT16, DT_INT32, DT_INT64, DT_UINT64, DT_FP64, DT_FP16, DT_FP32, DT_BF16 = range(9)
DT_UINT8, DT_UINT16, DT_UINT32, DT_FP8_E4M3, DT_INT4X2 = 9, 10, 11, 12, 13
# zbal_reduce_op_t
REDUCE_PROD, REDUCE_SUM, REDUCE_MAX, REDUCE_MIN = 0, 1, 2, 3
# zbal_quant_mode_t
NO_QUANT, QUANT_INT8, QUANT_FP8_B128, QUANT_W4A8_G128 = 0, 1, 2, 3
ROWMAX_CLEARED = 0x200   # ZBALHIP_ROWMAX_CLEARED: OR-ed into the mode of zbalhip_gmm1_swiglu_quant
# zbal_backend_t
BACKEND_GPU, BACKEND_DUMMY = 0, 1
WEIGHT_FORMAT_ND, WEIGHT_FORMAT_PREPACKED = 0, 1

Z_OK, Z_ERROR, Z_INVALID_PARAM = 0, -1, -2
Z_NOT_BOOTSTRAPPED, Z_CREATE_COMM_FAILED = -15, -16
Z_COMM_NOT_EXIST_BY_HANDLE, Z_COMM_DESTROY_GLOBAL_LAST = -20, -25


class TensorInfo(ctypes.Structure):
    """zbal_tensor_info_t (72 bytes)."""
    _fields_ = [("data", ctypes.c_void_p), ("dataType", ctypes.c_int32), ("dim", ctypes.c_uint16),
                ("shape", ctypes.c_uint32 * ZBAL_MAX_TENSOR_DIM), ("reserved", ctypes.c_uint16 * 1)]


class BootstrapOptions(ctypes.Structure):
    _fields_ = [("flags", ctypes.c_uint32), ("btType", ctypes.c_int32), ("ipPort", ctypes.c_char * 64),
                ("worldSize", ctypes.c_uint16), ("rankId", ctypes.c_uint16), ("deviceId", ctypes.c_uint16),
                ("startConfigServer", ctypes.c_uint16), ("deviceMemorySize", ctypes.c_uint64),
                ("dataOperationType", ctypes.c_uint32), ("commMetaSpaceSize", ctypes.c_uint16),
                ("commGroupCap", ctypes.c_uint16)]


class CommOptions(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char_p), ("backendType", ctypes.c_int32), ("flags", ctypes.c_uint32),
                ("isWorldGroup", ctypes.c_uint16), ("groupSize", ctypes.c_uint16), ("groupRankId", ctypes.c_uint16),
                ("symmetricMetaGva", ctypes.c_uint16)]


class CommProperty(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * ZBAL_COMM_NAME_MAX), ("backendType", ctypes.c_int32),
                ("flags", ctypes.c_uint32), ("isWorldGroup", ctypes.c_uint16), ("groupSize", ctypes.c_uint16),
                ("groupRankId", ctypes.c_uint16), ("symmetricMetaGva", ctypes.c_uint16), ("myGVA", ctypes.c_void_p),
                ("myMetaGVA", ctypes.c_void_p), ("myMetaGVAForOpParam", ctypes.c_void_p),
                ("myMetaGVAForOpExchange", ctypes.c_void_p), ("hostMemoryForProfiling", ctypes.c_void_p),
                ("devMemoryForProfiling", ctypes.c_void_p), ("sizeOfMetaArea", ctypes.c_uint64),
                ("sizeOfMetaForOpParam", ctypes.c_uint64), ("sizeOfMetaForAddressExchange", ctypes.c_uint64),
                ("tracePointPerCore", ctypes.c_uint64), ("localDeviceMemSize", ctypes.c_uint64),
                ("groupIndex", ctypes.c_uint32)]


ZBAL_MAX_RANKS = 1024


class CommGroupInfo(ctypes.Structure):
    """The reference's per-group record (include/zbal_comm_group_info.h, 2160 bytes) taken by the ZBALOp* launchers."""
    _fields_ = [("groupSize", ctypes.c_uint16), ("myGroupRank", ctypes.c_uint16), ("myMetaGva", ctypes.c_void_p),
                ("myParamDataGva", ctypes.c_void_p), ("myAddressExchangeGva", ctypes.c_void_p),
                ("sizeForCommGroupInfo", ctypes.c_uint64), ("sizeForParam", ctypes.c_uint64),
                ("sizeForExchangeAddress", ctypes.c_uint64), ("fftsConfig", ctypes.c_uint64),
                ("peerGroupRank2WorldRank", ctypes.c_uint16 * ZBAL_MAX_RANKS), ("localDeviceMemSize", ctypes.c_uint64),
                ("waitSymbol", ctypes.c_uint64), ("hostMemoryForProfiling", ctypes.c_void_p),
                ("devMemoryForProfiling", ctypes.c_void_p), ("tracePointPerCore", ctypes.c_uint64),
                ("groupIndex", ctypes.c_uint16), ("dataOpType", ctypes.c_uint32)]


_TI = ctypes.POINTER(TensorInfo)
_i64, _i32, _vp, _u16, _u32, _u64 = (ctypes.c_int64, ctypes.c_int32, ctypes.c_void_p, ctypes.c_uint16,
                                     ctypes.c_uint32, ctypes.c_uint64)

# name -> (restype, argtypes); every symbol include/*.h declares
SIGNATURES = {
    # zbal.h
    "zbal_version": (ctypes.c_char_p, []),
    "zbal_set_logger": (_i32, [_vp]),
    "zbal_set_logger_level": (_i32, [ctypes.c_int]),
    "zbal_get_last_error_msg": (ctypes.c_char_p, []),
    "zbal_get_and_clear_last_error_msg": (ctypes.c_char_p, []),
    # zbal_bootstrap.h
    "zbal_bootstrap_options_init": (_i32, [ctypes.POINTER(BootstrapOptions)]),
    "zbal_bootstrap": (_i32, [ctypes.POINTER(BootstrapOptions), _vp]),
    "zbal_unbootstrap": (_i32, [_u32]),
    # zbal_operations.h
    "zbal_comm_create": (_i32, [ctypes.POINTER(CommOptions), ctypes.POINTER(_vp)]),
    "zbal_comm_get_property": (_i32, [_vp, ctypes.POINTER(CommProperty)]),
    "zbal_comm_get_global": (_vp, []),
    "zbal_comm_get_by_name": (_vp, [ctypes.c_char_p]),
    "zbal_comm_destroy": (_i32, [_vp, _u32]),
    "zbal_comm_destroy_all": (None, [_u32]),
    "zbal_comm_register_peer_window": (_i32, [_vp, _u16, _vp, _u64]),
    "zbal_comm_dump_profiling_trace": (_i32, [_vp]),
    "zbal_all_reduce": (_i32, [_vp, _vp, _vp, ctypes.c_size_t, _i32, _i32, _vp, _vp]),
    "zbal_reduce_scatter": (_i32, [_vp, _vp, ctypes.c_size_t, _i32, _i32, _vp, _vp]),
    # exported for link compatibility; every one of them refuses (no transport between devices in this build)
    "zbal_all_gather": (_i32, [_vp, _vp, ctypes.c_size_t, _i32, _vp, _vp]),
    "zbal_all_to_all_v": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _vp, _vp]),
    "zbal_broadcast": (_i32, [_vp, ctypes.c_uint64, _i32, _u16, _vp, _vp]),
    "zbal_scatter": (_i32, [_vp, _vp, ctypes.c_uint64, _i32, _u16, _vp, _vp]),
    "zbal_gather": (_i32, [_vp, _vp, ctypes.c_uint64, _i32, _u16, _vp, _vp]),
    "zbal_barrier": (_i32, [_vp, _vp]),
    "zbal_send": (_i32, [_vp, _i32, _u32, _vp, _vp]),
    "zbal_recv": (_i32, [_vp, ctypes.c_size_t, _i32, _u32, _vp, _vp]),
    "zbal_dispatch_normal_notify": (_i32, [_TI, _i64, _i64, _TI, _TI, _TI, _TI, _TI, _vp, _vp, _i64]),
    "zbal_dispatch_normal_layout": (_i32, [_TI, _i64, _i64, _i64, _TI, _TI, _TI, _TI, _vp, _vp, _i64]),
    "zbal_dispatch_normal": (_i32, [_TI, _TI, _TI, _TI, _TI, _i64, _i32, _TI, _TI, _vp, _vp, _i64]),
    "zbal_combine_normal": (_i32, [_TI, _TI, _TI, _TI, _TI, _TI, _u16, _TI, _vp, _vp, _i64]),
    "zbal_dispatch_low_latency": (_i32, [_TI, _TI, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _TI, _TI, _TI, _TI, _TI,
                                         _TI, _TI, _vp, _vp, _i64]),
    "zbal_combine_low_latency": (_i32, [_TI, _TI, _TI, _TI, _TI, _TI, _i64, _vp, _vp, _i64]),
    "zbal_fused_deep_moe": (_i32, [_TI] * 18 + [_i64] * 6 + [_vp, _vp, _i64]),
    "zbal_fused_deep_moe_workspace_size": (_u64, [_i64] * 7),
    "zbal_moe_topk_route": (_i32, [_TI, _i64, _TI, _TI, _vp, _vp, _i64]),
    "zbal_moe_weight_prepack": (_i32, [_TI, _TI, _vp, _vp, _i64]),
    # zbal_hip_kernels.h
    "zbalhip_topk_route": (_i32, [_vp, _i64, _i64, _i64, _vp, _i32, _vp, _vp]),
    "zbalhip_dispatch_layout": (_i32, [_vp, _i32, _i64, _i64, _i64, _i32, _vp, _vp, _vp, _vp, _vp]),
    "zbalhip_dispatch_layout_static": (_i32, [_vp, _i32, _i64, _i64, _i64, _i32, _vp, _vp, _vp, _vp]),
    "zbalhip_dispatch_notify": (_i32, [_vp, _i32, _i32, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp]),
    "zbalhip_dispatch_normal": (_i32, [_vp, _i32, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _vp, _vp, _i32, _i32, _i64,
                                       _vp]),
    "zbalhip_combine": (_i32, [_vp, _i32, _i32, _i64, _i32, _vp, _i32, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp]),
    "zbalhip_dispatch_low_latency": (_i32, [_vp, _i32, _vp, _i64, _i64, _i64, _i64, _i32, _i32, _vp, _vp, _vp, _vp,
                                            _vp, _vp, _i32, _vp]),
    "zbalhip_reduce": (_i32, [ctypes.POINTER(_vp), _i32, _i64, _i32, _i32, _vp, _i32, _vp, _i64, _vp]),
    "zbalhip_trace_alloc": (_i32, [_i64, ctypes.POINTER(ctypes.POINTER(ctypes.c_uint64)), ctypes.POINTER(ctypes.POINTER(ctypes.c_uint64))]),
    "zbalhip_trace_sync": (_i32, []),
    "zbalhip_trace_free": (_i32, [ctypes.POINTER(ctypes.c_uint64)]),
    "zbalhip_weight_prepack": (_i32, [_vp, _i64, _i64, _i64, _i32, _vp, _vp]),
    "zbalhip_fill_i32": (_i32, [_vp, _i64, _i32, _vp]),
    "zbalhip_fused_permute_quant": (_i32, [_vp, _i32, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _vp, _vp, _vp, _vp, _vp,
                                           _vp, _i64, _vp, _i32, _vp]),
    "zbalhip_dispatch_low_latency_ranks": (_i32, [_vp, _i32, _vp, _i64, _i64, _i64, _i64, _i32, _i32, _vp, _vp, _i32, _i32, _i64,
                                                  _vp, _vp, _vp, _vp, _vp]),
    "zbalhip_gmm1_swiglu_quant": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _vp, _vp, _vp, _vp]),
    "zbalhip_gmm2_dequant": (_i32, [_vp, _vp, _vp, _vp, _i32, _vp, _i64, _i64, _i64, _i64, _i32, _i32, _vp, _vp]),
    "zbalhip_gemm_prepare": (_i32, []),
}

_lib = None


def load():
    """Load libzbal.so and attach the prototypes. Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("libzbal.so is missing (%s): build it with `python -m memfabric_hybrid_amd.build`; "
                           "there is no fallback implementation" % LIB_PATH)
    # Device memory comes from torch, so the library must bind to the HIP runtime torch ships: import torch
    # first so that its libamdhip64 is the one already resident when libzbal.so resolves its dependency.
    import torch  # noqa: F401
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


_GI = ctypes.POINTER(CommGroupInfo)
_f32, _bool = ctypes.c_float, ctypes.c_bool
# the C++-linkage launchers of include/zbal_amd_operators.h: name -> argument types (all return int32_t; references
# travel as pointers). ZBALOpFusedDeepMoe takes a std::string and is left to C++ callers.
CXX_SIGNATURES = {
    "ZBALOpReduceScatter": [_vp, _vp, ctypes.c_size_t, _i32, _vp, _i32, _GI],
    "ZBALOpAllReduce": [_vp, _vp, _vp, ctypes.c_size_t, _i32, _vp, _i32, _GI],
    "ZBALOpDispatchLayout": [_TI, _i64, _i64, _i64, _TI, _TI, _TI, _TI, _vp, _GI, _i64],
    "ZBALOpNotifyDispatch": [_TI, _i64, _i64, _TI, _TI, _TI, _TI, _TI, _f32, _f32, _vp, _GI, _i64],
    "ZBALOpDispatchNormal": [_TI, _TI, _TI, _TI, _TI, _i64, _i32, _TI, _TI, _bool, _vp, _GI, _i64],
    "ZBALOpCombineNormal": [_TI, _TI, _TI, _TI, _TI, _TI, _u16, _TI, _bool, _vp, _GI, _i64],
    "ZBALOpDispatchLowLatency": [_TI, _TI, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _TI, _TI, _TI, _TI, _TI, _TI, _TI, _vp,
                                 _GI, _i64],
    "ZBALOpCombineLowLatency": [_TI, _TI, _TI, _TI, _TI, _TI, _i64, _vp, _GI, _i64],
    # ... isTensorList, tilingDevBuf, const std::string &groupName (see std_string), stream, ep group, tp group, flags, needTilingCopy
    "ZBALOpFusedDeepMoe": [_TI] * 18 + [_i64] * 5 + [_bool, _vp, _vp, _vp, _GI, _GI, _i64, _bool],
}


def std_string(text=b""):
    """A libstdc++ std::string (the 32-byte small-string form) holding up to 15 bytes, for the one launcher that
    takes a `const std::string &`: pointer to the characters, length, then the in-object character buffer. Keep the
    returned buffer alive for the call and pass ctypes.addressof(buffer)."""
    assert len(text) <= 15
    buf = ctypes.create_string_buffer(32)
    ctypes.c_uint64.from_buffer(buf, 0).value = ctypes.addressof(buf) + 16
    ctypes.c_uint64.from_buffer(buf, 8).value = len(text)
    buf[16:16 + len(text)] = text
    return buf
_cxx = None


def cxx_symbols():
    """{name: mangled name} of the exported ZBALOp* functions, read from the library's dynamic symbol table (nm)."""
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", LIB_PATH], stdout=subprocess.PIPE, text=True, check=True).stdout
    table = {}
    for line in out.splitlines():
        sym = line.split()[-1]
        if sym.startswith("_Z") and "ZBALOp" in sym:
            digits = ""
            i = 2
            while sym[i].isdigit():
                digits += sym[i]
                i += 1
            table[sym[i:i + int(digits)]] = sym
    return table


def load_cxx():
    """The ZBALOp* launchers as ctypes functions, by their plain names."""
    global _cxx
    if _cxx is None:
        lib = load()
        table = cxx_symbols()
        fns = {}
        for name, args in CXX_SIGNATURES.items():
            fn = getattr(lib, table[name])
            fn.restype = _i32
            fn.argtypes = args
            fns[name] = fn
        _cxx = fns
    return _cxx


def last_error():
    return load().zbal_get_last_error_msg().decode()


class ZbalError(RuntimeError):
    def __init__(self, op, code):
        self.code = code
        super().__init__("%s returned %d: %s" % (op, code, last_error()))


def check(op, code):
    if code != 0:
        raise ZbalError(op, code)


_TORCH_DT = None


def _torch_dtype_map():
    global _TORCH_DT
    if _TORCH_DT is None:
        import torch
        _TORCH_DT = {torch.int8: DT_INT8, torch.int16: DT_INT16, torch.int32: DT_INT32, torch.int64: DT_INT64,
                     torch.float64: DT_FP64, torch.float16: DT_FP16, torch.float32: DT_FP32,
                     torch.bfloat16: DT_BF16, torch.uint8: DT_UINT8, torch.float8_e4m3fn: DT_FP8_E4M3}
    return _TORCH_DT


def tensor_info(t, dtype=None, weight_format=0, shape=None):
    """zbal_tensor_info_t for a contiguous torch tensor (None -> descriptor with a null data pointer)."""
    ti = TensorInfo()
    if t is None:
        return ti
    if not t.is_contiguous():
        raise ValueError("zbal tensors are dense row-major; got a non-contiguous tensor")
    shp = tuple(t.shape) if shape is None else tuple(shape)
    if len(shp) > ZBAL_MAX_TENSOR_DIM:
        raise ValueError("too many dimensions")
    ti.data = t.data_ptr()
    ti.dataType = _torch_dtype_map()[t.dtype] if dtype is None else dtype
    ti.dim = len(shp)
    for i, s in enumerate(shp):
        ti.shape[i] = int(s)
    ti.reserved[0] = weight_format
    return ti


def stream_ptr(stream=None):
    """hipStream_t of a torch stream (default: the current one) as an integer."""
    import torch
    s = torch.cuda.current_stream() if stream is None else stream
    return ctypes.c_void_p(s.cuda_stream)
