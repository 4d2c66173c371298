"""ctypes declarations for the C-ABI in include/paella_hip.h, paella_ops.h and paella_ring.h."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.environ.get("PAELLA_LIB_DIR") or os.path.join(_HERE, "lib")  # PAELLA_LIB_DIR: the libraries of another build
BIN_DIR = os.path.join(_HERE, "bin")
CSRC_DIR = os.path.join(_HERE, "csrc")

c_int, c_uint, c_float, c_double = ctypes.c_int, ctypes.c_uint, ctypes.c_float, ctypes.c_double
c_void_p, c_size_t, c_char_p = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_char_p
c_u32, c_u64 = ctypes.c_uint32, ctypes.c_uint64


from ._abi_types import LaunchDims  # noqa: E402


class ConvDesc(ctypes.Structure):
    _fields_ = [(n, c_int) for n in ("C", "H", "W", "K", "R", "S", "stride_h", "stride_w", "pad_h", "pad_w",
                                     "dil_h", "dil_w", "groups", "act")] + [("act_lo", c_float), ("act_hi", c_float)]


class ConvPlan(ctypes.Structure):
    _fields_ = [("d", ConvDesc), ("P", c_int), ("Q", c_int), ("kind", c_int), ("mi", c_int), ("ni", c_int),
                ("kw", c_int), ("splits", c_int), ("m_pad", c_int), ("k_pad", c_int), ("k_order", c_int), ("wg_order", c_int), ("fast_div", c_int), ("blob_bytes", c_size_t), ("workspace_bytes", c_size_t), ("dims", LaunchDims),
                ("flops", c_double), ("bytes", c_double), ("depth", c_int), ("pair_taps", c_int)]


class ConvOperands(ctypes.Structure):
    _fields_ = [("plan", ctypes.POINTER(ConvPlan))] + [(n, c_void_p) for n in ("x", "blob_dev", "bias", "residual", "slope", "y", "workspace")]


class PoolDesc(ctypes.Structure):
    _fields_ = [(n, c_int) for n in ("C", "H", "W", "R", "S", "stride_h", "stride_w", "pad_h", "pad_w",
                                     "ceil_mode", "is_avg", "count_include_pad")]


class DeviceCaps(ctypes.Structure):
    _fields_ = [(n, c_int) for n in ("num_cus", "wavefront_size", "max_threads_per_cu", "max_blocks_per_cu",
                                     "vgprs_per_cu", "lds_bytes_per_cu", "clock_khz", "l2_bytes")] + \
               [("name", ctypes.c_char * 64)]


# name -> (restype, argtypes); every symbol declared in include/*.h must appear here (tests check that).
HIP_SYMBOLS = {
    "llis_hip_device_count": (c_int, [ctypes.POINTER(c_int)]),
    "llis_hip_set_device": (c_int, [c_int]),
    "llis_hip_get_device_caps": (c_int, [ctypes.POINTER(DeviceCaps)]),
    "llis_hip_error_string": (c_char_p, [c_int]),
    "llis_hip_stream_create": (c_int, [ctypes.POINTER(c_void_p)]),
    "llis_hip_stream_destroy": (c_int, [c_void_p]),
    "llis_hip_stream_synchronize": (c_int, [c_void_p]),
    "llis_hip_stream_busy": (c_int, [c_void_p]),
    "llis_hip_device_synchronize": (c_int, []),
    "llis_hip_device_malloc": (c_int, [ctypes.POINTER(c_void_p), c_size_t]),
    "llis_hip_device_free": (c_int, [c_void_p]),
    "llis_hip_host_alloc_coherent": (c_int, [ctypes.POINTER(c_void_p), c_size_t]),
    "llis_hip_host_alloc_pinned": (c_int, [ctypes.POINTER(c_void_p), c_size_t]),
    "llis_hip_host_free": (c_int, [c_void_p]),
    "llis_hip_memcpy": (c_int, [c_void_p, c_void_p, c_size_t, c_int]),
    "llis_hip_memcpy_async": (c_int, [c_void_p, c_void_p, c_size_t, c_int, c_void_p]),
    "llis_hip_fill_u32_async": (c_int, [c_void_p, c_u32, c_size_t, c_void_p]),
    "llis_hip_launch_host_func": (c_int, [c_void_p, c_void_p, c_void_p]),
    "llis_hip_launch_ring_marker": (c_int, [c_void_p, c_void_p, c_uint, c_void_p, c_u64]),
    "llis_hip_event_create": (c_int, [ctypes.POINTER(c_void_p)]),
    "llis_hip_event_destroy": (c_int, [c_void_p]),
    "llis_hip_event_record": (c_int, [c_void_p, c_void_p]),
    "llis_hip_event_synchronize": (c_int, [c_void_p]),
    "llis_hip_event_elapsed_ms": (c_int, [c_void_p, c_void_p, ctypes.POINTER(c_float)]),
    "llis_hip_profiler_start": (c_int, []),
    "llis_hip_profiler_stop": (c_int, []),
}

_TAIL = [c_void_p, c_u32, c_void_p]  # stream, job_id, notifier

OPS_SYMBOLS = {
    "paella_conv2d_plan": (c_int, [ctypes.POINTER(ConvDesc), c_int, c_int, ctypes.POINTER(ConvPlan)]),
    "paella_conv2d_pack": (c_int, [ctypes.POINTER(ConvPlan), c_void_p, c_void_p]),
    "paella_conv2d_launch": (c_int, [ctypes.POINTER(ConvPlan)] + [c_void_p] * 7 + _TAIL),
    "paella_conv2d_plan_takes_input_transform": (c_int, [ctypes.POINTER(ConvPlan)]),
    "paella_conv2d_transformed_dims": (c_int, [ctypes.POINTER(ConvPlan), ctypes.POINTER(LaunchDims)]),
    "paella_conv2d_launch_transformed": (c_int, [ctypes.POINTER(ConvPlan)] + [c_void_p] * 3 + [c_int] + [c_void_p] * 6 + _TAIL),
    "paella_conv2d_pair_dims": (c_int, [ctypes.POINTER(ConvPlan), ctypes.POINTER(ConvPlan), ctypes.POINTER(LaunchDims)]),
    "paella_conv2d_launch_pair": (c_int, [ctypes.POINTER(ConvOperands), ctypes.POINTER(ConvOperands)] + _TAIL),
    "paella_conv2d_group_dims": (c_int, [ctypes.POINTER(ctypes.POINTER(ConvPlan)), c_int, ctypes.POINTER(LaunchDims)]),
    "paella_conv2d_launch_group": (c_int, [ctypes.POINTER(ConvOperands), c_int] + _TAIL),
    "paella_pack_enable": (c_int, [c_int]),
    "paella_pack_poll": (c_int, []),
    "paella_pack_flush": (c_int, []),
    "paella_pack_poll_hook": (None, []),
    "paella_pack_stats": (c_int, [ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint64)]),
    "paella_pack_sequence_begin": (c_int, [c_void_p, c_void_p]),
    "paella_pack_sequence_end": (c_int, []),
    "paella_conv2d_group_pool_dims": (c_int, [ctypes.POINTER(ctypes.POINTER(ConvPlan)), c_int, ctypes.POINTER(PoolDesc), ctypes.POINTER(LaunchDims)]),
    "paella_conv2d_launch_group_pool": (c_int, [ctypes.POINTER(ConvOperands), c_int, ctypes.POINTER(PoolDesc), c_void_p, c_void_p] + _TAIL),
    "paella_dense_dims": (c_int, [c_int, c_int, ctypes.POINTER(LaunchDims)]),
    "paella_dense_launch": (c_int, [c_void_p] * 4 + [c_int] * 3 + _TAIL),
    "paella_pool_out": (c_int, [c_int] * 5),
    "paella_pool2d_dims": (c_int, [ctypes.POINTER(PoolDesc), ctypes.POINTER(LaunchDims)]),
    "paella_pool2d_launch": (c_int, [ctypes.POINTER(PoolDesc), c_void_p, c_void_p] + _TAIL),
    "paella_global_avgpool_dims": (c_int, [c_int, c_int, ctypes.POINTER(LaunchDims)]),
    "paella_global_avgpool_launch": (c_int, [c_void_p, c_void_p, c_int, c_int] + _TAIL),
    "paella_eltwise_dims": (c_int, [c_int, c_int, ctypes.POINTER(LaunchDims)]),
    "paella_eltwise_launch": (c_int, [c_void_p] * 6 + [c_int, c_int, c_int, c_float, c_float] + _TAIL),
    "paella_copy_dims": (c_int, [c_size_t, ctypes.POINTER(LaunchDims)]),
    "paella_copy_launch": (c_int, [c_void_p, c_void_p, c_size_t] + _TAIL),
    "paella_softmax_dims": (c_int, [c_int, c_int, ctypes.POINTER(LaunchDims)]),
    "paella_softmax_launch": (c_int, [c_void_p, c_void_p, c_int, c_int] + _TAIL),
    "paella_lrn_dims": (c_int, [c_int, c_int, ctypes.POINTER(LaunchDims)]),
    "paella_lrn_launch": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_float, c_float] + _TAIL),
    "paella_kernel_vgprs": (c_int, [c_char_p, ctypes.POINTER(c_uint)]),
    "paella_conv_kernel_vgprs": (c_int, [c_int] * 4 + [ctypes.POINTER(c_uint)]),
    "paella_conv2d_launch_static": (c_int, [ctypes.POINTER(ConvPlan)] + [c_void_p] * 6 + _TAIL),
    "paella_conv2d_static_init": (c_int, []),
    "paella_conv2d_static_workspace": (c_int, [ctypes.POINTER(c_void_p)]),
    "paella_kernel_occupancy": (c_int, [c_char_p, c_uint, c_uint, ctypes.POINTER(c_int)]),
    "paella_conv_kernel_occupancy": (c_int, [c_int] * 6 + [c_uint, ctypes.POINTER(c_int), ctypes.POINTER(c_uint), ctypes.POINTER(c_uint)]),
    "paella_kernel_static_lds": (c_int, [c_char_p, ctypes.POINTER(c_uint)]),
    "paella_conv2d_dims": (c_int, [ctypes.POINTER(ConvPlan), ctypes.POINTER(LaunchDims)]),
    "paella_host_copy_submit": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p, c_void_p]),
    "paella_ops_time_launches": (c_int, [c_void_p, c_void_p]),
    "paella_direct_queue_create": (c_int, [ctypes.POINTER(c_void_p)]),
    "paella_direct_queue_set_ordered": (c_int, [c_void_p, c_int]),
    "paella_direct_queue_wait": (c_int, [c_void_p]),
    "paella_direct_queue_shared": (c_int, [ctypes.POINTER(c_void_p)]),
    "paella_direct_queue_destroy": (c_int, [c_void_p]),
}

RING_SYMBOLS = {
    "paella_ring_batch_size": (c_uint, []),
    "paella_ring_create": (c_int, [c_size_t, c_uint, ctypes.POINTER(c_void_p)]),
    "paella_ring_create_batched": (c_int, [c_size_t, c_uint, c_uint, ctypes.POINTER(c_void_p)]),
    "paella_ring_destroy": (c_int, [c_void_p]),
    "paella_ring_notifier": (c_void_p, [c_void_p, c_uint]),
    "paella_ring_channel": (c_void_p, [c_void_p]),
    "paella_ring_probe_launch": (c_int, [c_void_p, c_uint, c_uint, c_uint, c_uint, c_uint, c_u32, c_int, c_void_p]),
    "paella_ring_can_read": (c_int, [c_void_p]),
    "paella_ring_drain": (c_size_t, [c_void_p, c_void_p, c_size_t, c_double]),
    "paella_ring_bench_drain": (c_int, [c_void_p, c_uint, c_uint, c_int, c_int, ctypes.POINTER(c_double)]),
    "paella_ring_bench_pingpong": (c_int, [c_int, c_int, ctypes.POINTER(c_double), ctypes.POINTER(c_double), c_void_p]),
    "paella_ring_bench_echo": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p]),
}

# libpaella_probes.so (include/paella_probes.h): measurement only, loaded by the bench and the tests
PROBE_SYMBOLS = {
    "paella_empty_kernel_probe": (c_int, [c_int, ctypes.POINTER(c_double)]),
    "paella_mfma_peak_probe": (c_int, [ctypes.POINTER(c_double)]),
    "paella_mfma_valu_overlap_probe": (c_int, [c_int, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]),
    "paella_queue_concurrency_probe": (c_int, [ctypes.POINTER(ConvDesc), c_int, c_int, c_int, c_int, c_int, ctypes.POINTER(c_double)]),
}


def _bind(lib, table):
    for name, (res, args) in table.items():
        fn = getattr(lib, name)  # AttributeError here means the library does not export a declared symbol
        fn.restype = res
        fn.argtypes = args
    return lib


_cache = {}


def load(name):
    """Loads paella_amd/lib/lib<name>.so (RTLD_GLOBAL) and binds its declared symbols.  Raises if it is missing."""
    if name in _cache:
        return _cache[name]
    path = os.path.join(LIB_DIR, "lib%s.so" % name)
    if not os.path.exists(path):
        raise RuntimeError("%s is not built: run `make -C paella_amd/csrc` (there is no CPU fallback)" % path)
    lib = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
    if name == "llis_hip":
        _bind(lib, HIP_SYMBOLS)
    elif name == "paella_ops":
        _bind(lib, OPS_SYMBOLS)
        _bind(lib, RING_SYMBOLS)
        from . import _abi_models
        _abi_models.bind(lib)
    elif name == "paella_probes":
        _bind(lib, PROBE_SYMBOLS)
    _cache[name] = lib
    return lib


def hip():
    return load("llis_hip")


def ops():
    hip()
    return load("paella_ops")


def probes():
    ops()
    return load("paella_probes")


def check(rc, what=""):
    if rc != 0:
        msg = hip().llis_hip_error_string(rc).decode() if rc > 0 else {-1: "invalid argument", -2: "unsupported shape"}.get(rc, "?")
        raise RuntimeError("%s failed: %d (%s)" % (what or "call", rc, msg))
