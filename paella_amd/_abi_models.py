"""ctypes declarations for include/paella_models.h."""
import ctypes

from ._abi_types import LaunchDims

c_int, c_double, c_void_p, c_size_t, c_char_p, c_u32, c_u64 = (ctypes.c_int, ctypes.c_double, ctypes.c_void_p, ctypes.c_size_t,
                                                               ctypes.c_char_p, ctypes.c_uint32, ctypes.c_uint64)
_pd = ctypes.POINTER(c_double)

MODEL_SYMBOLS = {
    "paella_model_names": (c_char_p, []),
    "paella_model_io_bytes": (c_int, [c_char_p, ctypes.POINTER(c_size_t), ctypes.POINTER(c_size_t)]),
    "paella_model_describe": (c_int, [c_char_p, c_void_p, c_size_t, ctypes.POINTER(c_size_t)]),
    "paella_model_totals": (c_int, [c_char_p, _pd, _pd, _pd, _pd, ctypes.POINTER(c_int)]),
    "paella_model_weight_values": (c_int, [c_char_p, c_u64, c_int, c_void_p, c_size_t]),
    "paella_model_get": (c_int, [c_char_p, c_u64, ctypes.POINTER(c_void_p)]),
    "paella_model_launch_plan": (c_int, [ctypes.c_char_p, ctypes.POINTER(c_int), ctypes.c_size_t]),
    "paella_model_num_stages": (c_int, [c_void_p]),
    "paella_model_stage_nodes": (c_int, [c_void_p, c_int, ctypes.POINTER(c_int), c_int]),
    "paella_model_stage_dims": (c_int, [c_void_p, c_int, ctypes.POINTER(LaunchDims)]),
    "paella_model_stage_work": (c_int, [c_void_p, c_int, ctypes.POINTER(c_char_p), _pd, _pd]),
    "paella_exec_create": (c_int, [c_void_p, ctypes.POINTER(c_void_p)]),
    "paella_exec_destroy": (c_int, [c_void_p]),
    "paella_exec_bind_input": (c_int, [c_void_p, c_void_p]),
    "paella_exec_bind_output": (c_int, [c_void_p, c_void_p]),
    "paella_exec_input": (c_void_p, [c_void_p]),
    "paella_exec_output": (c_void_p, [c_void_p]),
    "paella_exec_launch_stage": (c_int, [c_void_p, c_int, c_void_p, c_u32, c_void_p]),
    "paella_exec_forward": (c_int, [c_void_p, c_void_p]),
    "paella_model_write_dim": (c_int, [ctypes.c_char_p, ctypes.c_char_p]),
}


def bind(lib):
    for name, (res, args) in MODEL_SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib
