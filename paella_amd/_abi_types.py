"""Plain C structs shared by the ctypes tables."""
import ctypes


class LaunchDims(ctypes.Structure):
    _fields_ = [("grid", ctypes.c_uint), ("block", ctypes.c_uint), ("lds_bytes", ctypes.c_uint), ("vgprs", ctypes.c_uint)]
