"""ctypes declarations for include/paella_models.h (bound when libpaella_ops.so exports them)."""


def bind(lib):
    return lib
