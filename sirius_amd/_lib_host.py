"""ctypes declarations for the host-runtime half of the C ABI (include/torch_col_host.h)."""

HOST_SYMBOLS = {}


def declare(handle):
    for name, (res, args) in HOST_SYMBOLS.items():
        fn = getattr(handle, name)
        fn.restype = res
        fn.argtypes = args
