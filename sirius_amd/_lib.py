"""ctypes binding of libtorch_col_hip.so, generated from the C ABI headers in include/.

There is no fallback: if the shared library has not been built, asking for the handle
raises, so no caller can silently run anything but the HIP path.
"""
import ctypes
import os
import re

_HERE = os.path.dirname(os.path.abspath(__file__))
# TCH_LIBRARY_PATH names another build of the same library (e.g. to compare two builds on one machine)
LIB_PATH = os.environ.get("TCH_LIBRARY_PATH") or os.path.join(_HERE, "lib", "libtorch_col_hip.so")
INCLUDE_DIR = os.path.join(os.path.dirname(_HERE), "include")
HEADERS = ("torch_col_hip.h", "torch_col_host.h")

_lib = None


class TorchColHipError(RuntimeError):
    pass


class KernelStat(ctypes.Structure):
    """Mirror of tch_kernel_stat (include/torch_col_hip.h)."""
    _fields_ = [("name", ctypes.c_char * 96), ("total_ms", ctypes.c_double), ("work", ctypes.c_double),
                ("launches", ctypes.c_int64), ("work_is_bytes", ctypes.c_int), ("bytes", ctypes.c_double)]


class LaunchStat(ctypes.Structure):
    """Mirror of tch_launch_stat (include/torch_col_hip.h)."""
    _fields_ = [("name", ctypes.c_char * 96), ("ms", ctypes.c_double), ("flops", ctypes.c_double),
                ("bytes", ctypes.c_double), ("lane", ctypes.c_int), ("workgroups", ctypes.c_int64)]


class CtrlMsg(ctypes.Structure):
    """Mirror of tch_ctrl_msg (include/torch_col_host.h)."""
    _fields_ = [("id", ctypes.c_uint64), ("event", ctypes.c_int), ("value", ctypes.c_int)]


_SCALARS = {
    "int": ctypes.c_int, "unsigned": ctypes.c_uint, "float": ctypes.c_float, "double": ctypes.c_double,
    "int32_t": ctypes.c_int32, "uint32_t": ctypes.c_uint32, "int64_t": ctypes.c_int64, "uint64_t": ctypes.c_uint64,
    "size_t": ctypes.c_size_t, "ptrdiff_t": ctypes.c_ssize_t,
}


def _ctype(decl, is_return):
    d = decl.replace("const", " ").strip()
    if "*" in d:
        base = d.replace("*", " ").split()[0]
        if base == "char":
            return ctypes.c_char_p if (is_return or "const" in decl) else ctypes.c_void_p
        return ctypes.c_void_p
    base = d.split()[0]
    if base == "void":
        return None
    return _SCALARS[base]


def parse_header(path):
    """{function name: (restype, [argtypes])} for every prototype in a C ABI header."""
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    text = re.sub(r"^\s*#.*$", " ", text, flags=re.M)
    text = re.sub(r"typedef\s+struct\s+\w+\s*\{.*?\}\s*\w+\s*;", " ", text, flags=re.S)
    text = re.sub(r"typedef[^;]*;", " ", text)
    text = text.replace('extern "C" {', " ").replace("}", " ")
    out = {}
    for m in re.finditer(r"([\w\s\*]+?)\b(tch_\w+)\s*\(([^;{]*?)\)\s*;", text):
        ret, name, args = m.group(1).strip(), m.group(2), m.group(3).strip()
        argtypes = []
        if args and args != "void":
            for a in args.split(","):
                a = a.strip()
                # drop the parameter name (last identifier not part of the type)
                a = re.sub(r"\b\w+$", "", a).strip() if re.search(r"[\*\s]\w+$", a) else a
                argtypes.append(_ctype(a, False))
        out[name] = (_ctype(ret, True), argtypes)
    return out


def declared_symbols():
    sig = {}
    for h in HEADERS:
        sig.update(parse_header(os.path.join(INCLUDE_DIR, h)))
    return sig


def lib():
    """The loaded shared library; raises if it was never built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise TorchColHipError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C sirius_amd/csrc`. There is no CPU fallback for this path.")
        handle = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
        for name, (res, args) in declared_symbols().items():
            fn = getattr(handle, name)  # AttributeError here = header and library disagree
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc, what=""):
    if rc < 0:
        msg = lib().tch_last_error()
        raise TorchColHipError(f"{what} failed ({rc}): {msg.decode() if msg else ''}")
    return rc


def check_host(rc, what=""):
    if rc < 0:
        msg = lib().tch_host_last_error()
        raise TorchColHipError(f"{what} failed ({rc}): {msg.decode() if msg else ''}")
    return rc
