"""ctypes binding of libttmi.so, generated from include/ttmi.h at import time.

The header is the single source of truth for the C ABI: every ``TTMI_API`` declaration is
parsed into a ctypes prototype, so a symbol missing from the library or a signature drift
shows up as an import error here rather than as a crash later.

    from turbotransformers_amd import capi
    lib = capi.load()                      # raises if libttmi.so has not been built
    capi.check(lib.ttmi_layer_norm(ptr, g, b, m, n, 1e-12, capi.F16, stream))
"""
import ctypes
import os
import re

_PKG = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(os.path.dirname(_PKG), "include", "ttmi.h")
LIB_PATH = os.path.join(_PKG, "lib", "libttmi.so")

F32, F16, BF16, I8, I32, I64 = range(6)
ACT_GELU, ACT_TANH, ACT_RELU = range(3)
H2D, D2H, D2D = range(3)
EPI_NONE, EPI_BIAS, EPI_BIAS_ACT, EPI_BIAS_RESIDUAL, EPI_QKV_SPLIT, EPI_QKV_SPLIT_PAD, EPI_F32_OUT = range(7)
QUANT_SCALE_FLOATS = 514  # TTMI_QUANT_SCALE_FLOATS
ABSMAX_SLOTS = 1024  # TTMI_ABSMAX_SLOTS


class EpilogueArgs(ctypes.Structure):
    """Mirror of ``ttmi_epilogue_args``."""
    _fields_ = [
        ("bias", ctypes.c_void_p), ("residual", ctypes.c_void_p), ("act", ctypes.c_int),
        ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
        ("seq", ctypes.c_int64), ("heads", ctypes.c_int64), ("head_dim", ctypes.c_int64),
        ("token_rows", ctypes.c_void_p), ("batch", ctypes.c_int64), ("v_seq_pitch", ctypes.c_int64),
    ]


_SCALARS = {
    "int": ctypes.c_int, "int64_t": ctypes.c_int64, "int32_t": ctypes.c_int32, "float": ctypes.c_float,
    "size_t": ctypes.c_size_t,
}


def _ctype_of(decl):
    decl = decl.strip()
    if "*" in decl:
        return ctypes.c_void_p
    words = [w for w in decl.replace("const", " ").split() if w]
    base = words[0]
    if base not in _SCALARS:
        raise ValueError("unknown C type in ttmi.h: %r" % decl)
    return _SCALARS[base]


def parse_header(path=HEADER):
    """-> {name: (restype, [argtypes])} for every TTMI_API declaration."""
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    protos = {}
    for m in re.finditer(r"TTMI_API\s+([\w\s\*]+?)\s*\b(ttmi_\w+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        ret, name, args = m.group(1).strip(), m.group(2), m.group(3).strip()
        restype = ctypes.c_char_p if "char" in ret else ctypes.c_int
        argtypes = [] if args in ("", "void") else [_ctype_of(a) for a in args.split(",")]
        protos[name] = (restype, argtypes)
    return protos


_lib = None


def load(path=LIB_PATH):
    """Load libttmi.so and attach prototypes; fails loudly when the library is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(path):
        raise RuntimeError("libttmi.so not built (%s); run `python turbotransformers_amd/build.py`" % path)
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in parse_header().items():
        fn = getattr(lib, name)  # AttributeError if a declared symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


class TtmiError(RuntimeError):
    pass


def check(rc):
    if rc != 0:
        msg = load().ttmi_last_error()
        raise TtmiError("ttmi error %d: %s" % (rc, msg.decode() if msg else "?"))


def dtype_of(torch_dtype):
    import torch
    return {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16, torch.int8: I8, torch.int32: I32,
            torch.int64: I64}[torch_dtype]
