"""ctypes binding of the C-ABI in include/dynet_hip.h (libdynet_hip.so)."""
import ctypes as C
import os
import re
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdynet_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "dynet_hip.h")
CSRC_DIR = os.path.join(_HERE, "csrc")

OK, ERR_INVALID_ARG, ERR_RUNTIME, ERR_OUT_OF_MEMORY, ERR_NO_DEVICE = range(5)
POOL_FXS, POOL_DEDFS, POOL_PS, POOL_SCS = range(4)
SCALAR_MINUSONE, SCALAR_ONE, SCALAR_ZERO = range(3)
OP_TANH, OP_LOGISTIC, OP_RECTIFY, OP_NEGATE, OP_IDENTITY = range(5)
LOGISTIC_PACKET, LOGISTIC_SCALAR = 0, 1
CWISE_SUM, CWISE_MULT, CWISE_QUOTIENT = range(3)
LN_STATIC_SCRATCH_BYTES = 4 << 20  # DYHIP_LN_STATIC_SCRATCH_BYTES


def build(force=True):
    """Compile every HIP source for gfx950 into libdynet_hip.so (hipcc cross-compiles without a GPU)."""
    args = ["make", "-C", CSRC_DIR, "-j8"]
    if force:
        args.append("-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)


def declared_symbols():
    """Names of every entry point the public header declares."""
    with open(HEADER_PATH) as f:
        text = f.read()
    return sorted(set(re.findall(r"\b(dyhip_[a-z0-9_]+)\s*\(", text)))


def _load():
    if not os.path.exists(LIB_PATH):
        build(force=False)
    if not os.path.exists(LIB_PATH):
        raise ImportError("libdynet_hip.so is missing and could not be built; there is no fallback path")
    return C.CDLL(LIB_PATH)


cdll = _load()
cdll.dyhip_last_error.restype = C.c_char_p
cdll.dyhip_last_error.argtypes = []


def last_error():
    msg = cdll.dyhip_last_error()
    return msg.decode("utf-8", "replace") if msg else ""
