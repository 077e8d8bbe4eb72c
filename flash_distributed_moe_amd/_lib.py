"""Loads libflashMoe.so (the C ABI of include/flash_moe.h) through ctypes.

There is no CPU fallback: if the library has not been built, loading raises.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libflashMoe.so")

F32, BF16 = 0, 1
SCHED_AUTO, SCHED_STREAM, SCHED_TILED = 0, 1, 2
FLAG_PACK_WEIGHTS = 1
FLAG_WEIGHTS_PREPACKED = 2
FLAG_RMSNORM = 4
FLAG_RESIDUAL = 8
NOALLOC_SCRATCH_BYTES = 64 << 20
HIP_SUCCESS = 0
HIP_ERROR_INVALID_VALUE = 1
HIP_ERROR_UNKNOWN = 999


class LayerDesc(ctypes.Structure):
    """Mirror of FlashMoeLayerDesc."""

    _fields_ = [
        ("experts", ctypes.c_int),
        ("hidden", ctypes.c_int),
        ("intermediate", ctypes.c_int),
        ("top_k", ctypes.c_int),
        ("dtype", ctypes.c_int),
        ("max_tokens", ctypes.c_int),
        ("sched", ctypes.c_int),
        ("flags", ctypes.c_int),
        ("gate_weights", ctypes.c_void_p),
        ("ffn1_weights", ctypes.c_void_p),
        ("ffn2_weights", ctypes.c_void_p),
        ("router_bias", ctypes.c_void_p),
        ("norm_weight", ctypes.c_void_p),
        ("norm_eps", ctypes.c_double),
    ]


# name -> (restype, argtypes); every symbol include/flash_moe.h declares
C_ABI = {
    "flashMoeVersion": (ctypes.c_char_p, []),
    "flashMoeWorkspaceBytes": (ctypes.c_int, [ctypes.POINTER(LayerDesc),
                                              ctypes.POINTER(ctypes.c_size_t)]),
    "flashMoeCreate": (ctypes.c_int, [ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(LayerDesc),
                                      ctypes.c_void_p]),
    "flashMoePackWeights": (ctypes.c_int, [ctypes.c_int] * 5 + [ctypes.c_void_p] * 3),
    "flashMoePackWeightsInPlace": (ctypes.c_int, [ctypes.c_int] * 5 + [ctypes.c_void_p] * 2),
    "flashMoeRefreshWeights": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p]),
    "flashMoeLaunch": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                      ctypes.c_int, ctypes.c_void_p]),
    "flashMoeLaunchNoAlloc": (ctypes.c_int, [ctypes.POINTER(LayerDesc), ctypes.c_void_p,
                                             ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]),
    "flashMoeDestroy": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p]),
    "flashMoeReadRouting": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
                                           ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                           ctypes.c_void_p, ctypes.c_void_p]),
    "flashMoeReadIntermediate": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
                                                ctypes.c_void_p]),
    "flashMoeStatus": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint),
                                      ctypes.POINTER(ctypes.c_uint), ctypes.c_void_p]),
    "flashMoeSetWaitLimitMs": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_double]),
    "flashMoeSchedFor": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int]),
    "flashMoeTraceEnable": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_uint]),
    "flashMoeTraceRead": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint,
                                         ctypes.c_void_p]),
    "flashMoeReadDownRows": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
                                            ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
                                            ctypes.c_void_p]),
    "flashMoeNoAllocStatus": (ctypes.c_int, [ctypes.POINTER(ctypes.c_uint), ctypes.c_void_p]),
    "flashMoeAbi": (ctypes.c_int, [ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_size_t)]),
    "flashMoeSetDenseSmallBatch": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int]),
}
ABI_VERSION = 3
# the C++-typed entry points of include/iMoeKernelLauncher.h (checked for presence only)
CXX_ABI = ["CreateLauncher", "CreateLauncherEx", "DestroyLauncher", "GetDistributedUniqueId",
           "LauncherHandle"]

_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libflashMoe.so is not built (expected %s); run "
                "`python -m flash_distributed_moe_amd.build`. There is no fallback path."
                % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in C_ABI.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        # a library built from another header revision would read the description wrongly
        version, desc_bytes = ctypes.c_int(0), ctypes.c_size_t(0)
        if lib.flashMoeAbi(ctypes.byref(version), ctypes.byref(desc_bytes)) != HIP_SUCCESS or \
                version.value != ABI_VERSION or desc_bytes.value != ctypes.sizeof(LayerDesc):
            raise RuntimeError("libflashMoe.so has interface revision %d with a %d-byte layer "
                               "description; this binding is written for revision %d and %d bytes: "
                               "rebuild the library" % (version.value, desc_bytes.value, ABI_VERSION,
                                                        ctypes.sizeof(LayerDesc)))
        _lib = lib
    return _lib
