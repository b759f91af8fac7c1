"""Loads librq_w4a4.so and declares the prototypes of include/rq_w4a4.h."""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
# RQ_LIB_PATH points the binding at another build of the same ABI (A/B measurements)
LIB_PATH = os.environ.get("RQ_LIB_PATH") or os.path.join(_HERE, "lib", "librq_w4a4.so")
CSRC = os.path.join(_HERE, "csrc")


class LibraryMissing(RuntimeError):
    pass


def build_library(jobs=8):
    """Compile every HIP source for gfx950 (hipcc cross-compiles without a GPU): the operator's library, the host
    program and the probe library of the benchmark."""
    subprocess.run(["make", "-C", CSRC, "-B", "-j%d" % jobs, "all"], check=True)
    return LIB_PATH


_lib = None

c_f32p = ctypes.POINTER(ctypes.c_float)
c_i64p = ctypes.POINTER(ctypes.c_int64)
c_intp = ctypes.POINTER(ctypes.c_int)

ABI_VERSION = 3   # RQ_ABI_VERSION of include/rq_w4a4.h

PROTOTYPES = {
    "rq_w4a4_abi_version": (ctypes.c_int, []),
    "rq_w4a4_supported": (ctypes.c_int, [ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                         ctypes.c_int64, ctypes.c_int64]),
    "rq_w4a4_hadamard_factor": (ctypes.c_int, [ctypes.c_int64, c_intp, c_intp]),
    "rq_w4a4_resolve_clip": (ctypes.c_float, [ctypes.c_void_p, ctypes.c_int]),
    "rq_w4a4_tensor_rot": (ctypes.c_int64, [ctypes.c_void_p, ctypes.c_int, ctypes.c_int64]),
    "rq_w4a4_act_group": (ctypes.c_int, []),
    "rq_w4a4_weight_group": (ctypes.c_int, [ctypes.c_void_p]),
    "rq_w4a4_prepared_bytes": (ctypes.c_size_t, [ctypes.c_int64, ctypes.c_int64]),
    "rq_w4a4_prepare": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
                                       ctypes.c_size_t, ctypes.c_void_p]),
    "rq_w4a4_plane6_bytes": (ctypes.c_size_t, [ctypes.c_int64, ctypes.c_int64]),
    "rq_w4a4_inplace_staging_bytes": (ctypes.c_size_t, [ctypes.c_int64, ctypes.c_int64]),
    "rq_w4a4_prepare_inplace": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
                                               ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "rq_w4a4_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64]),
    "rq_w4a4_mul_mat": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                                       ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
                                       ctypes.c_int64, ctypes.c_float, ctypes.c_int64, ctypes.c_void_p,
                                       ctypes.c_size_t, ctypes.c_void_p]),
    "rq_w4a4_mul_mat_static": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                                              ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
                                              ctypes.c_int64, ctypes.c_float, ctypes.c_int64, ctypes.c_void_p]),
    "rq_w4a4_mul_mat_stages": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                                              ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
                                              ctypes.c_int64, ctypes.c_float, ctypes.c_int64, ctypes.c_void_p,
                                              ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int]),
    "rq_w4a4_mul_mat_fused": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_void_p),
                                             ctypes.c_int64, c_i64p, ctypes.c_void_p, ctypes.c_int64,
                                             ctypes.c_int64, ctypes.POINTER(ctypes.c_void_p), c_i64p,
                                             ctypes.c_float, ctypes.c_int64, ctypes.c_void_p, ctypes.c_size_t,
                                             ctypes.c_void_p]),
    "rq_w4a4_hadamard": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                        ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]),
    "rq_w4a4_pack": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p]),
    "rq_w4a4_pack_groups": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                           ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p]),
    "rq_w4a4_set_clip": (None, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_float]),
    "rq_w4a4_set_rot_len": (None, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32]),
    "rq_w4a4_dequantize_rows": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p]),
    "rq_w4a4_quantize_weights_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int64, ctypes.c_int64,
                                                                  ctypes.c_int]),
    "rq_w4a4_quantize_weights": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                                                ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p,
                                                ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]),
    "rq_w4a4_dequantize": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                                          ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]),
    "rq_w4a4_stage_mask": (ctypes.c_int, [ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64]),
    "rq_w4a4_quantize_act": (ctypes.c_int, [ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                                            ctypes.c_int64, ctypes.c_float, ctypes.c_int64, ctypes.c_void_p,
                                            ctypes.c_void_p]),
}


def load_library():
    """Returns the ctypes handle of librq_w4a4.so; raises LibraryMissing when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LibraryMissing(
                "%s is missing: build it with `make -C %s` (or __graft_entry__.build()); there is no fallback path"
                % (LIB_PATH, CSRC))
        L = ctypes.CDLL(LIB_PATH)
        try:
            L.rq_w4a4_abi_version.restype = ctypes.c_int
            version = L.rq_w4a4_abi_version()
        except AttributeError:
            version = None
        if version != ABI_VERSION:
            raise LibraryMissing("%s reports ABI version %s, this binding is written for %d: rebuild it with `make -C %s`"
                                 % (LIB_PATH, version, ABI_VERSION, CSRC))
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


PROBE_PATH = os.path.join(_HERE, "lib", "librq_probe.so")
_probe = None


def load_probe_library():
    """ctypes handle of librq_probe.so (include/rq_probe.h): the machine-peak probe kernels of the benchmark."""
    global _probe
    if _probe is None:
        if not os.path.exists(PROBE_PATH):
            raise LibraryMissing("%s is missing: build it with `make -C %s`" % (PROBE_PATH, CSRC))
        P = ctypes.CDLL(PROBE_PATH)
        P.rq_probe.restype = ctypes.c_int
        P.rq_probe.argtypes = [ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                               ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        _probe = P
    return _probe
