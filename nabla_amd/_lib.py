"""ctypes binding of libnabla_optim.so (the C ABI of include/nabla_optim.h and, for
measurement, include/nabla_optim_bench.h).

The library is the product; there is no Python or CPU fallback.  If the shared
object is missing, or no gfx950 device can be initialised, importing is still
possible (so that CPU-only checks can inspect symbols) but every compute call
raises.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnabla_optim.so")

# nbo_status
OK = 0
ERR_LEN_MISMATCH = 1
ERR_COUNT_MISMATCH = 2
ERR_SHAPE = 3
ERR_STATE_KEY = 4
ERR_STATE_INDEX = 5
ERR_KIND = 6
ERR_DTYPE = 7
ERR_ARG = 8
ERR_NO_MASTER = 9
ERR_TOO_LARGE = 10
ERR_NO_DEVICE = 11
ERR_IO = 12
ERR_HIP = 1000

DT_F32, DT_BF16, DT_F64, DT_F16 = 0, 1, 2, 3
KIND_ADAMW, KIND_ADAM, KIND_SGD = 0, 1, 2

STEP_ZERO_GRADS = 1
STEP_SKIP_NONFINITE = 2
STEP_ZERO_ON_SKIP = 4
ACC_CHECK_FINITE = 1
ACC_WRITE_GRADS = 2


class Meta(C.Structure):
    _fields_ = [
        ("kind", C.c_int32),
        ("reserved", C.c_int32),
        ("lr", C.c_double),
        ("beta1", C.c_double),
        ("beta2", C.c_double),
        ("eps", C.c_double),
        ("weight_decay", C.c_double),
        ("momentum", C.c_double),
        ("step_count", C.c_uint64),
    ]


class ScalerState(C.Structure):
    _fields_ = [
        ("scale", C.c_double),
        ("growth_factor", C.c_double),
        ("backoff_factor", C.c_double),
        ("growth_interval", C.c_uint64),
        ("consecutive_ok", C.c_uint64),
    ]


class StepInfo(C.Structure):
    _fields_ = [
        ("scale", C.c_double),
        ("norm", C.c_double),
        ("step_count", C.c_uint64),
        ("found_inf", C.c_uint32),
        ("clipped", C.c_uint32),
    ]


# every symbol include/nabla_optim.h declares: name -> (restype, argtypes)
_P = C.c_void_p
_U64P = C.POINTER(C.c_uint64)
SYMBOLS = {
    "nbo_init": (C.c_int, []),
    "nbo_set_stream": (C.c_int, [_P]),
    "nbo_sync": (C.c_int, []),
    "nbo_last_error": (C.c_char_p, []),
    "nbo_status_string": (C.c_char_p, [C.c_int]),
    "nbo_version": (C.c_char_p, []),
    "nbo_list_create": (C.c_int, [C.c_uint64, _U64P, _U64P, C.c_int, C.POINTER(_P), C.POINTER(_P)]),
    "nbo_list_set_ptrs": (C.c_int, [_P, C.POINTER(_P)]),
    "nbo_list_destroy": (C.c_int, [_P]),
    "nbo_optim_create": (C.c_int, [C.POINTER(Meta), C.c_uint64, _U64P, _U64P, C.c_int, C.c_int,
                                   C.POINTER(_P)]),
    "nbo_optim_destroy": (C.c_int, [_P]),
    "nbo_optim_step": (C.c_int, [_P, _P, _P]),
    "nbo_optim_reset": (C.c_int, [_P]),
    "nbo_optim_set_lr": (C.c_int, [_P, C.c_double]),
    "nbo_optim_get_meta": (C.c_int, [_P, C.POINTER(Meta)]),
    "nbo_optim_load_meta": (C.c_int, [_P, C.POINTER(Meta)]),
    "nbo_optim_state_read": (C.c_int, [_P, C.c_char_p, _P, C.c_uint64, C.c_int]),
    "nbo_optim_state_write": (C.c_int, [_P, C.c_char_p, _P, C.c_uint64, C.c_int]),
    "nbo_optim_master_from_params": (C.c_int, [_P, _P]),
    "nbo_optim_params_from_master": (C.c_int, [_P, _P]),
    "nbo_optim_state_regions": (C.c_int, [_P, C.POINTER(C.c_int)]),
    "nbo_optim_state_placement_note": (C.c_int, [_P, C.c_char_p, C.c_uint64]),
    "nbo_scaler_create": (C.c_int, [C.POINTER(ScalerState), C.POINTER(_P)]),
    "nbo_scaler_destroy": (C.c_int, [_P]),
    "nbo_scaler_state_get": (C.c_int, [_P, C.POINTER(ScalerState)]),
    "nbo_scaler_load_state": (C.c_int, [_P, C.POINTER(ScalerState)]),
    "nbo_scaler_unscale_and_update": (C.c_int, [_P, _P, C.POINTER(C.c_int)]),
    "nbo_clip_grad_norm": (C.c_int, [_P, C.c_double, C.POINTER(C.c_double)]),
    "nbo_has_non_finite": (C.c_int, [_P, C.POINTER(C.c_int)]),
    "nbo_zero_grad": (C.c_int, [_P]),
    "nbo_scale_grad": (C.c_int, [_P, C.c_double]),
    "nbo_fused_step": (C.c_int, [_P, _P, _P, _P, C.c_double, C.c_uint32]),
    "nbo_fused_step_noalloc": (C.c_int, [_P, _P, _P, _P, C.c_double, C.c_uint32]),
    "nbo_fused_step_groups": (C.c_int, [C.c_uint64, C.POINTER(_P), C.POINTER(_P), C.POINTER(_P), _P, _P,
                                        C.c_double, C.c_uint32]),
    "nbo_accumulate": (C.c_int, [_P, _P, C.c_int]),
    "nbo_unscale_accumulate": (C.c_int, [_P, _P, _P, C.c_uint32, C.POINTER(C.c_int), C.POINTER(C.c_double)]),
    "nbo_fused_step_norm": (C.c_int, [_P, _P, _P, C.c_double, C.c_double, C.c_uint32]),
    "nbo_fused_step_groups_norm": (C.c_int, [C.c_uint64, C.POINTER(_P), C.POINTER(_P), C.POINTER(_P),
                                             C.c_double, C.c_double, C.c_uint32]),
    "nbo_backend_apply": (C.c_int, [C.c_int, _P, _P, _P, C.c_double]),
    "nbo_backend_cast": (C.c_int, [_P, _P]),
    "nbo_optim_last_step": (C.c_int, [_P, C.POINTER(StepInfo)]),
    "nbo_optim_trace_read": (C.c_int, [_P, C.POINTER(StepInfo), C.c_uint64, _U64P, _U64P]),
    "nbo_nbla_save_list": (C.c_int, [C.c_char_p, _P, C.POINTER(C.c_char_p)]),
    "nbo_nbla_load_list": (C.c_int, [C.c_char_p, _P, C.POINTER(C.c_char_p)]),
    "nbo_optim_save_state": (C.c_int, [_P, C.c_char_p]),
    "nbo_optim_load_state": (C.c_int, [_P, C.c_char_p]),
    "nbo_optim_save_master": (C.c_int, [_P, C.c_char_p, C.POINTER(C.c_char_p)]),
    "nbo_optim_load_master": (C.c_int, [_P, C.c_char_p, C.POINTER(C.c_char_p)]),
    "nbo_optim_save_state_groups": (C.c_int, [C.c_uint64, C.POINTER(_P), C.c_char_p]),
    "nbo_optim_load_state_groups": (C.c_int, [C.c_uint64, C.POINTER(_P), C.c_char_p]),
    "nbo_optim_save_params_groups": (C.c_int, [C.c_uint64, C.POINTER(_P), C.POINTER(_P), C.c_uint64,
                                               C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_char_p),
                                               C.c_char_p]),
    "nbo_optim_load_params_groups": (C.c_int, [C.c_uint64, C.POINTER(_P), C.POINTER(_P), C.c_uint64,
                                               C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_char_p),
                                               C.c_char_p]),
}
# every symbol include/nabla_optim_bench.h declares (measurement only)
BENCH_SYMBOLS = {
    "nbo_copy_bytes": (C.c_int, [_P, _P, C.c_uint64]),
    "nbo_hbm_ceiling": (C.c_int, [C.c_int, C.c_int, C.c_uint64, C.c_int, C.c_uint32, C.POINTER(C.c_double),
                                  C.POINTER(C.c_double), C.POINTER(C.c_int)]),
    "nbo_hbm_ceiling_shape": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_uint64, C.c_int, C.c_uint32,
                                        C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_int), _U64P]),
    "nbo_hbm_ceiling_compare": (C.c_int, [C.c_int, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_uint32), C.c_int,
                                          C.c_uint64, C.c_int, C.c_int, C.c_uint32, C.POINTER(C.c_double),
                                          C.POINTER(C.c_double), C.POINTER(C.c_int)]),
    "nbo_alloc_placed": (C.c_int, [C.c_uint32, C.c_uint64, C.POINTER(C.c_int), C.POINTER(_P), C.POINTER(_P)]),
    "nbo_free_placed": (C.c_int, [_P]),
    "nbo_placed_note": (C.c_int, [_P, C.c_char_p, C.c_uint64]),
    "nbo_profile_enable": (C.c_int, [C.c_int]),
    "nbo_profile_read": (C.c_int, [C.c_char_p, _U64P, C.POINTER(C.c_double)]),
    "nbo_selftest_half_arith": (C.c_int, [C.c_int, _U64P, _U64P, _U64P, _U64P]),
}


class NablaOptimError(RuntimeError):
    """A call into libnabla_optim.so returned a non-zero status."""

    def __init__(self, status: int, message: str):
        super().__init__(f"[nbo status {status}] {message}")
        self.status = status
        self.message = message


_lib = None


def load() -> C.CDLL:
    """Load the shared library and declare its symbols (no GPU call is made)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C nabla_amd/csrc` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`). "
            "There is no fallback path.")
    # A process must hold one HIP runtime.  PyTorch's ROCm wheels carry their own copy of it,
    # and if this library pulls in the system's copy first, torch finds no GPU afterwards; with
    # torch loaded first the library binds to the copy torch brought.  So where torch is
    # installed it is imported before the library is opened (callers that never use torch are
    # not affected: without it the system's runtime is the only one).
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in list(SYMBOLS.items()) + list(BENCH_SYMBOLS.items()):
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status: int) -> None:
    if status != OK:
        lib = load()
        msg = lib.nbo_last_error().decode("utf-8", "replace") or \
            lib.nbo_status_string(status).decode()
        raise NablaOptimError(status, msg)


def init() -> None:
    """Create the runtime on device 0; raises if there is no gfx950 device."""
    check(load().nbo_init())
