"""Loads libtrips_splat.so (the HIP kernels behind the C ABI of include/trips_splat.h).

There is no CPU fallback: if the library is missing or cannot be loaded, load() raises.
"""
import ctypes as C
import os

from . import abi

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libtrips_splat.so")

# every symbol include/trips_splat.h declares
SYMBOLS = [
    "trips_version", "trips_last_error_string", "trips_ctx_create", "trips_ctx_destroy", "trips_splat_layer_sizes",
    "trips_splat_workspace_size", "trips_splat_saved_size", "trips_splat_forward", "trips_splat_forward_static",
    "trips_splat_backward",
    "trips_splat_check", "trips_splat_check_static", "trips_splat_counters", "trips_splat_export_lists", "trips_splat_export_points",
    "trips_adam_step_fused", "trips_adam_points_state_size", "trips_adam_step_points", "trips_apply_tangent", "trips_profile_enable", "trips_profile_read",
    "trips_splat_pair_rows_mode",
]
# every symbol include/trips_unet.h declares
UNET_SYMBOLS = ["trips_unet_workspace_size", "trips_unet_saved_size", "trips_unet_backward_workspace_size",
                "trips_unet_forward", "trips_unet_backward", "trips_unet_flops"]


class TripsError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"trips_splat error {code}: {message}")
        self.code = code


_lib = None


def load():
    """Returns the ctypes handle of the device library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m trips_amd.build` "
                           "(there is no CPU fallback for the splat path)")
    lib = C.CDLL(LIB_PATH)
    vp, i32, i64 = C.c_void_p, C.c_int, C.c_int64
    lib.trips_version.restype = C.c_char_p
    lib.trips_last_error_string.restype = C.c_char_p
    lib.trips_ctx_create.argtypes = [C.POINTER(vp), i32]
    lib.trips_ctx_destroy.argtypes = [vp]
    lib.trips_splat_layer_sizes.argtypes = [C.POINTER(abi.TripsSplatDesc), C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
    lib.trips_splat_workspace_size.argtypes = [C.POINTER(abi.TripsSplatDesc), C.POINTER(C.c_size_t)]
    lib.trips_splat_saved_size.argtypes = [C.POINTER(abi.TripsSplatDesc), C.POINTER(C.c_size_t)]
    lib.trips_splat_forward.argtypes = [vp, C.POINTER(abi.TripsSplatDesc), C.POINTER(abi.TripsSplatIn),
                                        C.POINTER(abi.TripsSplatOut), vp, C.c_size_t, vp]
    lib.trips_splat_forward_static.argtypes = [vp, C.POINTER(abi.TripsSplatDesc), C.POINTER(abi.TripsSplatIn),
                                               C.POINTER(abi.TripsSplatOut), vp]
    lib.trips_splat_backward.argtypes = [vp, C.POINTER(abi.TripsSplatDesc), C.POINTER(abi.TripsSplatIn), vp,
                                         C.POINTER(vp), C.POINTER(abi.TripsSplatGrads), vp, C.c_size_t, vp]
    lib.trips_splat_check.argtypes = [vp, vp, vp]
    lib.trips_splat_check_static.argtypes = [vp, vp]
    lib.trips_splat_counters.argtypes = [vp, C.POINTER(abi.TripsSplatDesc), vp, i32, C.POINTER(i64), vp]
    lib.trips_splat_export_lists.argtypes = [vp, C.POINTER(abi.TripsSplatDesc), vp, i32, vp, vp, vp, vp]
    lib.trips_splat_export_points.argtypes = [vp, C.POINTER(abi.TripsSplatDesc), vp, i32, vp, vp, vp, vp, vp]
    lib.trips_adam_step_fused.argtypes = [vp, C.POINTER(abi.TripsAdamTensor), i32, vp]
    lib.trips_adam_points_state_size.argtypes = [i32, i32, C.POINTER(C.c_size_t), C.POINTER(i32)]
    lib.trips_adam_step_points.argtypes = [vp, C.POINTER(abi.TripsAdamTensor), i32, i32, vp, vp]
    lib.trips_apply_tangent.argtypes = [vp, vp, vp, i32, vp]
    lib.trips_unet_workspace_size.argtypes = [C.POINTER(abi.TripsUnetDesc), C.POINTER(C.c_size_t)]
    lib.trips_unet_flops.argtypes = [C.POINTER(abi.TripsUnetDesc), C.POINTER(C.c_double)]
    lib.trips_unet_saved_size.argtypes = [C.POINTER(abi.TripsUnetDesc), C.POINTER(C.c_size_t)]
    lib.trips_unet_backward_workspace_size.argtypes = [C.POINTER(abi.TripsUnetDesc), C.POINTER(C.c_size_t)]
    lib.trips_unet_forward.argtypes = [vp, C.POINTER(abi.TripsUnetDesc), C.POINTER(abi.TripsUnetWeights),
                                       C.POINTER(vp), vp, vp, vp, C.c_size_t, vp]
    lib.trips_unet_backward.argtypes = [vp, C.POINTER(abi.TripsUnetDesc), C.POINTER(abi.TripsUnetWeights),
                                        C.POINTER(vp), vp, vp, C.c_float, C.POINTER(abi.TripsUnetGrads), vp,
                                        C.c_size_t, vp]
    lib.trips_profile_enable.argtypes = [vp, i32]
    lib.trips_splat_pair_rows_mode.argtypes = [vp, i32]
    lib.trips_profile_read.argtypes = [vp, C.POINTER(i32), C.POINTER(C.c_char_p), C.POINTER(C.c_float),
                                       C.POINTER(i32)]
    for name in SYMBOLS:
        fn = getattr(lib, name)
        if name not in ("trips_version", "trips_last_error_string"):
            fn.restype = C.c_int
    _lib = lib
    return lib


def check(rc):
    if rc != 0:
        msg = load().trips_last_error_string()
        raise TripsError(rc, msg.decode() if msg else "")
