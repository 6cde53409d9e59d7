"""ctypes binding of ``libslayer_hip.so`` (the C ABI declared in ``include/slayer_hip.h``).

There is no CPU or PyTorch fallback: if the library is missing, the import error says how to
build it, and every call raises on a non-zero status.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libslayer_hip.so")

_f32p = ctypes.c_void_p          # device pointers travel as integers (tensor.data_ptr())
_i64 = ctypes.c_int64
_f32 = ctypes.c_float
_u32 = ctypes.c_uint32
_i32 = ctypes.c_int32
_stream = ctypes.c_void_p



class SynapseGeom(ctypes.Structure):
    """``slayer_synapse_geom``: input [N][C][H][W][T], weights [O][C/groups][KH][KW]."""
    _fields_ = [(k, ctypes.c_int32) for k in ("N", "C", "H", "W", "T", "O", "KH", "KW", "strideH", "strideW",
                                              "padH", "padW", "dilH", "dilW", "groups")]


_geomp = ctypes.POINTER(SynapseGeom)
_i32p = ctypes.POINTER(ctypes.c_int32)

# name -> (restype, argtypes); must list every symbol of include/slayer_hip.h
SIGNATURES = {
    "slayer_hip_abi_version": (ctypes.c_int, []),
    "slayer_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "slayer_last_hip_error": (ctypes.c_char_p, []),
    "slayer_force_generic_kernels": (ctypes.c_int, [ctypes.c_int]),
    "slayer_get_spikes_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _i64, _i64, _i64, _f32, _f32, _stream]),
    "slayer_conv_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _i64, _i64, _i64, _f32, _stream]),
    "slayer_corr_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _i64, _i64, _i64, _f32, _stream]),
    "slayer_shift_f32": (ctypes.c_int, [_f32p, _f32p, _f32, _i64, _i64, _f32, _stream]),
    "slayer_shift_lut_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _i64, _i64, _i64, _i64, _f32, _f32, _stream]),
    "slayer_psp_spike_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _f32p, _i64, _i64, _i64, _i64, _f32, _f32,
                                            _stream]),
    "slayer_psp_alpha_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _i64, _i64, _i64, _f32, _f32, _f32, ctypes.c_int,
                                            _stream]),
    "slayer_spike_bwd_psp_alpha_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _i64, _i64, _i64, _f32, _f32, _f32,
                                                      _f32, _f32, _f32, _stream]),
    "slayer_psp_spike_bwd_alpha_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _f32p, _i64, _i64, _i64, _f32, _f32,
                                                      _f32, _f32, _f32, _f32, _stream]),
    "slayer_spike_bwd_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32, _f32, _f32, _i64, _stream]),
    "slayer_spike_bwd_corr_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _i64, _i64, _i64, _f32, _f32, _f32, _f32,
                                                 _stream]),
    "slayer_get_spikes_delayed_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _i64, _f32, _f32, _i64, _i64, _i64,
                                                     _f32, _f32, _stream]),
    "slayer_spike_bwd_delayed_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _i64, _f32, _f32, _i64, _i64, _f32,
                                                    _f32, _f32, _stream]),
    "slayer_delay_grad_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "slayer_delay_grad_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _i64, _i64, _i64, _f32, _stream]),
    "slayer_delay_grad_static_max_rows": (_i64, []),
    "slayer_delay_grad_static_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _i64, _i64, _i64, _f32, _stream]),
    "slayer_loihi_get_spikes_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _i64, _i64, _u32, _i32,
                                                  _u32, _u32, _u32, _stream]),
    "slayer_loihi_get_spikes_delayed_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _i64, _i64, _u32, _i32,
                                                          _u32, _u32, _u32, _i32, _stream]),
    "slayer_bin_packed_events_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _i64, _f32p, _i64, _i64, _i32, _i32, _i32, _i32,
                                                    _i32, ctypes.c_double, _i32, _stream]),
    "slayer_bin_events_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _i64, _i64, _i32, _i32, _i32,
                                             _i32, ctypes.c_double, _i32, _stream]),
    "slayer_spike_loss_workspace_bytes": (_i64, [_i64]),
    "slayer_spike_loss_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p, _i64, _i64, _i64, _f32,
                                             _stream]),
    "slayer_synapse_out_shape": (ctypes.c_int, [_geomp, _i32p, _i32p]),
    "slayer_synapse_conv_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _geomp, _stream]),
    "slayer_synapse_conv_grad_input_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _geomp, _stream]),
    "slayer_synapse_conv_grad_weight_workspace_bytes": (_i64, [_geomp]),
    "slayer_synapse_conv_grad_weight_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _geomp, _stream]),
    "slayer_quantize_f32": (ctypes.c_int, [_f32p, _f32p, _i64, ctypes.c_double, _stream]),
    "slayer_dense_events_workspace_bytes": (_i64, [_i64, _i64, _i64, _i64]),
    "slayer_dense_events_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _i64, _i64, _i64, _i64, _stream]),
    "slayer_dense_events_grad_weight_workspace_bytes": (_i64, [_i64, _i64, _i64, _i64]),
    "slayer_dense_events_grad_weight_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _i64, _i64, _i64, _i64, _stream]),
    "slayer_dense_rows_supported": (ctypes.c_int, [_i64, _i64, _i64, _i64]),
    "slayer_dense_rows_workspace_bytes": (_i64, [_i64, _i64]),
    "slayer_dense_rows_grad_weight_supported": (ctypes.c_int, [_i64, _i64, _i64, _i64]),
    "slayer_dense_rows_grad_weight_workspace_bytes": (_i64, [_i64, _i64, _i64, _i64]),
    "slayer_dense_rows_grad_weight_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _i64, _i64, _i64, _i64, _stream]),
    "slayer_dense_rows_f32": (ctypes.c_int, [_f32p, _f32p, _f32p, _f32p, _i64, _i64, _i64, _i64, _i64, _i64, _stream]),
}

ABI_VERSION = 1

_lib = None


class SlayerHipError(RuntimeError):
    """A C-ABI entry point returned a non-zero status."""


def load():
    """Loads the shared library once and returns the ctypes handle."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libslayer_hip.so is not built (%s). Build it with `make -C %s` "
            "(hipcc --offload-arch=gfx950); there is no fallback implementation."
            % (LIB_PATH, os.path.join(_HERE, "csrc")))
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)      # AttributeError if the library lacks a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    got = lib.slayer_hip_abi_version()
    if got != ABI_VERSION:
        raise ImportError("libslayer_hip.so has ABI version %d, expected %d" % (got, ABI_VERSION))
    _lib = lib
    return lib


def check(status, what):
    """Raises :class:`SlayerHipError` for a non-zero status of entry point ``what``."""
    if status == 0:
        return
    lib = load()
    text = lib.slayer_status_string(status).decode()
    detail = lib.slayer_last_hip_error().decode() if status == 3 else ""
    raise SlayerHipError("%s failed: %s%s" % (what, text, (" (" + detail + ")") if detail else ""))
