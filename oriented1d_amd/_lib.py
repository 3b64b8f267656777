"""ctypes binding of libdwoconv1d_hip.so (the declarations of include/dwoconv1d_hip.h)."""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# DWOCONV1D_LIB overrides the library location (e.g. an instrumented build)
LIB_PATH = os.environ.get("DWOCONV1D_LIB") or os.path.join(HERE, "libdwoconv1d_hip.so")

F32, BF16, F16 = 0, 1, 2
NCHW, NHWC = 0, 1

_vp, _i, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t

# name -> (restype, argtypes); kept in the order of the header
SIGNATURES = {
    "dwo_version": (_i, []),
    "dwo_status_string": (ctypes.c_char_p, [_i]),
    "dwo_init": (_i, []),
    "dwo_taps_bytes": (_sz, [_i, _i]),
    "dwo_build_taps": (_i, [_vp, _i, _i, _vp]),
    "dwo_taps_get": (_i, [_vp, _i, _i, ctypes.POINTER(_i), ctypes.POINTER(_i)]),
    "dwo_fprop": (_i, [_vp, _vp, _vp, _vp, _vp] + [_i] * 8 + [_vp]),
    "dwo_dgrad": (_i, [_vp, _vp, _vp, _vp] + [_i] * 8 + [_vp]),
    "dwo_wgrad_scratch_bytes": (_sz, [_i] * 8),
    "dwo_wgrad": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _sz] + [_i] * 8 + [_vp]),
    "dwo_wgrad_static": (_i, [_vp, _vp, _vp, _vp, _vp] + [_i] * 8 + [_vp]),
    "dwo_set_wgrad_reduction": (_i, [_i]),
    "dwo_pointwise_fprop_nhwc": (_i, [_vp] * 7 + [_i] * 8 + [_vp]),
    "dwo_layernorm_nhwc": (_i, [_vp, _vp, _vp, _vp, _sz, _i, ctypes.c_float, _i, _i, _vp]),
    "dwo_nchw_layernorm_nhwc": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, ctypes.c_float, _i, _vp]),
    "dwo_nhwc_scale_add_nchw": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
}

_lib = None


def load():
    """Load the built library; there is no fallback when it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "libdwoconv1d_hip.so is not built (expected at %s); run "
            "`python -m oriented1d_amd.build` -- this operator has no CPU or PyTorch fallback"
            % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    _lib = lib
    return lib


_ready = set()


def ready(device):
    """The loaded library with its kernels set up on ``device`` (a torch CUDA device): the first
    use on a device runs ``dwo_init`` there, so no later call does anything but launch kernels."""
    import torch

    lib = load()
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _ready:
        with torch.cuda.device(index):
            check(lib.dwo_init(), "dwo_init")
        _ready.add(index)
    return lib


def launch(device, fn, *args):
    """Calls a launching entry point with ``device`` current: the library keeps its per-device
    state (occupancy figures, counters, the static scratch) under the current device, which
    must be the one the tensors and the stream live on."""
    import torch

    index = device.index if device.index is not None else torch.cuda.current_device()
    if index == torch.cuda.current_device():
        return fn(*args)
    with torch.cuda.device(index):
        return fn(*args)


def check(status, what):
    if status != 0:
        msg = load().dwo_status_string(status).decode()
        raise RuntimeError("%s failed: %s (status %d)" % (what, msg, status))
