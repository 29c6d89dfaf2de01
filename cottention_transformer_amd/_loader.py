"""ctypes binding of libcottention_hip.so (the C ABI declared in include/cottention.h).

There is no CPU or PyTorch fallback behind these entry points: if the library cannot be built or
loaded the import of this module's `lib()` raises.
"""
import ctypes
import os

_lib = None

OK, ERR_INVALID, ERR_UNSUPPORTED, ERR_WORKSPACE, ERR_HIP = 0, 1, 2, 3, 4
F32, F64, F16, BF16 = 0, 1, 2, 3

_vp, _i, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t

SIGNATURES = {
    "cott_version": (_i, []),
    "cott_last_error": (ctypes.c_char_p, []),
    "cott_causal_workspace_bytes": (_sz, [_i] * 6),
    "cott_causal_fwd": (_i, [_vp] * 4 + [_i] * 7 + [_vp, _sz, _vp]),
    "cott_noalloc_scratch_bytes": (_sz, []),
    "cott_causal_fwd_noalloc": (_i, [_vp] * 4 + [_i] * 7 + [_vp]),
    "cott_causal_fwd_prep_supported": (_i, [_i] * 7),
    "cott_causal_fwd_prep_preferred": (_i, [_i] * 7),
    "cott_causal_fwd_prep": (_i, [_vp] * 12 + [ctypes.c_longlong] + [_i] * 10 + [_vp, _sz, _vp]),
    "cott_causal_fwd_prep_save": (_i, [_vp] * 12 + [ctypes.c_longlong] + [_i] * 4 + [_vp] + [_i] * 8 + [_vp, _sz, _vp]),
    "cott_noncausal_fwd_prep_supported": (_i, [_i] * 6),
    "cott_noncausal_fwd_prep": (_i, [_vp] * 10 + [_i] * 8 + [_vp]),
    "cott_causal_fwd_state": (_i, [_vp] * 6 + [_i] * 6 + [_vp, _sz, _vp]),
    "cott_prep_fwd": (_i, [_vp] * 9 + [_i] * 7 + [_vp]),
    "cott_prep_bwd": (_i, [_vp] * 13 + [_i] * 7 + [_vp]),
    "cott_prep_ex_fwd": (_i, [_vp] * 11 + [_i] * 10 + [_vp]),
    "cott_prep_ex_bwd": (_i, [_vp] * 15 + [_i] * 10 + [_vp]),
    "cott_causal_fwd_may_alias_v": (_i, [_i] * 6),
    "cott_causal_bwd_workspace_bytes": (_sz, [_i] * 6),
    "cott_causal_bwd": (_i, [_vp] * 7 + [_i] * 6 + [_vp, _sz, _vp]),
    "cott_causal_saved_plan": (_i, [_i] * 6 + [ctypes.POINTER(_i)] * 3 + [ctypes.POINTER(_sz)]),
    "cott_causal_fwd_save": (_i, [_vp] * 5 + [_i] * 8 + [_vp, _sz, _vp]),
    "cott_causal_bwd_saved": (_i, [_vp] * 8 + [_i] * 8 + [_vp, _sz, _vp]),
    "cott_causal_fwd_save_bnhd": (_i, [_vp] * 5 + [_i] * 8 + [_vp, _sz, _vp]),
    "cott_causal_bwd_saved_bnhd": (_i, [_vp] * 8 + [_i] * 8 + [_vp, _sz, _vp]),
    "cott_causal_fwd_bnhd": (_i, [_vp] * 4 + [_i] * 6 + [_vp, _sz, _vp]),
    "cott_causal_bwd_bnhd": (_i, [_vp] * 7 + [_i] * 6 + [_vp, _sz, _vp]),
    "cott_noncausal_workspace_bytes": (_sz, [_i] * 6),
    "cott_noncausal_fwd": (_i, [_vp] * 4 + [_i] * 6 + [_vp, _sz, _vp]),
    "cott_noncausal_bwd": (_i, [_vp] * 7 + [_i] * 6 + [_vp, _sz, _vp]),
    "cott_noncausal_fwd_bnhd": (_i, [_vp] * 4 + [_i] * 6 + [_vp, _sz, _vp]),
    "cott_noncausal_bwd_bnhd": (_i, [_vp] * 7 + [_i] * 6 + [_vp, _sz, _vp]),
    "cott_decode_step": (_i, [_vp] * 5 + [_i] * 5 + [_vp]),
    "cott_decode_step_prep": (_i, [_vp] * 6 + [ctypes.c_float, _vp, ctypes.c_longlong] + [_i] * 7 + [_vp]),
    "cott_profile_enable": (_i, [_i]),
    "cott_profile_read": (_i, [_i, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_long)]),
    "cott_kernel_name": (ctypes.c_char_p, [_i]),
    "cott_stream_probe": (_i, [_vp, _vp, _sz, _i, _i, _i, _i, _vp]),
    "cott_plan_geometry": (_i, [_i, _i]),
    "cott_plan_describe": (_i, [_i] * 8 + [ctypes.POINTER(_i), ctypes.POINTER(_i)]),
}

KERNEL_IDS = {"group_state": 0, "state_prefix": 1, "scan": 2, "apply": 3, "scan_grad": 4, "generic": 5, "decode": 6,
              "prep": 7, "stream_probe": 8}


def profile_enable(on):
    lib().cott_profile_enable(int(bool(on)))


def profile_read(kernel):
    """(total_ms, launches) of one kernel family since the last read; waits for those launches."""
    ms, n = ctypes.c_double(0.0), ctypes.c_long(0)
    rc = lib().cott_profile_read(KERNEL_IDS[kernel], ctypes.byref(ms), ctypes.byref(n))
    if rc != OK:
        raise RuntimeError(last_error())
    return ms.value, n.value


def lib_path():
    """In-tree shared object; COTT_LIBRARY points at another build of the same ABI."""
    override = os.environ.get("COTT_LIBRARY")
    if override:
        return override
    from . import build as _build
    return _build.LIB_PATH


def lib():
    """The loaded library; built first if no shared object is present."""
    global _lib
    if _lib is None:
        path = lib_path()
        if not os.path.exists(path):
            from . import build as _build
            _build.build()
        handle = ctypes.CDLL(path)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError here = header and library disagree
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def last_error():
    return lib().cott_last_error().decode("utf-8", "replace")
