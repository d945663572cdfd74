"""ctypes binding of libkhan_aev.so (HIP kernels + C ABI, see include/khan_aev.h).

There is no CPU fallback: if the shared library is missing or fails to load, importing an op raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# KHAN_AEV_LIBRARY names another build of the same library (the measurement builds of khan_amd.build)
LIB_PATH = os.environ.get("KHAN_AEV_LIBRARY") or os.path.join(_HERE, "csrc", "libkhan_aev.so")

_c_i32p = ctypes.c_void_p   # all tensor arguments are raw device addresses
_ptr = ctypes.c_void_p

KHAN_OK = 0


class KhanError(RuntimeError):
    pass


def _featurize_sig():
    return [_ptr] * 3 + [_ptr] * 3 + [ctypes.c_int32, _ptr] + [_ptr] * 4 + [ctypes.POINTER(ctypes.c_int32), _ptr]


def _featurize_grad_sig():
    return [_ptr] * 3 + [_ptr] * 3 + [ctypes.c_int32, _ptr] + [_ptr] * 4 + [_ptr] * 3 + [
        ctypes.POINTER(ctypes.c_int32), _ptr]


def _ordered(sig):
    return sig[:-1] + [_ptr, ctypes.POINTER(ctypes.c_int32), _ptr]        # ..., acs_host, order, size_classes_host, stream


_SIGNATURES = {
    "khan_feature_size": (ctypes.c_int32, []),
    "khan_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "khan_last_hip_error": (ctypes.c_char_p, []),
    "khan_set_reproducible_gradients": (ctypes.c_int, [ctypes.c_int]),
    "khan_get_parameters": (None, [ctypes.POINTER(ctypes.c_float)] * 4),
    "khan_mol_offsets": (ctypes.c_int, [_ptr, ctypes.c_int64, ctypes.c_int32, _ptr, _ptr, _ptr]),
    "khan_ani_sort": (ctypes.c_int, [_ptr, ctypes.c_int64, _ptr, _ptr, _ptr, _ptr]),
    "khan_featurize_f32": (ctypes.c_int, _featurize_sig()),
    "khan_featurize_f64": (ctypes.c_int, _featurize_sig()),
    "khan_featurize_f32_noalloc": (ctypes.c_int, _featurize_sig()),
    "khan_featurize_grad_f32": (ctypes.c_int, _featurize_grad_sig()),
    "khan_featurize_grad_f64": (ctypes.c_int, _featurize_grad_sig()),
    "khan_featurize_grad_inverse_f32": (ctypes.c_int, _featurize_grad_sig()),
    "khan_featurize_grad_inverse_f64": (ctypes.c_int, _featurize_grad_sig()),
    "khan_size_order": (ctypes.c_int, [_ptr, ctypes.c_int32, _ptr, _ptr]),
    "khan_featurize_ordered_f32": (ctypes.c_int, _ordered(_featurize_sig())),
    "khan_featurize_ordered_f64": (ctypes.c_int, _ordered(_featurize_sig())),
    "khan_featurize_grad_ordered_f32": (ctypes.c_int, _ordered(_featurize_grad_sig())),
    "khan_featurize_grad_ordered_f64": (ctypes.c_int, _ordered(_featurize_grad_sig())),
    "khan_featurize_grad_inverse_ordered_f32": (ctypes.c_int, _ordered(_featurize_grad_sig())),
    "khan_featurize_grad_inverse_ordered_f64": (ctypes.c_int, _ordered(_featurize_grad_sig())),
    "khan_ani_charge_f32": (ctypes.c_int, [_ptr] * 6 + [ctypes.c_int32, _ptr, _ptr]),
    "khan_ani_charge_f64": (ctypes.c_int, [_ptr] * 6 + [ctypes.c_int32, _ptr, _ptr]),
    "khan_ani_charge_grad_f32": (ctypes.c_int, [_ptr] * 6 + [ctypes.c_int32, _ptr, _ptr, _ptr]),
    "khan_ani_charge_grad_f64": (ctypes.c_int, [_ptr] * 6 + [ctypes.c_int32, _ptr, _ptr, _ptr]),
    "khan_ani_charge_grad_xyz_f32": (ctypes.c_int, [_ptr] * 6 + [ctypes.c_int32] + [_ptr] * 6),
    "khan_ani_charge_grad_xyz_f64": (ctypes.c_int, [_ptr] * 6 + [ctypes.c_int32] + [_ptr] * 6),
    "khan_ani_charge_all_f32": (ctypes.c_int, [_ptr] * 6 + [ctypes.c_int32] + [_ptr] * 7),
    "khan_ani_charge_all_f64": (ctypes.c_int, [_ptr] * 6 + [ctypes.c_int32] + [_ptr] * 7),
    "khan_dense_first_f32": (ctypes.c_int, [ctypes.POINTER(_ptr), ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(_ptr),
                                            ctypes.POINTER(_ptr), ctypes.c_int32, ctypes.c_float, ctypes.POINTER(_ptr), _ptr]),
    "khan_dense_f32": (ctypes.c_int, [ctypes.POINTER(_ptr), ctypes.POINTER(ctypes.c_int32), ctypes.c_int32, ctypes.c_int32,
                                      ctypes.POINTER(_ptr), ctypes.POINTER(_ptr), ctypes.c_int32, ctypes.c_float,
                                      ctypes.POINTER(_ptr), ctypes.POINTER(_ptr), _ptr]),
    "khan_dense_head_f32": (ctypes.c_int, [ctypes.POINTER(_ptr), ctypes.POINTER(ctypes.c_int32), ctypes.c_int32, ctypes.c_int32,
                                           ctypes.POINTER(_ptr), ctypes.POINTER(_ptr), ctypes.c_int32, ctypes.c_float,
                                           ctypes.POINTER(_ptr), ctypes.POINTER(_ptr), ctypes.POINTER(_ptr),
                                           ctypes.POINTER(_ptr), _ptr]),
    "khan_dense_head_grad_f32": (ctypes.c_int, [ctypes.POINTER(_ptr), ctypes.POINTER(_ptr), ctypes.POINTER(ctypes.c_int32),
                                                ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(_ptr), ctypes.c_float,
                                                ctypes.POINTER(_ptr), ctypes.POINTER(_ptr), _ptr]),
    "khan_atomic_networks_packed_bytes": (ctypes.c_int64, []),
    "khan_atomic_networks_pack_f32": (ctypes.c_int, [ctypes.POINTER(_ptr), ctypes.POINTER(_ptr), _ptr, _ptr]),
    "khan_atomic_networks_f32": (ctypes.c_int, [ctypes.POINTER(_ptr), ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(_ptr),
                                                ctypes.POINTER(_ptr), _ptr] + [ctypes.POINTER(_ptr)] * 4
                                 + [ctypes.c_float, ctypes.POINTER(_ptr), ctypes.POINTER(_ptr), _ptr]),
    "khan_mol_energy_f32": (ctypes.c_int, [ctypes.POINTER(_ptr)] + [_ptr] * 4 + [ctypes.c_int32, _ptr, _ptr]),
    "khan_mol_energy_f64": (ctypes.c_int, [ctypes.POINTER(_ptr)] + [_ptr] * 4 + [ctypes.c_int32, _ptr, _ptr]),
    "khan_mol_energy_grad_f32": (ctypes.c_int, [_ptr] * 5 + [ctypes.c_int32, ctypes.POINTER(_ptr), _ptr]),
    "khan_mol_energy_grad_f64": (ctypes.c_int, [_ptr] * 5 + [ctypes.c_int32, ctypes.POINTER(_ptr), _ptr]),
    "khan_coulomb_f32": (ctypes.c_int, [_ptr] * 6 + [ctypes.c_int32, ctypes.c_float, _ptr, _ptr]),
    "khan_coulomb_f64": (ctypes.c_int, [_ptr] * 6 + [ctypes.c_int32, ctypes.c_double, _ptr, _ptr]),
    "khan_coulomb_grad_f32": (ctypes.c_int, [_ptr] * 6 + [ctypes.c_int32, _ptr, ctypes.c_float] + [_ptr] * 5),
    "khan_coulomb_grad_f64": (ctypes.c_int, [_ptr] * 6 + [ctypes.c_int32, _ptr, ctypes.c_double] + [_ptr] * 5),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib = None


def load():
    """Loads libkhan_aev.so once and declares every entry point's signature."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise KhanError(
            "%s is missing: build it with `python -m khan_amd.build` (hipcc, gfx950). "
            "This package has no CPU fallback." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status):
    if status != KHAN_OK:
        lib = load()
        msg = lib.khan_status_string(status).decode()
        detail = lib.khan_last_hip_error().decode()
        raise KhanError("libkhan_aev: %s%s" % (msg, (" (" + detail + ")") if detail else ""))
