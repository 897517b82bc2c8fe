"""ctypes binding of libscn_hip.so (the C ABI declared in include/scn_hip.h).

The library is loaded from this package directory, where
`python -m sparseconvnet_amd.build` puts it.  There is no fallback: without the
library every op raises."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libscn_hip.so")

_i64p = C.POINTER(C.c_int64)
_vp = C.c_void_p


class BnParams(C.Structure):
    """scn_bn_params of include/scn_hip.h: an eval-mode batch norm + leaky ReLU."""
    _fields_ = [("running_mean", _vp), ("running_var", _vp), ("gamma", _vp), ("beta", _vp),
                ("eps", C.c_float), ("leakiness", C.c_float)]


# name -> (restype, argtypes); mirrors include/scn_hip.h line by line
SIGNATURES = {
    "scn_last_error": (C.c_char_p, []),
    "scn_rulebook_bits": (C.c_int, []),
    "scn_md_create": (_vp, [C.c_int]),
    "scn_md_destroy": (None, [_vp]),
    "scn_md_clear": (C.c_int, [_vp]),
    "scn_set_build_stream": (C.c_int, [C.c_int]),
    "scn_md_set_bf16": (C.c_int, [_vp, C.c_int]),
    "scn_md_last_conv_kernel": (C.c_char_p, [_vp]),
    "scn_md_input_layer": (C.c_int, [_vp, _i64p, _vp, C.c_int64, C.c_int, C.c_int, C.c_int, _vp, _i64p]),
    "scn_md_input_layer_host": (C.c_int, [_vp, _i64p, _vp, C.c_int64, C.c_int, C.c_int, C.c_int, _vp, _i64p]),
    "scn_md_input_rules_header": (C.c_int, [_vp, C.POINTER(C.c_int32)]),
    "scn_md_input_rules": (C.c_int, [_vp, _vp, _vp]),
    "scn_md_bl_input_layer": (C.c_int, [_vp, _i64p, _vp, C.c_int64, C.c_int64, C.c_int, _vp, _i64p]),
    "scn_md_bl_rules_header": (C.c_int, [_vp, C.POINTER(C.c_int32)]),
    "scn_md_input_batch": (C.c_int, [_vp, _i64p, _vp, _vp, C.c_int64, C.c_int, C.c_int, _vp, _i64p]),
    "scn_md_generate_rulebooks": (C.c_int, [_vp, C.c_int, _vp]),
    "scn_md_nactive": (C.c_int, [_vp, _i64p, _i64p]),
    "scn_md_batch_size": (C.c_int, [_vp, _i64p, C.POINTER(C.c_int)]),
    "scn_md_spatial_locations": (C.c_int, [_vp, _i64p, _vp, _vp]),
    "scn_md_submanifold_rules": (C.c_int, [_vp, _i64p, _i64p, _vp]),
    "scn_md_strided_rules": (C.c_int, [_vp, _i64p, _i64p, _i64p, _i64p, _vp]),
    "scn_rules_count": (C.c_int, [_vp, C.c_int, _i64p, _i64p, _i64p, _i64p, _vp, C.POINTER(C.c_int)]),
    "scn_rules_sizes": (C.c_int, [_vp, C.c_int, _i64p, _i64p, _i64p, _i64p, _vp, _i64p]),
    "scn_rules_export": (C.c_int, [_vp, C.c_int, _i64p, _i64p, _i64p, _i64p, C.c_int, _vp, _vp]),
    "scn_md_take_macs": (C.c_int, [_vp, _vp, C.POINTER(C.c_double)]),
    "scn_input_layer_fwd": (C.c_int, [_vp, _vp, _vp, C.c_int, _vp]),
    "scn_output_layer_fwd": (C.c_int, [_vp, _vp, _vp, C.c_int, _vp]),
    "scn_subm_conv_fwd": (C.c_int, [_vp, _i64p, _i64p, _vp, _vp, _vp, _vp, C.c_int, C.c_int, C.c_int,
                                    _vp, C.POINTER(C.c_double)]),
    "scn_subm_conv_fwd_noalloc": (C.c_int, [_vp, _i64p, _i64p, _vp, _vp, _vp, _vp, C.c_int, C.c_int, _vp]),
    "scn_take_released_macs": (C.c_int, [C.POINTER(C.c_double)]),
    "scn_release_cache": (C.c_int, []),
    "scn_params_create": (_vp, []),
    "scn_params_destroy": (None, [_vp]),
    "scn_params_clear": (C.c_int, [_vp]),
    "scn_md_use_params": (C.c_int, [_vp, _vp]),
    "scn_active_pooling_fwd": (C.c_int, [_vp, _i64p, _vp, _vp, C.c_int, C.c_int, _vp]),
    "scn_active_pooling_bwd": (C.c_int, [_vp, _i64p, _vp, _vp, C.c_int, C.c_int, _vp]),
    "scn_md_next_output_stride": (C.c_int, [_vp, C.c_int64]),
    "scn_md_next_second_output": (C.c_int, [_vp, _vp, C.c_int64, C.POINTER(BnParams)]),
    "scn_sort_pairs": (C.c_int, [_vp, _vp, _vp, _vp, _vp, C.c_int64, C.c_int, _vp]),
    "scn_cache_stats": (C.c_int, [_i64p, _i64p, _i64p, _i64p]),
    "scn_conv_fwd": (C.c_int, [_vp, _i64p, _i64p, _i64p, _i64p, _vp, _vp, _vp, _vp, C.c_int, C.c_int,
                               C.c_int, _vp, C.POINTER(C.c_double)]),
    "scn_deconv_fwd": (C.c_int, [_vp, _i64p, _i64p, _i64p, _i64p, _vp, _vp, _vp, _vp, C.c_int, C.c_int,
                                 C.c_int, _vp, C.POINTER(C.c_double)]),
    "scn_conv_bn_fwd": (C.c_int, [_vp, C.c_int, _i64p, _i64p, _i64p, _i64p, _vp, _vp, _vp, _vp, C.c_int, C.c_int,
                                  C.c_int, C.POINTER(BnParams), C.POINTER(BnParams), _vp, C.POINTER(C.c_double)]),
    "scn_nin_fwd": (C.c_int, [_vp, _vp, _vp, _vp, _vp, C.c_int64, C.c_int, C.c_int, _vp, C.POINTER(C.c_double)]),
    "scn_maxpool_fwd": (C.c_int, [_vp, _i64p, _i64p, _i64p, _i64p, _vp, C.c_int, _vp, C.c_int, C.c_int,
                                  _vp]),
    "scn_avgpool_fwd": (C.c_int, [_vp, _i64p, _i64p, _i64p, _i64p, _vp, C.c_int, _vp, C.c_int, C.c_int,
                                  _vp]),
    "scn_unpool_fwd": (C.c_int, [_vp, _i64p, _i64p, _i64p, _i64p, _vp, C.c_int, _vp, C.c_int, C.c_int,
                                 _vp]),
    "scn_bn_eval_fwd": (C.c_int, [_vp, _vp, C.c_int64, C.c_int, C.c_int64, C.c_int64, _vp, _vp, _vp, _vp,
                                  C.c_float, C.c_float, _vp]),
    "scn_s2d_fwd": (C.c_int, [_vp, _i64p, _vp, _vp, C.c_int, _vp]),
    # backward pass
    "scn_subm_conv_bwd": (C.c_int, [_vp, _i64p, _i64p, _vp, _vp, _vp, _vp, _vp, _vp, C.c_int, C.c_int, C.c_int, _vp]),
    "scn_conv_bwd": (C.c_int, [_vp, _i64p, _i64p, _i64p, _i64p, _vp, _vp, _vp, _vp, _vp, _vp, C.c_int, C.c_int,
                               C.c_int, _vp]),
    "scn_deconv_bwd": (C.c_int, [_vp, _i64p, _i64p, _i64p, _i64p, _vp, _vp, _vp, _vp, _vp, _vp, C.c_int, C.c_int,
                                 C.c_int, _vp]),
    "scn_nin_bwd": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, C.c_int64, C.c_int, C.c_int, _vp]),
    "scn_bn_train_fwd": (C.c_int, [_vp, _vp, _vp, C.c_int64, C.c_int, C.c_int64, C.c_int64, _vp, _vp, _vp, _vp, _vp,
                                   _vp, C.c_float, C.c_float, C.c_float, _vp]),
    "scn_bn_bwd": (C.c_int, [_vp, _vp, _vp, _vp, _vp, C.c_int64, C.c_int, C.c_int64, C.c_int64, _vp, _vp, _vp, _vp,
                             _vp, C.c_float, _vp]),
    "scn_maxpool_bwd": (C.c_int, [_vp, _i64p, _i64p, _i64p, _i64p, _vp, _vp, C.c_int, _vp, _vp, C.c_int, C.c_int, _vp]),
    "scn_avgpool_bwd": (C.c_int, [_vp, _i64p, _i64p, _i64p, _i64p, _vp, C.c_int, _vp, C.c_int, C.c_int, _vp]),
    "scn_unpool_bwd": (C.c_int, [_vp, _i64p, _i64p, _i64p, _i64p, _vp, C.c_int, _vp, C.c_int, C.c_int, _vp]),
    "scn_input_layer_bwd": (C.c_int, [_vp, _vp, _vp, C.c_int, _vp]),
    "scn_output_layer_bwd": (C.c_int, [_vp, _vp, _vp, C.c_int, _vp]),
    "scn_s2d_bwd": (C.c_int, [_vp, _i64p, _vp, _vp, C.c_int, _vp]),
}

_lib = None


class ScnError(RuntimeError):
    pass


def lib():
    """The loaded library with argtypes set; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ScnError("libscn_hip.so is missing: run `python -m sparseconvnet_amd.build` "
                           "(there is no CPU fallback)")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            f = getattr(handle, name)
            f.restype = res
            f.argtypes = args
        _lib = handle
    return _lib


def check(status):
    if status != 0:
        raise ScnError(lib().scn_last_error().decode())


_sizes_made = {}


def sizes(dim, x):
    """A host int64[dim] ctypes array from an int, a sequence or a LongTensor.  The library only
    reads these arrays, and a network asks for the same few sizes in every pass: they are kept."""
    if hasattr(x, "tolist"):
        x = x.tolist()
    if isinstance(x, (int,)):
        x = (x,) * dim
    key = (dim, tuple(x))
    made = _sizes_made.get(key)
    if made is None:
        vals = [int(v) for v in key[1]]
        if len(vals) != dim:
            raise ValueError("expected %d sizes, got %r" % (dim, x))
        if len(_sizes_made) > 4096:
            _sizes_made.clear()
        made = _sizes_made[key] = (C.c_int64 * dim)(*vals)
    return made
