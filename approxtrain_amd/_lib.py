"""ctypes binding of libamsim.so.  There is no CPU fallback: if the library is
missing or does not load, importing the compute path raises."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

STATUS = {0: "ok", 1: "invalid argument", 2: "LUT file I/O error", 3: "bad LUT format",
          4: "HIP runtime error", 5: "workspace missing or too small", 6: "unsupported"}
PADDING = {"VALID": 1, "SAME": 2}


class AmsimError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"amsim status {status} ({STATUS.get(status, '?')}): {message}")
        self.status = status


def lib_path():
    return os.path.join(_HERE, "libamsim.so")


_i, _i64, _sz, _p, _f = C.c_int, C.c_int64, C.c_size_t, C.c_void_p, C.c_void_p

# name -> (restype, argtypes); mirrors include/amsim.h and include/amsim_bench.h declaration by declaration
SIGNATURES = {
    "amsim_status_string": (C.c_char_p, [_i]),
    "amsim_last_error": (C.c_char_p, []),
    "amsim_device_info": (_i, [C.c_char_p, _sz, C.POINTER(_i)]),
    "amsim_lut_load_file": (_i, [C.c_char_p, C.POINTER(_p)]),
    "amsim_lut_create": (_i, [_p, _sz, _i, _i, C.POINTER(_p)]),
    "amsim_lut_destroy": (_i, [_p]),
    "amsim_lut_mant_width": (_i, [_p]),
    "amsim_lut_params": (_i, [_p, C.POINTER(C.c_uint32), C.POINTER(_i), C.POINTER(_i)]),
    "amsim_lut_set_split_k": (_i, [_p, _i]),
    "amsim_lut_set_engine": (_i, [_p, _i]),
    "amsim_lut_generate": (_i, [_p, _p, _i, _i, _p, _sz]),
    "amsim_lut_generate_builtin": (_i, [C.c_char_p, _i, _i, _p, _sz]),
    "amsim_mul_f32": (_i, [_p, _f, _f, _f, _sz, _p]),
    "amsim_gemm_workspace_bytes": (_sz, [_i, _i, _i64, _i64, _i64, _i64]),
    "amsim_gemm_workspace_bytes_for": (_sz, [_p, _i, _i, _i64, _i64, _i64, _i64]),
    "amsim_gemm_plan_info": (_i, [_i, _i, _i64, _i64, _i64, _i64, C.POINTER(_i64)]),
    "amsim_lut_force_gather_zeroing": (_i, [_p, _i, C.POINTER(_i)]),
    "amsim_gemm_f32": (_i, [_p, _i, _i, _i, _i64, _i64, _i64, _f, _i64, _f, _i64, _f, _i64,
                            _i64, _i64, _i64, _i64, _p, _sz, _p]),
    "amsim_convam_workspace_bytes": (_sz, [_i] * 7),
    "amsim_convam_workspace_bytes_for": (_sz, [_p] + [_i] * 7),
    "amsim_convam_lean_workspace_bytes_for": (_sz, [_p] + [_i] * 9),
    "amsim_convam_f32": (_i, [_p, _f, _f] + [_i] * 13 + [_f, _p, _sz, _p]),
    "amsim_convam_noalloc_f32": (_i, [_p, _f, _f] + [_i] * 13 + [_f, _p]),
    "amsim_convam_bias_act_f32": (_i, [_p, _f, _f] + [_i] * 13 + [_f, _f, _i, _p, _sz, _p]),
    "amsim_convam_input_grad_workspace_bytes": (_sz, [_i] * 7),
    "amsim_convam_input_grad_strided_workspace_bytes": (_sz, [_i] * 11),
    "amsim_convam_input_grad_workspace_bytes_for": (_sz, [_p] + [_i] * 11),
    "amsim_convam_input_grad_f32": (_i, [_p, _f, _i, _i, _i, _i, _f] + [_i] * 9 + [_f, _i, _i, _p, _sz, _p]),
    "amsim_convam_filter_grad_workspace_bytes": (_sz, [_i] * 7),
    "amsim_convam_filter_grad_workspace_bytes_for": (_sz, [_p] + [_i] * 7),
    "amsim_convam_filter_grad_f32": (_i, [_p, _f, _f] + [_i] * 13 + [_f, _p, _sz, _p]),
    "amsim_denseam_workspace_bytes": (_sz, [_i] * 3),
    "amsim_denseam_workspace_bytes_for": (_sz, [_p] + [_i] * 3),
    "amsim_denseam_f32": (_i, [_p, _f, _f, _f, _i, _i, _i, _p, _sz, _p]),
    "amsim_denseam_bias_act_f32": (_i, [_p, _f, _f, _f, _i, _i, _i, _f, _i, _p, _sz, _p]),
    "amsim_denseam_weight_grad_f32": (_i, [_p, _f, _f, _f, _i, _i, _i, _p, _sz, _p]),
    "amsim_denseam_input_grad_f32": (_i, [_p, _f, _f, _f, _i, _i, _i, _p, _sz, _p]),
    "amsim_matmulam_workspace_bytes": (_sz, [_i] * 6),
    "amsim_matmulam_workspace_bytes_for": (_sz, [_p] + [_i] * 6),
    "amsim_matmulam_f32": (_i, [_p, _f, _f] + [_i] * 6 + [_f, _p, _sz, _p]),
    "amsim_attention_workspace_bytes": (_sz, [_i] * 5),
    "amsim_attention_workspace_bytes_for": (_sz, [_p] + [_i] * 5),
    "amsim_attention_f32": (_i, [_p, _f, _f, _f, _f, _i, _i64, _i64] + [_i] * 5 + [C.c_float, _f, _f, _p, _sz, _p]),
    "amsim_attention_grad_workspace_bytes": (_sz, [_i] * 5),
    "amsim_attention_grad_workspace_bytes_for": (_sz, [_p] + [_i] * 5),
    "amsim_attention_grad_f32": (_i, [_p, _f, _f, _f, _f, _f] + [_i] * 5 + [C.c_float, _f, _f, _f, _p, _sz, _p]),
    "amsim_conv_geometry": (_i, [_i, _i, _i, _i, C.POINTER(_i), C.POINTER(_i)]),
    "amsim_set_split_k": (_i, [_i]),
    "amsim_set_engine": (_i, [_i]),
    "amsim_calibration_copy": (_i, [_f, _f, _sz, _p]),
    "amsim_microbench_wide": (_i, [_i, _i, _i, _i, _p, _p, _sz, _f, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "amsim_microbench": (_i, [_i, _i, _i, _i, _p, _f, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
}


def load_library():
    """Loads libamsim.so (built by ``__graft_entry__.build()`` or
    ``make -C approxtrain_amd/csrc``).  Raises if it is absent: the product
    path never falls back to anything else."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = lib_path()
    if not os.path.exists(path):
        raise ImportError(f"{path} not built: run `make -C approxtrain_amd/csrc` (needs hipcc)")
    # PyTorch ships its own copy of the HIP runtime.  Loading torch first makes libamsim.so bind to
    # that copy, so the process holds one runtime and torch's device pointers and streams are valid
    # in the library; loaded the other way round, the second runtime finds no device.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = C.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    _LIB = lib
    return lib


def check(status):
    if status != 0:
        raise AmsimError(status, load_library().amsim_last_error().decode())


def conv_geometry(in_size, filter_size, stride, padding):
    """(out_size, pad_before) of one spatial dimension; padding 'VALID' | 'SAME'."""
    o, p = _i(0), _i(0)
    check(load_library().amsim_conv_geometry(in_size, filter_size, stride, PADDING[padding], C.byref(o), C.byref(p)))
    return o.value, p.value
