"""ctypes binding of libtagi_hip.so (declared in include/tagi_hip.h).

This is the only way Python reaches the kernels: plain pointers and sizes over
the C ABI, no torch types in any signature. Callers hand in anything that has a
`data_ptr()` (torch tensors are used for device memory and streams only) or a
raw integer address. There is no CPU fallback: if the library was not built the
import of this module fails with instructions to build it.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtagi_hip.so")

OK = 0
ERR_INVALID_ARG = -1
ERR_UNSUPPORTED = -2
ERR_NO_DEVICE = -3

_vp = ctypes.c_void_p
_i = ctypes.c_int
_f = ctypes.c_float
_sz = ctypes.c_size_t
_ip = ctypes.POINTER(ctypes.c_int)

# name -> (restype, argtypes); mirrors include/tagi_hip.h one to one
SIGNATURES = {
    "tagi_hip_version": (_i, []),
    "tagi_hip_device_count": (_i, [_ip]),
    "tagi_hip_error_string": (ctypes.c_char_p, [_i]),
    "tagi_hip_workspace_reserve": (_i, [_sz, _vp]),
    "tagi_hip_device_info": (_i, [_ip, _ip, ctypes.c_char_p, _sz]),
    "tagi_hip_shutdown": (_i, []),
    "tagi_hip_tune": (_i, [ctypes.c_char_p, _i]),
    "tagi_linear_fwd": (_i, [_vp] * 6 + [_i] * 4 + [_vp] * 3),
    "tagi_linear_fwd_act": (_i, [_vp] * 6 + [_i] * 5 + [_vp] * 4),
    "tagi_linear_fwd_static": (_i, [_vp] * 6 + [_i] * 4 + [_vp] * 3),
    "tagi_linear_bwd_dz": (_i, [_vp] * 4 + [_i] * 3 + [_vp] * 3),
    "tagi_linear_bwd_dw": (_i, [_vp] * 4 + [_i] * 3 + [_vp] * 3),
    "tagi_linear_bwd_db": (_i, [_vp] * 3 + [_i] * 2 + [_vp] * 3),
    "tagi_linear_bwd": (_i, [_vp] * 7 + [_i] * 6 + [_vp] * 7),
    "tagi_conv2d_out_size": (_i, [_i] * 6 + [_ip, _ip]),
    "tagi_conv2d_build_idx": (_i, [_i] * 7 + [_ip] * 5),
    "tagi_conv2d_fwd": (_i, [_vp] * 7 + [_i] * 7 + [_vp] * 3),
    "tagi_conv2d_fwd_act": (_i, [_vp] * 7 + [_i] * 8 + [_vp] * 4),
    "tagi_conv2d_bwd_dz": (_i, [_vp] * 6 + [_i] * 7 + [_vp] * 3),
    "tagi_conv2d_bwd_dz_res": (_i, [_vp] * 6 + [_i] * 7 + [_vp, _vp, _i] + [_vp] * 3),
    "tagi_conv2d_bwd_dw": (_i, [_vp] * 6 + [_i] * 7 + [_vp] * 5),
    "tagi_store_states": (_i, [_vp, _vp, _sz, _vp, _vp, _vp, _sz, _vp]),
    "tagi_param_update": (_i, [_vp, _vp, _f, _sz, _vp, _vp, _vp, _vp]),
    "tagi_param_raw_update": (_i, [_vp, _vp, _sz, _vp, _vp, _vp]),
    "tagi_model_update": (_i, [_vp, _i, _vp]),
    "tagi_layer_update": (_i, [_vp, _vp, _sz, _vp, _vp, _vp, _vp, _sz, _vp, _vp, _f, _vp, _i, _vp]),
    "tagi_cap_factor": (_f, [_i, _f]),
    "tagi_out_update_dense": (_i, [_vp] * 5 + [_i] + [_vp] * 3),
    "tagi_out_update_heteros": (_i, [_vp] * 4 + [_i] + [_vp] * 3),
    "tagi_out_update_indexed": (_i, [_vp] * 6 + [_i] * 3 + [_vp] * 3),
    "tagi_out_update_indexed_reset": (_i, [_vp] * 6 + [_i, _i, _i, _vp, _vp, _sz, _vp]),
    "tagi_conv2d_bwd": (_i, [_vp] * 10 + [_i] * 10 + [_vp, _vp, _i] + [_vp] * 7),
    "tagi_batchnorm2d_fwd_train": (_i, [_vp] * 8 + [_i, _f, _f, _i, _i, _i] + [_vp] * 7),
    "tagi_upload_input": (_i, [_vp, _vp, _sz, _vp, _vp, _vp]),
    "tagi_download_outputs": (_i, [_vp, _vp, _sz, _vp, _vp, _vp, ctypes.c_uint, _vp]),
    "tagi_relu_fwd": (_i, [_vp, _vp, _sz, _vp, _vp, _vp, _vp]),
    "tagi_mixture_relu_fwd": (_i, [_vp, _vp, _sz, _vp, _vp, _vp, _vp]),
    "tagi_batchnorm2d_stats": (_i, [_vp, _vp, _i, _i, _i, _f] + [_vp] * 5),
    "tagi_batchnorm2d_fwd": (_i, [_vp] * 8 + [_i, _f, _i, _i, _i] + [_vp] * 3),
    "tagi_batchnorm2d_fwd_res": (_i, [_vp] * 10 + [_i, _f, _i, _i, _i] + [_vp] * 3),
    "tagi_batchnorm2d_bwd": (_i, [_vp] * 9 + [_f] + [_i] * 6 + [_vp] * 7),
    "tagi_avgpool2d_build_idx": (_i, [_i] * 6 + [_ip] * 5),
    "tagi_avgpool2d_fwd": (_i, [_vp] * 3 + [_i] * 4 + [_vp] * 3),
    "tagi_avgpool2d_bwd_dz": (_i, [_vp] * 4 + [_i] * 7 + [_vp] * 3),
    "tagi_add_shortcut": (_i, [_vp, _vp, _sz, _vp, _vp, _vp]),
    "tagi_add_shortcut_delta": (_i, [_vp, _vp, _vp, _sz, _vp, _vp, _vp]),
}


class UpdateItem(ctypes.Structure):
    """tagi_update_item of include/tagi_hip.h."""
    _fields_ = [("delta_mu_w", _vp), ("delta_var_w", _vp), ("mu_w", _vp), ("var_w", _vp),
                ("num_weights", _sz), ("delta_mu_b", _vp), ("delta_var_b", _vp), ("mu_b", _vp),
                ("var_b", _vp), ("num_biases", _sz), ("cap_factor", _f),
                ("neg_var_count", _vp), ("slot", _i)]


class TagiHipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("%s (code %d)" % (message, code))
        self.code = code


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libtagi_hip.so is not built: run `python -m cutagi_amd.build` "
            "(needs hipcc; cross-compiles for gfx950 without a GPU). "
            "There is no CPU fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def ptr(x):
    """Address of a tensor-like (data_ptr()), an int address, or None."""
    if x is None:
        return None
    if isinstance(x, int):
        return x
    return x.data_ptr()


def check(code):
    if code != OK:
        raise TagiHipError(code, lib.tagi_hip_error_string(code).decode())


def version():
    return lib.tagi_hip_version()


def device_count():
    n = ctypes.c_int(0)
    check(lib.tagi_hip_device_count(ctypes.byref(n)))
    return n.value


def device_info():
    """(compute units, clock in MHz, name) of the current device."""
    cus, mhz = ctypes.c_int(0), ctypes.c_int(0)
    name = ctypes.create_string_buffer(256)
    check(lib.tagi_hip_device_info(ctypes.byref(cus), ctypes.byref(mhz), name, 256))
    return cus.value, mhz.value, name.value.decode()


def tune(key, value):
    check(lib.tagi_hip_tune(key.encode(), int(value)))


def cap_factor(batch_size, prev=1.0):
    return float(lib.tagi_cap_factor(int(batch_size), float(prev)))


def conv2d_out_size(kernel, stride, wi, hi, pad, pad_type):
    wo, ho = ctypes.c_int(0), ctypes.c_int(0)
    check(lib.tagi_conv2d_out_size(kernel, stride, wi, hi, pad, pad_type,
                                   ctypes.byref(wo), ctypes.byref(ho)))
    return wo.value, ho.value


def avgpool2d_build_idx(kernel, stride, wi, hi, pad, pad_type):
    """Host pooling tables as numpy int32 arrays (see tagi_avgpool2d_build_idx)."""
    import numpy as np
    wo, ho = conv2d_out_size(kernel, stride, wi, hi, pad, pad_type)
    k2 = kernel * kernel
    pool = np.zeros(wo * ho * k2, np.int32)
    zud = np.zeros(wi * hi * k2, np.int32)
    w, h, ov = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
    as_ip = lambda a: a.ctypes.data_as(_ip)
    check(lib.tagi_avgpool2d_build_idx(kernel, stride, wi, hi, pad, pad_type, as_ip(pool),
                                       as_ip(zud), ctypes.byref(w), ctypes.byref(h),
                                       ctypes.byref(ov)))
    return dict(pool_idx=pool, z_ud_idx=zud[:w.value * h.value].copy(), w=w.value, h=h.value,
                overlap=bool(ov.value), wo=wo, ho=ho)


def conv2d_build_idx(kernel, stride, wi, hi, pad, pad_type, param_pad_idx):
    """Host index tables as numpy int32 arrays (see tagi_conv2d_build_idx)."""
    import numpy as np
    wo, ho = conv2d_out_size(kernel, stride, wi, hi, pad, pad_type)
    k2 = kernel * kernel
    fm = np.zeros(wo * ho * k2, np.int32)
    zw = np.zeros(wi * hi * k2, np.int32)
    zud = np.zeros(wi * hi * k2, np.int32)
    w, h = ctypes.c_int(0), ctypes.c_int(0)
    as_ip = lambda a: a.ctypes.data_as(_ip)
    check(lib.tagi_conv2d_build_idx(kernel, stride, wi, hi, pad, pad_type,
                                    param_pad_idx, as_ip(fm), as_ip(zw),
                                    as_ip(zud), ctypes.byref(w),
                                    ctypes.byref(h)))
    n = w.value * h.value
    return dict(Fmwa_2=fm, FCzwa_1=zw[:n].copy(), Szz_ud=zud[:n].copy(),
                w=w.value, h=h.value, wo=wo, ho=ho)
