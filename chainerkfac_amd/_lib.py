"""ctypes binding of libkfac_hip.so (the C ABI declared in include/kfac_hip.h).

There is no fallback: if the shared library is missing, or a call fails, an
exception is raised.  Device memory is whatever the caller owns (torch-ROCm
tensors in this package); only raw pointers cross the boundary.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'libkfac_hip.so')

c_int = ctypes.c_int
c_i32p = ctypes.POINTER(ctypes.c_int32)
c_i64 = ctypes.c_int64
c_i64p = ctypes.POINTER(ctypes.c_int64)
c_f = ctypes.c_float
c_d = ctypes.c_double
c_dp = ctypes.POINTER(ctypes.c_double)
c_vp = ctypes.c_void_p
c_vpp = ctypes.POINTER(ctypes.c_void_p)
c_sz = ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/kfac_hip.h
PROTOTYPES = {
    'kfac_abi_version': (c_int, []),
    'kfac_last_error_string': (ctypes.c_char_p, []),
    'kfac_option_set': (c_int, [ctypes.c_char_p, c_d]),
    'kfac_option_unset': (c_int, [ctypes.c_char_p]),
    'kfac_option_get': (c_int, [ctypes.c_char_p, c_dp, ctypes.POINTER(c_int)]),
    'kfac_option_count': (c_int, []),
    'kfac_option_name': (ctypes.c_char_p, [c_int]),
    'kfac_packed_nelems': (c_i64, [c_int, c_i64p, c_i32p]),
    'kfac_pack_plan_create': (c_int, [c_int, c_vpp, c_i64p, c_i32p, c_i32p, c_vpp]),
    'kfac_pack_plan_set_ptrs': (c_int, [c_vp, c_vpp, c_vp]),
    'kfac_pack_plan_nelems': (c_i64, [c_vp]),
    'kfac_pack_plan_destroy': (c_int, [c_vp]),
    'kfac_pack_f32': (c_int, [c_vp, c_vp, c_i64, c_int, c_vp]),
    'kfac_unpack_f32': (c_int, [c_vp, c_vp, c_i64, c_int, c_int, c_vp]),
    'kfac_pack_f16': (c_int, [c_vp, c_vp, c_i64, c_int, c_vp]),
    'kfac_unpack_f16': (c_int, [c_vp, c_vp, c_i64, c_int, c_int, c_vp]),
    'kfac_cov_workspace_bytes': (c_sz, [c_int, c_i64]),
    'kfac_cov_linear_f32': (c_int, [c_vp, c_int, c_int, c_int, c_f, c_f, c_vp, c_vp, c_sz, c_vp]),
    'kfac_cov_conv_a_f32': (c_int, [c_vp] + [c_int] * 11 + [c_f, c_f, c_vp, c_vp, c_sz, c_vp]),
    'kfac_cov_conv_a_last_route': (c_int, []),
    'kfac_cov_conv_g_f32': (c_int, [c_vp, c_int, c_int, c_int, c_f, c_f, c_vp, c_vp, c_sz, c_vp]),
    'kfac_cov_group_create': (c_int, [c_int, c_vp, c_vpp]),
    'kfac_cov_group_workspace_bytes': (c_sz, [c_vp]),
    'kfac_cov_group_destroy': (c_int, [c_vp]),
    'kfac_cov_group_set_capture_origin': (c_int, [c_vp, c_int]),
    'kfac_cov_group_run_f32': (c_int, [c_vp, c_vpp, c_vpp, c_vp, c_vp, c_vp, c_sz, c_vp]),
    'kfac_bn_workspace_bytes': (c_sz, [c_int, c_int]),
    'kfac_bn_grad_matrix_f32': (c_int, [c_vp, c_vp, c_int, c_int, c_int, c_f, c_f, c_int, c_int,
                                        c_vp, c_vp, c_sz, c_vp]),
    'kfac_bn_stats_f32': (c_int, [c_vp, c_vp, c_int, c_int, c_int, c_vp, c_sz, c_vp]),
    'kfac_bn_finish_batch_create': (c_int, [c_vp]),
    'kfac_bn_finish_batch_destroy': (c_int, [c_vp]),
    'kfac_bn_finish_batched_f32': (c_int, [c_vp, c_int, c_vpp, c_vpp, c_i32p, c_i32p, c_i32p, c_vp, c_vp,
                                           c_i32p, c_i32p, c_vp]),
    'kfac_axpby_f32': (c_int, [c_vp, c_vp, c_i64, c_f, c_f, c_vp]),
    'kfac_axpby_batch_create': (c_int, [c_vp]),
    'kfac_axpby_batch_destroy': (c_int, [c_vp]),
    'kfac_axpby_batched_f32': (c_int, [c_vp, c_int, c_vp, c_vp, c_vp, c_f, c_f, c_vp]),
    'kfac_div_batched_f32': (c_int, [c_vp, c_int, c_vp, c_vp, c_f, c_vp]),
    'kfac_inverse_plan_create': (c_int, [c_int, c_i32p, c_vpp]),
    'kfac_inverse_plan_workspace_bytes': (c_sz, [c_vp]),
    'kfac_inverse_plan_destroy': (c_int, [c_vp]),
    'kfac_inverse_plan_set_capture_origin': (c_int, [c_vp, c_int]),
    'kfac_spd_inverse_batched_f32': (c_int, [c_vp, c_vpp, c_vpp, c_vp, c_vp, c_sz, c_vp]),
    'kfac_damp_plan_create': (c_int, [c_int, c_i32p, c_i32p, c_vpp]),
    'kfac_damp_plan_destroy': (c_int, [c_vp]),
    'kfac_pi_damp_batched_f32': (c_int, [c_vp, c_vpp, c_vpp, c_dp, c_int, c_vp, c_vp]),
    'kfac_bn_lowrank_plan_create': (c_int, [c_int, c_int, c_i32p, c_i32p, c_vpp]),
    'kfac_bn_lowrank_workspace_bytes': (c_sz, [c_vp]),
    'kfac_bn_lowrank_plan_destroy': (c_int, [c_vp]),
    'kfac_bn_lowrank_inverse_batched_f32': (c_int, [c_vp, c_vpp, c_vpp, c_dp, c_dp, c_vp, c_vp, c_sz, c_vp]),
    'kfac_add_diag_f32': (c_int, [c_vp, c_int, c_int, c_d, c_d, c_vp]),
    'kfac_keep_diag_f32': (c_int, [c_vp, c_int, c_vp]),
    'kfac_recip_add_f32': (c_int, [c_vp, c_i64, c_d, c_d, c_vp, c_i64, c_vp]),
    'kfac_diag_batch_create': (c_int, [c_vp]),
    'kfac_diag_batch_destroy': (c_int, [c_vp]),
    'kfac_add_diag_batched_f32': (c_int, [c_vp, c_int, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp]),
    'kfac_precond_conn_workspace_bytes': (c_sz, [c_int, c_int]),
    'kfac_precond_conn_f32': (c_int, [c_vp, c_int, c_vp, c_int, c_vp, c_vp, c_vp, c_vp, c_vp, c_sz, c_vp]),
    'kfac_precond_group_create': (c_int, [c_int, c_i32p, c_i32p, c_i32p, c_vpp]),
    'kfac_precond_group_workspace_bytes': (c_sz, [c_vp]),
    'kfac_precond_group_destroy': (c_int, [c_vp]),
    'kfac_precond_group_set_capture_origin': (c_int, [c_vp, c_int]),
    'kfac_precond_group_run_f32': (c_int, [c_vp, c_vpp, c_vpp, c_vpp, c_vpp, c_vpp, c_vpp, c_vp, c_sz, c_vp]),
    'kfac_precond_bn_workspace_bytes': (c_sz, [c_int]),
    'kfac_precond_bn_f32': (c_int, [c_vp, c_int, c_vp, c_int, c_vp, c_int, c_vp, c_vp, c_vp, c_vp, c_sz, c_vp]),
    'kfac_precond_bn_batch_create': (c_int, [c_vp]),
    'kfac_precond_bn_batch_destroy': (c_int, [c_vp]),
    'kfac_precond_bn_batched_workspace_bytes': (c_sz, [c_int, c_i32p]),
    'kfac_precond_bn_batched_f32': (c_int, [c_vp, c_int, c_vpp, c_i32p, c_vpp, c_i32p, c_vpp, c_vpp, c_vpp, c_vpp,
                                            c_vp, c_sz, c_vp]),
    'kfac_precond_bn_static_f32': (c_int, [c_vp, c_int, c_vp, c_int, c_vp, c_int, c_vp, c_vp, c_vp, c_vp]),
    'kfac_momentum_update_f32': (c_int, [c_vp, c_vp, c_vp, c_i64, c_f, c_f, c_vp]),
    'kfac_momentum_batch_create': (c_int, [c_vp]),
    'kfac_momentum_batch_destroy': (c_int, [c_vp]),
    'kfac_momentum_update_batched_f32': (c_int, [c_vp, c_int, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_f, c_f, c_f,
                                                 c_vp]),
    'kfac_stream_copy_f32': (c_int, [c_vp, c_vp, c_i64, c_vp]),
    'kfac_stream_fanout_f32': (c_int, [c_vp, c_vp, c_vp, c_i64, c_vp]),
    'kfac_timing_enable': (c_int, [c_int]),
    'kfac_timing_read': (c_int, [c_int, c_i64p, c_dp]),
}


class KfacHipError(RuntimeError):
    pass


_lib = None


def load():
    """Load libkfac_hip.so and attach prototypes.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise KfacHipError(
            'libkfac_hip.so is not built (expected at {}); run '
            '`python -c "import __graft_entry__ as g; g.build()"` from the '
            'repository root'.format(LIB_PATH))
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)   # AttributeError if the export is missing
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.kfac_abi_version() != 1:
        raise KfacHipError('libkfac_hip.so ABI version mismatch')
    _lib = lib
    return lib


def check(status):
    if status != 0:
        msg = load().kfac_last_error_string().decode('utf-8', 'replace')
        raise KfacHipError('libkfac_hip error {}: {}'.format(status, msg))


def set_option(name, value):
    """Sets a tuning option of the library (None restores the built-in default)."""
    lib = load()
    if value is None:
        check(lib.kfac_option_unset(name.encode()))
    else:
        check(lib.kfac_option_set(name.encode(), float(value)))


def get_option(name):
    """The value an option was set to, or None while the built-in default is in force."""
    value, is_set = ctypes.c_double(), ctypes.c_int()
    check(load().kfac_option_get(name.encode(), ctypes.byref(value), ctypes.byref(is_set)))
    return value.value if is_set.value else None


class options(object):
    """``with options(inverse_group=3): ...`` -- options set for the block, restored after."""

    def __init__(self, **values):
        self._values = values
        self._saved = {}

    def __enter__(self):
        for k, v in self._values.items():
            self._saved[k] = get_option(k)
            set_option(k, v)
        return self

    def __exit__(self, *exc):
        for k, v in self._saved.items():
            set_option(k, v)
        return False


def i32_array(values):
    return (ctypes.c_int32 * len(values))(*[int(v) for v in values])


def i64_array(values):
    return (ctypes.c_int64 * len(values))(*[int(v) for v in values])


def f64_array(values):
    return (ctypes.c_double * len(values))(*[float(v) for v in values])


def f32_array(values):
    return (ctypes.c_float * len(values))(*[float(v) for v in values])


def ptr_array(values):
    return (ctypes.c_void_p * len(values))(*[int(v) for v in values])
