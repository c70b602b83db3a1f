"""ctypes view of libcnet_hip.so, the C-ABI device library (include/cnet_hip.h).

This module is plumbing for Python callers (tests, bench): it loads the in-tree library, declares every entry
point's signature, turns non-zero status codes into exceptions and moves numpy arrays to and from device memory.
There is no fallback of any kind: a missing library or a missing GPU raises.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libcnet_hip.so")

c_fp = C.c_void_p  # device pointers travel as integers
_i = C.c_int
_l = C.c_int64

# name -> argument types, exactly as declared in include/cnet_hip.h
SIGNATURES = {
    "cnet_init": [_i],
    "cnet_shutdown": [],
    "cnet_get_device_info": [C.c_void_p],
    "cnet_stream": [],
    "cnet_set_stream": [C.c_void_p],
    "cnet_sync": [],
    "cnet_alloc": [C.c_size_t, C.POINTER(C.c_void_p)],
    "cnet_free": [C.c_void_p],
    "cnet_memcpy_h2d": [C.c_void_p, C.c_void_p, C.c_size_t],
    "cnet_host_alloc": [C.c_size_t, C.POINTER(C.c_void_p)],
    "cnet_host_free": [C.c_void_p],
    "cnet_memcpy_h2d_async": [C.c_void_p, C.c_void_p, C.c_size_t],
    "cnet_memcpy_d2h_async": [C.c_void_p, C.c_void_p, C.c_size_t],
    "cnet_upload_async": [C.c_void_p, C.c_void_p, C.c_size_t],
    "cnet_upload_zero": [C.c_void_p, C.c_size_t],
    "cnet_upload_pair": [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p, C.c_size_t],
    "cnet_upload_gather_rows": [c_fp, _l, _l, c_fp, _l, _l, _i, _i, C.c_void_p, c_fp, c_fp, _i, _i],
    "cnet_gather_rows": [c_fp, _l, _l, c_fp, _l, _l, _i, _i, C.c_void_p, c_fp, c_fp, _i, _i],
    "cnet_upload_wait_compute": [],
    "cnet_mark_compute": [_i],
    "cnet_upload_wait_marker": [_i],
    "cnet_compute_wait_upload": [],
    "cnet_mark_upload": [_i],
    "cnet_compute_wait_upload_marker": [_i],
    "cnet_upload_sync": [],
    "cnet_copy_ticket": [_i, C.POINTER(C.c_int64)],
    "cnet_copy_wait": [C.c_int64],
    "cnet_compute_wait_ticket": [C.c_int64],
    "cnet_graph_begin": [],
    "cnet_graph_end": [C.POINTER(C.c_void_p)],
    "cnet_graph_launch": [C.c_void_p],
    "cnet_graph_destroy": [C.c_void_p],
    "cnet_memcpy_d2h": [C.c_void_p, C.c_void_p, C.c_size_t],
    "cnet_memcpy_d2d": [C.c_void_p, C.c_void_p, C.c_size_t],
    "cnet_memset_zero": [C.c_void_p, C.c_size_t],
    "cnet_cgemm": [_i, _i, _i, _i, _i, _i, c_fp, c_fp, _l, c_fp, c_fp, _l, c_fp, c_fp, _l, _i],
    "cnet_cgemm_batched": [_i, _i, _i, _i, _i, _i, _i, c_fp, c_fp, _l, _l, c_fp, c_fp, _l, _l, c_fp, c_fp, _l, _l, _i, _i],
    "cnet_clinear_fwd": [c_fp, c_fp, _l, c_fp, c_fp, _l, c_fp, c_fp, _l, _i, _i, _i, _i],
    "cnet_clinear_cgelu_fwd": [c_fp, c_fp, _l, c_fp, c_fp, _l, c_fp, c_fp, c_fp, c_fp, _l, _i, _i, _i, _i],
    "cnet_clinear_bwd_input": [c_fp] * 4 + [_l] + [c_fp] * 2 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i, _i],
    "cnet_clinear_bwd_weight": [c_fp] * 4 + [_l] + [c_fp] * 2 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i, _i],
    "cnet_clinear_bwd_input_sym": [c_fp] * 2 + [_l] + [c_fp] * 2 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i, _i],
    "cnet_clinear_bwd_weight_sym": [c_fp] * 2 + [_l] + [c_fp] * 2 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i, _i],
    "cnet_clinear_hadamard_cgelu_bwd_sym": [c_fp] * 2 + [_l] + [c_fp] * 2 + [_l] + [c_fp] * 2 + [_l] + ([c_fp] * 4 + [_l, _i]) * 2 +
                                           [c_fp] * 2 + [_l] + [c_fp] * 2 + ([c_fp] * 4 + [_l]) * 2 + [c_fp] * 4 + [_i, _i, _i, _i],
    "cnet_clinear_bwd_sym": [c_fp] * 2 + [_l] + [c_fp] * 2 + [_l] + [c_fp] * 2 + [_l] + [c_fp] * 4 + [_l, _i] + [c_fp] * 4 + [_l, _i, _i, _i, _i],
    "cnet_clinear_cross_entropy_fwd_bwd_sym": [c_fp, c_fp, _l, c_fp, c_fp, _l, c_fp, c_fp, _l, c_fp, c_fp, c_fp, _l, c_fp, c_fp, c_fp] +
                                              [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_cdft_plan": [_i],
    "cnet_cdft_twiddle": [_i, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p)],
    "cnet_cdft_set_forward_matrix": [_i, C.c_void_p, C.c_void_p],
    "cnet_cgemm_set_products": [_i],
    "cnet_cgemm_get_products": [],
    "cnet_cdft_fwd": [c_fp, c_fp, _l, c_fp, c_fp, _l, _i, _i, _i],
    "cnet_cdft_fwd_real_input": [c_fp, c_fp, _l, c_fp, c_fp, _l, _i, _i],
    "cnet_cdft_hadamard_cgelu_fwd": [c_fp, c_fp, _l] + [c_fp] * 8 + [_l, _i, _i],
    "cnet_cdft_bwd": [c_fp] * 4 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_cdft_bwd_sym": [c_fp] * 2 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_ctriang_dft_bwd_sym": [c_fp] * 2 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_ctriang_dft_plan": [_i],
    "cnet_ctriang_dft_fwd": [c_fp, c_fp, _l, c_fp, c_fp, _l, _i, _i, _i],
    "cnet_ctriang_dft_bwd": [c_fp] * 4 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_hadamard_fwd": [c_fp, c_fp, _l, c_fp, c_fp, _l, c_fp, c_fp, _l, _i, _i],
    "cnet_hadamard_bwd": [c_fp, c_fp, _l, c_fp, c_fp, _l] + [c_fp] * 4 + [_l] + [c_fp] * 4 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_cgelu_fwd": [c_fp, c_fp, _l, c_fp, c_fp, _l, _i, _i],
    "cnet_cgelu_bwd": [c_fp, c_fp, _l] + [c_fp] * 4 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_crelu_fwd": [c_fp, c_fp, _l, c_fp, c_fp, _l, _i, _i],
    "cnet_crelu_bwd": [c_fp, c_fp, _l] + [c_fp] * 4 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_residual_fwd": [c_fp, c_fp, _l, c_fp, c_fp, _l, c_fp, c_fp, _l, _i, _i],
    "cnet_residual_bwd": [c_fp] * 4 + [_l] + [c_fp] * 4 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_l2norm_fwd": [c_fp, c_fp, _l, c_fp, c_fp, _l, c_fp, _i, _i],
    "cnet_l2norm_bwd": [c_fp, c_fp, _l, c_fp] + [c_fp] * 4 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_cross_entropy_fwd": [c_fp, c_fp, _l, c_fp, c_fp, c_fp, _l, c_fp, c_fp, c_fp, _i, _i],
    "cnet_cross_entropy_bwd": [c_fp, c_fp, _l, c_fp, c_fp] + [c_fp] * 4 + [_l, _i, _i],
    "cnet_l2out_fwd": [c_fp, c_fp, _l, c_fp, _i, _i],
    "cnet_l2out_bwd": [c_fp, c_fp, _l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_hadamard_bwd_sym": [c_fp, c_fp, _l, c_fp, c_fp, _l, c_fp, c_fp, _l] + [c_fp] * 4 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_cgelu_bwd_sym": [c_fp, c_fp, _l, c_fp, c_fp, _l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_hadamard_cgelu_fwd": [c_fp, c_fp, _l, c_fp, c_fp, _l, c_fp, c_fp, _l, c_fp, c_fp, _l, _i, _i],
    "cnet_hadamard_cgelu_bwd_sym": [c_fp, c_fp, _l, c_fp, c_fp, _l, c_fp, c_fp, _l] + ([c_fp] * 4 + [_l]) * 3 + [_i, _i, _i],
    "cnet_crelu_bwd_sym": [c_fp, c_fp, _l, c_fp, c_fp, _l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_residual_bwd_sym": [c_fp, c_fp, _l] + [c_fp] * 4 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_residual_bwd_sym2": [c_fp, c_fp, _l, c_fp, c_fp, _l] + [c_fp] * 4 + [_l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_residual_cgelu_bwd_sym": [c_fp, c_fp, _l, c_fp, c_fp, _l, c_fp, c_fp, _l] + ([c_fp] * 4 + [_l]) * 3 + [_i, _i],
    "cnet_l2norm_bwd_sym": [c_fp, c_fp, _l, c_fp, c_fp, c_fp, _l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_l2out_bwd_sym": [c_fp, c_fp, _l] + [c_fp] * 4 + [_l, _i, _i, _i],
    "cnet_cross_entropy_bwd_sym": [c_fp, c_fp, _l, c_fp, c_fp] + [c_fp] * 4 + [_l, _i, _i],
    "cnet_cross_entropy_fwd_bwd_sym": [c_fp, c_fp, _l, c_fp, c_fp, c_fp, _l, c_fp, c_fp, c_fp] + [c_fp] * 4 + [_l, _i, _i],
    "cnet_copy2d": [c_fp, _l, c_fp, _l, _i, _i],
    "cnet_add2d": [c_fp, _l, c_fp, _l, _i, _i],
    "cnet_add_multi": [_i, C.c_void_p, C.c_void_p, C.c_void_p],
    "cnet_batch_sum": [c_fp, _l, c_fp, _i, _i, _i],
    "cnet_batch_sum_noalloc": [c_fp, _l, c_fp, _i, _i, _i],
    "cnet_sgd_update": [c_fp, c_fp, c_fp, c_fp, _l, C.c_float, _i],
    "cnet_sgd_update_multi": [_i, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, _i],
    "cnet_adam_update": [c_fp] * 6 + [_l, C.c_float, C.c_float, _i, _i],
    "cnet_embedding_fwd": [c_fp, c_fp, _i, _i, c_fp, c_fp, c_fp, _l, _i, _i],
    "cnet_embedding_bwd": [c_fp, c_fp, c_fp, _l, c_fp, c_fp, _i, _i, _i, _i, _i],
    "cnet_last_error": [],
}


class DeviceInfo(C.Structure):
    _fields_ = [("name", C.c_char * 256), ("arch", C.c_char * 64), ("compute_units", C.c_int),
                ("clock_khz", C.c_int), ("wavefront_size", C.c_int), ("lds_bytes_per_block", C.c_int),
                ("hbm_bytes", C.c_int64), ("fp32_matrix_peak_tflops", C.c_double)]


class CnetError(RuntimeError):
    pass


_lib = None


def load():
    """Load the library and declare signatures (no GPU needed for this)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise CnetError("libcnet_hip.so is not built: run `python -m cnet_amd.build` (%s)" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, args in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the header and the library disagree
            fn.argtypes = args
            fn.restype = _i
        lib.cnet_last_error.restype = C.c_char_p
        lib.cnet_stream.restype = C.c_void_p
        _lib = lib
    return _lib


def check(rc, what=""):
    if rc != 0:
        raise CnetError("%s failed with status %d: %s" % (what or "cnet call", rc, load().cnet_last_error().decode()))


def call(name, *args):
    check(getattr(load(), name)(*args), name)


def init(device=0):
    call("cnet_init", device)


def shutdown():
    call("cnet_shutdown")


def sync():
    call("cnet_sync")


def device_info():
    info = DeviceInfo()
    call("cnet_get_device_info", C.byref(info))
    return info


class DevArray:
    """A C-contiguous fp32/int32 array in device memory allocated through cnet_alloc."""

    def __init__(self, shape, dtype=np.float32):
        self.shape = tuple(int(s) for s in np.atleast_1d(shape))
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = C.c_void_p()
        call("cnet_alloc", max(self.nbytes, 16), C.byref(p))
        self.ptr = p.value

    @property
    def ld(self):
        return self.shape[-1]

    def at(self, *index):
        """Device address of an element (row-major)."""
        off = 0
        for k, i in enumerate(index):
            off = off * self.shape[k] + i
        for k in range(len(index), len(self.shape)):
            off *= self.shape[k]
        return self.ptr + off * self.dtype.itemsize

    def upload(self, host):
        host = np.ascontiguousarray(host, self.dtype)
        assert host.shape == self.shape, (host.shape, self.shape)
        call("cnet_memcpy_h2d", self.ptr, host.ctypes.data, self.nbytes)
        return self

    def download(self):
        out = np.empty(self.shape, self.dtype)
        call("cnet_memcpy_d2h", out.ctypes.data, self.ptr, self.nbytes)
        return out

    def zero(self):
        call("cnet_memset_zero", self.ptr, self.nbytes)
        return self

    def free(self):
        if self.ptr:
            call("cnet_free", self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def to_device(host):
    host = np.ascontiguousarray(host)
    return DevArray(host.shape, host.dtype).upload(host)


def empty(shape, dtype=np.float32):
    return DevArray(shape, dtype)


def zeros(shape, dtype=np.float32):
    return DevArray(shape, dtype).zero()
