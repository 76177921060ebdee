"""ctypes binding of libe3x.so, the C ABI of the HIP kernels.

The library is built in-tree by ``e3nn_amd.csrc.build``; nothing here falls back to
another implementation: if the shared object is missing, importing a symbol raises.
"""
import ctypes
import os

import torch  # noqa: F401  (loads the HIP runtime the library links against)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libe3x.so")

F32, BF16 = 0, 1
MODE_UVW, MODE_UVU = 0, 1
NORM_INTEGRAL, NORM_COMPONENT, NORM_NORM = 0, 1, 2
ERR_INDEX = -4
ERR_INVALID = -1

c_void_p, c_int, c_int32, c_int64, c_size_t = ctypes.c_void_p, ctypes.c_int, ctypes.c_int32, ctypes.c_int64, ctypes.c_size_t


class Irrep(ctypes.Structure):
    _fields_ = [("mul", c_int32), ("l", c_int32), ("p", c_int32)]


class Instruction(ctypes.Structure):
    _fields_ = [("i_in1", c_int32), ("i_in2", c_int32), ("i_out", c_int32), ("mode", c_int32),
                ("has_weight", c_int32), ("path_weight", ctypes.c_double)]  # fmt: skip


class TpDesc(ctypes.Structure):
    _fields_ = [("n_in1", c_int32), ("n_in2", c_int32), ("n_out", c_int32), ("n_ins", c_int32),
                ("in1", ctypes.POINTER(Irrep)), ("in2", ctypes.POINTER(Irrep)), ("out", ctypes.POINTER(Irrep)),
                ("ins", ctypes.POINTER(Instruction)), ("shared_weights", c_int32), ("dtype", c_int32)]  # fmt: skip


_SIGNATURES = {
    "e3x_last_error": (ctypes.c_char_p, []),
    "e3x_version": (c_int, []),
    "e3x_wigner_3j": (c_int, [c_int, c_int, c_int, ctypes.POINTER(ctypes.c_double)]),
    "e3x_tp_plan_create": (c_int, [ctypes.POINTER(TpDesc), ctypes.POINTER(c_void_p)]),
    "e3x_tp_plan_destroy": (c_int, [c_void_p]),
    "e3x_tp_plan_info": (c_int, [c_void_p, ctypes.POINTER(c_int64), ctypes.POINTER(c_int64), ctypes.POINTER(c_int64),
                                 ctypes.POINTER(c_int64), ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(ctypes.c_char_p)]),
    "e3x_tp_plan_arithmetic": (ctypes.c_char_p, [c_void_p, c_int]),
    "e3x_tp_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "e3x_tp_forward_workspace_bytes": (c_size_t, [c_void_p]),
    "e3x_tp_forward_ws": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_size_t, c_void_p]),
    "e3x_csr_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "e3x_csr_build": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "e3x_csr_static_scratch_bytes": (c_size_t, []),
    "e3x_csr_build_static": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p]),
    "e3x_index_check": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p]),
    "e3x_tp_gather_scatter": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                      c_void_p, c_int64, c_int64, c_int64, c_void_p]),
    "e3x_row_order_workspace_bytes": (c_size_t, [c_int64]),
    "e3x_row_order_build": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p,
                                    ctypes.POINTER(c_int32), c_void_p, c_size_t, c_void_p]),
    "e3x_tp_gather_scatter_ordered": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                              c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p]),
    "e3x_tp_gather_scatter_workspace_bytes": (c_size_t, [c_void_p, c_int64]),
    "e3x_tp_gather_scatter_ws": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                         c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "e3x_tp_plan_prepare_gather_scatter_sh": (c_int, [c_void_p, c_int32, c_int32]),
    "e3x_tp_gather_scatter_sh": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                         c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int32, c_int32, c_void_p]),
    "e3x_src_rows_build": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_int64, c_void_p, c_void_p]),
    "e3x_tp_gather_scatter_radial": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32,
                                             ctypes.c_double, ctypes.c_double, ctypes.c_double, c_void_p, c_int, c_void_p,
                                             c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p]),
    "e3x_tp_plan_prepare_radial": (c_int, [c_void_p, c_int32, c_int32, c_int32, ctypes.c_double, ctypes.c_double, ctypes.c_double]),
    "e3x_tp_backward_w_x2": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                     c_void_p, c_int64, c_int64, c_int64, c_void_p]),
    "e3x_tp_plan_prepare_backward_w": (c_int, [c_void_p]),
    "e3x_tp_plan_prepare_gather_scatter_grad_w": (c_int, [c_void_p]),
    "e3x_tp_gather_scatter_grad_w": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                             c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                             c_int64, c_void_p]),
    "e3x_tp_backward_w_uvw": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "e3x_gate_forward": (c_int, [c_void_p, c_int32, c_void_p, c_int32, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int32, c_void_p]),
    "e3x_gate_backward": (c_int, [c_void_p, c_int32, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int32, c_void_p]),
    "e3x_gate_backward2": (c_int, [c_void_p, c_int32, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                   c_int64, c_int64, c_int32, c_void_p]),
    "e3x_sh_forward": (c_int, [ctypes.POINTER(c_int32), c_int32, c_int32, c_int32, c_void_p, c_void_p, c_int64,
                               c_int32, c_void_p]),
    "e3x_sh_backward": (c_int, [ctypes.POINTER(c_int32), c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_int64,
                                c_int32, c_void_p]),
    "e3x_sh_backward2": (c_int, [ctypes.POINTER(c_int32), c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_int64, c_int32, c_void_p]),
    "e3x_fc_plan_create": (c_int, [ctypes.POINTER(c_int32), c_int32, c_int32, ctypes.c_double, c_int32, ctypes.c_double,
                                   ctypes.c_double, c_int32, ctypes.POINTER(c_void_p)]),
    "e3x_fc_plan_create_fused": (c_int, [ctypes.POINTER(c_int32), c_int32, c_int32, ctypes.c_double, c_int32, ctypes.c_double,
                                         ctypes.c_double, c_int32, c_int32, ctypes.c_double, c_int32, ctypes.c_double,
                                         ctypes.POINTER(c_void_p)]),
    "e3x_fc_forward_epilogue": (c_int, [c_void_p, c_void_p, ctypes.POINTER(c_void_p), c_void_p, c_void_p, c_int64, c_void_p,
                                        c_size_t, c_void_p]),
    "e3x_fc_plan_destroy": (c_int, [c_void_p]),
    "e3x_fc_workspace_bytes": (c_size_t, [c_void_p]),
    "e3x_fc_plan_key": (ctypes.c_char_p, [c_void_p]),
    "e3x_fc_forward": (c_int, [c_void_p, c_void_p, ctypes.POINTER(c_void_p), c_void_p, c_int64, c_void_p, c_size_t, c_void_p]),
    "e3x_fc_plan_prepare_backward_w": (c_int, [c_void_p]),
    "e3x_fc_backward_w": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "e3x_copy_bytes": (c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "e3x_stream_rows": (c_int, [c_void_p, c_size_t, c_int64, c_void_p, c_size_t, c_void_p]),
}  # fmt: skip

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m e3nn_amd.csrc.build` "
                "(there is no fallback implementation)"
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


class E3xError(RuntimeError):
    pass


def check(rc):
    if rc != 0:
        msg = lib().e3x_last_error().decode()
        if rc == ERR_INDEX:
            raise IndexError(msg)
        raise E3xError(msg)


def stream_ptr(device):
    return c_void_p(torch.cuda.current_stream(device).cuda_stream)


def ptr(t):
    return c_void_p(t.data_ptr()) if t is not None and t.numel() > 0 else c_void_p(0)
