"""Real-basis Wigner 3j symbols, computed by the C library (host code, no GPU needed).

Same contract as the reference's ``e3nn.o3.wigner_3j`` (e3nn/o3/_wigner.py:102-147):
a ``[2l1+1, 2l2+1, 2l3+1]`` tensor, invariant under simultaneous rotation of the three
indices, of Frobenius norm 1.
"""
import ctypes

import numpy as np
import torch

from .. import _lib


def wigner_3j(l1: int, l2: int, l3: int, dtype=None, device=None) -> torch.Tensor:
    assert isinstance(l1, int) and isinstance(l2, int) and isinstance(l3, int)
    assert abs(l2 - l3) <= l1 <= l2 + l3
    d = (2 * l1 + 1, 2 * l2 + 1, 2 * l3 + 1)
    buf = np.empty(d, dtype=np.float64)
    _lib.check(_lib.lib().e3x_wigner_3j(l1, l2, l3, buf.ctypes.data_as(ctypes.POINTER(ctypes.c_double))))
    if dtype is None:
        dtype = torch.get_default_dtype()
    return torch.from_numpy(buf).to(dtype=dtype, device=device, copy=True)
