"""The package's instruction-set list with the golden cases of tests/golden switched on."""
import os

from e3nn_amd import kernel_sets as _ks

_ks.use_golden(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))

from e3nn_amd.kernel_sets import *  # noqa: E402,F401,F403
from e3nn_amd.kernel_sets import GOLDEN_GPU_CASES, BACKWARD_CASES, BACKWARD_BF16_CASES, FUSED_FC_CASES, SH2, SH3  # noqa: E402,F401
