from .irreps import Irrep, Irreps  # noqa: F401
from .linear import Linear  # noqa: F401
from .spherical_harmonics import SphericalHarmonics, spherical_harmonics  # noqa: F401
from .tensor_product import FullyConnectedTensorProduct, Instruction, TensorProduct  # noqa: F401
from .wigner import wigner_3j  # noqa: F401
