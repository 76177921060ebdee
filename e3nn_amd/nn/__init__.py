from .activation import Activation, Gate  # noqa: F401
from .convolution import Convolution  # noqa: F401
from .edges import DstSortedEdges  # noqa: F401
from .fc import FullyConnectedNet  # noqa: F401
