from .kernel import Kernel  # noqa: F401
from .diff_kernel import DiffKernel  # noqa: F401
from .distance_kernel import GaussianKernel, LaplacianKernel, MaternKernel  # noqa: F401
