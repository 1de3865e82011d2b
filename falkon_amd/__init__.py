"""falkon_amd: MI355X-native kernel-vector products (Gaussian, Laplacian, Matern) behind Falkon's kernel API."""
from .options import FalkonOptions  # noqa: F401
from .kernels import GaussianKernel, LaplacianKernel, MaternKernel  # noqa: F401
from .mmv_ops import fdmmv, fmmv  # noqa: F401
from .models import Falkon, InCoreFalkon, LogisticFalkon  # noqa: F401
from . import gsc_losses  # noqa: F401

__version__ = "0.1.0"
