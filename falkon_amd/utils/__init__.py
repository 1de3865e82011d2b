from .tensor_helpers import create_C, create_fortran, create_same_stride, is_contig, is_f_contig  # noqa: F401
from .helpers import check_same_device, check_same_dtype, sizeof_dtype  # noqa: F401
