"""MI355X-native implementation of Deconver's nonnegative-deconvolution (NDC) update."""

from . import _lib, ops  # noqa: F401
from .functional import deconv_update, hip_kernels_apply  # noqa: F401
