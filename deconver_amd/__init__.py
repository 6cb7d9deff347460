"""MI355X-native implementation of Deconver's nonnegative-deconvolution (NDC) update.

``Deconv`` / ``NDC`` is the drop-in layer; ``deconv_update`` is the operator boundary
(one multiplicative update as an autograd node over ``libdeconver_ndc.so``)."""

from . import _lib, ops  # noqa: F401
from .functional import DeconvUpdate, deconv_update, hip_kernels_apply, matrix_kernels, save_ratio  # noqa: F401
from .layers import (MLP, LayerNorm, Linear, PatchConv1d, PatchConv2d, PatchConv3d,  # noqa: F401
                     PatchConvTranspose1d, PatchConvTranspose2d, PatchConvTranspose3d, UnfoldConv1d,
                     UnfoldConv2d, UnfoldConv3d)
from .model import Deconver, DeconverBlock, DeconverStage, DeconvMixer, Stem  # noqa: F401
from .ndc import NDC, Deconv, Initializer  # noqa: F401
from .norm import InstanceNorm1d, InstanceNorm2d, InstanceNorm3d, instance_norm  # noqa: F401
