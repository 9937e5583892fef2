"""The image-processing ops of the CNN hot path (reference cgt/nn_ops/)."""
from . import conv_col, conv_same, cross_channel_lrn, im2col, max_pool_2d  # noqa: F401
