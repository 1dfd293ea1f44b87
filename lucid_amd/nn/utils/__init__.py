from . import rnn
from .fusion import fuse_conv_bn_eval

__all__ = ["fuse_conv_bn_eval", "rnn"]
