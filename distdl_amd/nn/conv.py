"""Public convolution selectors (reference: nn/conv.py:15-88).  Only the
feature-partitioned implementation exists in this build: a selector called with
``P_x`` alone returns it, any other combination raises."""

from .conv_feature import DistributedFeatureConv1d
from .conv_feature import DistributedFeatureConv2d
from .conv_feature import DistributedFeatureConv3d


class DistributedConvSelector:

    DistributedFeatureConvType = None

    def __new__(cls, P_x, P_y=None, P_w=None, buffer_manager=None, *args, **kwargs):
        if P_y is None and P_w is None:
            return cls.DistributedFeatureConvType(P_x, buffer_manager=buffer_manager, *args, **kwargs)
        if P_y is not None and P_w is not None:
            raise NotImplementedError("channel-partitioned and general convolutions are not part of this build")
        raise ValueError("Cannot determine valid matching class.")


class DistributedConv1d(DistributedConvSelector):
    DistributedFeatureConvType = DistributedFeatureConv1d


class DistributedConv2d(DistributedConvSelector):
    DistributedFeatureConvType = DistributedFeatureConv2d


class DistributedConv3d(DistributedConvSelector):
    DistributedFeatureConvType = DistributedFeatureConv3d
