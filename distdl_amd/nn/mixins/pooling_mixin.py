"""Input range a pooling window touches (reference: nn/mixins/pooling_mixin.py:34-91);
the same arithmetic as a convolution kernel."""

from .conv_mixin import ConvMixin


class PoolingMixin(ConvMixin):
    pass
