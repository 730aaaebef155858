"""Input range a convolution kernel touches (reference: nn/mixins/conv_mixin.py:34-91)."""


class ConvMixin:

    def _compute_min_input_range(self, idx, kernel_size, stride, padding, dilation):
        """Left-most input index read to produce output index ``idx``."""
        return stride * idx - padding

    def _compute_max_input_range(self, idx, kernel_size, stride, padding, dilation):
        """Right-most input index read to produce output index ``idx``."""
        return stride * idx + dilation * (kernel_size - 1) - padding
