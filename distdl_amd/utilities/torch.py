"""Small torch-side helpers shared by the layers (reference: utilities/torch.py)."""

import numpy as np
import torch


def zero_volume_tensor(b=None, dtype=None, requires_grad=False, device=None):
    """The tensor an inactive worker holds: shape ``(0,)``, or ``(b, 0)`` when a
    batch size has to survive (utilities/torch.py:5-13)."""
    if dtype is None:
        dtype = torch.get_default_dtype()
    shape = (0,) if b is None else (b, 0)
    return torch.empty(shape, dtype=dtype, requires_grad=requires_grad, device=device)


class TensorStructure:
    """(shape, dtype, requires_grad) of a tensor; layers re-run their setup when
    it changes (utilities/torch.py:16-40)."""

    __slots__ = ("shape", "dtype", "requires_grad")

    def __init__(self, tensor=None):
        self.shape = self.dtype = self.requires_grad = None      # "nothing seen yet"
        if tensor is not None:
            self.fill_from_tensor(tensor)

    def fill_from_tensor(self, tensor):
        self.shape, self.dtype, self.requires_grad = tensor.shape, tensor.dtype, tensor.requires_grad

    def _key(self):
        shape = None if self.shape is None else tuple(int(s) for s in self.shape)
        return (shape, self.dtype, self.requires_grad)

    def __eq__(self, other):
        return self._key() == other._key()

    def __ne__(self, other):
        return not self.__eq__(other)

    def __repr__(self):
        return "TensorStructure(shape=%s, dtype=%s, requires_grad=%s)" % self._key()


def distdl_padding_to_torch_padding(pad):
    """``[[a_0, b_0], ..., [a_n, b_n]] -> (a_n, b_n, ..., a_0, b_0)``, the order
    ``torch.nn.functional.pad`` wants (utilities/torch.py:43-49)."""
    return tuple(int(v) for row in reversed(list(pad)) for v in np.atleast_1d(row))
