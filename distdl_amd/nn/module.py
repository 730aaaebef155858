"""Base class of every layer (reference: nn/module.py:6-112): binds the backend
selected at construction time and re-runs the layer's setup from a forward
pre-hook whenever the structure of the input changes."""

import torch

from .. import backends
from .. import config


class Module(torch.nn.Module):

    def __init__(self):
        super().__init__()
        self._distdl_backend = backends.backend
        self._distdl_is_setup = False
        self.register_forward_pre_hook(self._distdl_forward_pre_hook)

    @staticmethod
    def _distdl_forward_pre_hook(self, input):
        if self._distdl_module_requires_reset(input):
            if self._distdl_is_setup:
                self._distdl_module_teardown(input)
            self._distdl_module_setup(input)

    def _distdl_module_setup(self, input):
        pass

    def _distdl_module_teardown(self, input):
        pass

    def _distdl_input_changed(self, input):
        pass

    def _distdl_module_requires_reset(self, input):
        if config.check_input_changed:
            return not self._distdl_is_setup or self._distdl_input_changed(input)
        return not self._distdl_is_setup
