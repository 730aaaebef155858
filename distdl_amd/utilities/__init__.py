from . import slicing  # noqa: F401
from . import tensor_decomposition  # noqa: F401
from . import torch  # noqa: F401
