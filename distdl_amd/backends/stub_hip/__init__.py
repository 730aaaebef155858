"""``stub_hip`` backend: hand-written HIP kernels for the per-rank local work,
in-process stand-ins for partitions and the wire.  Exports the names a DistDL
backend module provides (reference: backends/mpi_numpy/__init__.py:1-15)."""

from . import buffer_allocator  # noqa: F401
from . import functional  # noqa: F401
from . import tensor_comm  # noqa: F401
from . import tensor_decomposition  # noqa: F401
from . import transport  # noqa: F401
from .buffer import BufferManager  # noqa: F401
from .buffer import ExpandableBuffer  # noqa: F401
from .device import get_device  # noqa: F401
from .device import set_device  # noqa: F401
from .partition import CartesianPartition  # noqa: F401
from .partition import Partition  # noqa: F401
from .partition import SimWorld  # noqa: F401
from .tensor_comm import assemble_global_tensor_structure  # noqa: F401
from .tensor_comm import assemble_global_tensor_structure_along_axis  # noqa: F401
from .tensor_comm import broadcast_tensor_structure  # noqa: F401

__name__ = 'stub_hip'
