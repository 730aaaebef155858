"""Layers of the per-rank hot path, under the names the reference exports
(reference: nn/__init__.py:69-133)."""

from .all_gather import AllGather  # noqa: F401
from .all_sum_reduce import AllSumReduce  # noqa: F401
from .broadcast import Broadcast  # noqa: F401
from .conv import DistributedConv1d  # noqa: F401
from .conv import DistributedConv2d  # noqa: F401
from .conv import DistributedConv3d  # noqa: F401
from .conv_feature import DistributedFeatureConv1d  # noqa: F401
from .conv_feature import DistributedFeatureConv2d  # noqa: F401
from .conv_feature import DistributedFeatureConv3d  # noqa: F401
from .embedding import DistributedEmbedding  # noqa: F401
from .halo_exchange import HaloExchange  # noqa: F401
from .layernorm import DistributedLayerNorm  # noqa: F401
from .linear import DistributedLinear  # noqa: F401
from .linear_ag import DistributedLinearAllGather  # noqa: F401
from .linear_rs import DistributedLinearReduceScatter  # noqa: F401
from .reduce_scatter import ReduceScatter  # noqa: F401
from .module import Module  # noqa: F401
from .repartition import Repartition  # noqa: F401
from .sum_reduce import SumReduce  # noqa: F401
from .transpose import DistributedTranspose  # noqa: F401

__all__ = [
    "AllGather", "AllSumReduce", "Broadcast", "DistributedConv1d", "DistributedConv2d", "DistributedConv3d",
    "DistributedFeatureConv1d", "DistributedFeatureConv2d", "DistributedFeatureConv3d", "DistributedEmbedding",
    "HaloExchange", "DistributedLayerNorm", "DistributedLinear", "DistributedLinearAllGather", "DistributedLinearReduceScatter", "Module", "ReduceScatter",
    "Repartition", "SumReduce", "DistributedTranspose",
]
