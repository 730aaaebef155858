"""``DistributedTranspose`` is the historical name of Repartition (reference: nn/transpose.py)."""

from .repartition import Repartition as DistributedTranspose  # noqa: F401
