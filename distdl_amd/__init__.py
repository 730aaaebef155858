"""distdl_amd: MI355X-native per-rank hot path of DistDL (Repartition and halo
pack / unpack, LayerNorm / Embedding / Linear shard compute) behind DistDL's own
backend seam and layer signatures."""

__version__ = "0.1.0"

from . import backends  # noqa: F401
from . import config  # noqa: F401
from . import utilities  # noqa: F401

config.set_backend()

from . import nn  # noqa: E402,F401
