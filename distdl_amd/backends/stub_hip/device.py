"""Device selection of the stub backend (reference: backends/mpi_cupy/device.py:5-15).

One process drives one GPU, so every simulated rank maps to the current device.
Without a GPU the device is ``cpu``: tensors and buffers can then be created
and the host-side setup exercised, but every kernel call raises.
"""

import torch


def get_device(requested_device=None, rank=None):
    if requested_device is not None:
        return torch.device(requested_device)
    if torch.cuda.is_available():
        return torch.device("cuda", torch.cuda.current_device())
    return torch.device("cpu")


def set_device(requested_device=None, rank=None):
    return get_device(requested_device, rank)
