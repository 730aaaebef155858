"""Backend selection (reference: config.py:8-76).

``set_backend(backend_comm, backend_array, check_input_changed)`` keeps the
reference's signature and environment variables; the only pair this package
ships is ``("stub", "hip")``, which is also the default.  An unknown pair is an
error here -- the reference falls back silently to its CPU backend, and this
package has no CPU compute path to fall back to.
"""

import os

from . import backends
from .backends import supported_backends

BACKEND_COMM_ENV = "DISTDL_BACKEND_COMM"
BACKEND_ARRAY_ENV = "DISTDL_BACKEND_ARRAY"
PRE_HOOK_CHECK_INPUT_CHANGED_ENV = "DISTDL_CHECK_INPUT_CHANGED"

check_input_changed = True

# Debug aid of DistributedEmbedding (no counterpart in the reference, whose
# torch lookup raises by itself): check every forward's ids against
# [0, num_embeddings) on the host before the gather kernel runs.
CHECK_EMBEDDING_IDS_ENV = "DISTDL_CHECK_EMBEDDING_IDS"
check_embedding_ids = os.environ.get(CHECK_EMBEDDING_IDS_ENV, "0") in ("1", "True")


def get_default_comm():
    return os.environ.get(BACKEND_COMM_ENV, "stub")


def get_default_array():
    return os.environ.get(BACKEND_ARRAY_ENV, "hip")


def get_default_pre_hook_setting():
    value = os.environ.get(PRE_HOOK_CHECK_INPUT_CHANGED_ENV)
    if value is None:
        return True
    if value in ("0", "1"):
        return bool(int(value))
    if value in ("False", "True"):
        return value == "True"
    raise ValueError(f"{PRE_HOOK_CHECK_INPUT_CHANGED_ENV}={value!r} is not one of 0, 1, False, True")


def set_backend(backend_comm=None, backend_array=None, check_input_changed=None):
    if backend_comm is None:
        backend_comm = get_default_comm()
    if backend_array is None:
        backend_array = get_default_array()
    if check_input_changed is None:
        check_input_changed = get_default_pre_hook_setting()
    globals()["check_input_changed"] = bool(check_input_changed)

    name = "_".join([backend_comm, backend_array])
    module = supported_backends.get(name)
    if module is None:
        raise ValueError(f"backend {name!r} is not available; supported: {sorted(supported_backends)}")
    backends.backend = module
    return module
