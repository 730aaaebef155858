"""Backend registry (reference: backends/__init__.py:7-19).

``supported_backends`` maps ``"<comm>_<array>"`` to a backend module; the one
selected by :func:`distdl_amd.config.set_backend` is ``backends.backend``.
This package ships a single backend, ``stub_hip``: HIP kernels for the local
work, in-process stand-ins for the wire.
"""

import importlib
import logging

supported_backends = {
    "stub_hip": None,
}

backend = None

for _name in list(supported_backends):
    try:
        supported_backends[_name] = importlib.import_module(__name__ + "." + _name)
    except Exception as exc:  # pragma: no cover - import problems are reported, not hidden
        logging.getLogger("distdl_amd").warning("Could not load %s backend: %s", _name, exc)
