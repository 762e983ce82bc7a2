"""qfactory for MI355X: weight-only-quantized linear layers on hand-written gfx950 kernels.

Same public surface as the reference package (``qfactory/__init__.py:26-27``): ``QLinear`` and
``QMatmul``, logging level from ``QFACTORY_LOG_LEVEL``.
"""
import logging
import os

_levels = {None: logging.INFO, "DEBUG": logging.DEBUG, "INFO": logging.INFO, "WARNING": logging.WARNING,
           "ERROR": logging.ERROR, "CRITICAL": logging.CRITICAL}
_env_level = os.environ.get("QFACTORY_LOG_LEVEL")
assert _env_level in _levels, f"Unknown log level {_env_level}"

logging.basicConfig(
    format="%(levelname)s %(asctime)s [%(filename)s:%(lineno)d] %(message)s",
    level=_levels[_env_level],
)

from .core import QMatmul, Matmul   # noqa: E402
from .qlinear import QLinear        # noqa: E402

__all__ = ["QLinear", "QMatmul", "Matmul"]
