"""dryft_amd: a small model library with generation of its own for one AMD MI355X GPU."""

from .engine import Engine, SeqStep  # noqa: F401
from .models import known_architectures, register_architecture  # noqa: F401
from .parts import register_block, register_part  # noqa: F401

__version__ = "0.1.0"
