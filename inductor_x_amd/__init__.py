"""MI355X-native TorchInductor backend (gfx950).  Importing the package has
side effects only, like the reference's import hook
(reference inductor_x/__init__.py:1-63); see `_register` below.
"""
from __future__ import annotations

__version__ = "0.1.0"

from . import config  # noqa: F401
