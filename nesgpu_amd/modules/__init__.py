"""Layer API mirroring the reference's ``modules`` package (binary layers only)."""
from . import base, binary  # noqa: F401
