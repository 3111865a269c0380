"""Python op layer mirroring the reference's ``extensions`` package."""
from . import booleanOperations, boolop_cuda, boolutil_cuda  # noqa: F401
