from . import build, ops  # noqa: F401
