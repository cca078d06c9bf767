from . import build, ops

__all__ = ["build", "ops"]
