from .engine import Engine, GenResult
from .hybrid import HybridEngine

__all__ = ["Engine", "GenResult", "HybridEngine"]
