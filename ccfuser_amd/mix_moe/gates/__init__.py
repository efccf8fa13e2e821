from .base_gate import BaseGate
from .naive_gate import NaiveGate

__all__ = ["BaseGate", "NaiveGate"]
