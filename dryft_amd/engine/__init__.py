from .engine import Engine
from .step import SeqStep, Stepper

__all__ = ["Engine", "SeqStep", "Stepper"]
