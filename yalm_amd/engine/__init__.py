from .engine import Engine, StepError
from .model import Model

__all__ = ["Engine", "Model", "StepError"]
