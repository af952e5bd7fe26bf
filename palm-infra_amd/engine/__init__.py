"""The model built from its description, the step function, the generation loop and trace replay."""
from .engine import Engine, FedTokens, StepEntry, StepError, resolve_dtype
from .model import DecoderModel

__all__ = ["Engine", "FedTokens", "StepEntry", "StepError", "resolve_dtype", "DecoderModel"]
