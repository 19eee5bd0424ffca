from .batch import StepEntry
from .runner import ModelRunner, parse_dtype

__all__ = ["StepEntry", "ModelRunner", "parse_dtype"]
