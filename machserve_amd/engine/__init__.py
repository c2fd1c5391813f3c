from .step import StepEntry, StepError, StepFunction
from .loading import LoadedModel, load_model, parse_dtype

__all__ = ["StepEntry", "StepError", "StepFunction", "LoadedModel", "load_model", "parse_dtype"]
