from .batch import DeviceMeta, SeqStep, StepPlan
from .model import DecoderModel, expected_parameters, model_parameters, resolve_dtype
from .session import Session

__all__ = ["DeviceMeta", "SeqStep", "StepPlan", "DecoderModel", "expected_parameters",
           "model_parameters", "resolve_dtype", "Session"]
