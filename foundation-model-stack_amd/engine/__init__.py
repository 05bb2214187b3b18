from .batch import StepBatch, build_batch
from .engine import Engine
from .model import DecoderModel

__all__ = ["StepBatch", "build_batch", "Engine", "DecoderModel"]
