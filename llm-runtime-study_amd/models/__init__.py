"""Model assembly: the neutral ModelSpec, the decoder that runs it, and the architectures."""

from .decoder import DecoderModel
from .spec import ModelSpec, ScheduleEntry

__all__ = ["DecoderModel", "ModelSpec", "ScheduleEntry"]
