from .engine import DecodeEngine, GenerateOutput, GenerationConfig, generate
from .stepper import SequenceStepper

__all__ = ["DecodeEngine", "GenerateOutput", "GenerationConfig", "generate", "SequenceStepper"]
