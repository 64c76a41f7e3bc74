"""placeholder"""
from dataclasses import dataclass
@dataclass
class GenerationResult:
    tokens: list
class Generator:
    pass
