"""Sampling parameters of a request (mirror of ``infer/sampling_params.py:3-8``)."""
from dataclasses import dataclass


@dataclass
class SamplingParams:
    temperature: float = 1.0
    max_tokens: int = 64
    ignore_eos: bool = False
