"""Sampling options, with the reference's names, meanings and defaults
(src/runtime/engine.h:15-22): temperature 0.7 (<= 0: greedy), top_k 50,
top_p 0.95, repetition_penalty 1.05, seed 0 (= not fixed), max_new_tokens 512."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass
class SamplingParams:
    temperature: float = 0.7
    top_k: int = 50
    top_p: float = 0.95
    repetition_penalty: float = 1.05
    seed: int = 0
    max_new_tokens: int = 512

    @staticmethod
    def greedy(max_new_tokens: int = 512) -> "SamplingParams":
        return SamplingParams(temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0,
                              seed=0, max_new_tokens=max_new_tokens)
