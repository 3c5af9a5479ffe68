"""Sampling: per-request parameters, the device kernel's driver and the host sampler."""
from .params import SamplingParams
from .sampler import (Sampler, apply_repetition_penalty, argmax, draw, lowbias32, nucleus,
                      row_key, sample_on_device)

__all__ = ["Sampler", "SamplingParams", "apply_repetition_penalty", "argmax", "draw",
           "lowbias32", "nucleus", "row_key", "sample_on_device"]
