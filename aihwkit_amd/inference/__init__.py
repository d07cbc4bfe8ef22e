"""Inference weight pipeline on the GPU tile: the reference's ``aihwkit.inference`` noise model and drift
compensation (src/aihwkit/inference/noise/pcm.py, compensation/drift.py) and the inference-tile methods that
use them (src/aihwkit/simulator/tiles/inference.py:161-282), with the matrix kept in HBM."""
from .pcm import GlobalDriftCompensation, InferenceTile, PCMLikeNoiseModel

__all__ = ["GlobalDriftCompensation", "InferenceTile", "PCMLikeNoiseModel"]
