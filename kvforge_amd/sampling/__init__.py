from kvforge_amd.sampling.params import SamplingParams
from kvforge_amd.sampling.rng import uniform

__all__ = ["SamplingParams", "uniform"]
