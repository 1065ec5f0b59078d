from pyre_amd.sampling.params import SamplingParams
from pyre_amd.sampling.rng import uniform

__all__ = ["SamplingParams", "uniform"]
