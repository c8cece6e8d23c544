from tokasaurus_amd.sampling.params import SamplingParams  # noqa: F401
from tokasaurus_amd.sampling.sampler import uniform_for  # noqa: F401
