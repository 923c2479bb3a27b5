from .host import sample_host
from .params import SamplingParams
from .rng import Xoshiro256
