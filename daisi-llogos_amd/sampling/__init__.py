from .params import GenerationParams
from .rng import uniform
from .sampler import Sampler
