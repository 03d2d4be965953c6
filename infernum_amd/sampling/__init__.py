from .params import GenerateOptions, SamplingParams
from .rng import token_uniform
from .sampler import RowRequest, Sampler
