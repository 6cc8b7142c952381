from .params import UNSEEDED, SamplingParams, philox_uniform
