from .params import SamplingParams
from .sampler import Sampler, SampleRow, uniform, pack_rows
