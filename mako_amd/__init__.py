"""MI355X-native token sampler with the call surface of mako's gen::Sampler."""
from .api import (PARAMS_DTYPE, Batch, Desc, MakoError, SamplerContext, make_params, sample)  # noqa: F401
