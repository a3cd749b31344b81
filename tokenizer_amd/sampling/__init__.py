from .host import Rng, SampleError, check_params, greedy_token, sample_token, sample_with_uniform

__all__ = ["Rng", "SampleError", "check_params", "greedy_token", "sample_token", "sample_with_uniform"]
