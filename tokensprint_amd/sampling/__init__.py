from tokensprint_amd.sampling.sampler import Sampler, mix64, noise_key

__all__ = ["Sampler", "mix64", "noise_key"]
