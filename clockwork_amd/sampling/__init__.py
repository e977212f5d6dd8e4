from clockwork_amd.sampling.sampler import Sampler

__all__ = ["Sampler"]
