from .sampler import DeviceSampler, validate_temperature

__all__ = ["DeviceSampler", "validate_temperature"]
