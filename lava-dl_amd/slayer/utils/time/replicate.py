"""Repeat a tensor along a new trailing time axis (utils/time/replicate.py:9-36 in the reference)."""


def replicate(input, num_steps):
    """``input [N, C, ...]`` -> ``[N, C, ..., num_steps]``, every step a copy of the input."""
    return input.unsqueeze(-1).expand(*input.shape, num_steps).contiguous()
