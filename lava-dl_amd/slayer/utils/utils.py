"""Small helpers of the reference's utils/utils.py (:9-83)."""
import torch


class dotdict(dict):
    """Dictionary whose keys read and write as attributes; a missing key reads as None."""
    __getattr__ = dict.get
    __setattr__ = dict.__setitem__
    __delattr__ = dict.__delitem__


class staticproperty(property):
    """Property of the class itself: ``Class.name`` calls the wrapped function without arguments."""

    def __get__(self, instance, owner):
        return self.fget()


def diagonal_mask(dim, num_diagonals):
    """``[dim, dim]`` mask with ones on the main diagonal and on ``num_diagonals // 2`` diagonals
    either side of it (the count is rounded up to an odd number)."""
    if num_diagonals == 0:
        raise Exception(f'Expected positive number of diagonals. Found {num_diagonals=}.')
    i = torch.arange(dim)
    return ((i[:, None] - i[None, :]).abs() <= num_diagonals // 2).float()


def event_rate(x):
    """Fraction of non-zero entries; with more than one time step the first step is left out (it
    holds initialisation events)."""
    events = x if x.shape[-1] == 1 else x[..., 1:]
    return (events != 0).to(x.dtype).mean().item()
