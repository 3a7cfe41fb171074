"""Shape and initialisation helpers of the convolution modules
(reference: sphconv/utils/__init__.py:27-124)."""
import math
from itertools import repeat
from typing import Iterable, List, Sequence

import torch


def out_spatial(in_spatial: Sequence[int], kernel_size: Sequence[int], stride: Sequence[int],
                padding: Sequence[int], dilation: Sequence[int] = (1, 1, 1)) -> List[int]:
    """Output size per axis: floor((i + 2p - d(k-1) - 1)/s + 1) (utils/__init__.py:27-44)."""
    return [int(math.floor((i + 2 * p - d * (k - 1) - 1) / s + 1))
            for i, k, s, p, d in zip(in_spatial, kernel_size, stride, padding, dilation)]


def _triple(x):
    """An int becomes (x, x, x); an iterable is passed through (utils/__init__.py:47-51)."""
    if isinstance(x, Iterable):
        return tuple(x)
    return tuple(repeat(x, 3))


def _calculate_fan_in_and_fan_out(tensor: torch.Tensor):
    """Fans of a [K0,K1,K2,iC,oC] weight the way the reference computes them
    (utils/__init__.py:57-80): fan_in = size(-1) * receptive field, i.e. oC * KV,
    fan_out = size(-2) * receptive field."""
    if tensor.dim() < 2:
        raise ValueError("fan in/out needs at least 2 dimensions")
    if tensor.dim() == 2:
        return tensor.size(-2), tensor.size(-1)
    receptive = 1
    for s in tensor.shape[:-2]:
        receptive *= s
    return tensor.size(-1) * receptive, tensor.size(-2) * receptive


def kaiming_uniform_(tensor: torch.Tensor, a: float = 0, mode: str = "fan_in",
                     nonlinearity: str = "leaky_relu") -> torch.Tensor:
    """He-uniform initialisation with the fans above (utils/__init__.py:96-124)."""
    fan_in, fan_out = _calculate_fan_in_and_fan_out(tensor)
    fan = fan_in if mode == "fan_in" else fan_out
    gain = torch.nn.init.calculate_gain(nonlinearity, a)
    bound = math.sqrt(3.0) * gain / math.sqrt(fan)
    with torch.no_grad():
        return tensor.uniform_(-bound, bound)
