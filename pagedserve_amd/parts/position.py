"""Position encodings."""

from ..weights.loader import TABLE, ParamSpec
from .base import PositionEncoding
from .registry import register_position


@register_position("learned_absolute")
class LearnedAbsolutePositions(PositionEncoding):
    """A table row per position, added to the token embedding
    (src/model/paged_decoder.py:289,311-313).  Positions must lie in ``[0, max_positions)``
    (src/model/paged_decoder.py:519-522)."""

    graph_safe = True

    def __init__(self, width: int, dtype, max_positions: int):
        self.width = width
        self.dtype = dtype
        self.max_positions = max_positions

    def parameters(self):
        return {"table": ParamSpec((self.max_positions, self.width), TABLE)}

    def embedding_table(self):
        return self.table


@register_position("none")
class NoPositions(PositionEncoding):
    """Nothing is added and nothing is rotated."""

    graph_safe = True

    def __init__(self, width: int, dtype, max_positions: int = 0):
        self.width = width
        self.dtype = dtype
        self.max_positions = max_positions


def rotary_frequencies(dims: int, base: float, scaling=None):
    """(frequencies of the ``dims / 2`` rotated pairs as 64-bit floats, factor on cosine and sine).

    Pair ``i`` turns by ``position * f_i`` with ``f_i = base^(-2i / dims)``.  ``scaling = (factor,
    original, fast, slow)`` stretches them in the manner of YaRN (Peng et al., "YaRN: Efficient
    Context Window Extension of Large Language Models"): a pair that makes ``t`` turns over
    ``original`` positions has index ``n(t) = dims * ln(original / (2 pi t)) / (2 ln base)``;
    with ``lo = max(floor(n(fast)), 0)``, ``hi = min(ceil(n(slow)), dims - 1)`` and ``ramp_i =
    clamp((i - lo) / max(hi - lo, 0.001), 0, 1)`` the frequency becomes ``f_i / factor * ramp_i +
    f_i * (1 - ramp_i)`` (fast pairs keep theirs, slow ones are divided by the factor), and
    cosine and sine are multiplied by ``0.1 ln(factor) + 1``."""
    import math

    import torch

    steps = torch.arange(dims // 2, dtype=torch.float64)
    freqs = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * steps / dims)
    if scaling is None:
        return freqs, 1.0
    factor, original, fast, slow = (float(value) for value in scaling)

    def index_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    low = max(math.floor(index_of(fast)), 0)
    high = min(math.ceil(index_of(slow)), dims - 1)
    ramp = torch.clamp((steps - low) / max(high - low, 0.001), 0.0, 1.0)
    return freqs / factor * ramp + freqs * (1.0 - ramp), 0.1 * math.log(factor) + 1.0
