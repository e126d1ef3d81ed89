"""How a sublayer is connected to a residual stream that is kept in several copies."""

from ..ops import kernels
from ..weights.loader import VECTOR, ParamSpec
from .base import Part
from .registry import register_connection


@register_connection("hyper")
class HyperConnection(Part):
    """The residual stream as ``streams`` copies ``x_1 .. x_s`` of the width.  A sublayer reads
    ``u = sum_s in[s] x_s`` and its result ``y`` is written back while the copies are mixed:
    ``x'_t = sum_s mix[s, t] x_s + out[t] y``, every new copy from the old ones.  Three
    parameters: ``in [s]``, ``out [s]``, ``mix [s, s]`` (indexed from, to), all 32-bit."""

    graph_safe = True

    def __init__(self, width: int, dtype, streams: int):
        if not 1 <= streams <= kernels.MAX_STREAMS:
            raise ValueError(f"{streams} streams; the kernel takes 1..{kernels.MAX_STREAMS}")
        self.width = width
        self.dtype = dtype
        self.streams = streams

    def parameters(self):
        return {"in": ParamSpec((self.streams,), VECTOR), "out": ParamSpec((self.streams,), VECTOR),
                "mix": ParamSpec((self.streams, self.streams), VECTOR)}

    def bind(self, tensors):
        self.in_weights = tensors["in"]
        self.out_weights = tensors["out"]
        self.mix = tensors["mix"]

    def write_of(self, y):
        """What ``kernels.hyper_step`` needs to write the sublayer's result ``y`` back."""
        return (y, self.mix, self.out_weights)

    def read_of(self, norm, normed):
        """What ``kernels.hyper_step`` needs to hand the sublayer its normed input."""
        pending = norm.pending(None, normed)
        if pending is None or not pending.rms or pending.beta is not None:
            raise NotImplementedError("a hyper-connected sublayer takes an RMS norm without a shift")
        return (self.in_weights, pending.gamma, pending.eps, normed)


@register_connection("column_scale")
class ColumnScale(Part):
    """A learned factor per column on what a sublayer adds to the stream ("layer scale"):
    ``x <- x + weight * sublayer(norm(x))``, element by element.  One parameter, ``weight
    [width]``, 32-bit."""

    graph_safe = True

    def __init__(self, width: int, dtype):
        self.width = width
        self.dtype = dtype

    def parameters(self):
        return {"weight": ParamSpec((self.width,), VECTOR)}

    def bind(self, tensors):
        self.weight = tensors["weight"]
