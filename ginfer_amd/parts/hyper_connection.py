"""Hyper-connections: the residual stream kept as several streams side by side, and how a sublayer reads and writes them."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part
from .registry import register_connection, register_stream


@register_stream("hyper_streams")
class HyperStreams(Part):
    """The residual stream as `streams` copies, float32 [T, streams, W]: all equal to the embedding's output at the start
    (`open`), added up at the end (`close`, at the rows whose logits are wanted)."""

    capturable = True

    def __init__(self, streams, dtype, device):
        self.streams = int(streams)
        if not 1 <= self.streams <= ops.HYPER_MAX_STREAMS:
            raise ValueError("1 to %d streams, got %r" % (ops.HYPER_MAX_STREAMS, streams))
        self.dtype, self.device = dtype, device

    def kernel_modules(self):
        return ["hyper_connection"]

    def open(self, x):
        return ops.hyper_open(x, self.streams)

    def close(self, X, rows=None):
        return ops.hyper_sum(X, rows)


@register_connection("hyper_connection")
class HyperConnection(Part):
    """One sublayer's link to the streams X: it reads u = sum_s in[s] X_s (through its norm: `read`), and its result y enters
    as X_j <- sum_s mix[s, j] X_s + out[j] * y for all j at once from the old streams (`write`; mix is indexed [from, to]).
    `write` can make the rows that the next sublayer reads in the same launch.  Tensors: in [S], out [S], mix [S, S];
    everything 32-bit.  learned=False: no tensors, every weight 1 on one stream, which is the plain residual sum x <- x + y."""

    capturable = True

    def __init__(self, streams, dtype, device, learned=True):
        self.streams, self.learned = int(streams), bool(learned)
        if not self.learned and self.streams != 1:
            raise ValueError("the plain residual sum has one stream")
        if not 1 <= self.streams <= ops.HYPER_MAX_STREAMS:
            raise ValueError("1 to %d streams, got %r" % (ops.HYPER_MAX_STREAMS, streams))
        self.dtype, self.device = dtype, device
        self.w_in = self.w_out = self.w_mix = None

    def weight_specs(self):
        S = self.streams
        if not self.learned:
            return {}
        return {"in": WeightSpec((S,), init="unit_interval", keep_32bit=True),
                "out": WeightSpec((S,), init="one_plus_normal", std=0.1, keep_32bit=True),
                "mix": WeightSpec((S, S), std=0.5, keep_32bit=True)}

    def bind_weights(self, t):
        if not self.learned:
            one = torch.ones((1,), dtype=torch.float32, device=self.device)
            self.w_in, self.w_out, self.w_mix = one, one.clone(), one.clone().view(1, 1)
            return
        self.w_in, self.w_out, self.w_mix = (t[n].float().contiguous() for n in ("in", "out", "mix"))

    def kernel_modules(self):
        return ["hyper_connection"]

    @staticmethod
    def _gain(norm):
        """The norm's gain in 32-bit, converted once (a checkpoint may store it in the compute dtype)."""
        if norm.weight.dtype == torch.float32:
            return norm.weight
        kept = getattr(norm, "_gain32", None)
        if kept is None or kept[0] is not norm.weight:
            kept = (norm.weight, norm.weight.float().contiguous())
            norm._gain32 = kept
        return kept[1]

    def read(self, X, norm):
        """The rows of `norm` (a gain over the root mean square) of what this sublayer reads."""
        return ops.hyper_read(X, self.w_in, self._gain(norm), norm.eps, norm.dtype)

    def write(self, X, y, then=None):
        """Adds the sublayer's result y into the streams; then = (the next sublayer's connection, its norm): returns the rows
        that it reads."""
        if then is None:
            return ops.hyper_write(X, self.w_mix, self.w_out, y)
        link, norm = then
        return ops.hyper_write(X, self.w_mix, self.w_out, y, link.w_in, self._gain(norm), norm.eps, norm.dtype)
