"""Gates on the way from a block's sublayers into the residual stream."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part
from .linear import linear
from .registry import register_residual_gate


@register_residual_gate("sigmoid_projection")
class SigmoidProjectionGate(Part):
    """Every gated sublayer's result is multiplied, channel by channel, by sigmoid(R x + r), x being what the sublayer itself
    read; a matrix R and a bias r per sublayer.  `names`: the tensors' names, one per gated sublayer (the bias is the name with
    ".b" behind it).  The gates of a block are one product over the stacked matrices, left in 32-bit; the sigmoid, the
    products with the results and the sum into the 32-bit stream are one launch (`add`), which can also hand back the rows of
    the norm that is read next."""

    capturable = True

    def __init__(self, hidden_size, names, dtype, device):
        self.hidden_size, self.names = int(hidden_size), [str(n) for n in names]
        if not 1 <= len(self.names) <= 2:
            raise ValueError("a block gates one or two sublayers, got %r" % (names,))
        self.dtype, self.device = dtype, device
        self.weight = self.bias = None

    def weight_specs(self):
        H = self.hidden_size
        specs = {}
        for n in self.names:
            specs[n] = WeightSpec((H, H))
            specs[n + ".b"] = WeightSpec((H,), std=1.0)
        return specs

    def bind_weights(self, t):
        self.weight = torch.cat([t[n] for n in self.names], dim=0).contiguous()
        self.bias = torch.cat([t[n + ".b"] for n in self.names], dim=0).contiguous()

    def kernel_modules(self):
        return ["gated_residual", "gemm"] + (["gemm_skinny"] if self.dtype == torch.bfloat16 else [])

    def logits(self, x):
        """float32 [T, gates * H]: what the sigmoids are taken of."""
        if self.weight is None:
            raise RuntimeError("the gates' matrix was handed to the part that reads the same rows: take its extra columns")
        return linear(x, self.weight, self.bias, out_dtype=torch.float32)

    def hand_over(self, taker):
        """Gives the gates' matrix and bias to a part that reads the same rows and can stack them behind its own projection
        (`append_columns(weight, bias)`; its forward then leaves the logits in `extra_columns`).  True if it took them: this
        part then keeps no copy."""
        take = getattr(taker, "append_columns", None)
        if take is None or self.weight is None or not take(self.weight, self.bias):
            return False
        self.weight = self.bias = None
        return True

    def add(self, residual, z, results, then=None):
        """residual += sum_i sigmoid(z_i) * results[i] (the gated results added to each other first).  then: a norm with a
        plain gain (`weight`, `eps`, `dtype`) whose rows of the new stream come back."""
        if len(results) != len(self.names):
            raise ValueError("%d results for %d gates" % (len(results), len(self.names)))
        y2 = results[1] if len(results) > 1 else None
        if then is None:
            return ops.gated_residual_add(residual, z, results[0], y2)
        gain = then.weight if then.weight.dtype == torch.float32 else then.weight.float()
        return ops.gated_residual_add(residual, z, results[0], y2, next_gain=gain, next_eps=then.eps, dtype=then.dtype)
