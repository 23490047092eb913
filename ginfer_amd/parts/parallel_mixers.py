"""Several mixers side by side on the same input, their results added with a factor each."""
import torch

from ..kernels import ops
from .base import Part
from .registry import register_mixer


@register_mixer("parallel_sum")
class ParallelSum(Part):
    """out = sum_i scale_i * mixer_i(x): `branches` are mixers of any kind (the model builds them from their `PartSpec`s),
    `names` the prefixes of their tensors inside this part, `scales` a factor each.  What a run keeps per request is the
    branches' caches one after the other (every branch gets its own share of the list of views, in the shape it
    declared).  The sum is taken in 32-bit."""

    def __init__(self, branches, names, scales, dtype, device):
        self.branches, self.names, self.scales = list(branches), [str(n) for n in names], [float(s) for s in scales]
        if not (len(self.branches) == len(self.names) == len(self.scales) == 2):
            raise ValueError("two mixers side by side, each with a name and a factor; got %d, %d, %d"
                             % (len(self.branches), len(self.names), len(self.scales)))
        self.dtype, self.device = dtype, device
        self.capturable = all(getattr(b, "capturable", False) for b in self.branches)

    def _shares(self):
        """Per branch: (its spec as it declared it, how many places of the common list it takes)."""
        out = []
        for b in self.branches:
            spec = b.cache_spec()
            out.append((spec, len(spec) if isinstance(spec, (list, tuple)) else 1))
        return out

    def cache_spec(self):
        specs = []
        for spec, _ in self._shares():
            specs += list(spec) if isinstance(spec, (list, tuple)) else [spec]
        return specs

    def weight_specs(self):
        return {n + "." + local: ws for n, b in zip(self.names, self.branches) for local, ws in b.weight_specs().items()}

    def bind_weights(self, tensors):
        for n, b in zip(self.names, self.branches):
            b.bind_weights({local: tensors[n + "." + local] for local in b.weight_specs()})

    def kernel_modules(self):
        mods = ["activation"]
        for b in self.branches:
            mods += [m for m in b.kernel_modules() if m not in mods]
        return mods

    def forward(self, x, step, cache):
        results, at = [], 0
        for b, (spec, n) in zip(self.branches, self._shares()):
            share = cache[at:at + n]
            at += n
            # (a result may be the 32-bit partial sums of a product whose K was split: the sum's kernel adds them up)
            results.append(b.forward(x, step, share if isinstance(spec, (list, tuple)) else share[0]))
        return ops.scaled_sum(results[0], results[1], self.scales[0], self.scales[1], self.dtype)
