"""How a layer's parts are arranged around the residual stream."""
from ..kernels import ops
from .registry import register_arrangement


class Arrangement:
    """How a layer's parts sit around the residual stream.  A kind of arrangement says which roles it has and of which
    family each is (`roles`: role -> "mixer" | "feed_forward" | "norm"); the model builds the parts that a layer names
    for exactly these roles and hands them over as a dictionary.  Every part becomes an attribute under its role's
    name.  forward(residual float32 [T, H], delta, step, cache) takes the output of the block before as a pending
    `delta` (it is added to the residual by the first norm that runs) and returns its own last output as the next one.
    cache_spec(): what one run of the block keeps per request; the mixer's, unless the kind says otherwise (a block with
    several parts that keep something returns the list of their specs and gets the list of views as `cache`)."""

    roles = {}
    optional_roles = ()      # roles that a layer of this kind may leave out

    def __init__(self, parts):
        self._parts = dict(parts)
        for role, part in self._parts.items():
            setattr(self, role, part)

    def parts(self):
        """(role, part) pairs; the roles are what `LayerSpec.names` gives tensor prefixes for."""
        return list(self._parts.items())

    def cache_spec(self):
        mixer = self._parts.get("mixer")
        return mixer.cache_spec() if mixer is not None else None

    def forward(self, residual, delta, step, cache):
        raise NotImplementedError


@register_arrangement("prenorm")
class PreNormBlock(Arrangement):
    """n = norm1(x); h = x + mixer(n); n = norm2(h); x = h + feed_forward(n)
    (ginfer/core/layer/transformer/encoder.cc:33-39).  The residual stream is kept in 32-bit and every add
    is fused into the norm that follows it, so a block takes the previous block's output as a pending
    `delta` and returns its own feed-forward output as the next one.  Where the mixer says `folds_norm`, the
    feed-forward `takes_scaled_rows` and the norm between them is `foldable`, the mixer may add its result to
    the residual itself and hand the norm's rows on in two factors (ops.ScaledRows): then the second norm makes
    no pass over memory of its own.  The same holds across blocks: a block whose feed-forward `folds_norm` may be
    given the first norm of the block that runs next (`into_norm`), if that block says `takes_folded_input()`;
    it then returns ops.ScaledRows in place of its delta, and the next block skips its first norm."""

    roles = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "norm", "feed_forward_norm": "norm"}

    def __init__(self, parts):
        super().__init__(parts)
        mixer, feed_forward, feed_forward_norm = self.mixer, self.feed_forward, self.feed_forward_norm
        self.folds = (getattr(mixer, "folds_norm", False) and getattr(feed_forward, "takes_scaled_rows", False)
                      and getattr(feed_forward_norm, "foldable", False))

    @property
    def folds_output(self):
        """Whether forward() takes `into_norm`."""
        return bool(getattr(self.feed_forward, "folds_norm", False))

    def takes_folded_input(self):
        """The norm whose rows this block takes in two factors (ops.ScaledRows) in place of a delta, or None."""
        if getattr(self.mixer, "takes_scaled_rows", False) and getattr(self.mixer_norm, "foldable", False):
            return self.mixer_norm
        return None

    def forward(self, residual, delta, step, cache, into_norm=None):
        if isinstance(delta, ops.ScaledRows):      # the block before has added its output and folded this norm
            n = delta
        else:
            n = self.mixer_norm.forward(residual, whole(delta, self.mixer_norm))
        if self.folds:
            a = self.mixer.forward(n, step, cache, into_norm=(residual, self.feed_forward_norm))
        else:
            a = self.mixer.forward(n, step, cache)
        if not isinstance(a, ops.ScaledRows):
            a = self.feed_forward_norm.forward(residual, whole(a, self.feed_forward_norm))
        if into_norm is not None:
            return self.feed_forward.forward(a, into_norm=(residual, into_norm))
        return self.feed_forward.forward(a)


@register_arrangement("outnorm")
class OutputNormBlock(Arrangement):
    """x <- x + norm1(mixer(conv(x)));  x <- x + norm2(feed_forward(x)): the norms sit on the sublayers' OUTPUTS, and the
    sublayers read the residual stream itself (the mixer through an optional short convolution over time).  A layer may
    have no feed-forward (then it has no second norm either) and no convolution.  The norms are of a kind that offers
    `add_normed(residual, y, copy)`.  The 32-bit stream is updated in place; nothing is left pending for the next block.
    What a run keeps per request is the convolution's state followed by the mixer's cache, as a list."""

    roles = {"mixer": "mixer", "mixer_norm": "norm", "feed_forward": "feed_forward", "feed_forward_norm": "norm",
             "input_conv": "convolution"}
    optional_roles = ("feed_forward", "feed_forward_norm", "input_conv")

    def __init__(self, parts):
        super().__init__(parts)
        self.input_conv = self._parts.get("input_conv")
        self.feed_forward = self._parts.get("feed_forward")
        self.feed_forward_norm = self._parts.get("feed_forward_norm")
        if (self.feed_forward is None) != (self.feed_forward_norm is None):
            raise ValueError("a block names its feed-forward and that feed-forward's norm together, or neither")
        for norm in (self.mixer_norm, self.feed_forward_norm):
            if norm is not None and not hasattr(norm, "add_normed"):
                raise ValueError("the norms of this block sit on the sublayers' outputs: %s has no add_normed"
                                 % type(norm).__name__)

    def cache_spec(self):
        conv = self.input_conv.cache_spec() if self.input_conv is not None else None
        return [conv, self.mixer.cache_spec()]

    def forward(self, residual, delta, step, cache):
        if delta is not None:                     # what a block of another kind left pending
            residual.add_(whole(delta).to(residual.dtype))
        conv_cache, mixer_cache = cache
        dtype = self.mixer_norm.dtype
        if self.input_conv is not None:
            h = self.input_conv.forward(residual, step, conv_cache)
        else:
            h = residual if dtype == residual.dtype else residual.to(dtype)
        m = self.mixer.forward(h, step, mixer_cache)
        x = self.mixer_norm.add_normed(residual, m, copy=self.feed_forward is not None)
        if self.feed_forward is not None:
            self.feed_forward_norm.add_normed(residual, self.feed_forward.forward(x))
        return None


class NormedRows:
    """What a block hands to the next one in place of a pending delta when it has already added its own output into the
    stream and made the rows of the next block's first norm in the same launch."""

    def __init__(self, rows):
        self.rows = rows


@register_arrangement("sandwich")
class SandwichBlock(Arrangement):
    """x <- x + out_norm1(mixer(norm1(x)));  x <- x + out_norm2(feed_forward(norm2(x))): a norm in front of every
    sublayer and one on its output (which may bring a factor per channel along).  A layer may have no feed-forward (then
    it has neither of that sublayer's norms).  The output norms are of a kind that offers `add_normed(residual, y,
    then)`; the norm in front of the feed-forward is handed to the mixer's output norm as `then`, so that one launch
    adds the mixer's result and makes the rows the feed-forward reads; in the same way the block's last output norm
    makes the rows of the NEXT block's first norm where the model hands that norm over (`into_norm`; the next block then
    gets `NormedRows` in place of a delta).  The 32-bit stream is updated in place; nothing is left pending."""

    roles = {"mixer": "mixer", "mixer_norm": "norm", "mixer_out_norm": "norm", "feed_forward": "feed_forward",
             "feed_forward_norm": "norm", "feed_forward_out_norm": "norm"}
    optional_roles = ("feed_forward", "feed_forward_norm", "feed_forward_out_norm")

    def __init__(self, parts):
        super().__init__(parts)
        self.feed_forward = self._parts.get("feed_forward")
        self.feed_forward_norm = self._parts.get("feed_forward_norm")
        self.feed_forward_out_norm = self._parts.get("feed_forward_out_norm")
        present = [p is not None for p in (self.feed_forward, self.feed_forward_norm, self.feed_forward_out_norm)]
        if any(present) != all(present):
            raise ValueError("a block names its feed-forward and that feed-forward's two norms together, or none of them")
        for norm in (self.mixer_out_norm, self.feed_forward_out_norm):
            if norm is not None and not hasattr(norm, "add_normed"):
                raise ValueError("the output norms of this block add into the stream: %s has no add_normed"
                                 % type(norm).__name__)
        # the rows of the second norm come out of the first output norm's launch where that norm is a plain gain
        self._fused_second = self.feed_forward_norm is not None and self._plain_gain(self.feed_forward_norm)

    @staticmethod
    def _plain_gain(norm):
        """Whether an output norm's launch can make this norm's rows: a gain per channel over the root mean square."""
        return hasattr(norm, "weight") and hasattr(norm, "eps") and getattr(norm, "size", None) is not None \
            and not getattr(norm, "has_bias", False) and type(norm).__name__ == "RMSNorm"

    folds_output = True              # forward() takes `into_norm`

    def takes_folded_input(self):
        """The norm whose rows this block takes ready-made (NormedRows) in place of a delta, or None."""
        return self.mixer_norm if self._plain_gain(self.mixer_norm) else None

    def forward(self, residual, delta, step, cache, into_norm=None):
        if isinstance(delta, NormedRows):           # the block before has made this block's first rows
            n = delta.rows
        else:
            n = self.mixer_norm.forward(residual, whole(delta, self.mixer_norm))
        m = self.mixer.forward(n, step, cache)
        if self.feed_forward is None:
            rows = self.mixer_out_norm.add_normed(residual, m, then=into_norm)
            return NormedRows(rows) if into_norm is not None else None
        if self._fused_second:
            n = self.mixer_out_norm.add_normed(residual, m, then=self.feed_forward_norm)
        else:
            self.mixer_out_norm.add_normed(residual, m)
            n = self.feed_forward_norm.forward(residual, None)
        rows = self.feed_forward_out_norm.add_normed(residual, self.feed_forward.forward(n), then=into_norm)
        return NormedRows(rows) if into_norm is not None else None


def whole(delta, norm=None):
    """A mixer or feed-forward may hand on float32 partial sums [parts, T, H] of a K-split product.  A norm
    that says `accepts_partial_sums` adds them up itself; for any other (or for none) they are added up here."""
    if delta is not None and delta.dim() == 3 and not getattr(norm, "accepts_partial_sums", False):
        total = delta.sum(dim=0)
        return total.to(norm.dtype) if norm is not None else total
    return delta


@register_arrangement("parallel_gated")
class ParallelGatedBlock(Arrangement):
    """n = norm(x);  x <- x + (gate1(n) * mixer(n) + gate2(n) * feed_forward(n)): ONE norm, both sublayers read its rows side
    by side, and each result enters the stream through a gate that reads the same rows (a part of the `residual_gate`
    family: `logits(n)`, `add(residual, z, results, then)`).  A layer may have no feed-forward (its gate part then names one
    gate).  Where the gate part can hand its matrix to the mixer (`hand_over`; the mixer has `append_columns`), the gates'
    logits come out of the mixer's own projection: both read the same rows.  The 32-bit stream is updated in place; where the model hands over the norm of the block that runs next
    (`into_norm`), the launch that adds the results also makes that norm's rows (the next block then gets `NormedRows` in
    place of a delta)."""

    roles = {"norm": "norm", "mixer": "mixer", "feed_forward": "feed_forward", "gate": "residual_gate"}
    optional_roles = ("feed_forward",)

    folds_output = True              # forward() takes `into_norm`

    def __init__(self, parts):
        super().__init__(parts)
        self.feed_forward = self._parts.get("feed_forward")
        self._one_product = None
        gates = len(getattr(self.gate, "names", ()))
        if gates != (1 if self.feed_forward is None else 2):
            raise ValueError("a block gates each of its sublayers: %d gates for %d sublayers"
                             % (gates, 1 if self.feed_forward is None else 2))

    def takes_folded_input(self):
        """The norm whose rows this block takes ready-made (NormedRows) in place of a delta, or None."""
        return self.norm if SandwichBlock._plain_gain(self.norm) else None

    def forward(self, residual, delta, step, cache, into_norm=None):
        if isinstance(delta, NormedRows):           # the block before has made this block's rows
            n = delta.rows
        else:
            n = self.norm.forward(residual, whole(delta, self.norm))
        if self._one_product is None:           # once the weights are bound: the gates' matrix behind the mixer's own projection
            hand = getattr(self.gate, "hand_over", None)
            self._one_product = bool(hand is not None and hand(self.mixer))
        if self._one_product:
            results = [self.mixer.forward(n, step, cache)]
            z = self.mixer.extra_columns
        else:
            z = self.gate.logits(n)
            results = [self.mixer.forward(n, step, cache)]
        if self.feed_forward is not None:
            results.append(self.feed_forward.forward(n))
        rows = self.gate.add(residual, z, [whole(r).to(n.dtype) if r.dim() == 3 else r for r in results], then=into_norm)
        return NormedRows(rows) if into_norm is not None else None


@register_arrangement("hyper_prenorm")
class HyperPreNormBlock(Arrangement):
    """A pre-norm block around several residual streams X (float32 [T, S, W]; the model's `stream` part makes them): every
    sublayer reads the norm of a weighted sum of the streams and writes its result back into all of them through its
    connection (a part of the `connection` family: `read(X, norm)`, `write(X, y, then)`), first the mixer, then the
    feed-forward; a layer may have no feed-forward (then neither its norm nor its connection).  The launch that writes a
    sublayer's result also makes the rows that the next sublayer reads: the feed-forward's inside the block, and the next
    block's mixer's where the model hands that block's first connection and norm over (`into_norm`; the next block then
    gets `NormedRows` in place of a delta).  The streams are updated in place; nothing is left pending."""

    roles = {"mixer": "mixer", "mixer_norm": "norm", "mixer_link": "connection", "feed_forward": "feed_forward",
             "feed_forward_norm": "norm", "feed_forward_link": "connection"}
    optional_roles = ("feed_forward", "feed_forward_norm", "feed_forward_link")

    folds_output = True              # forward() takes `into_norm`

    def __init__(self, parts):
        super().__init__(parts)
        self.feed_forward = self._parts.get("feed_forward")
        self.feed_forward_norm = self._parts.get("feed_forward_norm")
        self.feed_forward_link = self._parts.get("feed_forward_link")
        present = [p is not None for p in (self.feed_forward, self.feed_forward_norm, self.feed_forward_link)]
        if any(present) != all(present):
            raise ValueError("a block names its feed-forward, that feed-forward's norm and its connection together, or none of them")
        for norm in (self.mixer_norm, self.feed_forward_norm):
            if norm is not None and not SandwichBlock._plain_gain(norm):
                raise ValueError("the norms of this block are plain gains over the root mean square: %s is not" % type(norm).__name__)

    def takes_folded_input(self):
        """(connection, norm) of the block's first sublayer: the block before can make its rows."""
        return (self.mixer_link, self.mixer_norm)

    def forward(self, residual, delta, step, cache, into_norm=None):
        if residual.dim() != 3:
            raise ValueError("this block runs around several streams [T, S, W]; the model needs a `stream` part")
        if isinstance(delta, NormedRows):
            n = delta.rows
        else:
            if delta is not None:
                raise ValueError("a block around several streams cannot take another block's pending output")
            n = self.mixer_link.read(residual, self.mixer_norm)
        m = self.mixer.forward(n, step, cache)
        if self.feed_forward is None:
            rows = self.mixer_link.write(residual, m, then=into_norm)
            return NormedRows(rows) if into_norm is not None else None
        n = self.mixer_link.write(residual, m, then=(self.feed_forward_link, self.feed_forward_norm))
        rows = self.feed_forward_link.write(residual, self.feed_forward.forward(n), then=into_norm)
        return NormedRows(rows) if into_norm is not None else None
