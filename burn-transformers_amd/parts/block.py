"""Arrangements of parts in a layer.

pre_norm: y = x + mixer(norm(x)); z = y + feed_forward(norm(y)), the feed-forward optional
(src/models/gpt2/model.rs:218-270).  A part adds its contribution to the stream itself or
returns it as a Delta, which stays pending until the next norm reads the stream.

output_norm: y = x + m * norm(mixer(x)); z = y + m * norm(feed_forward(y)), the feed-forward
optional.  The parts read the stream itself; what is normalised is what they add.  ``m`` is the
block's parameter ``mult``.  With gates (``mixer_gate``, ``ff_gate``: parts of role "gate") a sublayer's
output is multiplied, element by element, by sigmoid(gate(x)) before it is normalised: a gated residual.

sandwich_norm: y = x + post(mixer(pre(x))); z = y + post'(feed_forward(pre'(y))), the feed-forward
optional: a norm before AND behind every sublayer, four norms a layer with tensors of their own.

transform: x = t(x), one part of role "transform" and nothing else: what stands between two runs of
layers (it keeps nothing in the cache; its schedule entry names no cache entry).
"""

from .base import Block, SublayerOutput, Transform, offers_chunked
from .registry import register

# Most rows of a step whose first norm is folded too.  Measured at GPT-2 XL sizes, ms a decode step
# without / with it: 1.87 / 1.81 at one row, 1.89 / 1.84 at two, 1.96 / 1.94 at four, 2.14 / 2.23 at
# eight (there the feed-forward's second product misses its split of K more than the norm costs).
# With the limit at eight rows instead, ms a step of eight rows at widths 768 / 1,024 / 1,600 (12, 24
# and 12 layers): 0.395 -> 0.388, 0.781 -> 0.785, 0.531 -> 0.546; so four at every width.
MIXER_FOLD_ROWS = 4


@register("block", "pre_norm")
class PreNormBlock(Block):
    ROLES = {"mixer_norm": "norm", "mixer": "mixer", "ff_norm": "norm", "ff": "feed_forward"}
    OPTIONAL = ("ff_norm", "ff")
    only_launches_kernels = True

    def __init__(self, parts, params=None):
        super().__init__(parts, params)
        if ("ff" in parts) != ("ff_norm" in parts):
            raise ValueError("pre_norm block: a feed-forward and its norm come together")

    def forward(self, stream, step, memory):
        parts = self.parts
        mixer, mixer_norm = parts["mixer"], parts["mixer_norm"]
        rows = stream.x.shape[0]
        if "ff" not in parts:             # a layer that is its mixer alone
            h = _apply(mixer_norm, stream, step, mixer.takes_deferred_norm)
            delta = mixer.forward(h, step, memory, stream)
            if delta is not None:
                stream.add(delta)
            return
        ff, ff_norm = parts["ff"], parts["ff_norm"]
        # In a small decode step a norm can be folded into the product that follows it (one kernel
        # fewer) if the part before it leaves its output in the stream itself instead of pending
        # partial sums.  For the second norm that costs the attention output its split of K, which is
        # cheap; for the first norm it costs the feed-forward's second product its split, which pays
        # only for the very smallest steps (MIXER_FOLD_ROWS).
        fold_ff = ff.takes_deferred_norm and _can_defer(ff_norm, step, rows)
        fold_mixer = mixer.takes_deferred_norm and rows <= MIXER_FOLD_ROWS and _can_defer(mixer_norm, step, rows)
        h = mixer_norm.deferred(stream, step) if fold_mixer else None
        if h is None:
            h = _apply(mixer_norm, stream, step, mixer.takes_deferred_norm)
        stream.in_place = fold_ff
        delta = mixer.forward(h, step, memory, stream)
        stream.in_place = False
        if delta is not None:
            stream.add(delta)
        h = ff_norm.deferred(stream, step) if fold_ff else None
        if h is None:
            h = _apply(ff_norm, stream, step, ff.takes_deferred_norm)
        stream.in_place = fold_mixer          # for the next layer's first norm (or the final one, which does not mind)
        delta = ff.forward(h, step, stream)
        stream.in_place = False
        if delta is not None:
            stream.add(delta)


def _apply(norm, stream, step, only_multiplied):
    """The normalised rows; for a part that only hands them to ``gemm``, in the chunk-major layout
    if the norm offers it (the norm decides by the number of rows)."""
    if only_multiplied and offers_chunked(norm):
        return norm.apply(stream, step, chunked=True)
    return norm.apply(stream, step)


def _can_defer(norm, step, rows):
    possible = getattr(norm, "deferred_possible", None)
    return possible is not None and possible(step, rows)


@register("block", "output_norm")
class OutputNormBlock(Block):
    """Sublayers that read the residual stream as it is and whose outputs are normalised (and scaled
    by ``mult``) before they join it.  The norms are of a kind with ``add_output`` (rms_norm).  A
    layer without a feed-forward leaves ``ff`` and ``ff_norm`` out."""
    ROLES = {"mixer": "mixer", "mixer_norm": "norm", "ff": "feed_forward", "ff_norm": "norm",
             "mixer_gate": "gate", "ff_gate": "gate"}
    OPTIONAL = ("ff", "ff_norm", "mixer_gate", "ff_gate")
    only_launches_kernels = True

    def __init__(self, parts, params=None):
        super().__init__(parts, params)
        self.mult = float(self.params.get("mult", 1.0))
        if ("ff" in parts) != ("ff_norm" in parts):
            raise ValueError("output_norm block: a feed-forward and its norm come together")
        if "ff_gate" in parts and "ff" not in parts:
            raise ValueError("output_norm block: a gate on a feed-forward that is not there")
        for gate, norm in (("mixer_gate", "mixer_norm"), ("ff_gate", "ff_norm")):
            if gate in parts and not getattr(parts[norm], "takes_weighted_output", False):
                raise ValueError(f"output_norm block: {type(parts[norm]).__name__} takes no gate on what it normalises")
        for name in ("mixer_norm", "ff_norm"):
            if name in parts and not hasattr(parts[name], "add_output"):
                raise ValueError(f"output_norm block: {type(parts[name]).__name__} cannot normalise a sublayer's output")
        # a gate reads what its sublayer reads: where the mixer's first product can take the gate's rows along, it does
        self.mixer_rider = None
        gate = parts.get("mixer_gate")
        if gate is not None and hasattr(gate, "stored") and hasattr(gate, "handed_over"):
            self.mixer_rider = parts["mixer"].ride_along(gate.stored, gate.bias)
            if self.mixer_rider is not None:
                gate.handed_over()

    def forward(self, stream, step, memory):
        parts = self.parts
        output = SublayerOutput()
        h = stream.operand(step)
        gate = {}
        if "mixer_gate" in parts and self.mixer_rider is None:
            gate = {"gate": parts["mixer_gate"].logits(h, step, "block.gate")}
        delta = parts["mixer"].forward(h, step, memory, output)
        if self.mixer_rider is not None:
            gate = {"gate": self.mixer_rider(step)}
        parts["mixer_norm"].add_output(stream, step, delta if delta is not None else output.take(), self.mult, **gate)
        if "ff" in parts:
            h = stream.operand(step)
            gate = {"gate": parts["ff_gate"].logits(h, step, "block.gate")} if "ff_gate" in parts else {}
            delta = parts["ff"].forward(h, step, output)
            parts["ff_norm"].add_output(stream, step, delta if delta is not None else output.take(), self.mult, **gate)


@register("block", "sandwich_norm")
class SandwichNormBlock(Block):
    """A norm before and a norm behind each sublayer: the sublayer reads a norm of the stream, and
    its output is normalised again before it joins the stream.  The norms behind are of a kind with
    ``add_output`` (layer_norm, rms_norm).  A layer without a feed-forward leaves ``ff`` and its two
    norms out."""
    ROLES = {"mixer_norm": "norm", "mixer": "mixer", "mixer_post": "norm",
             "ff_norm": "norm", "ff": "feed_forward", "ff_post": "norm"}
    OPTIONAL = ("ff_norm", "ff", "ff_post")
    only_launches_kernels = True

    def __init__(self, parts, params=None):
        super().__init__(parts, params)
        if len({name in parts for name in ("ff_norm", "ff", "ff_post")}) != 1:
            raise ValueError("sandwich_norm block: a feed-forward and its two norms come together")
        for name in ("mixer_post", "ff_post"):
            if name in parts and not hasattr(parts[name], "add_output"):
                raise ValueError(f"sandwich_norm block: {type(parts[name]).__name__} cannot normalise a sublayer's output")

    def forward(self, stream, step, memory):
        parts = self.parts
        output = SublayerOutput()
        mixer = parts["mixer"]
        h = _apply(parts["mixer_norm"], stream, step, mixer.takes_deferred_norm)
        delta = mixer.forward(h, step, memory, output)
        # what a sublayer adds is normalised by the kernel that normalises the stream for the next one
        stream.defer_output(parts["mixer_post"], step, delta if delta is not None else output.take())
        if "ff" in parts:
            ff = parts["ff"]
            h = _apply(parts["ff_norm"], stream, step, ff.takes_deferred_norm)
            delta = ff.forward(h, step, output)
            stream.defer_output(parts["ff_post"], step, delta if delta is not None else output.take())


@register("block", "transform")
class TransformBlock(Block):
    """One part that replaces the stream's rows; no mixer, nothing in the cache."""
    ROLES = {"transform": "transform"}
    only_launches_kernels = True

    def __init__(self, parts, params=None):
        super().__init__(parts, params)
        if not isinstance(parts["transform"], Transform):
            raise ValueError(f"transform block: {type(parts['transform']).__name__} is no transform")

    def forward(self, stream, step, memory):
        self.parts["transform"].forward(stream, step)
