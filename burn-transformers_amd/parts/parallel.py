"""Two mixers side by side: both read the same rows, and the layer's mixer output is
left_scale * left(h) + right_scale * right(h).

parallel_mixers: parameters left and right ({"kind": a registered mixer, "params": its parameters}),
left_scale, right_scale.  Tensors: the two mixers' own, with their roles prefixed ``left.`` and ``right.``.

A layer's run has one cache entry, so at most one of the two keeps keys and values and at most one a state of
fixed size; each gets the entry's memory and takes from it what it keeps.  The two outputs stay apart as
32-bit partial sums and meet, with their factors, in the norm of the sublayer's output (a ``Delta`` with a
second term), so the sum costs no kernel of its own; the arrangement therefore belongs in blocks that normalise
what a sublayer adds.
"""

from .base import Delta, Mixer, SublayerOutput
from .registry import lookup, register


@register("mixer", "parallel_mixers")
class ParallelMixers(Mixer):
    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.sides = []
        for side in ("left", "right"):
            spec = params[side]
            own = {role[len(side) + 1:]: tensor for role, tensor in tensors.items() if role.startswith(side + ".")}
            mixer = lookup("mixer", spec["kind"])(spec["params"], own)
            self.sides.append((side, mixer, float(params[side + "_scale"])))
        mixers = [mixer for _, mixer, _ in self.sides]
        if sum(m.kv_spec() is not None for m in mixers) > 1 or sum(m.state_spec() is not None for m in mixers) > 1:
            raise ValueError("parallel mixers: a layer's run has one cache entry; two mixers that both keep keys and "
                             "values, or both a state, do not fit side by side")
        self.only_launches_kernels = all(m.only_launches_kernels for m in mixers)
        self.graph_safe = all(m.graph_safe for m in mixers)

    def kv_spec(self):
        return next((m.kv_spec() for _, m, _ in self.sides if m.kv_spec() is not None), None)

    def state_spec(self):
        return next((m.state_spec() for _, m, _ in self.sides if m.state_spec() is not None), None)

    def kernel_modules(self, dtype):
        return tuple(name for _, m, _ in self.sides for name in m.kernel_modules(dtype))

    def ride_along(self, weight, bias=None):
        for _, mixer, _ in self.sides:
            rider = mixer.ride_along(weight, bias)
            if rider is not None:
                return rider
        return None

    def forward(self, h, step, memory, stream):
        terms = []
        for side, mixer, scale in self.sides:
            output = SublayerOutput(key=f"parallel.{side}.partials")
            delta = mixer.forward(h, step, memory, output)
            delta = delta if delta is not None else output.take()
            if not delta.plain:
                raise ValueError("parallel mixers: a side's output is itself a weighted sum")
            terms.append(Delta(delta.partials, delta.bias, scale))
        return Delta(terms[0].partials, terms[0].bias, terms[0].scale, other=terms[1])
