"""Gates on a sublayer's output: logits = W h + b from what the sublayer reads; the norm of the output
multiplies by their sigmoid (``parts.block.OutputNormBlock``, roles ``mixer_gate`` / ``ff_gate``).

sigmoid_projection: parameters width (of h) and out (of the output; default width).  Tensors: weight
[out, width], bias [out] (optional).  The logits are 32-bit sums.  Where the sublayer starts with a product of
the same rows that leaves 32-bit sums, the block lets the gate's rows ride in it (``Mixer.ride_along``).
"""

from ..kernels import library as K
from .base import Gate, operand_columns, pad_columns
from .registry import register


@register("gate", "sigmoid_projection")
class SigmoidProjection(Gate):
    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width = params["width"]
        self.out = params.get("out", self.width)
        weight, self.bias = tensors["weight"], tensors.get("bias")
        if tuple(weight.shape) != (self.out, self.width) or (self.bias is not None and tuple(self.bias.shape) != (self.out,)):
            raise ValueError(f"sigmoid_projection: weight {tuple(weight.shape)}, expected {(self.out, self.width)} with a bias of {(self.out,)}")
        self.stored = weight
        self.weight = pad_columns(weight, operand_columns(self.width, weight.dtype))
        self.packed = K.PackedWeight(self.weight) if self.weight.is_cuda else None

    def handed_over(self):
        """The projection rides in another part's product (``Mixer.ride_along``): the copies for a product of its own go."""
        self.weight = self.packed = None

    def logits(self, h, step, key):
        out = step.buffer(key, h.shape[0], self.out, "float32")
        K.gemm(h, self.weight, K.epilogue_f32(out, self.bias), packed=self.packed)
        return out
