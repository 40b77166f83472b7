"""Readout: logits = h . table^T in float32, no bias; the table is [vocab, width] and may be
the token table itself (src/models/gpt2/model.rs:500-513, src/operations.rs:675-728).  Parameter
``soft_cap`` (default none): logits <- cap * tanh(logits / cap), in 32-bit."""

from ..kernels import library as K
from .base import Readout, operand_columns, pad_columns
from .registry import register


@register("readout", "linear_readout")
class LinearReadout(Readout):
    only_launches_kernels = True
    takes_deferred_norm = True       # the rows are only handed to ``gemm``: the final norm may leave them chunk-major

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.vocab_size = params["width"], params["vocab_size"]
        self.weight = tensors["weight"]
        self.soft_cap = float(params.get("soft_cap") or 0.0)
        if self.soft_cap < 0.0 or self.soft_cap != self.soft_cap:
            raise ValueError(f"readout: the logits' cap {self.soft_cap} must be positive")
        if tuple(self.weight.shape) != (self.vocab_size, self.width):
            raise ValueError(f"readout: table is {tuple(self.weight.shape)}, expected "
                             f"{(self.vocab_size, self.width)}")
        # a second copy for steps of few rows, which read the table and little else (the token
        # embedding looks rows up in the table as it is stored)
        # (rows that a bfloat16 product reads 16 bytes at a time: a width that is no multiple of that gets zero columns,
        # which meet the zero columns behind the normalised rows)
        self.matrix = pad_columns(self.weight, operand_columns(self.width, self.weight.dtype))
        self.packed = K.PackedWeight(self.matrix) if self.weight.is_cuda else None

    def logits(self, h, step):
        out = step.buffer("readout.logits", h.shape[0], self.vocab_size, "float32")
        K.gemm(h, self.matrix, K.epilogue_f32(out), packed=self.packed)
        if self.soft_cap:
            K.soft_cap(out, self.soft_cap)
        return out
