"""Dense feed-forward: down(act(up(x)))  (src/feed_forward.rs:111-114).

Parameters: width, inner, activation ("gelu_tanh": 0.5x(1+tanh(sqrt(2/pi)(x+0.044715x^3))),
"gelu_erf": x(1+erf(x/sqrt 2))/2; src/feed_forward.rs:351-387).  The activation runs in 32-bit
inside the up projection's epilogue (src/feed_forward.rs:397-406 widens half inputs too); the
down projection adds into the residual stream.

"poly_norm" is an activation that is a norm: a N(z) + b N(z^2) + c N(z^3) + e with powers taken
element by element and N(v) = v / sqrt(mean(v^2) + eps) over a token's whole inner vector; the four
numbers are the tensor ``act_coefficients``, ``eps`` a parameter.  It needs a whole row, so the up
projection leaves 32-bit sums and a kernel of its own applies it.

gated_dense: down(silu(gate x) * (up x)), no biases.  Parameters width, inner; tensors gate_weight and
up_weight [inner, width], down_weight [width, inner].  ONE product with the two matrices laid one behind the
other, the kernel of the routed experts' units for the single unit every token uses, and the down product.

The MFMA kernels read operands 16 bytes at a time, so an inner width that is no multiple of 8 is
padded once, when the part is built: zero rows (and zero bias) in the up projection give
act(0) = 0 in the padded columns, which meet zero columns of the down projection.
"""

import torch

from ..kernels import library as K
from .base import FeedForward, operand_columns, packed_for_stream, pad_columns, pad_rows
from .registry import register


@register("feed_forward", "dense")
class DenseFeedForward(FeedForward):
    takes_deferred_norm = True
    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.inner, self.activation = params["width"], params["inner"], params["activation"]
        if self.activation not in K.ACTIVATIONS and self.activation != "poly_norm":
            raise ValueError(f"feed-forward: unknown activation {self.activation!r}")
        if self.activation == "poly_norm":
            self.coefficients, self.eps = tensors["act_coefficients"], float(params["eps"])
            if tuple(self.coefficients.shape) != (4,):
                raise ValueError(f"feed-forward: poly_norm takes four numbers, got {tuple(self.coefficients.shape)}")
        self.up_weight, self.up_bias = tensors["up_weight"], tensors.get("up_bias")
        self.down_weight, self.down_bias = tensors["down_weight"], tensors.get("down_bias")
        if tuple(self.up_weight.shape) != (self.inner, self.width) or \
                tuple(self.down_weight.shape) != (self.width, self.inner):
            raise ValueError(f"feed-forward: projections are {tuple(self.up_weight.shape)} and "
                             f"{tuple(self.down_weight.shape)}, expected {(self.inner, self.width)} and "
                             f"{(self.width, self.inner)}")
        self.padded = (self.inner + 7) // 8 * 8
        extra = self.padded - self.inner
        if extra:
            up, down = self.up_weight, self.down_weight
            self.up_weight = torch.cat([up, up.new_zeros(extra, self.width)]).contiguous()
            self.down_weight = torch.cat([down, down.new_zeros(self.width, extra)], dim=1).contiguous()
            if self.up_bias is not None:
                self.up_bias = torch.cat([self.up_bias, self.up_bias.new_zeros(extra)]).contiguous()

        # second copies for decode steps, which read the weights and little else
        self.up_packed = K.PackedWeight(self.up_weight) if self.up_weight.is_cuda else None
        self.down_packed = packed_for_stream(self.down_weight) if self.down_weight.is_cuda else None

    def forward(self, h, step, stream):
        tokens = h.shape[0]
        if self.activation == "poly_norm":
            z = step.buffer("feed_forward.sums", tokens, self.padded, "float32")
            hidden = step.buffer("feed_forward.hidden", tokens, self.padded, step.dtype)
            K.gemm(h, self.up_weight, K.epilogue_f32(z, self.up_bias), packed=self.up_packed)
            K.poly_norm(z, self.inner, self.coefficients, self.eps, hidden)
            stream.add_product(step, hidden, self.down_weight, self.down_bias, packed=self.down_packed)
            return
        if K.Chunked.wanted(tokens) and (step.dtype_is_bf16 or self.padded % 4 == 0):
            hidden = K.Chunked.take(step, "feed_forward.hidden", tokens, self.padded, step.dtype)   # read by the next product only
        else:
            hidden = step.buffer("feed_forward.hidden", tokens, self.padded, step.dtype)
        K.gemm(h, self.up_weight, K.epilogue_act(hidden, self.activation, self.up_bias), packed=self.up_packed)
        stream.add_product(step, hidden, self.down_weight, self.down_bias, packed=self.down_packed)


@register("feed_forward", "gated_dense")
class GatedDenseFeedForward(FeedForward):
    takes_deferred_norm = False
    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.inner = params["width"], params["inner"]
        gate, up, down = tensors["gate_weight"], tensors["up_weight"], tensors["down_weight"]
        if tuple(gate.shape) != (self.inner, self.width) or tuple(up.shape) != (self.inner, self.width) or \
                tuple(down.shape) != (self.width, self.inner):
            raise ValueError(f"gated feed-forward: projections {tuple(gate.shape)}, {tuple(up.shape)}, {tuple(down.shape)} do "
                             f"not fit width {self.width} and inner width {self.inner}")
        dtype = gate.dtype
        columns = operand_columns(self.width, dtype)
        self.hidden_cols = operand_columns(self.inner, dtype)
        self.fused_cols = operand_columns(2 * self.inner, dtype)
        self.in_weight = pad_columns(pad_rows(torch.cat([gate, up]), self.fused_cols), columns)
        self.down_weight = pad_columns(down, self.hidden_cols)
        self.in_packed = K.PackedWeight(self.in_weight) if self.in_weight.is_cuda else None
        self.down_packed = packed_for_stream(self.down_weight) if self.down_weight.is_cuda else None

    def kernel_modules(self, dtype):
        return ("experts",)

    def forward(self, h, step, stream):
        tokens = h.shape[0]
        fused = step.buffer("feed_forward.fused", tokens, self.fused_cols, step.dtype)
        K.gemm(h, self.in_weight, K.epilogue_store(fused), packed=self.in_packed)
        hidden = step.buffer("feed_forward.hidden", tokens, self.hidden_cols, step.dtype)
        K.gated_experts(fused, None, None, 0, 1, self.inner, 0, hidden)
        stream.add_product(step, hidden, self.down_weight, packed=self.down_packed)
