"""Normalisations over the channel axis, with 32-bit statistics in both precisions.

layer_norm: y = (x - mean) / sqrt(var + eps) * weight + bias, var the population variance
            (src/models/gpt2/model.rs:8, 143-148).
rms_norm:   y = x / sqrt(mean(x^2) + eps) * weight   (src/normalization.rs:158-171).

Parameter ``offset`` (default 0): the scale is stored as its distance from ``offset`` and the norm
multiplies by offset + weight (1 for scales stored around zero); the sum is formed once, in
float32, when the part is built.

Parameter ``gain`` (default 1): scale and shift are multiplied by it once, in float32, when the part
is built (a model that scales what it reads off the normalised rows, its logits for one, states
the factor here).

Parameter ``groups`` (default 1, rms_norm only): the row is split into that many equal consecutive parts,
each divided by its own root mean square; the scale still has one entry a column.

``apply`` first adds what is pending on the residual stream, in the same pass.  ``add_output`` is
the norm of a sublayer's OUTPUT: x += mult * norm(output), for layers that normalise what they add
to the stream (with or without a norm of the sublayer's input as well).
"""

from ..kernels import library as K
from .base import Norm, operand_columns
from .registry import register


class _KernelNorm(Norm):
    KIND = None
    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.eps = params["width"], float(params["eps"])
        self.weight, self.bias = tensors["weight"], tensors.get("bias")
        if tuple(self.weight.shape) != (self.width,):
            raise ValueError(f"{self.KIND}: scale is {tuple(self.weight.shape)}, expected {(self.width,)}")
        self.offset = float(params.get("offset", 0.0))
        if self.offset:
            self.weight = (self.weight.float() + self.offset).contiguous()
        self.groups = int(params.get("groups") or 1)
        if self.groups != 1 and (self.KIND != "rms_norm" or self.groups < 1 or self.width % self.groups != 0):
            raise ValueError(f"{self.KIND}: {self.groups} parts of a row of {self.width}: only an RMS norm is taken in "
                             f"parts, and they must divide the width")
        gain = float(params.get("gain", 1.0))
        if gain != 1.0:
            self.weight = (self.weight.float() * gain).contiguous()
            self.bias = (self.bias.float() * gain).contiguous() if self.bias is not None else None

    def apply(self, stream, step, rows=None, chunked=False):
        count = rows.numel() if rows is not None else stream.x.shape[0]
        if self.groups > 1 or (self.KIND == "rms_norm" and operand_columns(self.width, step.dtype) != self.width):
            # (also rows that a product reads 16 bytes at a time and that are no multiple of that long: zeros behind them)
            stream.flush()
            out = step.buffer("norm.out" if rows is None else "norm.selected", count, operand_columns(self.width, step.dtype),
                              step.dtype)
            K.group_norm_rows(stream.x, self.weight, self.groups, self.eps, out, rows=rows)
            return out
        if chunked and K.Chunked.wanted(count) and self.width % 4 == 0:
            out = K.Chunked.take(step, "norm.out" if rows is None else "norm.selected", count, self.width, step.dtype)     # for a part that only hands it to `gemm`
        else:
            out = step.buffer("norm.out" if rows is None else "norm.selected", count, self.width, step.dtype)
        if stream.pending_output is not None:
            if rows is None and not isinstance(out, K.Chunked):
                # the norm of the last sublayer's output is still to join the stream: one kernel for both
                post, post_step, delta, mult = stream.take_pending_output()
                post.add_output(stream, post_step, delta, mult, keep_operand=False,
                                then=(self.KIND, self.weight, self.bias, self.eps, out))
                return out
            stream.flush()
        pending = stream.pending
        K.add_norm(stream.x, out, self.weight, self.bias, self.eps, self.KIND,
                   delta=pending.partials if pending else None, bias=pending.bias if pending else None,
                   rows=rows, write_back=rows is None)
        if rows is None:
            stream.pending = None
        return out

    def deferred_possible(self, step, rows):
        return self.groups == 1 and step.dtype_is_bf16 and self.width % 8 == 0 and K.Normalized.worth_it(rows, self.width)

    def deferred(self, stream, step):
        if stream.pending is not None or stream.pending_output is not None or \
                not self.deferred_possible(step, stream.x.shape[0]):
            return None
        return K.Normalized(stream.x, self.weight, self.bias, self.eps, self.KIND)


    @property
    def takes_weighted_output(self):
        """Whether ``add_output`` takes a gate and a ``Delta`` of two weighted terms."""
        return self.KIND == "rms_norm"

    def add_output(self, stream, step, delta, mult=1.0, accumulate=True, keep_operand=True, then=None, gate=None):
        """x (+)= mult * norm(v), v = the sublayer's output ``delta`` (a ``Delta``; None: the stream's
        own rows, normalised in place).  ``gate``: float32 logits [tokens, width]; v is multiplied by their
        sigmoid first.  In a bfloat16 model the new rows are also left as the
        stream's copy in the products' type (``stream.operand``) unless ``keep_operand`` is False
        (layers whose sublayers read a norm of the stream have no use for it).  ``then``: the norm
        that reads the stream next, computed in the same pass (``kernels.library.output_norm``)."""
        if stream.pending is not None or stream.pending_output is not None:
            stream.flush()
        cast = None
        if keep_operand and step.dtype != stream.x.dtype:
            cast = step.buffer("stream.operand", stream.x.shape[0], operand_columns(self.width, step.dtype), step.dtype)
        if self.groups > 1 or gate is not None or (delta is not None and not delta.plain):
            if not self.takes_weighted_output or delta is None or then is not None:
                raise ValueError(f"{self.KIND}: a gate, parts of the row or a weighted sum of two outputs go with an RMS "
                                 f"norm of a sublayer's output, and the norm that follows runs on its own")
            other = delta.other
            if other is not None and other.other is not None:
                raise ValueError("a sublayer's output has at most two terms")
            K.group_norm_output(stream.x, self.weight, self.groups, self.eps, delta.partials, delta.bias, delta.scale,
                                other.partials if other else None, other.bias if other else None,
                                other.scale if other else 1.0, gate=gate, mult=mult, accumulate=accumulate, cast=cast)
            stream.cast = cast
            return
        K.output_norm(stream.x, self.weight, self.eps, mult, delta=delta.partials if delta is not None else None,
                      bias=delta.bias if delta is not None else None, accumulate=accumulate, cast=cast,
                      kind=self.KIND, beta=self.bias, then=then)
        stream.cast = cast


@register("norm", "layer_norm")
class LayerNorm(_KernelNorm):
    KIND = "layer_norm"


@register("norm", "rms_norm")
class RMSNorm(_KernelNorm):
    KIND = "rms_norm"
