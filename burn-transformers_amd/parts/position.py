"""Token embedding and position encodings that act at the embedding.

learned_positions: x0[t] = tokens[id[t]] + positions[pos[t]]  (src/models/gpt2/model.rs:447-448);
the table's length bounds a sequence's length.  token_only: x0[t] = scale * tokens[id[t]] (for models
whose position encoding lives in the mixer; ``scale`` defaults to 1; with ``keep_origin`` the rows
are also kept beside the stream, ``stream.origin``, for parts that read the embedding's output again; with
``keep_operand`` a bfloat16 model also gets the rows in the products' type, ``stream.cast``, for layers whose
sublayers multiply by the stream itself).  normalized_tokens: x0[t] = rms_norm(tokens[id[t]]) with
a scale of its own (stored as its distance from ``offset``), for models that normalise the
embedding before the first layer; it also leaves the stream's copy in the products' type.
"""

from ..kernels import library as K
from .base import Embedding, ResidualStream, operand_columns
from .registry import register


@register("embedding", "learned_positions")
class LearnedPositionEmbedding(Embedding):
    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.vocab_size = params["width"], params["vocab_size"]
        self.max_positions = params["max_positions"]
        self.token_table, self.position_table = tensors["tokens"], tensors["positions"]
        if tuple(self.token_table.shape) != (self.vocab_size, self.width) or \
                tuple(self.position_table.shape) != (self.max_positions, self.width):
            raise ValueError("embedding: tables do not have the configured sizes")

    def embed(self, step):
        x = step.buffer("stream.x", step.n_tokens, self.width, "float32")
        K.embed(step.tok_ids, step.tok_pos, self.token_table, self.position_table, x)
        return ResidualStream(x)


@register("embedding", "token_only")
class TokenEmbedding(Embedding):
    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.vocab_size = params["width"], params["vocab_size"]
        self.max_positions = params.get("max_positions", 2 ** 31 - 1)
        self.scale, self.keep_origin = float(params.get("scale", 1.0)), bool(params.get("keep_origin", False))
        # for layers whose sublayers multiply by the stream itself: its rows in the products' type beside it
        self.keep_operand = bool(params.get("keep_operand", False))
        self.token_table = tensors["tokens"]
        if tuple(self.token_table.shape) != (self.vocab_size, self.width):
            raise ValueError("embedding: the table does not have the configured sizes")

    def embed(self, step):
        x = step.buffer("stream.x", step.n_tokens, self.width, "float32")
        origin = step.buffer("stream.origin", step.n_tokens, self.width, "float32") if self.keep_origin else None
        cast = None
        if self.keep_operand and step.dtype != x.dtype:
            cast = step.buffer("stream.operand", step.n_tokens, operand_columns(self.width, step.dtype), step.dtype)
        K.embed(step.tok_ids, None, self.token_table, None, x, scale=self.scale, copy=origin, cast=cast)
        stream = ResidualStream(x)
        stream.origin, stream.cast = origin, cast
        return stream


@register("embedding", "normalized_tokens")
class NormalizedTokenEmbedding(Embedding):
    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.vocab_size = params["width"], params["vocab_size"]
        self.max_positions = params.get("max_positions", 2 ** 31 - 1)
        self.eps = float(params["eps"])
        self.token_table = tensors["tokens"]
        self.scale = (tensors["norm_weight"].float() + float(params.get("offset", 0.0))).contiguous()
        if tuple(self.token_table.shape) != (self.vocab_size, self.width) or tuple(self.scale.shape) != (self.width,):
            raise ValueError("embedding: table or scale do not have the configured sizes")
        if self.token_table.dtype != self.scale.dtype and self.width % 8 != 0:
            # the layers multiply by the stream's bfloat16 copy, whose rows the MFMA kernels read 16 bytes at a time
            raise ValueError(f"embedding: the bfloat16 kernels take widths that are multiples of 8, not {self.width}; "
                             f"load the model with dtype float32, which takes any width")

    def embed(self, step):
        x = step.buffer("stream.x", step.n_tokens, self.width, "float32")
        K.embed(step.tok_ids, None, self.token_table, None, x)
        stream = ResidualStream(x)
        if step.dtype != x.dtype:
            stream.cast = step.buffer("stream.operand", step.n_tokens, operand_columns(self.width, step.dtype), step.dtype)
        K.output_norm(x, self.scale, self.eps, 1.0, accumulate=False, cast=stream.cast)
        return stream
