"""Routed feed-forward: a mixture of gated experts, with optional identity experts and an expert
that every token uses.

Parameters: width, experts (experts with tensors), ff (an expert's inner width), identity (experts
without tensors whose output is their input; they are the LAST router outputs), top (experts a
token uses), groups / keep (the experts, identity experts included, form ``groups`` equal groups of
neighbours, and only experts of the ``keep`` groups with the best score can be chosen; groups <= 1:
all can), shared_ff (inner width of the expert every token uses; 0: none), score ("softmax", the default,
or "sigmoid": each router logit's own sigmoid), group_rank (a group's score is the sum of its so many best
scores; default 1, its best), normalize (default true; false: the weights are the chosen experts' scores as
they are), limit and alpha (with a limit an expert's unit is g' * sigmoid(alpha g') * (u' + 1) with
g' = min(gate h, limit), u' = clamp(up h, -limit, limit), instead of silu(gate h) * (up h)), unit ("gated", the
default; "gelu_erf" or "silu": experts WITHOUT a gate, down(act(up h)), act the exact (erf) GELU or the SiLU; such
experts have no ``gate_<e>`` / ``shared_gate`` tensors).
Tensors: router [experts + identity, width] and correction [experts + identity] in float32, per
expert gate / up [ff, width] and down [width, ff] (``gate_<e>``, ``up_<e>``, ``down_<e>``), and for the
shared expert shared_gate / shared_up / shared_down and, optionally, shared_mix [1, width] (without it the shared
expert's output is added as it is).

    z = router . h (32-bit), s = softmax(z) over all router outputs
    chosen = the ``top`` largest of s + correction among the open groups (a group's score is its
             largest s + correction); weights = s[chosen] / (sum of s[chosen] + 1e-20)
    out = sum over chosen e of weights_e * expert_e(h), expert(h) = down (silu(gate h) * (up h)),
          an identity expert's output being h itself,
        + sigmoid(shared_mix . h) * shared(h)

How a step computes it: ONE product with every expert's gate and up matrices laid one behind the
other (the shared expert's last), a kernel that applies silu(gate) * up times the token's weight of
that expert (zero where it was not chosen, the sigmoid gate for the shared expert), and ONE product
with the down matrices laid side by side, which so sums the weighted outputs.  No token is moved
and nothing depends on the host knowing the choice, so the step is a fixed list of kernels like
every other; the price is that every expert multiplies every token.  In decode steps that costs
little once tokens * top reaches the number of experts (all matrices are read anyway); a prompt does
experts / top times the routed arithmetic, which a grouped product over tokens sorted by expert
would save.
"""

import torch

from ..kernels import library as K
from .base import Delta, FeedForward, operand_columns, packed_for_stream, pad_columns, pad_rows, stream_product_splits
from .registry import register


@register("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    takes_deferred_norm = False          # the router reads the rows themselves
    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        p = params
        self.width, self.experts, self.ff = p["width"], p["experts"], p["ff"]
        self.identity, self.top = int(p.get("identity") or 0), p["top"]
        self.groups, self.keep = int(p.get("groups") or 1), int(p.get("keep") or 1)
        self.shared_ff = int(p.get("shared_ff") or 0)
        self.score, self.group_rank = p.get("score", "softmax"), int(p.get("group_rank") or 1)
        self.normalize = bool(p.get("normalize", True))
        self.limit = float(p["limit"]) if p.get("limit") is not None else None
        self.alpha = float(p.get("alpha", 1.0))
        self.unit = p.get("unit", "gated")
        if self.unit not in ("gated", "gelu_erf", "silu"):
            raise ValueError(f"routed experts: unknown unit {self.unit!r}")
        if self.unit != "gated" and self.limit is not None:
            raise ValueError("routed experts: the clamped unit has a gate")
        self.gated = self.unit == "gated"
        if self.score not in ("softmax", "sigmoid"):
            raise ValueError(f"routed experts: unknown score {self.score!r}")
        if self.limit is not None and not self.limit > 0.0:
            raise ValueError(f"routed experts: the limit {self.limit} must be positive")
        self.outputs = self.experts + self.identity
        if not (0 < self.top <= self.outputs):
            raise ValueError(f"routed experts: {self.top} of {self.outputs} experts a token")
        if self.groups > 1 and (self.outputs % self.groups != 0 or not (0 < self.keep <= self.groups)
                                or self.keep * (self.outputs // self.groups) < self.top):
            raise ValueError(f"routed experts: {self.groups} groups of which {self.keep} stay open do not fit "
                             f"{self.outputs} experts of which a token uses {self.top}")
        self.router, self.correction = tensors["router"], tensors.get("correction")
        if tuple(self.router.shape) != (self.outputs, self.width) or self.router.dtype != torch.float32:
            raise ValueError(f"routed experts: the router is {tuple(self.router.shape)} {self.router.dtype}, expected "
                             f"{(self.outputs, self.width)} in float32")
        rows, columns = [], []
        for e in range(self.experts):
            up, down = tensors[f"up_{e}"], tensors[f"down_{e}"]
            gate = tensors[f"gate_{e}"] if self.gated else up
            if tuple(gate.shape) != (self.ff, self.width) or tuple(up.shape) != (self.ff, self.width) or \
                    tuple(down.shape) != (self.width, self.ff):
                raise ValueError(f"routed experts: expert {e}'s matrices do not have the configured sizes")
            rows += [gate, up] if self.gated else [up]
            columns.append(down)
        self.shared_mix = None
        if self.shared_ff:
            up, down = tensors["shared_up"], tensors["shared_down"]
            gate = tensors["shared_gate"] if self.gated else up
            if tuple(gate.shape) != (self.shared_ff, self.width) or tuple(up.shape) != (self.shared_ff, self.width) or \
                    tuple(down.shape) != (self.width, self.shared_ff):
                raise ValueError("routed experts: the shared expert's matrices do not have the configured sizes")
            rows += [gate, up] if self.gated else [up]
            columns.append(down)
            if "shared_mix" in tensors:
                self.shared_mix = tensors["shared_mix"].reshape(-1).contiguous()
                if tuple(self.shared_mix.shape) != (self.width,) or self.shared_mix.dtype != torch.float32:
                    raise ValueError("routed experts: the shared expert's gate is one float32 row of the model's width")
        if not rows:
            raise ValueError("routed experts: no expert has tensors")
        dtype = rows[0].dtype
        self.inner = self.experts * self.ff + self.shared_ff
        self.hidden_cols = operand_columns(self.inner, dtype)
        self.fused_cols = operand_columns((2 if self.gated else 1) * self.inner, dtype)      # (rows of the fused product's output start where 16-byte stores may)
        # [2 * inner, or inner without gates (+ zero rows), width (+ zero columns, where the rows it multiplies carry them)]
        self.in_weight = pad_columns(pad_rows(torch.cat(rows), self.fused_cols), operand_columns(self.width, dtype))
        self.down_weight = pad_columns(torch.cat(columns, dim=1), self.hidden_cols)           # [width, inner (+ zeros)]
        on_gpu = self.in_weight.is_cuda
        self.in_packed = K.PackedWeight(self.in_weight) if on_gpu else None
        self.down_packed = packed_for_stream(self.down_weight) if on_gpu else None

    def kernel_modules(self, dtype):
        return ("experts",)

    def forward(self, h, step, stream):
        tokens = h.shape[0]
        weights = step.buffer("experts.weights", tokens, self.outputs, "float32")
        mix = step.buffer("experts.mix", tokens, 1, "float32") if self.shared_mix is not None else None
        K.route(h, self.router, self.correction, self.top, self.groups, self.keep, weights, self.shared_mix, mix,
                score=self.score, group_rank=self.group_rank, normalize=self.normalize)
        fused = step.buffer("experts.fused", tokens, self.fused_cols, step.dtype)
        K.gemm(h, self.in_weight, K.epilogue_store(fused), packed=self.in_packed)
        hidden = step.buffer("experts.hidden", tokens, self.hidden_cols, step.dtype)
        splits = stream_product_splits(step, hidden, self.down_weight)
        extra = 1 if self.identity else 0
        partials = step.partial_sums("experts.partials", splits + extra, tokens, self.width)
        K.gated_experts(fused, weights, mix, self.experts, self.ff, self.shared_ff, self.identity, hidden,
                        h=h if self.identity else None, identity_out=partials[splits] if self.identity else None,
                        limit=self.limit, alpha=self.alpha, unit=None if self.gated else self.unit)
        K.gemm(hidden, self.down_weight, K.epilogue_f32(partials[:splits]), splits=splits, packed=self.down_packed)
        return Delta(partials, None)
