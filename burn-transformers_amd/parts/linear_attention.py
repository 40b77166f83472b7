"""Mixers that are linear attention with a matrix state per head: no softmax and no cache of keys, a state
S [dim, vdim] per head and sequence in 32-bit that every token lets decay per key channel and then writes
into (``csrc/linear_attention.hip``).

gated_delta_rule: parameters width, heads (of values, decays and the state), kv_heads (of queries and keys;
head h uses h // (heads // kv_heads)), dim, vdim, taps, eps (of the output norm), unit_eps (default 1e-6).
Tensors: q_weight, k_weight [kv_heads * dim, width], v_weight [heads * vdim, width], q_conv, k_conv, v_conv
[channels, taps] (the last tap meets the current token; no bias), beta_weight [heads, width], a1 [r, width],
a2 [heads * dim, r], dt_bias [heads * dim], A_log [heads], g1 [r', width], g2 [heads * vdim, r'], norm_weight
[vdim] (shared by the heads), out_weight [width, heads * vdim].
    q, k, v <- silu(conv(W h));   q <- q / sqrt(sum q^2 + unit_eps) * dim^-1/2,  k <- k / sqrt(sum k^2 + unit_eps)  per head
    beta = sigmoid(beta_weight h);   g = exp(-exp(A_log) * softplus(a2 (a1 h) + dt_bias))  per head and key channel
    S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
    out = out_weight (o / rms(o over vdim) * norm_weight * sigmoid(g2 (g1 h)))
  Parameters of the rule's variants: low_rank (default true; false: the step sizes' and the output gate's projections
  are single matrices ``a_weight`` and ``g_weight`` in place of a1, a2 and g1, g2), decay_span ("channel", the
  default, or "head": ONE decay per head for all its key channels, a_weight [heads, width], dt_bias [heads]),
  gate_act ("sigmoid", the default, or "silu": the output is multiplied by z sigmoid(z) of the gate's sums z).

forget_gate_attention: parameters width, heads, dim, vdim, eps.  Tensors: q_weight, f_weight [heads * dim,
width], f_bias, lower [heads * dim], v_weight [heads * vdim, width], norm_weight [vdim], out_weight.
    f = lower + (1 - lower) * sigmoid(f_weight h + f_bias);   q = silu(q_weight h);   v = v_weight h
    S <- diag(f) S + (1 - f) v^T;  o = S^T q;   out = out_weight (o / rms(o over vdim) * norm_weight)

Both: ONE product with all projections of h laid one behind the other leaves 32-bit sums; everything behind
it that enters the recurrence stays 32-bit.  The convolution's last taps - 1 inputs and S are the sequence's
state: one float32 row per sequence (``StateSpec``), zero for a new sequence.  A step may bring any number of
a sequence's tokens; the kernels walk them in order from the state the last step left.
"""

import torch

from ..cache.storage import StateSpec
from ..kernels import library as K
from .base import Mixer, operand_columns, packed_for_stream, pad_columns
from .registry import register


def _check(kind, tensors, shapes):
    for role, shape in shapes.items():
        if tuple(tensors[role].shape) != shape:
            raise ValueError(f"{kind}: {role} is {tuple(tensors[role].shape)}, expected {shape}")


class _MatrixState(Mixer):
    only_launches_kernels = True

    def kernel_modules(self, dtype):
        return ("linear_attention", "state_space")

    def state_spec(self):
        return StateSpec((self.conv_state + self.scan_state,), "float32")

    def _sizes(self, params):
        self.width, self.heads, self.dim, self.vdim = params["width"], params["heads"], params["dim"], params["vdim"]
        self.eps = float(params["eps"])
        if not 1 <= self.dim <= 256:
            raise ValueError(f"{type(self).__name__}: keys of {self.dim} channels outside 1..256, what the scan takes")
        self.inner = self.heads * self.vdim
        # (the scan lays a head's state out in tiles of four value channels)
        self.scan_state = self.heads * self.dim * ((self.vdim + 3) // 4 * 4)

    def _finish(self, fused_rows, out_weight):
        dtype = out_weight.dtype
        self.in_weight = pad_columns(torch.cat(fused_rows), operand_columns(self.width, dtype))
        self.fused_cols = self.in_weight.shape[0]
        self.inner_cols = operand_columns(self.inner, dtype)
        self.out_weight = pad_columns(out_weight, self.inner_cols)
        on_gpu = self.in_weight.is_cuda
        self.in_packed = K.PackedWeight(self.in_weight) if on_gpu else None
        self.out_packed = packed_for_stream(self.out_weight) if on_gpu else None
        self.in_bias, self.fused = None, None

    def ride_along(self, weight, bias=None):
        if self.in_bias is not None or weight.dtype != self.in_weight.dtype or weight.shape[1] != self.width:
            return None
        first, rows = self.fused_cols, weight.shape[0]
        self.in_weight = torch.cat([self.in_weight, pad_columns(weight, self.in_weight.shape[1])]).contiguous()
        self.fused_cols = self.in_weight.shape[0]
        self.in_packed = K.PackedWeight(self.in_weight) if self.in_weight.is_cuda else None
        self.in_bias = torch.zeros(self.fused_cols, dtype=torch.float32, device=weight.device)
        if bias is not None:
            self.in_bias[first:] = bias.float()
        return lambda step: self.fused[:, first:first + rows]

    def _project(self, h, step, key):
        """The mixer's first product: every projection of h, and what rides along, as 32-bit sums."""
        self.fused = step.buffer(key, h.shape[0], self.fused_cols, "float32")
        K.gemm(h, self.in_weight, K.epilogue_f32(self.fused, self.in_bias), packed=self.in_packed)
        return self.fused


@register("mixer", "gated_delta_rule")
class GatedDeltaRule(_MatrixState):
    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self._sizes(params)
        self.kv_heads, self.taps = params["kv_heads"], int(params["taps"])
        self.unit_eps = float(params.get("unit_eps", 1e-6))
        self.low_rank = bool(params.get("low_rank", True))
        self.per_head = {"channel": False, "head": True}[params.get("decay_span", "channel")]
        self.gate_act = params.get("gate_act", "sigmoid")
        if self.gate_act not in ("sigmoid", "silu"):
            raise ValueError(f"gated_delta_rule: unknown activation {self.gate_act!r} of the output gate")
        if self.heads % self.kv_heads != 0:
            raise ValueError(f"gated_delta_rule: {self.heads} heads cannot share {self.kv_heads} heads of queries and keys")
        qk, t = self.kv_heads * self.dim, tensors
        self.decays = self.heads if self.per_head else self.heads * self.dim
        shapes = {"q_weight": (qk, self.width), "k_weight": (qk, self.width), "v_weight": (self.inner, self.width),
                  "q_conv": (qk, self.taps), "k_conv": (qk, self.taps), "v_conv": (self.inner, self.taps),
                  "beta_weight": (self.heads, self.width), "dt_bias": (self.decays,), "A_log": (self.heads,),
                  "norm_weight": (self.vdim,), "out_weight": (self.width, self.inner)}
        if self.low_rank:
            self.rank_a, self.rank_g = t["a1"].shape[0], t["g1"].shape[0]
            shapes.update(a1=(self.rank_a, self.width), a2=(self.decays, self.rank_a), g1=(self.rank_g, self.width),
                          g2=(self.inner, self.rank_g))
        else:
            self.rank_a, self.rank_g = self.decays, self.inner          # the fused product's columns are the sums themselves
            shapes.update(a_weight=(self.decays, self.width), g_weight=(self.inner, self.width))
        _check("gated_delta_rule", t, shapes)
        self.qk, self.channels = qk, 2 * qk + self.inner
        self.at_beta = self.channels
        self.at_a, self.at_g = self.at_beta + self.heads, self.at_beta + self.heads + self.rank_a
        first, second = (t["a1"], t["g1"]) if self.low_rank else (t["a_weight"], t["g_weight"])
        self._finish([t["q_weight"], t["k_weight"], t["v_weight"], t["beta_weight"], first, second], t["out_weight"])
        self.conv_weight = torch.cat([t["q_conv"], t["k_conv"], t["v_conv"]]).float().contiguous()
        if self.low_rank:
            self.a2, self.g2 = t["a2"].contiguous(), t["g2"].contiguous()
        self.dt_bias, self.A_log, self.norm_weight = t["dt_bias"], t["A_log"], t["norm_weight"]
        self.conv_state = (self.taps - 1) * self.channels

    def forward(self, h, step, memory, stream):
        tokens, qk = h.shape[0], self.qk
        rows = memory.state()
        conv_state, scan_state = rows[:, :self.conv_state], rows[:, self.conv_state:]
        fused = self._project(h, step, "delta.in")
        qkv = step.buffer("delta.qkv", tokens, self.channels, "float32")
        K.causal_conv(fused[:, :self.channels], self.conv_weight, None, qkv, conv_state, step)
        if self.low_rank:
            dt = step.buffer("delta.dt", tokens, self.decays, "float32")
            K.dt_project(fused[:, self.at_a:self.at_a + self.rank_a], self.a2, self.dt_bias, dt, act="softplus")
            gate = step.buffer("delta.gate", tokens, self.inner, "float32")
            K.dt_project(fused[:, self.at_g:self.at_g + self.rank_g], self.g2, None, gate, act="none")
            raw = None
        else:            # the sums are in the fused product's rows: the scan adds the bias and takes the softplus itself
            dt, gate, raw = fused[:, self.at_a:self.at_a + self.decays], fused[:, self.at_g:self.at_g + self.inner], self.dt_bias
        y = step.buffer("delta.y", tokens, self.inner, "float32")
        K.keyed_scan(qkv[:, :qk], qkv[:, qk:2 * qk], qkv[:, 2 * qk:], dt, y, scan_state, step, self.heads, self.kv_heads,
                     self.dim, self.vdim, "delta", beta=fused[:, self.at_beta:self.at_beta + self.heads], A_log=self.A_log,
                     unit=True, unit_eps=self.unit_eps, q_scale=self.dim ** -0.5, decay_per_head=self.per_head, dt_bias=raw)
        gated = step.buffer("delta.gated", tokens, self.inner_cols, step.dtype)
        K.head_norm_gate(y, self.norm_weight, self.heads, self.vdim, self.eps, gated, gate=gate, gate_act=self.gate_act)
        stream.add_product(step, gated, self.out_weight, packed=self.out_packed)


@register("mixer", "forget_gate_attention")
class ForgetGateAttention(_MatrixState):
    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self._sizes(params)
        qk, t = self.heads * self.dim, tensors
        _check("forget_gate_attention", t, {
            "q_weight": (qk, self.width), "f_weight": (qk, self.width), "f_bias": (qk,), "lower": (qk,),
            "v_weight": (self.inner, self.width), "norm_weight": (self.vdim,), "out_weight": (self.width, self.inner)})
        self.qk = qk
        self._finish([t["q_weight"], t["f_weight"], t["v_weight"]], t["out_weight"])
        self.f_bias, self.lower, self.norm_weight = t["f_bias"], t["lower"], t["norm_weight"]
        self.conv_state = 0

    def forward(self, h, step, memory, stream):
        tokens, qk = h.shape[0], self.qk
        fused = self._project(h, step, "forget.in")
        y = step.buffer("forget.y", tokens, self.inner, "float32")
        K.keyed_scan(fused[:, :qk], None, fused[:, 2 * qk:], fused[:, qk:2 * qk], y, memory.state(), step, self.heads,
                     self.heads, self.dim, self.vdim, "forget", g_bias=self.f_bias, lower=self.lower,
                     carry=K.scan_carry(step, self.scan_state, self.heads * self.dim))
        normed = step.buffer("forget.normed", tokens, self.inner_cols, step.dtype)
        K.head_norm_gate(y, self.norm_weight, self.heads, self.vdim, self.eps, normed)
        stream.add_product(step, normed, self.out_weight, packed=self.out_packed)
