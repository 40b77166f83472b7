"""Causal self-attention whose queries and keys are normalised per head and turned by their
positions (rotary positions), with grouped heads over the paged cache.

Parameters (all from the plan): width, heads, kv_heads, dim (a query's and a key's head size), vdim
(a value's head size, which may differ), scale (multiplies q.k), eps (of the head norms), head_norm
(whether queries and keys are divided by their root mean square per head, times the scales
``q_norm`` / ``k_norm`` [dim] that all heads share), rot_dims (the first so many channels of every
query and key head are turned, channel i with channel i + rot_dims / 2, by the angle position *
f_i), rot_base (f_i = rot_base^(-2 i / rot_dims)), rot_scaling (None, or factor / low / high /
original: frequencies whose wavelength is beyond original / low are divided by factor, those whose
wavelength is below original / high are kept, and between the two the division is blended in
linearly in original / wavelength; or, with the keys factor / original / fast / slow, the schedule that
blends by a pair's INDEX: with turns(i) the index at which a wave turns that many times in ``original`` positions,
pairs up to turns(fast) are kept, pairs from turns(slow) on are divided by factor, a linear ramp over the index
between, and every sine and cosine is multiplied by 0.1 ln(factor) + 1), rot_pairing ("halves", the default: channel i with channel i + rot_dims / 2;
"neighbours": channel 2 i with channel 2 i + 1), norm_span ("head", the default; "whole": the root mean square
is taken over a token's whole query (key) projection before it is split into heads, and the scales ``q_norm`` /
``k_norm`` are [heads * dim] / [kv_heads * dim]), window and chunk (which earlier keys a query sees, as in
``parts/attention.py``), taps (default 0; with taps > 0 every channel of the query, key and value projections
passes a short causal convolution over its sequence's tokens, tensors ``q_conv`` / ``k_conv`` / ``v_conv``
[channels, taps], the last tap meeting the current token, no bias, no activation, before norms and rotation;
the projections' last taps - 1 outputs are then a state of the sequence beside its keys and values).  Optional
tensors ``q_bias`` / ``k_bias`` / ``v_bias``: added in the projection.  Optional tensor ``sink`` [heads]: a learned logit per head that stands in the softmax's
denominator beside the keys', with no key and no value.  Tensors: q_weight [heads * dim, width], k_weight [kv_heads * dim, width],
v_weight [kv_heads * vdim, width], out_weight [width, heads * vdim], no biases.

One step: ONE product with the three projections laid one behind the other leaves 32-bit sums; a
kernel normalises and turns the heads, writes the queries to a buffer and the keys (turned) and
values straight into the cache at each token's position; the framework's attention kernels read the
cache; the output projection adds to the stream.  The cache keeps heads of one size, max(dim, vdim)
rounded up to what the kernels take, with zeros behind a head's own channels; the output
projection's columns are spread the same way, so the zeros meet zeros.
"""

import math

import torch

from ..cache.storage import StateSpec
from ..kernels import library as K
from .attention import CausalSelfAttention
from .base import Mixer, operand_columns, packed_for_stream, pad_columns
from .registry import register


def rotary_frequencies(dims, base, scaling=None):
    """f_i for i < dims / 2 (float64): base^(-2 i / dims), rescaled by ``scaling`` as the module's text says."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    if scaling and "fast" in scaling:
        factor, original = float(scaling["factor"]), float(scaling["original"])
        # the (fractional) pair index whose wave turns ``turns`` times in ``original`` positions
        index = lambda turns: dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))
        first = max(math.floor(index(float(scaling["fast"]))), 0)
        last = min(math.ceil(index(float(scaling["slow"]))), dims - 1)
        ramp = torch.clamp((i - first) / max(last - first, 0.001), 0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
    elif scaling:
        factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
        wavelength = 2.0 * math.pi / f
        blend = (original / wavelength - low) / (high - low)
        between = (1.0 - blend) * f / factor + blend * f
        f = torch.where(wavelength < original / high, f, torch.where(wavelength > original / low, f / factor, between))
    return f


def rotary_amplitude(scaling=None):
    """The factor on every sine and cosine that goes with ``scaling``: 0.1 ln(factor) + 1 for the schedule that
    blends by index, 1 otherwise."""
    return 0.1 * math.log(float(scaling["factor"])) + 1.0 if scaling and "fast" in scaling else 1.0


@register("mixer", "rotary_attention")
class RotaryAttention(CausalSelfAttention):
    takes_deferred_norm = False          # (its first product leaves 32-bit sums; the rows come normalised)
    only_launches_kernels = True

    def __init__(self, params, tensors):
        Mixer.__init__(self, params, tensors)
        p = params
        self.width, self.heads, self.kv_heads = p["width"], p["heads"], p["kv_heads"]
        self.dim, self.vdim = p["dim"], p["vdim"]
        self.scale, self.eps = float(p["scale"]), float(p.get("eps", 0.0))
        self.window, self.chunk = int(p.get("window") or 0), int(p.get("chunk") or 0)
        self.rot_dims = int(p.get("rot_dims") or 0)
        if self.heads % self.kv_heads != 0:
            raise ValueError(f"rotary attention: {self.heads} query heads cannot share {self.kv_heads} key/value heads")
        if self.rot_dims % 2 != 0 or self.rot_dims > self.dim:
            raise ValueError(f"rotary attention: {self.rot_dims} turned channels must be even and at most the head size {self.dim}")
        shapes = {"q_weight": (self.heads * self.dim, self.width), "k_weight": (self.kv_heads * self.dim, self.width),
                  "v_weight": (self.kv_heads * self.vdim, self.width), "out_weight": (self.width, self.heads * self.vdim)}
        self.neighbours = {"halves": False, "neighbours": True}[p.get("rot_pairing", "halves")]
        self.whole_norm = {"head": False, "whole": True}[p.get("norm_span", "head")]
        if p.get("head_norm", True):
            shapes.update(q_norm=(self.heads * self.dim,), k_norm=(self.kv_heads * self.dim,)) if self.whole_norm else \
                shapes.update(q_norm=(self.dim,), k_norm=(self.dim,))
        if "sink" in tensors:
            shapes["sink"] = (self.heads,)
        self.taps = int(p.get("taps") or 0)
        for name, rows in (("q", self.heads * self.dim), ("k", self.kv_heads * self.dim), ("v", self.kv_heads * self.vdim)):
            if name + "_bias" in tensors:
                shapes[name + "_bias"] = (rows,)
            if self.taps:
                shapes[name + "_conv"] = (rows, self.taps)
        for role, shape in shapes.items():
            if tuple(tensors[role].shape) != shape:
                raise ValueError(f"rotary attention: {role} is {tuple(tensors[role].shape)}, expected {shape}")
        self.q_norm, self.k_norm = tensors.get("q_norm"), tensors.get("k_norm")
        self.sink = tensors["sink"].float().contiguous() if "sink" in tensors else None
        dtype = tensors["q_weight"].dtype
        bf16 = dtype == torch.bfloat16
        # the cached head: the larger of the two head sizes, in the steps of 16 the MFMA kernels take
        self.head_dim = (max(self.dim, self.vdim) + 15) // 16 * 16
        if self.head_dim > 256:
            raise ValueError(f"rotary attention: heads of {max(self.dim, self.vdim)} are beyond 256, the most any kernel here takes")
        # the MFMA kernels take heads of up to 128 in bfloat16; larger ones run on the plain attention kernel
        self.plain_only = bf16 and self.head_dim > 128
        self.plain_decode = bf16 and self.heads // self.kv_heads > 16
        self.n_q, self.n_kv = self.heads * self.head_dim, self.kv_heads * self.head_dim
        self.fused_cols = (self.heads + self.kv_heads) * self.dim + self.kv_heads * self.vdim
        self.qkv_weight = pad_columns(torch.cat([tensors["q_weight"], tensors["k_weight"], tensors["v_weight"]]),
                                      operand_columns(self.width, dtype))
        # the output projection reads heads of head_dim: its columns are spread, zeros between them
        out = tensors["out_weight"]
        spread = out.new_zeros(self.width, self.heads, self.head_dim)
        spread[:, :, :self.vdim] = out.view(self.width, self.heads, self.vdim)
        self.out_weight = spread.view(self.width, self.n_q).contiguous()
        self.out_bias = None
        device = self.qkv_weight.device
        self.inv_freq = rotary_frequencies(self.rot_dims, p["rot_base"], p.get("rot_scaling")).to(torch.float32).to(device) \
            if self.rot_dims else None
        self.amplitude = rotary_amplitude(p.get("rot_scaling")) if self.rot_dims else 1.0
        self.qkv_bias = None
        if any(name + "_bias" in tensors for name in "qkv"):
            self.qkv_bias = torch.cat([tensors[name + "_bias"].float() if name + "_bias" in tensors
                                       else torch.zeros(rows, dtype=torch.float32, device=device)
                                       for name, rows in (("q", self.heads * self.dim), ("k", self.kv_heads * self.dim),
                                                          ("v", self.kv_heads * self.vdim))]).contiguous()
        self.conv_weight, self.conv_state = None, 0
        if self.taps:
            self.conv_weight = torch.cat([tensors["q_conv"], tensors["k_conv"], tensors["v_conv"]]).float().contiguous()
            self.conv_state = (self.taps - 1) * self.fused_cols
            self.no_state = torch.zeros(1, 1, dtype=torch.float32, device=device)       # what one tap keeps: nothing
        on_gpu = self.qkv_weight.is_cuda
        self.qkv_packed = K.PackedWeight(self.qkv_weight) if on_gpu else None
        self.out_packed = packed_for_stream(self.out_weight) if on_gpu else None

    def kernel_modules(self, dtype):
        return ("rotary",) + (("state_space",) if self.taps else ()) + tuple(super().kernel_modules(dtype))

    def state_spec(self):
        return StateSpec((self.conv_state,), "float32") if self.conv_state else None

    def forward(self, h, step, memory, stream):
        tokens = h.shape[0]
        if not memory.writes:
            raise ValueError("rotary attention: every run keeps a cache entry of its own")
        kv = memory.kv()
        fused = step.buffer("rotary.fused", tokens, self.fused_cols, "float32")
        K.gemm(h, self.qkv_weight, K.epilogue_f32(fused, self.qkv_bias), packed=self.qkv_packed)
        if self.taps:
            mixed_in_time = step.buffer("rotary.conv", tokens, self.fused_cols, "float32")
            K.causal_conv(fused, self.conv_weight, None, mixed_in_time, memory.state() if self.conv_state else self.no_state,
                          step, act="none")
            fused = mixed_in_time
        q = step.buffer("attention.q", tokens, self.n_q, step.dtype)
        K.head_rotary(fused, self.heads, self.kv_heads, self.dim, self.vdim, self.rot_dims, self.inv_freq,
                      self.q_norm, self.k_norm, self.eps, q, step.tok_seq, step.tok_pos, kv, step.dtype,
                      neighbours=self.neighbours, whole_norm=self.whole_norm, amplitude=self.amplitude)
        plain = self.plain_only or (self.plain_decode and step.decode)
        if step.decode and step.dtype_is_bf16 and K.Chunked.wanted(tokens) and not plain:
            mixed = K.Chunked.take(step, "attention.mixed", tokens, self.n_q, step.dtype)
        else:
            mixed = step.buffer("attention.mixed", tokens, self.n_q, step.dtype)
        partial, runs = None, 1 if plain else self.decode_runs(step, h.device)
        if runs > 1:
            partial = step.buffer("attention.partial", step.n_seqs * self.heads * runs, self.head_dim + 2, "float32")
        args = K.attention_args(q, mixed, kv, step.tok_seq, step.tok_pos, step.seq_off, step.seq_start,
                                self.heads, step.n_seqs, step.max_count, self.scale, self.window, partial,
                                chunk=self.chunk, sink=self.sink)
        # (the bfloat16 decode kernel takes up to 16 query heads on a cached head; beyond, the plain kernel)
        K.attention(args, step.dtype, step.decode, impl="plain" if plain else "auto")
        stream.add_product(step, mixed, self.out_weight, None, packed=self.out_packed)
