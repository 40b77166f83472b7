"""Causal attention through low-rank latents, with an optional output gate and an optional key part that is
turned by position and shared by all heads.

Parameters: width, heads, dim (query/key size per head), vdim (value size per head), q_rank,
kv_rank, scale (multiplies q.k), eps (of the two latent norms), window (default 0: every earlier key; else the
latest so many positions), rot_dim (default 0), rot_base, rot_scaling, rot_pairing ("neighbours", the default, or
"halves"; frequencies and pairing as in ``parts/rotary_attention.py``).  Tensors, all [out, in]:
down_q [q_rank, width], q_norm [q_rank], up_q [heads*(dim + rot_dim), q_rank] (per head its dim plain rows, then
its rot_dim turned rows), down_kv [kv_rank + rot_dim, width] (the latent's rows, then the shared turned key part's,
which is not normalised), kv_norm [kv_rank], up_k [heads*dim, kv_rank], up_v [heads*vdim, kv_rank], optional
gate [heads*vdim, width], out_weight [width, heads*vdim].

With rot_dim > 0 a head's score is q_plain . k_plain + turn(q_turned) . turn(k_shared): the cached head is
[c; turn(k_shared)], its values c with zeros behind, and the absorbed query of head i is
[up_k_i^T up_q_i,plain c_q; turn(up_q_i,turned c_q)], so the same one-head attention serves.

With c_q = rms_norm(down_q h) and c = rms_norm(down_kv h), head i has queries q_i = up_q_i c_q,
keys k_i = up_k_i c and values v_i = up_v_i c.  Both up-projections of c are linear, so
    q_i . k_i(j) = (up_k_i^T up_q_i c_q) . c(j)        and        sum_j p_j v_i(j) = up_v_i sum_j p_j c(j):
attention runs on the latent itself.  Only c is cached, as ONE shared head of size kv_rank whose
keys and values are the same vector, and the heads' queries against it are the grouped-query case
of the attention kernels (all heads of a token read each cached vector once).  The matrix
up_k_i^T up_q_i is formed once when the part is built (in float64, rounded to the products' type).

One step: a fused product [down_q; down_kv; gate] h (32-bit sums) -> the two norms, c straight into
the paged cache -> absorbed queries (one product) -> attention over the cache -> per head up_v and
sigmoid gate -> output projection (the sublayer's output).
"""

import torch

from ..cache.storage import KVSpec
from ..kernels import library as K
from .attention import CausalSelfAttention
from .base import Mixer, compute_units, operand_columns, packed_for_stream, pad_columns, pad_rows
from .registry import register
from .rotary_attention import rotary_amplitude, rotary_frequencies


@register("mixer", "latent_attention")
class LatentAttention(Mixer):
    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        p = params
        self.width, self.heads, self.dim, self.vdim = p["width"], p["heads"], p["dim"], p["vdim"]
        self.q_rank, self.kv_rank = p["q_rank"], p["kv_rank"]
        self.scale, self.eps = float(p["scale"]), float(p["eps"])
        self.window, self.rot_dim = int(p.get("window") or 0), int(p.get("rot_dim") or 0)
        self.neighbours = {"halves": False, "neighbours": True}[p.get("rot_pairing", "neighbours")]
        if self.rot_dim % 2 != 0:
            raise ValueError(f"latent attention: {self.rot_dim} turned channels must be even")
        self.gated = "gate" in tensors
        shapes = {"down_q": (self.q_rank, self.width), "q_norm": (self.q_rank,),
                  "up_q": (self.heads * (self.dim + self.rot_dim), self.q_rank),
                  "down_kv": (self.kv_rank + self.rot_dim, self.width),
                  "kv_norm": (self.kv_rank,), "up_k": (self.heads * self.dim, self.kv_rank),
                  "up_v": (self.heads * self.vdim, self.kv_rank), "out_weight": (self.width, self.heads * self.vdim)}
        if self.gated:
            shapes["gate"] = (self.heads * self.vdim, self.width)
        for role, shape in shapes.items():
            if tuple(tensors[role].shape) != shape:
                raise ValueError(f"latent attention: {role} is {tuple(tensors[role].shape)}, expected {shape}")
        dtype = tensors["down_q"].dtype
        self.bf16 = dtype == torch.bfloat16
        # the cached head: the latent, padded to what the attention kernels take (zeros that meet zeros)
        self.head_dim = (self.kv_rank + self.rot_dim + 15) // 16 * 16
        if self.head_dim > 768:
            raise ValueError(f"latent attention: a cached head of {self.kv_rank} + {self.rot_dim} is beyond 768, the most any "
                             f"attention kernel here takes")
        # the MFMA kernels take heads of up to 128 (bfloat16) and up to 16 query heads per cached head
        # in decode steps; everything else runs on the plain attention kernel
        self.plain_only = self.bf16 and (self.head_dim > 128 or self.heads > 16)
        # segments of the fused first product, each padded so that the next starts where 16-byte loads may
        self.q_cols = operand_columns(self.q_rank, dtype)
        self.kv_offset = (self.q_rank + 3) // 4 * 4
        self.gate_offset = self.kv_offset + (self.kv_rank + self.rot_dim + 3) // 4 * 4
        self.fused_cols = self.gate_offset + (self.heads * self.vdim if self.gated else 0)
        self.fused_weight = torch.cat([pad_rows(tensors["down_q"], self.kv_offset),
                                       pad_rows(tensors["down_kv"], self.gate_offset - self.kv_offset)] +
                                      ([tensors["gate"]] if self.gated else []))
        # (the rows it multiplies carry zero columns where the width is no multiple of what 16-byte loads take)
        self.fused_weight = pad_columns(self.fused_weight, operand_columns(self.width, dtype))
        self.q_norm, self.kv_norm = tensors["q_norm"], tensors["kv_norm"]
        # absorbed queries: rows i * head_dim .. of W are up_k_i^T up_q_i  ([kv_rank, q_rank]), and behind them
        # the head's turned rows of up_q as they are
        up_q = tensors["up_q"].double().view(self.heads, self.dim + self.rot_dim, self.q_rank)
        up_k = tensors["up_k"].double().view(self.heads, self.dim, self.kv_rank)
        absorbed = torch.einsum("hdr,hdq->hrq", up_k, up_q[:, :self.dim])
        full = absorbed.new_zeros(self.heads, self.head_dim, self.q_cols)
        full[:, :self.kv_rank, :self.q_rank] = absorbed
        full[:, self.kv_rank:self.kv_rank + self.rot_dim, :self.q_rank] = up_q[:, self.dim:]
        device = tensors["down_q"].device
        self.inv_freq, self.amplitude = None, 1.0
        if self.rot_dim:
            self.inv_freq = rotary_frequencies(self.rot_dim, p["rot_base"], p.get("rot_scaling")).to(torch.float32).to(device)
            self.amplitude = rotary_amplitude(p.get("rot_scaling"))
        self.query_weight = full.view(self.heads * self.head_dim, self.q_cols).to(dtype).contiguous()
        self.up_v = tensors["up_v"].contiguous()
        self.mixed_cols = operand_columns(self.heads * self.vdim, dtype)
        self.out_weight = pad_columns(tensors["out_weight"], self.mixed_cols)
        self.n_q = self.heads * self.head_dim
        # second copies for decode steps, which read the weights and little else
        on_gpu = self.fused_weight.is_cuda
        self.fused_packed = K.PackedWeight(self.fused_weight) if on_gpu else None
        self.query_packed = K.PackedWeight(self.query_weight) if on_gpu else None
        self.out_packed = packed_for_stream(self.out_weight) if on_gpu else None

    def kv_spec(self):
        return KVSpec(1, self.head_dim, self.window)

    def kernel_modules(self, dtype):
        names = ["latent"]
        if not self.plain_only:
            if dtype == torch.bfloat16:
                names.append(f"attention_bf16_hd{self.head_dim}")
            elif self.head_dim <= 128:
                names.append("attention_f32")
        return tuple(names)

    # the planning of a prompt's runs of keys is the ordinary attention's: one cached head, ``heads`` query heads
    kv_heads = 1
    chunk = 0
    prompt_runs = CausalSelfAttention.prompt_runs

    def decode_runs(self, step, device):
        """Into how many runs a decode step's keys are cut.  All heads share one cached head, so a
        step has only as many work-groups as sequences unless the keys are cut, and they are cut much
        earlier than where every head brings keys of its own: from ``SPLIT_BYTES`` of a sequence's
        cached vectors on, into runs of at least ``RUN_BYTES``, as many as give every work-group a
        compute unit.  Planned for the step's class of context, like the ordinary attention's."""
        if not step.decode:
            return 1
        keys = min(step.context_limit, self.window + 32) if self.window else step.context_limit
        pair_bytes = keys * self.head_dim * 2 * (2 if step.dtype_is_bf16 else 4)
        if pair_bytes <= self.SPLIT_BYTES:
            return 1
        return max(1, min(compute_units(device) // step.n_seqs, pair_bytes // self.RUN_BYTES, 64))

    SPLIT_BYTES = 128 << 10
    RUN_BYTES = 64 << 10

    def forward(self, h, step, memory, stream):
        tokens = h.shape[0]
        kv = memory.kv()
        fused = step.buffer("latent.fused", tokens, self.fused_cols, "float32")
        K.gemm(h, self.fused_weight, K.epilogue_f32(fused), packed=self.fused_packed)
        c_q = step.buffer("latent.query_latent", tokens, self.q_cols, step.dtype)
        if not memory.writes:
            raise ValueError("latent attention: every run keeps a cache entry of its own")
        K.latent_norm(fused, self.q_rank, self.kv_offset, self.kv_rank, self.q_norm, self.kv_norm, self.eps, c_q,
                      step.tok_seq, step.tok_pos, kv, step.dtype, rot_dim=self.rot_dim, inv_freq=self.inv_freq,
                      neighbours=self.neighbours, amplitude=self.amplitude)
        q = step.buffer("latent.queries", tokens, self.n_q, step.dtype)
        if self.rot_dim:         # the turned part of every head is rotated from the 32-bit sums
            sums = step.buffer("latent.query_sums", tokens, self.n_q, "float32")
            K.gemm(c_q, self.query_weight, K.epilogue_f32(sums), packed=self.query_packed)
            K.latent_query(sums, self.heads, self.head_dim, self.kv_rank, self.rot_dim, self.inv_freq, step.tok_pos, q,
                           neighbours=self.neighbours, amplitude=self.amplitude)
        else:
            K.gemm(c_q, self.query_weight, K.epilogue_store(q), packed=self.query_packed)
        ctx = step.buffer("latent.context", tokens, self.n_q, step.dtype)
        partial, runs, prompt_runs = None, self.decode_runs(step, h.device), self.prompt_runs(step, h.device)
        if self.plain_only:
            runs = prompt_runs = 1
        if runs > 1:
            partial = step.buffer("attention.partial", step.n_seqs * self.heads * runs, self.head_dim + 2, "float32")
        elif prompt_runs > 1:
            partial = step.buffer("attention.partial", tokens * self.heads * prompt_runs, self.head_dim + 2, "float32")
        args = K.attention_args(q, ctx, kv, step.tok_seq, step.tok_pos, step.seq_off, step.seq_start, self.heads,
                                step.n_seqs, step.max_count, self.scale, self.window, partial,
                                runs=prompt_runs if prompt_runs > 1 else None)
        K.attention(args, step.dtype, step.decode, impl="plain" if self.plain_only else "auto")
        mixed = step.buffer("latent.mixed", tokens, self.mixed_cols, step.dtype)
        K.head_project(ctx, self.up_v, self.heads, self.vdim, self.kv_rank, self.head_dim, mixed,
                       gate=fused[:, self.gate_offset:] if self.gated else None)
        stream.add_product(step, mixed, self.out_weight, packed=self.out_packed)
