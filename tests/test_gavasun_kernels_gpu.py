"""The kernel forms that came with Gavasun's mechanisms, each alone against float64: the delta rule's scan with one
decay per head and its step sizes taken raw (bias and softplus in the kernel), the head norm with a SiLU gate, the
convolution without an activation, the latent norms with a turned key part into the cache, the rotation of the
absorbed queries, sines and cosines with an amplitude, experts' units without a gate, and the plain attention kernel
on heads beyond 256."""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu

import plain_gavasun as plain  # noqa: E402
from burn_transformers_amd.kernels import library as K  # noqa: E402
from burn_transformers_amd.parts.rotary_attention import rotary_amplitude, rotary_frequencies  # noqa: E402
from kernel_helpers import PagedCase  # noqa: E402
from step_helpers import make_step  # noqa: E402

DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F64 = torch.float64


def rel_err(got, want):
    got = got.detach().cpu().double()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(4, 2, 16, 24), (3, 1, 20, 12), (2, 2, 128, 32), (1, 1, 200, 70), (5, 5, 8, 4)])
def test_delta_rule_scan_with_one_decay_a_head(heads, kv_heads, dim, vdim):
    """S <- g S with g = exp(-exp(A_log) softplus(raw + dt_bias)) one number a head; three sequences in slots of their
    own, in portions down to one token, from the state the last portion left."""
    gen = torch.Generator().manual_seed(heads * 100 + dim)
    lengths, qk, inner = [140, 5, 70], kv_heads * dim, heads * vdim
    seqs = [torch.randn(n, 2 * qk + inner + 2 * heads, generator=gen) for n in lengths]
    A_log = torch.log(torch.rand(heads, generator=gen) * 3.0 + 0.5)
    dt_bias = torch.randn(heads, generator=gen) - 2.0
    want = []
    for rows in seqs:
        r = rows.double()
        q, k = r[:, :qk].view(-1, kv_heads, dim), r[:, qk:2 * qk].view(-1, kv_heads, dim)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        v = r[:, 2 * qk:2 * qk + inner].view(-1, heads, vdim)
        decay = torch.exp(-torch.exp(A_log.double()) * plain.softplus(r[:, 2 * qk + inner:2 * qk + inner + heads] + dt_bias.double()))
        beta = plain.sigmoid(r[:, 2 * qk + inner + heads:])
        out = torch.zeros(rows.shape[0], heads, vdim, dtype=F64)
        for h in range(heads):
            j, S = h // (heads // kv_heads), torch.zeros(dim, vdim, dtype=F64)
            for t in range(rows.shape[0]):
                S = decay[t, h] * S
                u = beta[t, h] * (v[t, h] - S.T @ k[t, j])
                S = S + k[t, j][:, None] * u[None, :]
                out[t, h] = S.T @ q[t, j]
        want.append(out.reshape(rows.shape[0], inner))
    slots = [2, 1, 0]
    state = torch.zeros(3, heads * dim * ((vdim + 3) // 4 * 4) + 5, device=DEV)
    got = [torch.zeros(n, inner, dtype=F64) for n in lengths]
    cuts = [2, 3, 64, 129]
    bounds = [[0] + [c for c in cuts if c < n] + [n] for n in lengths]
    for turn in range(max(len(b) for b in bounds) - 1):
        spans = [(s, b[turn], b[turn + 1]) for s, b in enumerate(bounds) if turn + 1 < len(b)]
        step = make_step(torch.float32, [b - a for _, a, b in spans], starts=[a for _, a, _ in spans], slots=[slots[s] for s, _, _ in spans])
        rows = torch.cat([seqs[s][a:b] for s, a, b in spans]).to(DEV)
        y = torch.full((rows.shape[0], inner), float("nan"), device=DEV)
        K.keyed_scan(rows[:, :qk], rows[:, qk:2 * qk], rows[:, 2 * qk:2 * qk + inner], rows[:, 2 * qk + inner:2 * qk + inner + heads], y,
                     state, step, heads, kv_heads, dim, vdim, "delta", beta=rows[:, 2 * qk + inner + heads:], A_log=A_log.to(DEV),
                     unit=True, unit_eps=1e-6, q_scale=dim ** -0.5, decay_per_head=True, dt_bias=dt_bias.to(DEV))
        at = 0
        for s, a, b in spans:
            got[s][a:b] = y[at:at + b - a].cpu().double()
            at += b - a
    for g, w in zip(got, want):
        assert rel_err(g, w) < 2e-5


@pytest.mark.parametrize("out_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("gate_act", ["silu", "sigmoid"])
def test_head_norm_with_a_gate(out_dtype, gate_act):
    gen = torch.Generator().manual_seed(5)
    tokens, heads, vdim, eps = 37, 5, 20, 1e-4
    y, gate, weight = torch.randn(tokens, heads * vdim, generator=gen), torch.randn(tokens, heads * vdim, generator=gen), torch.randn(vdim, generator=gen)
    out = torch.full((tokens, heads * vdim + 4), float("nan"), dtype=DTYPES[out_dtype], device=DEV)
    K.head_norm_gate(y.to(DEV), weight.to(DEV), heads, vdim, eps, out, gate=gate.to(DEV), gate_act=gate_act)
    factor = plain.silu(gate.double()) if gate_act == "silu" else plain.sigmoid(gate.double())
    want = (plain.unit_rms(y.double().view(tokens, heads, vdim), eps) * weight.double()).reshape(tokens, -1) * factor
    assert rel_err(out[:, :heads * vdim], want) < (1e-5 if out_dtype == "float32" else 1e-2)
    assert float(out[:, heads * vdim:].float().abs().max()) == 0.0


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_convolution_without_activation_in_portions(taps):
    """Two sequences in portions of unequal length (shorter than the taps too); inputs before a portion come from
    the state, which starts at zero."""
    gen = torch.Generator().manual_seed(taps)
    channels, lengths = 13, [23, 9]
    seqs = [torch.randn(n, channels, generator=gen) for n in lengths]
    weight = torch.randn(channels, taps, generator=gen)
    want = [plain.short_conv(s.double(), weight.double()) for s in seqs]
    state = torch.zeros(3, max(taps - 1, 1) * channels + 2, device=DEV)
    got = [torch.zeros(n, channels, dtype=F64) for n in lengths]
    at = [0, 0]
    for portion in ([1, 2], [2, 1], [5, 1], [15, 5]):
        live = [s for s in range(2) if at[s] < lengths[s]]
        counts = [min(portion[s], lengths[s] - at[s]) for s in live]
        step = make_step(torch.float32, counts, starts=[at[s] for s in live], slots=[[2, 0][s] for s in live])
        rows = torch.cat([seqs[s][at[s]:at[s] + c] for s, c in zip(live, counts)]).to(DEV)
        out = torch.full((rows.shape[0], channels), float("nan"), device=DEV)
        K.causal_conv(rows, weight.to(DEV), None, out, state, step, act="none")
        row = 0
        for s, c in zip(live, counts):
            got[s][at[s]:at[s] + c] = out[row:row + c].cpu().double()
            row += c
            at[s] += c
    assert at == lengths
    for g, w in zip(got, want):
        assert rel_err(g, w) < 1e-6


SCALINGS = [None, {"factor": 6.0, "original": 64, "fast": 24.0, "slow": 1.0}, {"factor": 3.0, "original": 4096, "fast": 4.0, "slow": 0.5}]


@pytest.mark.parametrize("scaling", SCALINGS)
@pytest.mark.parametrize("dims,base", [(32, 300000.0), (6, 50.0), (64, 7000.0)])
def test_frequencies_and_amplitude(dims, base, scaling):
    rot = {"dims": dims, "base": base, "scaling": scaling}
    f, amplitude = plain.frequencies(rot)
    assert torch.allclose(rotary_frequencies(dims, base, scaling), f, rtol=1e-12, atol=0.0)
    assert rotary_amplitude(scaling) == pytest.approx(amplitude)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("q_rank,kv_rank,rot_dim,neighbours", [(24, 32, 8, True), (7, 9, 6, True), (40, 250, 64, False), (16, 48, 0, True)])
def test_latent_norms_with_a_turned_key_part(dtype, q_rank, kv_rank, rot_dim, neighbours):
    """The query latent normalised into a buffer; the key/value latent normalised into the cached head's keys and
    values, the turned part behind it in the keys only (zeros in the values)."""
    totals = [70, 5]
    hd = (kv_rank + rot_dim + 15) // 16 * 16
    case = PagedCase(totals, totals, 1, hd, DTYPES[dtype], DEV, seed=3)
    gen = torch.Generator().manual_seed(q_rank)
    kv_offset = (q_rank + 3) // 4 * 4
    tokens = sum(totals)
    fused = torch.randn(tokens, kv_offset + kv_rank + rot_dim + 3, generator=gen)
    q_gamma, kv_gamma = torch.randn(q_rank, generator=gen), torch.randn(kv_rank, generator=gen)
    scaling = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}
    rot = {"dims": rot_dim, "base": 300.0, "scaling": scaling} if rot_dim else None
    inv_freq = rotary_frequencies(rot_dim, 300.0, scaling).float().to(DEV) if rot_dim else None
    q_out = torch.full((tokens, q_rank + 2), float("nan"), dtype=DTYPES[dtype], device=DEV)
    K.latent_norm(fused.to(DEV), q_rank, kv_offset, kv_rank, q_gamma.to(DEV), kv_gamma.to(DEV), 1e-5, q_out, case.tok_seq, case.tok_pos,
                  case.view(), DTYPES[dtype], rot_dim=rot_dim, inv_freq=inv_freq, neighbours=neighbours,
                  amplitude=rotary_amplitude(scaling) if rot_dim else 1.0)
    bound = 1e-5 if dtype == "float32" else 1e-2
    f = fused.double()
    assert rel_err(q_out[:, :q_rank], plain.unit_rms(f[:, :q_rank], 1e-5) * q_gamma.double()) < bound
    assert float(q_out[:, q_rank:].float().abs().max()) == 0.0
    c = plain.unit_rms(f[:, kv_offset:kv_offset + kv_rank], 1e-5) * kv_gamma.double()
    positions = torch.cat([torch.arange(t) for t in totals])
    keys, values = case.read_back()
    assert rel_err(keys[:, :kv_rank], c) < bound and rel_err(values[:, :kv_rank], c) < bound
    if rot_dim:
        turned = plain.turn(f[:, None, kv_offset + kv_rank:kv_offset + kv_rank + rot_dim], positions, rot,
                            "neighbours" if neighbours else "halves")[:, 0]
        assert rel_err(keys[:, kv_rank:kv_rank + rot_dim], turned) < bound
    assert hd == kv_rank or float(values[:, kv_rank:].float().abs().max()) == 0.0
    assert hd == kv_rank + rot_dim or float(keys[:, kv_rank + rot_dim:].float().abs().max()) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,pitch,rot_at,rot_dim,neighbours", [(3, 48, 32, 8, True), (2, 16, 9, 6, False), (5, 320, 250, 64, True), (1, 16, 16, 0, True)])
def test_rotation_of_the_absorbed_queries(dtype, heads, pitch, rot_at, rot_dim, neighbours):
    gen = torch.Generator().manual_seed(pitch)
    tokens = 45
    sums = torch.randn(tokens, heads * pitch, generator=gen)
    positions = torch.randint(0, 3000, (tokens,), generator=gen)
    scaling = {"factor": 2.0, "original": 128, "fast": 16.0, "slow": 1.0}
    inv_freq = rotary_frequencies(rot_dim, 5000.0, scaling).float().to(DEV) if rot_dim else None
    out = torch.full((tokens, heads * pitch), float("nan"), dtype=DTYPES[dtype], device=DEV)
    K.latent_query(sums.to(DEV), heads, pitch, rot_at, rot_dim, inv_freq, positions.to(torch.int32).to(DEV), out, neighbours=neighbours,
                   amplitude=rotary_amplitude(scaling))
    want = sums.double().view(tokens, heads, pitch).clone()
    if rot_dim:
        want[..., rot_at:rot_at + rot_dim] = plain.turn(want[..., rot_at:rot_at + rot_dim], positions,
                                                        {"dims": rot_dim, "base": 5000.0, "scaling": scaling},
                                                        "neighbours" if neighbours else "halves")
    # (angles are 32-bit products of position and frequency: at position 3,000 they are off by 2e-4)
    assert rel_err(out, want.reshape(tokens, -1)) < (1e-3 if dtype == "float32" else 1e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_head_rotary_with_an_amplitude(dtype):
    """Halves turned together with slowed frequencies; sine and cosine carry the schedule's factor."""
    heads, kv_heads, dim, vdim, rot_dims = 4, 2, 24, 16, 12
    totals = [40, 3]
    case = PagedCase(totals, totals, kv_heads, 32, DTYPES[dtype], DEV, seed=2)
    gen = torch.Generator().manual_seed(1)
    tokens = sum(totals)
    fused = torch.randn(tokens, (heads + kv_heads) * dim + kv_heads * vdim, generator=gen)
    scaling = {"factor": 8.0, "original": 16, "fast": 4.0, "slow": 1.0}
    rot = {"dims": rot_dims, "base": 100.0, "scaling": scaling}
    q_out = torch.zeros(tokens, heads * 32, dtype=DTYPES[dtype], device=DEV)
    K.head_rotary(fused.to(DEV), heads, kv_heads, dim, vdim, rot_dims, rotary_frequencies(rot_dims, 100.0, scaling).float().to(DEV),
                  None, None, 0.0, q_out, case.tok_seq, case.tok_pos, case.view(), DTYPES[dtype], amplitude=rotary_amplitude(scaling))
    positions = torch.cat([torch.arange(t) for t in totals])
    f = fused.double()
    want_q = plain.turn(f[:, :heads * dim].view(tokens, heads, dim), positions, rot, "halves")
    want_k = plain.turn(f[:, heads * dim:(heads + kv_heads) * dim].view(tokens, kv_heads, dim), positions, rot, "halves")
    bound = 1e-5 if dtype == "float32" else 1e-2
    assert rel_err(q_out.view(tokens, heads, 32)[..., :dim], want_q) < bound
    keys, _ = case.read_back()
    assert rel_err(keys.view(tokens, kv_heads, 32)[..., :dim], want_k) < bound
    assert rotary_amplitude(scaling) > 1.2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("unit", ["gelu_erf", "silu"])
@pytest.mark.parametrize("experts,ff,shared", [(4, 12, 20), (3, 5, 0), (1, 8, 8)])
def test_units_without_a_gate(dtype, unit, experts, ff, shared):
    gen = torch.Generator().manual_seed(experts)
    tokens, inner = 19, experts * ff + shared
    up = torch.randn(tokens, inner + 3, generator=gen).to(DTYPES[dtype])
    weights = torch.rand(tokens, experts, generator=gen)
    weights[weights < 0.4] = 0.0
    hidden = torch.full((tokens, inner + 2), float("nan"), dtype=DTYPES[dtype], device=DEV)
    K.gated_experts(up.to(DEV), weights.to(DEV), None, experts, ff, shared, 0, hidden, unit=unit)
    act = plain.gelu_erf if unit == "gelu_erf" else plain.silu
    want = act(up.double()[:, :inner])
    want[:, :experts * ff] *= weights.double().repeat_interleave(ff, dim=1)
    assert rel_err(hidden[:, :inner], want) < (1e-6 if dtype == "float32" else 1e-2)
    assert float(hidden[:, inner:].float().abs().max()) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("hd,window", [(320, 0), (576, 70), (768, 0)])
def test_plain_attention_on_heads_beyond_256(dtype, hd, window):
    totals, counts, q_heads = [150, 9], [20, 9], 3
    case = PagedCase(totals, counts, 1, hd, DTYPES[dtype], DEV, seed=hd)
    gen = torch.Generator().manual_seed(7)
    q = (torch.randn(case.n_tokens, q_heads * hd, generator=gen) * 0.5).to(DTYPES[dtype])
    out = torch.zeros(case.n_tokens, q_heads * hd, dtype=DTYPES[dtype], device=DEV)
    args = K.attention_args(q.to(DEV), out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start, q_heads,
                            len(totals), max(counts), 1.0 / math.sqrt(hd), window)
    K.attention(args, DTYPES[dtype], False, impl="plain")
    assert rel_err(out, case.reference(q, q_heads, 1.0 / math.sqrt(hd), window)) < (1e-5 if dtype == "float32" else 2e-2)
