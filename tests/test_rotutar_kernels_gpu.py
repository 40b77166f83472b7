"""The kernels that came with Rotutar's mechanisms, each alone against float64: the scans with a matrix state
(forget gate, delta rule), the head norm with a gate, the norm in parts of a sublayer's output with its gate and
two weighted terms, capped logits, the sigmoid router with groups ranked by their two best, the clamped experts'
unit, the root mean square over a whole projection with neighbouring channels turned, the embedding's copy, and a
sink in every attention kernel, with one dominant key placed just inside and just outside the window."""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu

import plain_rotutar as plain  # noqa: E402
from burn_transformers_amd.kernels import library as K  # noqa: E402
from kernel_helpers import PagedCase  # noqa: E402
from step_helpers import make_step  # noqa: E402

DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F64 = torch.float64


def rel_err(got, want):
    got = got.detach().cpu().double()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


def spans_of(lengths, cuts):
    """Steps of several sequences: every sequence is cut at ``cuts`` (positions), a step brings each sequence's
    next span (sequences that have ended drop out)."""
    bounds = [[0] + [c for c in cuts if c < n] + [n] for n in lengths]
    steps = []
    for k in range(max(len(b) for b in bounds) - 1):
        steps.append([(s, b[k], b[k + 1]) for s, b in enumerate(bounds) if k + 1 < len(b)])
    return steps


@pytest.mark.parametrize("heads,dim,vdim,lengths,cuts,spans", [
    (2, 16, 32, [150, 7, 66], [1, 3, 64, 65, 130], False), (3, 12, 20, [150, 7, 66], [1, 3, 64, 65, 130], False),
    (1, 36, 4, [150, 7, 66], [1, 3, 64, 65, 130], False), (2, 64, 48, [150, 7, 66], [1, 3, 64, 65, 130], False),
    (1, 200, 70, [150, 7, 66], [1, 3, 64, 65, 130], False), (4, 8, 8, [150, 7, 66], [1, 3, 64, 65, 130], False),
    (2, 16, 32, [700, 40, 330], [5, 505], True), (1, 128, 20, [450, 193, 1], [200], True)])
def test_forget_gate_scan_in_portions(heads, dim, vdim, lengths, cuts, spans):
    """S <- diag(f) S + (1 - f) v^T, o = S^T silu(q): three sequences in slots of their own, cut into portions of
    unequal length, down to one token, from the state the last portion left; with room for it, long portions are
    scanned in spans side by side (beside short ones that are not cut, from a state that is not zero)."""
    gen = torch.Generator().manual_seed(heads * 100 + dim)
    qk, inner = heads * dim, heads * vdim
    seqs = [torch.randn(n, 2 * qk + inner, generator=gen) for n in lengths]
    f_bias, lower = torch.randn(qk, generator=gen), torch.rand(qk, generator=gen) * 0.9
    want = []
    for rows in seqs:
        q = plain.silu(rows[:, :qk].double()).view(-1, heads, dim)
        f = (lower.double() + (1.0 - lower.double()) * plain.sigmoid(rows[:, qk:2 * qk].double() + f_bias.double())).view(-1, heads, dim)
        v = rows[:, 2 * qk:].double().view(-1, heads, vdim)
        out = torch.zeros(rows.shape[0], heads, vdim, dtype=F64)
        for h in range(heads):
            S = torch.zeros(dim, vdim, dtype=F64)
            for t in range(rows.shape[0]):
                S = f[t, h][:, None] * S + (1.0 - f[t, h])[:, None] * v[t, h][None, :]
                out[t, h] = S.T @ q[t, h]
        want.append(out.reshape(rows.shape[0], inner))
    slots = [3, 0, 1]
    state = torch.zeros(4, heads * dim * ((vdim + 3) // 4 * 4), device=DEV)
    got = [torch.zeros(n, inner, dtype=F64) for n in lengths]
    for step_spans in spans_of(lengths, cuts):
        step = make_step(torch.float32, [b - a for _, a, b in step_spans], starts=[a for _, a, _ in step_spans],
                         slots=[slots[s] for s, _, _ in step_spans])
        rows = torch.cat([seqs[s][a:b] for s, a, b in step_spans]).to(DEV)
        y = torch.full((rows.shape[0], inner + 2), float("nan"), device=DEV)
        carry = K.scan_carry(step, state.shape[1], heads * dim) if spans else None
        assert not spans or step.max_count < 192 or carry is not None
        K.keyed_scan(rows[:, :qk], None, rows[:, 2 * qk:], rows[:, qk:2 * qk], y, state, step, heads, heads, dim, vdim,
                     "forget", g_bias=f_bias.to(DEV), lower=lower.to(DEV), carry=carry)
        at = 0
        for s, a, b in step_spans:
            got[s][a:b] = y[at:at + b - a, :inner].cpu().double()
            at += b - a
    for g, w in zip(got, want):
        assert rel_err(g, w) < 5e-6


@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(4, 2, 16, 24), (2, 1, 20, 12), (3, 3, 40, 8), (2, 2, 128, 32), (1, 1, 200, 70)])
def test_delta_rule_scan_in_portions(heads, kv_heads, dim, vdim):
    """S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q with unit keys and queries per head."""
    gen = torch.Generator().manual_seed(heads * 100 + dim)
    lengths, qk, inner, decays = [140, 5, 70], kv_heads * dim, heads * vdim, heads * dim
    seqs = [torch.randn(n, 2 * qk + inner + decays + heads, generator=gen) for n in lengths]
    A_log = torch.log(torch.rand(heads, generator=gen) * 3.0 + 0.5)
    want = []
    for rows in seqs:
        r = rows.double()
        q, k = r[:, :qk].view(-1, kv_heads, dim), r[:, qk:2 * qk].view(-1, kv_heads, dim)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        v = r[:, 2 * qk:2 * qk + inner].view(-1, heads, vdim)
        dt = r[:, 2 * qk + inner:2 * qk + inner + decays].abs().view(-1, heads, dim) * 0.2
        beta = plain.sigmoid(r[:, 2 * qk + inner + decays:])
        out = torch.zeros(rows.shape[0], heads, vdim, dtype=F64)
        for h in range(heads):
            j, S = h // (heads // kv_heads), torch.zeros(dim, vdim, dtype=F64)
            for t in range(rows.shape[0]):
                S = torch.exp(-torch.exp(A_log[h].double()) * dt[t, h])[:, None] * S
                u = beta[t, h] * (v[t, h] - S.T @ k[t, j])
                S = S + k[t, j][:, None] * u[None, :]
                out[t, h] = S.T @ q[t, j]
        want.append(out.reshape(rows.shape[0], inner))
    slots = [2, 1, 0]
    state = torch.zeros(3, heads * dim * ((vdim + 3) // 4 * 4) + 5, device=DEV)
    got = [torch.zeros(n, inner, dtype=F64) for n in lengths]
    for step_spans in spans_of(lengths, [2, 3, 64, 129]):
        step = make_step(torch.float32, [b - a for _, a, b in step_spans], starts=[a for _, a, _ in step_spans],
                         slots=[slots[s] for s, _, _ in step_spans])
        rows = torch.cat([seqs[s][a:b] for s, a, b in step_spans]).to(DEV)
        dt = (rows[:, 2 * qk + inner:2 * qk + inner + decays].abs() * 0.2).contiguous()
        y = torch.full((rows.shape[0], inner), float("nan"), device=DEV)
        K.keyed_scan(rows[:, :qk], rows[:, qk:2 * qk], rows[:, 2 * qk:2 * qk + inner], dt, y, state, step, heads, kv_heads,
                     dim, vdim, "delta", beta=rows[:, 2 * qk + inner + decays:], A_log=A_log.to(DEV), unit=True,
                     unit_eps=1e-6, q_scale=dim ** -0.5)
        at = 0
        for s, a, b in step_spans:
            got[s][a:b] = y[at:at + b - a].cpu().double()
            at += b - a
    for g, w in zip(got, want):
        assert rel_err(g, w) < 2e-5


def test_delta_rule_takes_off_what_the_state_answers():
    """Inputs made so that the rule shows: with beta = 1 and no decay, writing the same unit key twice leaves the
    second value alone in the state (a plain sum would hold both)."""
    dim, vdim = 16, 8
    k = torch.zeros(2, dim)
    k[:, 3] = 5.0
    v = torch.tensor([[1.0] * vdim, [7.0] * vdim])
    q = k.clone()
    beta = torch.full((2, 1), 40.0)                   # sigmoid -> 1
    dt = torch.zeros(2, dim)                          # decay exp(0) = 1
    state = torch.zeros(1, dim * vdim, device=DEV)
    y = torch.empty(2, vdim, device=DEV)
    step = make_step(torch.float32, [2])
    K.keyed_scan(q.to(DEV), k.to(DEV), v.to(DEV), dt.to(DEV), y, state, step, 1, 1, dim, vdim, "delta", beta=beta.to(DEV),
                 A_log=torch.zeros(1, device=DEV), unit=True, unit_eps=1e-6, q_scale=1.0)
    assert float((y[0].cpu() - 1.0).abs().max()) < 1e-4 and float((y[1].cpu() - 7.0).abs().max()) < 1e-4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,vdim,gated", [(4, 24, True), (3, 20, False), (1, 70, True), (5, 128, True)])
def test_head_norm_with_a_gate(dtype, heads, vdim, gated):
    gen = torch.Generator().manual_seed(vdim)
    y = torch.randn(19, heads * vdim + 3, generator=gen) * 3.0
    gate = torch.randn(19, heads * vdim, generator=gen)
    weight = torch.randn(vdim, generator=gen) + 1.0
    cols = (heads * vdim + 7) // 8 * 8
    out = torch.full((19, cols), float("nan"), dtype=DTYPES[dtype], device=DEV)
    K.head_norm_gate(y.to(DEV)[:, :heads * vdim], weight.to(DEV), heads, vdim, 1e-3, out, gate=gate.to(DEV) if gated else None)
    rows = plain.unit_rms(y[:, :heads * vdim].double().view(19, heads, vdim), 1e-3) * weight.double()
    if gated:
        rows = rows * plain.sigmoid(gate.double()).view(19, heads, vdim)
    want = torch.zeros(19, cols, dtype=F64)
    want[:, :heads * vdim] = rows.reshape(19, -1)
    assert rel_err(out, want) < (2e-6 if dtype == "float32" else 5e-3)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("width,groups,two,gated", [(64, 2, True, True), (40, 1, False, True), (40, 5, True, False),
                                                  (96, 3, False, False), (192, 64, True, True)])
def test_norm_in_parts_of_a_sublayers_output(dtype, width, groups, two, gated):
    """x += N(gate * (a * (sum of partials + bias) + b * (sum of other partials))), N in equal parts of the row."""
    gen = torch.Generator().manual_seed(width + groups)
    tokens = 23
    x = torch.randn(tokens, width, generator=gen)
    d1, d2 = torch.randn(3, tokens, width, generator=gen), torch.randn(2, tokens, width, generator=gen)
    bias, gate, gamma = torch.randn(width, generator=gen), torch.randn(tokens, width, generator=gen), torch.randn(width, generator=gen) + 1.0
    v = 0.7 * (d1.double().sum(0) + bias.double())
    if two:
        v = v + 1.3 * d2.double().sum(0)
    if gated:
        v = v * plain.sigmoid(gate.double())
    want = x.double() + 0.5 * plain.group_norm(v, gamma.double(), groups, 1e-4)
    xs = x.to(DEV).clone()
    cols = (width + 7) // 8 * 8 + 8
    cast = torch.full((tokens, cols), float("nan"), dtype=DTYPES[dtype], device=DEV)
    K.group_norm_output(xs, gamma.to(DEV), groups, 1e-4, d1.to(DEV), bias.to(DEV), 0.7, d2.to(DEV) if two else None, None, 1.3,
                        gate=gate.to(DEV) if gated else None, mult=0.5, cast=cast)
    assert rel_err(xs, want) < 2e-6
    assert rel_err(cast[:, :width], want) < (2e-6 if dtype == "float32" else 5e-3) and float(cast[:, width:].abs().max()) == 0.0
    # rows of the stream itself, chosen ones
    rows = torch.tensor([5, 0, 22], dtype=torch.int32, device=DEV)
    out = torch.full((3, cols), float("nan"), dtype=DTYPES[dtype], device=DEV)
    K.group_norm_rows(xs, gamma.to(DEV), groups, 1e-4, out, rows=rows)
    picked = plain.group_norm(want[[5, 0, 22]], gamma.double(), groups, 1e-4)
    assert rel_err(out[:, :width], picked) < (4e-6 if dtype == "float32" else 5e-3)


def test_capped_logits():
    gen = torch.Generator().manual_seed(0)
    logits = torch.randn(5, 3001, generator=gen) * 40.0
    got = logits.to(DEV)[:, :3000]
    K.soft_cap(got, 30.0)
    assert rel_err(got, 30.0 * torch.tanh(logits[:, :3000].double() / 30.0)) < 1e-6


def plain_weights(h, router, mlp_router):
    scores = plain.sigmoid(h.double() @ router.double().T)
    out = torch.zeros_like(scores)
    for t in range(h.shape[0]):
        for e in plain.choose(scores[t], mlp_router):
            out[t, e] = scores[t, e]
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("experts,top,groups,keep,width", [(12, 3, 3, 2, 64), (5, 1, 0, 0, 40), (4, 4, 2, 2, 32),
                                                           (6, 2, 6, 3, 96), (64, 6, 8, 3, 128), (9, 2, 3, 1, 24)])
def test_sigmoid_router_with_groups_ranked_by_their_two_best(dtype, experts, top, groups, keep, width):
    gen = torch.Generator().manual_seed(experts)
    h = torch.randn(41, width, generator=gen).to(DTYPES[dtype])
    router = torch.randn(experts, width, generator=gen) * (1.5 / math.sqrt(width))
    weights = torch.full((41, experts), float("nan"), device=DEV)
    K.route(h.to(DEV), router.to(DEV), None, top, groups, keep, weights, score="sigmoid", group_rank=2, normalize=False)
    want = plain_weights(h.float(), router, {"experts": experts, "top": top,
                                             "groups": {"count": groups, "keep": keep} if groups else None})
    assert torch.equal(weights.cpu() != 0, want != 0), "another expert was chosen"
    assert float((weights.cpu().double() - want).abs().max()) < 2e-6


def test_a_groups_rank_is_the_sum_of_its_two_best():
    """Made so that the rule shows: the best single expert sits in a group whose second best is low, and two groups
    with two good experts each shut it out."""
    width = 8
    h = torch.zeros(1, width)
    h[0, 0] = 1.0
    logits = torch.tensor([3.0, -4.0, -4.0, 1.0, 0.9, -4.0, 0.8, 0.7, -4.0])      # three groups of three
    router = torch.zeros(9, width)
    router[:, 0] = logits
    weights = torch.empty(1, 9, device=DEV)
    K.route(h.to(DEV), router.to(DEV), None, 2, 3, 2, weights, score="sigmoid", group_rank=2, normalize=False)
    want = torch.zeros(9, dtype=F64)
    want[3], want[4] = plain.sigmoid(logits[3].double()), plain.sigmoid(logits[4].double())
    assert float((weights.cpu().double()[0] - want).abs().max()) < 1e-6
    K.route(h.to(DEV), router.to(DEV), None, 2, 3, 2, weights, score="sigmoid", group_rank=1, normalize=False)
    assert float(weights[0, 0]) > 0.9                 # ranked by its best alone, the first group stays open


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_clamped_experts_unit(dtype):
    gen = torch.Generator().manual_seed(3)
    experts, ff, tokens, limit = 3, 20, 9, 0.8
    gu = (torch.randn(tokens, 2 * experts * ff, generator=gen) * 1.5).to(DTYPES[dtype])
    weights = torch.rand(tokens, experts, generator=gen)
    weights[:, 1] = 0.0
    hidden = torch.full((tokens, experts * ff + 4), float("nan"), dtype=DTYPES[dtype], device=DEV)
    K.gated_experts(gu.to(DEV), weights.to(DEV), None, experts, ff, 0, 0, hidden, limit=limit, alpha=1.702)
    x = gu.double().view(tokens, experts, 2, ff)
    g, u = torch.clamp(x[:, :, 0], max=limit), torch.clamp(x[:, :, 1], -limit, limit)
    want = torch.zeros(tokens, experts * ff + 4, dtype=F64)
    want[:, :experts * ff] = (weights.double()[:, :, None] * g * plain.sigmoid(1.702 * g) * (u + 1.0)).reshape(tokens, -1)
    assert rel_err(hidden, want) < (2e-6 if dtype == "float32" else 5e-3)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,rot", [(4, 2, 16, 32, 8), (3, 3, 24, 10, 24), (6, 1, 8, 8, 0), (2, 1, 144, 20, 100)])
def test_whole_projection_norm_and_neighbours_turned_into_the_cache(dtype, heads, kv_heads, dim, vdim, rot):
    dt = DTYPES[dtype]
    hd = (max(dim, vdim) + 15) // 16 * 16
    totals, counts = [70, 5, 131], [70, 2, 3]
    case = PagedCase(totals, counts, kv_heads, hd, dt, DEV, seed=1)
    gen = torch.Generator().manual_seed(2)
    cols = (heads + kv_heads) * dim + kv_heads * vdim
    fused = torch.randn(case.n_tokens, cols + 3, generator=gen)
    q_gamma, k_gamma = torch.randn(heads * dim, generator=gen) + 1.0, torch.randn(kv_heads * dim, generator=gen) + 1.0
    inv_freq = (1000.0 ** (-2.0 * torch.arange(rot // 2, dtype=F64) / max(rot, 1))).float()
    q_out = torch.full((case.n_tokens, heads * hd), float("nan"), dtype=dt, device=DEV)
    K.head_rotary(fused.to(DEV)[:, :cols], heads, kv_heads, dim, vdim, rot, inv_freq.to(DEV) if rot else None,
                  q_gamma.to(DEV), k_gamma.to(DEV), 1e-3, q_out, case.tok_seq, case.tok_pos, case.view(), dt,
                  neighbours=True, whole_norm=True)
    x, pos = fused.double(), case.tok_pos.cpu()

    def heads_of(first, count, size, gamma):
        rows = x[:, first:first + count * size]
        if gamma is not None:
            rows = plain.unit_rms(rows, 1e-3) * gamma.double()
        rows = rows.reshape(-1, count, size)
        if gamma is not None and rot:
            angle = (pos[:, None].float() * inv_freq[None, :]).double()          # the angle itself is a 32-bit product
            cos, sin = torch.cos(angle)[:, None], torch.sin(angle)[:, None]
            a, b = rows[..., 0:rot:2], rows[..., 1:rot:2]
            rows = rows.clone()
            rows[..., 0:rot:2], rows[..., 1:rot:2] = a * cos - b * sin, b * cos + a * sin
        out = torch.zeros(rows.shape[0], count, hd, dtype=F64)
        out[..., :size] = rows
        return out.reshape(rows.shape[0], count * hd)

    bound = 2e-6 if dtype == "float32" else 6e-3
    assert rel_err(q_out, heads_of(0, heads, dim, q_gamma)) < bound
    k_all, v_all = case.read_back()
    step_rows, at = [], 0
    for total, count in zip(totals, counts):
        step_rows += list(range(at + total - count, at + total))
        at += total
    assert rel_err(k_all[step_rows], heads_of(heads * dim, kv_heads, dim, k_gamma)) < bound
    assert rel_err(v_all[step_rows], heads_of((heads + kv_heads) * dim, kv_heads, vdim, None)) < bound


def test_angles_of_neighbouring_channels_are_pinned_by_a_shift_of_positions():
    """The plain rotation itself: turning by p then taking scores equals turning both by p + s (scores depend on
    the distance only), and channel 2i is paired with 2i + 1, not with i + dims / 2."""
    gen = torch.Generator().manual_seed(5)
    x = torch.randn(6, 1, 8, generator=gen, dtype=F64)
    rot = {"dims": 8, "base": 100.0}
    a, b = plain.turn_pairs(x, torch.arange(6), rot), plain.turn_pairs(x, torch.arange(6) + 11, rot)
    assert float(((a[:, 0] @ a[:, 0].T) - (b[:, 0] @ b[:, 0].T)).abs().max()) < 1e-12
    one = torch.zeros(1, 1, 8, dtype=F64)
    one[0, 0, 0] = 1.0
    turned = plain.turn_pairs(one, torch.tensor([1]), rot)[0, 0]
    assert abs(float(turned[0]) - math.cos(1.0)) < 1e-12 and abs(float(turned[1]) - math.sin(1.0)) < 1e-12
    assert float(turned[2:].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embedding_leaves_the_products_copy(dtype):
    gen = torch.Generator().manual_seed(1)
    dt = DTYPES[dtype]
    table = torch.randn(50, 20, generator=gen).to(dt)
    ids = torch.randint(0, 50, (13,), generator=gen, dtype=torch.int32)
    rows = torch.empty(13, 20, device=DEV)
    cast = torch.full((13, 24), float("nan"), dtype=dt, device=DEV)
    K.embed(ids.to(DEV), None, table.to(DEV), None, rows, cast=cast)
    assert torch.equal(rows.cpu(), table[ids.long()].float())
    assert torch.equal(cast[:, :20].cpu(), table[ids.long()]) and float(cast[:, 20:].abs().max()) == 0.0


def sink_reference(case, q, q_heads, scale, window, sink):
    """float64 attention of the step's queries over the last ``window`` keys, with exp(sink) in the denominator."""
    hd, group = case.head_dim, q_heads // case.kv_heads
    out = torch.zeros(case.n_tokens, q_heads * hd, dtype=F64)
    q = q.detach().cpu().double()
    row = 0
    for s, (total, count) in enumerate(zip(case.totals, case.counts)):
        k = case.k_rows[s].double().view(total, case.kv_heads, hd)
        v = case.v_rows[s].double().view(total, case.kv_heads, hd)
        for i in range(count):
            pos = total - count + i
            lo = max(0, pos - window + 1) if window else 0
            for h in range(q_heads):
                scores = (k[lo:pos + 1, h // group] @ q[row, h * hd:(h + 1) * hd]) * scale
                top = max(float(scores.max()), float(sink[h]) if sink is not None else -math.inf)
                e = torch.exp(scores - top)
                den = e.sum() + (math.exp(float(sink[h]) - top) if sink is not None else 0.0)
                out[row, h * hd:(h + 1) * hd] = (e / den) @ v[lo:pos + 1, h // group]
            row += 1
    return out


IMPLS = {"float32": ["plain", "tiled"], "bfloat16": ["plain", "mfma"]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("q_heads,kv_heads,hd,window", [(4, 2, 32, 24), (2, 2, 64, 64), (3, 1, 48, 100), (2, 1, 128, 7),
                                                        (6, 2, 48, 0), (2, 1, 128, 200), (4, 4, 16, 1)])
def test_attention_with_a_sink_in_a_window(dtype, q_heads, kv_heads, hd, window):
    """Prompts, portions that start inside a window, and single tokens, on every attention kernel; sinks from far
    below every score to far above."""
    dt = DTYPES[dtype]
    scale = 0.4 / math.sqrt(hd)
    sink = torch.linspace(-6.0, 5.0, q_heads)
    for totals, counts in (([130, 5, 300], [130, 5, 300]), ([250, 64, 201], [50, 3, 200]), ([257, 24, 100, 449], [1, 1, 1, 1]),
                           ([940, 600], [940, 152]), ([940, 897], [1, 1])):
        case = PagedCase(totals, counts, kv_heads, hd, dt, DEV, seed=4, poison=True)
        gen = torch.Generator().manual_seed(7)
        q = torch.randn(case.n_tokens, q_heads * hd, generator=gen).to(dt).to(DEV)
        want = sink_reference(case, q, q_heads, scale, window, sink)
        for impl in IMPLS[dtype]:
            for decode in ([False, True] if max(counts) == 1 and impl != "plain" else [max(counts) == 1]):
                out = torch.full((case.n_tokens, q_heads * hd), float("nan"), dtype=dt, device=DEV)
                args = K.attention_args(q, out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                                        q_heads, len(totals), max(counts), scale, window, sink=sink.to(DEV))
                K.attention(args, dt, decode=decode, impl=impl)
                assert rel_err(out, want) < (4e-6 if dtype == "float32" else 1.2e-2), (impl, decode, totals, counts)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [48, 64, 96, 200])
def test_one_dominant_key_just_inside_and_just_outside_the_window(dtype, window):
    """One key is made to take all the weight.  At the window's first position it must be found (the output is its
    value row, less the sink's share); one position earlier it must not be seen at all.  A sink made dominant
    instead leaves nearly nothing of any value."""
    dt, hd, total = DTYPES[dtype], 64, 5 * window + 11
    start = total - window                                      # the first position the last query sees
    for target, found in ((start, True), (start - 1, False), (total - 1, True), (0, False)):
        for counts in ([1], [window + 5], [total]):
            case = PagedCase([total], counts, 1, hd, dt, DEV, seed=target)
            case.k_rows[0][:] *= 0.05
            case.k_rows[0][target, 3] = 8.0
            seq = torch.zeros(total, dtype=torch.int32, device=DEV)
            pos = torch.arange(total, dtype=torch.int32, device=DEV)
            K.kv_copy(case.k_rows[0].to(DEV), case.v_rows[0].to(DEV), seq, pos, case.view(), True)
            q = torch.zeros(case.n_tokens, hd)
            q[-1, 3] = 8.0                                       # the last query looks for the key; the others look nowhere
            q = q.to(dt).to(DEV)
            for sink_value, drowned in ((0.0, False), (80.0, True)):
                sink = torch.tensor([sink_value])
                want = sink_reference(case, q, 1, 1.0, window, sink)
                hit = float((want[-1] - case.v_rows[0][target].double()).abs().max()) < 1e-3
                assert hit == (found and not drowned)
                if drowned:
                    assert float(want[-1].abs().max()) < 1e-6
                for impl in IMPLS[dtype]:
                    out = torch.empty(case.n_tokens, hd, dtype=dt, device=DEV)
                    args = K.attention_args(q, out, case.view(), case.tok_seq, case.tok_pos, case.seq_off, case.seq_start,
                                            1, 1, max(counts), 1.0, window, sink=sink.to(DEV))
                    K.attention(args, dt, decode=max(counts) == 1, impl=impl)
                    err = float((out[-1].cpu().double() - want[-1]).abs().max())
                    assert err < (1e-5 if dtype == "float32" else 1e-2) * max(1.0, float(want[-1].abs().max())), (target, counts, impl, sink_value)


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_short_convolution_without_a_bias_across_portions(taps):
    gen = torch.Generator().manual_seed(taps)
    channels, lengths = 20, [9, 3]
    seqs = [torch.randn(n, channels, generator=gen) for n in lengths]
    weight = torch.randn(channels, taps, generator=gen)
    want = [plain.short_conv(s.double(), weight.double()) for s in seqs]
    state = torch.zeros(3, max(1, (taps - 1) * channels), device=DEV)
    got = [torch.zeros(n, channels, dtype=F64) for n in lengths]
    for step_spans in spans_of(lengths, [1, 2, 4]):
        step = make_step(torch.float32, [b - a for _, a, b in step_spans], starts=[a for _, a, _ in step_spans],
                         slots=[[2, 0][s] for s, _, _ in step_spans])
        rows = torch.cat([seqs[s][a:b] for s, a, b in step_spans]).to(DEV)
        out = torch.empty_like(rows)
        K.causal_conv(rows, weight.to(DEV), None, out, state, step)
        at = 0
        for s, a, b in step_spans:
            got[s][a:b] = out[at:at + b - a].cpu().double()
            at += b - a
    for g, w in zip(got, want):
        assert rel_err(g, w) < 2e-6


@pytest.mark.parametrize("act", ["softplus", "sigmoid", "none"])
def test_low_rank_projection_with_an_activation(act):
    gen = torch.Generator().manual_seed(9)
    low, weight, bias = torch.randn(21, 6, generator=gen), torch.randn(50, 6, generator=gen), torch.randn(50, generator=gen)
    out = torch.empty(21, 50, device=DEV)
    K.dt_project(low.to(DEV), weight.to(DEV), bias.to(DEV) if act != "none" else None, out, act=act)
    z = low.double() @ weight.double().T + (bias.double() if act != "none" else 0.0)
    want = {"softplus": plain.softplus, "sigmoid": plain.sigmoid, "none": lambda v: v}[act](z)
    assert rel_err(out, want) < 2e-6
