"""A plain, slow Rotutar in float64: whole sequences, no cache, one function per mechanism.

It shares no code with the package: configuration is read from the config.json dictionary as it
is, tensors by their checkpoint names.  Notation: x the residual stream [T, width], p the position
of a token in its sequence (from 0), H heads, S a head's state [dim, vdim].
"""

import math

import torch

F64 = torch.float64


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x, scale, groups, eps):
    """Each of `groups` equal consecutive parts of the last axis over its own root mean square; the
    whole times `scale`."""
    T, n = x.shape
    parts = unit_rms(x.view(T, groups, n // groups), eps)
    return parts.reshape(T, n) * scale


def turn_pairs(x, positions, rot):
    """x [T, heads, dim]: channels 2i and 2i + 1 (i < dims / 2) of every head are a pair, rotated by the
    angle p * base^(-2i / dims); channels from dims on stay."""
    if not rot or not rot.get("dims"):
        return x
    dims = rot["dims"]
    f = torch.tensor([rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    angle = positions.to(F64)[:, None] * f[None, :]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def window_attention(h, w, prefix, sizes, eps):
    """Softmax attention over the last mask.size positions, with a learned logit per head in the
    denominator that has no key and no value."""
    T = h.shape[0]
    H, G, D, V = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    positions = torch.arange(T)
    q = unit_rms(h @ w[prefix + "q"].T, eps) * w[prefix + "q.norm"]          # over the whole projection
    k = unit_rms(h @ w[prefix + "k"].T, eps) * w[prefix + "k.norm"]
    q = turn_pairs(q.view(T, H, D), positions, sizes.get("rot"))
    k = turn_pairs(k.view(T, G, D), positions, sizes.get("rot"))
    v = (h @ w[prefix + "v"].T).view(T, G, V)
    distance = positions[:, None] - positions[None, :]
    seen = distance >= 0
    if sizes.get("mask") and sizes["mask"].get("size"):
        seen = seen & (distance < sizes["mask"]["size"])
    out = torch.zeros(T, H, V, dtype=F64)
    for head in range(H):
        shared = head // (H // G)
        scores = (q[:, head] @ k[:, shared].T) * sizes["scale"]
        scores = scores.masked_fill(~seen, -math.inf)
        sink = w[prefix + "sink"][head] if prefix + "sink" in w else None
        top = scores.max(-1, keepdim=True).values
        if sink is not None:
            top = torch.maximum(top, sink.expand_as(top))
        e = torch.exp(scores - top)
        denominator = e.sum(-1, keepdim=True)
        if sink is not None:
            denominator = denominator + torch.exp(sink - top)
        out[:, head] = (e / denominator) @ v[:, shared]
    return out.reshape(T, H * V) @ w[prefix + "o"].T


def short_conv(x, taps_weight):
    """Per channel, y[t] = sum_j taps[c, j] x[t - (taps - 1 - j)], zeros before the start; then silu."""
    T, _ = x.shape
    taps = taps_weight.shape[1]
    y = torch.zeros_like(x)
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            y[back:] += x[:T - back] * taps_weight[:, j]
    return silu(y)


def delta_rule(h, w, prefix, sizes, eps):
    """Per head S <- g * S (g per key channel); u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T = h.shape[0]
    H, G, D, V = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    q = short_conv(h @ w[prefix + "q"].T, w[prefix + "q.conv"]).view(T, G, D)
    k = short_conv(h @ w[prefix + "k"].T, w[prefix + "k.conv"]).view(T, G, D)
    v = short_conv(h @ w[prefix + "v"].T, w[prefix + "v.conv"]).view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = sigmoid(h @ w[prefix + "b"].T)                                                    # [T, H]
    low = (h @ w[prefix + "a1"].T) @ w[prefix + "a2"].T + w[prefix + "dt_bias"]
    decay = torch.exp(-torch.exp(w[prefix + "A_log"])[None, :, None] * softplus(low).view(T, H, D))
    gate = sigmoid((h @ w[prefix + "g1"].T) @ w[prefix + "g2"].T).view(T, H, V)
    out = torch.zeros(T, H, V, dtype=F64)
    for head in range(H):
        shared = head // (H // G)
        S = torch.zeros(D, V, dtype=F64)
        for t in range(T):
            S = decay[t, head][:, None] * S
            kt = k[t, shared]
            u = beta[t, head] * (v[t, head] - S.T @ kt)
            S = S + kt[:, None] * u[None, :]
            out[t, head] = S.T @ q[t, shared]
    out = unit_rms(out, eps) * w[prefix + "norm"] * gate
    return out.reshape(T, H * V) @ w[prefix + "o"].T


def parallel(h, w, prefix, sizes, eps):
    left = window_attention(h, w, prefix + "left.", sizes["left"], eps)
    right = delta_rule(h, w, prefix + "right.", sizes["right"], eps)
    return sizes["left_scale"] * left + sizes["right_scale"] * right


def hgrn2(h, w, prefix, sizes, eps):
    """S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, o_t = S_t^T q_t, with a lower bound on f."""
    T = h.shape[0]
    H, D, V = sizes["heads"], sizes["dim"], sizes["vdim"]
    q = silu(h @ w[prefix + "q"].T).view(T, H, D)
    v = (h @ w[prefix + "v"].T).view(T, H, V)
    lower = w[prefix + "lower"]
    f = (lower + (1.0 - lower) * sigmoid(h @ w[prefix + "f"].T + w[prefix + "f.b"])).view(T, H, D)
    out = torch.zeros(T, H, V, dtype=F64)
    for head in range(H):
        S = torch.zeros(D, V, dtype=F64)
        for t in range(T):
            S = f[t, head][:, None] * S + (1.0 - f[t, head])[:, None] * v[t, head][None, :]
            out[t, head] = S.T @ q[t, head]
    out = unit_rms(out, eps) * w[prefix + "norm"]
    return out.reshape(T, H * V) @ w[prefix + "o"].T


def dense(h, w, prefix):
    return (silu(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


def choose(scores, router):
    """The experts one token uses: the `top` largest scores among the experts of the best groups (a
    group's score is the sum of its two largest); lowest index among equals."""
    n, top = router["experts"], router["top"]
    allowed = torch.ones(n, dtype=torch.bool)
    groups = router.get("groups")
    if groups and groups.get("count", 0) > 1:
        size = n // groups["count"]
        ranks = []
        for g in range(groups["count"]):
            part = torch.sort(scores[g * size:(g + 1) * size], descending=True).values
            ranks.append(float(part[:2].sum()))
        order = sorted(range(groups["count"]), key=lambda g: (-ranks[g], g))
        allowed[:] = False
        for g in order[:groups["keep"]]:
            allowed[g * size:(g + 1) * size] = True
    order = sorted((e for e in range(n) if allowed[e]), key=lambda e: (-float(scores[e]), e))
    return order[:top]


def experts(h, w, prefix, mlp):
    router, limit = mlp["router"], mlp["expert"]["limit"]
    scores = sigmoid(h @ w[prefix + "router"].T)
    out = torch.zeros(h.shape[0], w[prefix + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for e in choose(scores[t], router):
            g = torch.clamp(h[t] @ w[f"{prefix}e{e}.gate"].T, max=limit)
            u = torch.clamp(h[t] @ w[f"{prefix}e{e}.up"].T, -limit, limit)
            y = g * sigmoid(1.702 * g) * (u + 1.0)
            out[t] += scores[t, e] * (w[f"{prefix}e{e}.down"] @ y)
    return out


def feed_forward(h, w, prefix, mlp):
    return dense(h, w, prefix) if mlp["kind"] == "dense" else experts(h, w, prefix, mlp)


def mixer(h, w, prefix, layer, eps):
    if layer["type"] == "hgrn2":
        return hgrn2(h, w, prefix, layer["mixer"], eps)
    if layer["type"] == "parallel":
        return parallel(h, w, prefix, layer["mixer"], eps)
    raise ValueError(layer["type"])


def forward(ids, weights, config, streams=None):
    """float64 logits [T, vocab] of one whole sequence; `streams`, a list, receives the residual stream
    after every layer."""
    w = {name: tensor.to(F64) for name, tensor in weights.items()}
    eps, groups = config["norm"]["eps"], config["norm"]["groups"]
    x = w["embed"][torch.as_tensor(ids)]
    for index, layer in enumerate(config["layers"]):
        p = f"l{index}."
        out = mixer(x, w, p + "mix.", layer, eps) * sigmoid(x @ w[p + "rg1"].T + w[p + "rg1.b"])
        x = x + group_norm(out, w[p + "norm1"], groups, eps)
        if layer.get("mlp") is not None:
            out = feed_forward(x, w, p + "mlp.", layer["mlp"]) * sigmoid(x @ w[p + "rg2"].T + w[p + "rg2.b"])
            x = x + group_norm(out, w[p + "norm2"], groups, eps)
        if streams is not None:
            streams.append(x.clone())
    logits = group_norm(x, w["final.norm"], groups, eps) @ w["head"].T
    cap = config.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


def greedy(ids, weights, config, new_tokens):
    """The `new_tokens` tokens with the largest logit, each fed back."""
    ids, made = list(ids), []
    for _ in range(new_tokens):
        token = int(forward(ids, weights, config)[-1].argmax())
        made.append(token)
        ids.append(token)
    return made
