"""A plain, slow Gavasun in float64: whole sequences, no cache, one function per mechanism.

It shares no code with the package: configuration is read from the config.json dictionary as it
is, tensors by their checkpoint names.  Notation: x the residual stream [T, width], p the position
of a token in its sequence (from 0), H query heads, G shared key/value heads, S a head's state
[dim, vdim], c the key/value latent of latent attention.
"""

import math

import torch

F64 = torch.float64


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, stored, eps):
    """The layers' norm: its scale is stored as the distance from one."""
    return unit_rms(x, eps) * (1.0 + stored)


def frequencies(rot):
    """(f [dims / 2], amplitude): f_i = base^(-2i / dims); with `scaling`, waves longer than
    original / slow turns are slowed by `factor`, those shorter than original / fast turns are kept,
    a linear ramp over the pair index between, and sine and cosine grow by 0.1 ln(factor) + 1."""
    dims, base = rot["dims"], rot["base"]
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    scaling = rot.get("scaling")
    if not scaling:
        return f, 1.0
    factor, original = scaling["factor"], scaling["original"]

    def pair_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(scaling["fast"])), 0)
    hi = min(math.ceil(pair_of(scaling["slow"])), dims - 1)
    i = torch.arange(dims // 2, dtype=F64)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def turn(x, positions, rot, pairing):
    """x [T, heads, n]: the first rot.dims channels of every head in pairs, (i, i + dims / 2) for
    "halves", (2i, 2i + 1) for "neighbours", each rotated by p * f_i; the rest stays."""
    if not rot or not rot.get("dims"):
        return x
    dims = rot["dims"]
    f, amplitude = frequencies(rot)
    angle = positions.to(F64)[:, None] * f[None, :]
    cos, sin = (torch.cos(angle) * amplitude)[:, None, :], (torch.sin(angle) * amplitude)[:, None, :]
    first = slice(0, dims // 2) if pairing == "halves" else slice(0, dims, 2)
    second = slice(dims // 2, dims) if pairing == "halves" else slice(1, dims, 2)
    u, v = x[..., first], x[..., second]
    out = x.clone()
    out[..., first] = u * cos - v * sin
    out[..., second] = v * cos + u * sin
    return out


def short_conv(x, taps_weight):
    """Per channel, y[t] = sum_j taps[c, j] x[t - (taps - 1 - j)], zeros before the start."""
    T, _ = x.shape
    taps = taps_weight.shape[1]
    y = torch.zeros_like(x)
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            y[back:] += x[:T - back] * taps_weight[:, j]
    return y


def softmax_over(scores, seen):
    scores = scores.masked_fill(~seen, -math.inf)
    e = torch.exp(scores - scores.max(-1, keepdim=True).values)
    return e / e.sum(-1, keepdim=True)


def chunk_attention(h, w, prefix, sizes, eps):
    """Biased projections, a short convolution on each, norms over the whole query and key
    projections, halves turned together, keys of the query's own chunk only."""
    T = h.shape[0]
    H, G, D, V = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    positions = torch.arange(T)
    rows = {}
    for name in ("q", "k", "v"):
        y = h @ w[prefix + name].T + w[prefix + name + ".b"]
        if prefix + name + ".conv" in w:
            y = short_conv(y, w[prefix + name + ".conv"])
        rows[name] = y
    q = unit_rms(rows["q"], eps) * w[prefix + "q.norm"]
    k = unit_rms(rows["k"], eps) * w[prefix + "k.norm"]
    q = turn(q.view(T, H, D), positions, sizes.get("rot"), "halves")
    k = turn(k.view(T, G, D), positions, sizes.get("rot"), "halves")
    v = rows["v"].view(T, G, V)
    seen = positions[:, None] >= positions[None, :]
    if sizes.get("mask") and sizes["mask"].get("size"):
        c = sizes["mask"]["size"]
        seen = seen & ((positions[:, None] // c) == (positions[None, :] // c))
    out = torch.zeros(T, H, V, dtype=F64)
    for head in range(H):
        shared = head // (H // G)
        p = softmax_over((q[:, head] @ k[:, shared].T) * sizes["scale"], seen)
        out[:, head] = p @ v[:, shared]
    return out.reshape(T, H * V) @ w[prefix + "o"].T


def latent_attention(h, w, prefix, sizes, eps):
    """Queries and keys/values through normalised latents; one turned key part for all heads beside
    each head's own unturned keys; the last mask.size positions are seen."""
    T = h.shape[0]
    H, D, R, V, rank = sizes["heads"], sizes["dim"], sizes["rot_dim"], sizes["vdim"], sizes["kv_rank"]
    positions = torch.arange(T)
    rot = dict(sizes["rot"], dims=R) if sizes.get("rot") else None
    c_q = unit_rms(h @ w[prefix + "dq"].T, eps) * w[prefix + "dq.norm"]
    q = (c_q @ w[prefix + "uq"].T).view(T, H, D + R)
    q_plain, q_turned = q[..., :D], turn(q[..., D:], positions, rot, "neighbours")
    down = h @ w[prefix + "dkv"].T
    c = unit_rms(down[:, :rank], eps) * w[prefix + "dkv.norm"]
    k_turned = turn(down[:, None, rank:], positions, rot, "neighbours")[:, 0]          # [T, R]
    k_plain = (c @ w[prefix + "uk"].T).view(T, H, D)
    v = (c @ w[prefix + "uv"].T).view(T, H, V)
    distance = positions[:, None] - positions[None, :]
    seen = distance >= 0
    if sizes.get("mask") and sizes["mask"].get("size"):
        seen = seen & (distance < sizes["mask"]["size"])
    out = torch.zeros(T, H, V, dtype=F64)
    for head in range(H):
        scores = (q_plain[:, head] @ k_plain[:, head].T + q_turned[:, head] @ k_turned.T) * sizes["scale"]
        out[:, head] = softmax_over(scores, seen) @ v[:, head]
    return out.reshape(T, H * V) @ w[prefix + "o"].T


def delta_rule(h, w, prefix, sizes, eps):
    """Per head S <- g S (one g a head); u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T = h.shape[0]
    H, G, D, V = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    q = silu(short_conv(h @ w[prefix + "q"].T, w[prefix + "q.conv"])).view(T, G, D)
    k = silu(short_conv(h @ w[prefix + "k"].T, w[prefix + "k.conv"])).view(T, G, D)
    v = silu(short_conv(h @ w[prefix + "v"].T, w[prefix + "v.conv"])).view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = sigmoid(h @ w[prefix + "b"].T)                                                    # [T, H]
    decay = torch.exp(-torch.exp(w[prefix + "A_log"]) * softplus(h @ w[prefix + "a"].T + w[prefix + "dt_bias"]))
    out = torch.zeros(T, H, V, dtype=F64)
    for head in range(H):
        shared = head // (H // G)
        S = torch.zeros(D, V, dtype=F64)
        for t in range(T):
            S = decay[t, head] * S
            kt = k[t, shared]
            u = beta[t, head] * (v[t, head] - S.T @ kt)
            S = S + kt[:, None] * u[None, :]
            out[t, head] = S.T @ q[t, shared]
    out = unit_rms(out, eps) * w[prefix + "norm"] * silu(h @ w[prefix + "g"].T).view(T, H, V)
    return out.reshape(T, H * V) @ w[prefix + "o"].T


def dense(h, w, prefix):
    return (silu(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


def unit(h, w, prefix):
    return gelu_erf(h @ w[prefix + "up"].T) @ w[prefix + "down"].T


def experts(h, w, prefix, mlp):
    top = mlp["router"]["top"]
    z = h @ w[prefix + "router"].T
    scores = torch.softmax(z, -1)
    out = torch.zeros(h.shape[0], h.shape[1], dtype=F64)
    for t in range(h.shape[0]):
        chosen = sorted(range(scores.shape[1]), key=lambda e: (-float(scores[t, e]), e))[:top]
        total = sum(scores[t, e] for e in chosen) + 1e-20
        for e in chosen:
            out[t] += scores[t, e] / total * unit(h[t:t + 1], w, f"{prefix}e{e}.")[0]
    if mlp.get("shared"):
        out = out + unit(h, w, prefix + "shared.")
    return out


def feed_forward(h, w, prefix, mlp):
    return dense(h, w, prefix) if mlp["kind"] == "dense" else experts(h, w, prefix, mlp)


MIXERS = {"attention": chunk_attention, "latent_attention": latent_attention, "delta": delta_rule}


def runs(config):
    """The layers in the order they run: a looped stretch several times over."""
    count, loop = len(config["layers"]), config.get("loop")
    if not loop:
        return list(range(count))
    stretch = list(range(loop["start"], loop["stop"]))
    return list(range(loop["start"])) + stretch * loop["times"] + list(range(loop["stop"], count))


def forward(ids, weights, config, streams=None):
    """float64 logits [T, vocab] of one whole sequence; `streams`, a list, receives the residual stream
    after every run of a layer."""
    w = {name: tensor.to(F64) for name, tensor in weights.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.as_tensor(ids)] * config["embedding"]["scale"]
    for index in runs(config):
        layer, p = config["layers"][index], f"l{index}."
        x = x + MIXERS[layer["type"]](layer_norm(x, w[p + "norm1"], eps), w, p + "mix.", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            x = x + feed_forward(layer_norm(x, w[p + "norm2"], eps), w, p + "mlp.", layer["mlp"])
        if streams is not None:
            streams.append(x.clone())
    return layer_norm(x, w["final.norm"], eps) @ w["head"].T


def greedy(ids, weights, config, new_tokens):
    """The `new_tokens` tokens with the largest logit, each fed back."""
    ids, made = list(ids), []
    for _ in range(new_tokens):
        token = int(forward(ids, weights, config)[-1].argmax())
        made.append(token)
        ids.append(token)
    return made
