"""Tiny Rotutar configurations and helpers shared by the tests of that family."""

import torch

import burn_transformers_amd as bt
import plain_rotutar as plain


def forget(heads, dim, vdim):
    return "hgrn2", {"heads": heads, "dim": dim, "vdim": vdim}


def window_attention(heads, kv_heads, dim, vdim, scale, rot_dims=None, base=10000.0, window=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
            "rot": {"dims": rot_dims, "base": base} if rot_dims else None, "mask": {"size": window} if window else None}


def delta(heads, kv_heads, dim, vdim, taps, rank=None):
    sizes = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps}
    if rank:
        sizes["rank"] = rank
    return sizes


def side_by_side(left, right, left_scale=1.0, right_scale=1.0):
    return "parallel", {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, ff, top, limit, groups=None):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "top": top, "groups": {"count": groups[0], "keep": groups[1]} if groups else None}}


def layer(mixer, mlp=None):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def model_config(layers, width=64, vocab=211, groups=2, eps=1e-5, cap=20.0):
    return {"architecture": "Rotutar", "vocab": vocab, "width": width, "logit_softcap": cap,
            "norm": {"eps": eps, "groups": groups}, "layers": layers}


# both kinds of layer and of feed-forward: values wider than keys, part of a head turned, a window that is no
# multiple of a tile, shared heads on both sides, experts in three groups of which two stay open
BASIC = model_config([layer(forget(2, 16, 32), dense(96)),
                      layer(side_by_side(window_attention(4, 2, 16, 32, 0.25, rot_dims=8, base=500.0, window=24),
                                         delta(4, 2, 16, 24, 3, rank=6), 0.7, 1.3), moe(6, 24, 3, 1.0, groups=(3, 2))),
                      layer(forget(4, 8, 8), moe(4, 16, 2, 2.0))])
# sizes the kernels do not divide, one part a row (the norm's groups), no cap, a layer without a feed-forward, the
# mixers side by side first, no rotation and no window in one layer, one tap, one expert a token, every expert chosen
ODD = model_config([layer(side_by_side(window_attention(3, 3, 24, 10, 0.2, rot_dims=24, base=100.0, window=7),
                                       delta(2, 1, 20, 12, 2, rank=5), 1.0, 0.5)),
                    layer(forget(3, 12, 20), moe(5, 12, 1, 0.5)),
                    layer(side_by_side(window_attention(6, 1, 8, 8, 0.4), delta(3, 3, 40, 8, 1, rank=3), 2.0, 1.0), dense(50)),
                    layer(forget(1, 36, 4), moe(3, 20, 3, 3.0, groups=(3, 3)))],
                   width=40, vocab=97, groups=1, eps=1e-3, cap=None)
# each mechanism alone: one layer, the other side of the pair switched off by its factor
FORGET_ONLY = model_config([layer(forget(3, 16, 24))], width=48, vocab=101, groups=3)
ATTENTION_ONLY = model_config([layer(side_by_side(window_attention(4, 2, 32, 32, 0.18, rot_dims=16, base=1000.0, window=40),
                                                  delta(1, 1, 8, 8, 2, rank=2), 1.0, 0.0))], width=64, vocab=101, groups=4)
DELTA_ONLY = model_config([layer(side_by_side(window_attention(1, 1, 16, 16, 0.25, window=5),
                                              delta(4, 2, 24, 16, 4, rank=8), 0.0, 1.0))], width=64, vocab=101, groups=1)
DENSE_ONLY = model_config([layer(forget(1, 8, 8), dense(72))], width=32, vocab=61, groups=2)
EXPERTS_ONLY = model_config([layer(forget(1, 8, 8), moe(8, 16, 2, 1.0, groups=(4, 2)))], width=32, vocab=61, groups=2)
# a window that spans several blocks of the cache, heads of 128 and of 64, states of 128 key channels
LONG = model_config([layer(side_by_side(window_attention(2, 1, 128, 64, 0.09, rot_dims=64, base=300000.0, window=200),
                                        delta(2, 2, 128, 32, 4, rank=8), 1.0, 1.0), dense(64)),
                     layer(forget(2, 64, 48), moe(4, 32, 2, 1.5))], width=96, vocab=151, groups=2)
# more query heads on a cached head than a decode tile takes; heads wider than any MFMA attention kernel's
MANY_HEADS = model_config([layer(side_by_side(window_attention(20, 1, 16, 16, 0.25, rot_dims=16, window=48),
                                              delta(2, 1, 16, 16, 2, rank=4), 1.0, 1.0), dense(24))], width=48, vocab=71, groups=2)
WIDE_HEADS = model_config([layer(side_by_side(window_attention(2, 1, 144, 20, 0.08, rot_dims=100, window=30),
                                              delta(1, 1, 200, 70, 3, rank=4), 1.0, 1.0))], width=32, vocab=53, groups=1)
# nothing a multiple of eight: a width of 36 in three parts, heads of 10, 12, 6 and 20, feed-forwards of 10 and 22
UNALIGNED = model_config([layer(forget(2, 10, 6), moe(3, 10, 2, 1.0)),
                          layer(side_by_side(window_attention(2, 1, 12, 20, 0.3, rot_dims=6, window=9),
                                             delta(2, 2, 10, 6, 3, rank=3), 1.0, 1.0), dense(22))], width=36, vocab=53, groups=3)
CONFIGS = {"unaligned": (UNALIGNED, 11), "basic": (BASIC, 1), "odd": (ODD, 2), "forget": (FORGET_ONLY, 3), "attention": (ATTENTION_ONLY, 4),
           "delta": (DELTA_ONLY, 5), "dense": (DENSE_ONLY, 6), "experts": (EXPERTS_ONLY, 7), "long": (LONG, 8),
           "many_heads": (MANY_HEADS, 9), "wide_heads": (WIDE_HEADS, 10)}

_weights, _models = {}, {}


def config_for(name, dtype="float32"):
    """The configuration a run uses.  bfloat16 runs let every token use every expert (``top`` = experts, every
    group open): with operands rounded to 8 bits a near tie between two experts' scores falls the other way now and
    then, the token's whole feed-forward output is then another, and no bound on rounding holds.  The weights, which
    are the experts' scores, still differ from token to token; the choice itself is made in the float32 runs, which
    go through the same kernels."""
    config = CONFIGS[name][0]
    if dtype != "bfloat16":
        return config
    layers = []
    for entry in config["layers"]:
        mlp = entry["mlp"]
        if mlp and mlp["kind"] == "moe":
            groups = mlp["router"]["groups"]
            router = dict(mlp["router"], top=mlp["router"]["experts"],
                          groups=dict(groups, keep=groups["count"]) if groups else None)
            entry = dict(entry, mlp=dict(mlp, router=router))
        layers.append(entry)
    return dict(config, layers=layers)


def weights_for(name, sharpen=1.0, dtype="float32"):
    """float32 weights as a load will see them (rounded to bfloat16).  ``sharpen`` multiplies the scale of
    the queries' norm, so that attention puts its weight on few keys and a lost key shows."""
    key = (name, sharpen)
    if key not in _weights:
        config, seed = CONFIGS[name]
        _, tensors = bt.random_tensors(config, seed)
        if sharpen != 1.0:
            tensors = {k: (v * sharpen if k.endswith(".left.q.norm") else v) for k, v in tensors.items()}
        _weights[key] = {k: v.to(torch.bfloat16).float() for k, v in tensors.items()}
    return _weights[key]


def model_for(name, dtype, sharpen=1.0):
    key = (name, dtype, sharpen)
    if key not in _models:
        stored = {k: v.to(torch.bfloat16) for k, v in weights_for(name, sharpen, dtype).items()}
        _models[key] = bt.model_from_tensors(config_for(name, dtype), stored, dtype, "cuda:0")
    return _models[key]


def engine_for(name, dtype, max_tokens=4096, sharpen=1.0, **options):
    return bt.Engine(model_for(name, dtype, sharpen), max_tokens=max_tokens, **options)


def plain_logits(name, ids, sharpen=1.0, dtype="float32"):
    return plain.forward(ids, weights_for(name, sharpen, dtype), config_for(name, dtype))


def prompts_for(name, lengths, seed=0):
    gen = torch.Generator().manual_seed(seed)
    return [torch.randint(0, CONFIGS[name][0]["vocab"], (n,), generator=gen).tolist() for n in lengths]


def tolerance(dtype, reference):
    """Largest allowed absolute error of logits: float32 differs from float64 by the rounding of sums;
    bfloat16 rounds the operands of every product to 8 bits."""
    scale = float(reference.abs().max())
    return 2e-5 + 3e-5 * scale if dtype == "float32" else 3e-2 * scale


def random_config(seed):
    """A configuration drawn from a seed: two to five layers of either kind in any order, with any of the three
    feed-forwards or none, sizes, windows, taps, parts of the norm and constants from short lists."""
    import random
    rng = random.Random(seed)
    width = rng.choice([64, 96, 128, 160, 256])
    layers = []
    for _ in range(rng.randint(2, 5)):
        if rng.random() < 0.5:
            mixer = forget(rng.choice([1, 2, 4, 6]), rng.choice([16, 32, 48, 64, 96]), rng.choice([16, 32, 64]))
        else:
            kv, dim = rng.choice([1, 2, 4]), rng.choice([16, 32, 48, 64, 80, 128])
            left = window_attention(kv * rng.choice([1, 2, 3, 4]), kv, dim, rng.choice([16, 32, 48, 64, 128]),
                                    dim ** -0.5 * rng.choice([0.7, 1.0, 1.5]), rot_dims=rng.choice([0, dim // 4 * 2, dim]),
                                    base=rng.choice([100.0, 10000.0, 500000.0]),
                                    window=rng.choice([5, 32, 64, 96, 100, 160]) if rng.random() < 0.85 else None)
            shared = rng.choice([1, 2, 4])
            right = delta(shared * rng.choice([1, 2]), shared, rng.choice([16, 32, 64, 128]), rng.choice([16, 32, 64]),
                          rng.choice([1, 2, 3, 4, 5]), rank=rng.choice([4, 16, 24]))
            mixer = side_by_side(left, right, rng.choice([0.5, 1.0, 1.2]), rng.choice([0.9, 1.0, 2.0]))
        kind = rng.random()
        if kind < 0.15:
            mlp = None
        elif kind < 0.45:
            mlp = dense(rng.choice([64, 200, 256]))
        else:
            count, per = rng.choice([1, 2, 4]), rng.choice([1, 2, 3, 4])
            keep = rng.randint(1, count)
            grouped = rng.random() < 0.8
            mlp = moe(count * per, rng.choice([32, 64]), rng.randint(1, keep * per if grouped else count * per),
                      rng.choice([0.7, 1.5, 7.0]), groups=(count, keep) if grouped else None)
        layers.append(layer(mixer, mlp))
    return model_config(layers, width=width, vocab=rng.choice([97, 320, 1000]), groups=rng.choice([g for g in (1, 2, 4, 8) if width % g == 0]),
                        eps=rng.choice([1e-5, 1e-6]), cap=rng.choice([None, 15.0, 30.0]))
