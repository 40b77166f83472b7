"""Tiny Gavasun configurations and helpers shared by the tests of that family."""

import torch

import burn_transformers_amd as bt
import plain_gavasun as plain


def rotation(dims, base=10000.0, scaling=None):
    """scaling: (factor, original, fast, slow) or None."""
    if not dims:
        return None
    keys = ("factor", "original", "fast", "slow")
    return {"dims": dims, "base": base, "scaling": dict(zip(keys, scaling)) if scaling else None}


def attention(heads, kv_heads, dim, vdim, scale, taps=None, rot=None, chunk=None):
    sizes = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot,
             "mask": {"size": chunk} if chunk else None}
    if taps:
        sizes["conv"] = taps
    return "attention", sizes


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base=10000.0, scaling=None, window=None):
    return "latent_attention", {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                                "scale": scale, "rot": rotation(rot_dim, base, scaling), "mask": {"size": window} if window else None}


def delta(heads, kv_heads, dim, vdim, taps):
    return "delta", {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, ff, top, shared=None):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top},
            "shared": {"ff": shared} if shared else None}


def layer(mixer, mlp=None):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def model_config(layers, width=64, vocab=211, eps=1e-5, scale=2.0, loop=None):
    return {"architecture": "Gavasun", "vocab": vocab, "width": width, "embedding": {"scale": scale}, "norm": {"eps": eps},
            "loop": dict(zip(("start", "stop", "times"), loop)) if loop else None, "layers": layers}


# all three mixers and all three feed-forwards; the middle two layers run twice; shared heads on both sides, values wider
# than keys, part of a head turned, a chunk and a window that are no multiple of a tile and differ, both schedules of slowing
BASIC = model_config([layer(attention(4, 2, 16, 32, 0.25, taps=3, rot=rotation(8, 500.0, (4.0, 64, 16.0, 2.0)), chunk=24), dense(96)),
                      layer(delta(4, 2, 16, 24, 4), moe(6, 24, 3, shared=40)),
                      layer(latent(3, 16, 8, 24, 40, 32, 0.2, base=2000.0, scaling=(2.0, 128, 8.0, 1.0), window=20), moe(4, 16, 2)),
                      layer(attention(2, 2, 32, 16, 0.18, taps=2, rot=rotation(32, 10000.0), chunk=50))], loop=(1, 3, 2))
# sizes the kernels do not divide, the loop over the first layers, one tap, no convolution, no rotation, no mask, a layer
# without a feed-forward, one expert a token, every expert chosen, no shared expert, the whole head turned
ODD = model_config([layer(delta(3, 1, 20, 12, 1), moe(5, 12, 1)),
                    layer(latent(5, 24, 6, 10, 18, 44, 0.2, base=100.0, window=7)),
                    layer(attention(3, 3, 24, 10, 0.2, taps=5, rot=rotation(24, 100.0, (3.0, 40, 4.0, 0.5)), chunk=7), dense(50)),
                    layer(attention(6, 1, 8, 8, 0.4), moe(3, 20, 3, shared=9)),
                    layer(latent(2, 12, 0, 20, 30, 20, 0.3), dense(22)),
                    layer(delta(2, 2, 40, 8, 2))], width=40, vocab=97, eps=1e-3, scale=0.5, loop=(0, 2, 3))
# each mechanism alone, in a model of one layer
ATTENTION_ONLY = model_config([layer(attention(4, 2, 32, 32, 0.18, taps=4, rot=rotation(16, 1000.0, (6.0, 32, 24.0, 1.0)), chunk=40))],
                              vocab=101)
LATENT_ONLY = model_config([layer(latent(4, 32, 16, 24, 48, 64, 0.15, base=5000.0, scaling=(4.0, 64, 16.0, 1.0), window=33))], vocab=101)
DELTA_ONLY = model_config([layer(delta(4, 2, 24, 16, 4))], vocab=101)
DENSE_ONLY = model_config([layer(delta(1, 1, 8, 8, 2), dense(72))], width=32, vocab=61)
EXPERTS_ONLY = model_config([layer(delta(1, 1, 8, 8, 2), moe(8, 16, 2, shared=24))], width=32, vocab=61)
# chunks and windows that span several blocks of the cache, heads of 128, a latent wider than any MFMA attention kernel's head
LONG = model_config([layer(attention(2, 1, 128, 64, 0.09, taps=4, rot=rotation(64, 300000.0, (5.0, 256, 24.0, 1.5)), chunk=200), dense(64)),
                     layer(latent(2, 64, 32, 48, 64, 112, 0.1, base=30000.0, scaling=(3.0, 512, 16.0, 1.0), window=150), moe(4, 32, 2, shared=16)),
                     layer(delta(2, 2, 128, 32, 4))], width=96, vocab=151)
# a latent whose cached head fits the MFMA kernels (96 + 32), more query heads on a cached head than a decode tile takes
NARROW_LATENT = model_config([layer(latent(4, 32, 32, 32, 48, 96, 0.12, window=70), dense(48)),
                              layer(latent(20, 8, 8, 8, 24, 40, 0.3, window=48)),
                              layer(attention(20, 1, 16, 16, 0.25, taps=2, rot=rotation(16), chunk=48))], width=48, vocab=71)
# heads wider than any MFMA attention kernel's, a state of 200 key channels
WIDE_HEADS = model_config([layer(attention(2, 1, 144, 20, 0.08, taps=3, rot=rotation(100, 1000.0, (2.0, 64, 8.0, 1.0)), chunk=30)),
                           layer(delta(1, 1, 200, 70, 3)),
                           layer(latent(2, 40, 64, 144, 72, 250, 0.1, window=64))], width=32, vocab=53)
# nothing a multiple of eight
UNALIGNED = model_config([layer(delta(2, 2, 10, 6, 3), moe(3, 10, 2, shared=7)),
                          layer(attention(2, 1, 12, 20, 0.3, taps=3, rot=rotation(6), chunk=9), dense(22)),
                          layer(latent(3, 10, 6, 5, 7, 9, 0.3, window=11), moe(3, 5, 1))], width=36, vocab=53, loop=(2, 3, 2))
CONFIGS = {"basic": (BASIC, 1), "odd": (ODD, 2), "attention": (ATTENTION_ONLY, 3), "latent": (LATENT_ONLY, 4), "delta": (DELTA_ONLY, 5),
           "dense": (DENSE_ONLY, 6), "experts": (EXPERTS_ONLY, 7), "long": (LONG, 8), "narrow_latent": (NARROW_LATENT, 9),
           "wide_heads": (WIDE_HEADS, 10), "unaligned": (UNALIGNED, 11)}

_weights, _models = {}, {}


def config_for(name, dtype="float32"):
    """The configuration a run uses.  bfloat16 runs let every token use every expert (``top`` = experts): with
    operands rounded to 8 bits a near tie between two experts' scores falls the other way now and then, the token's
    whole feed-forward output is then another, and no bound on rounding holds.  The weights, which are the experts'
    scores, still differ from token to token; the choice itself is made in the float32 runs, which go through the
    same kernels."""
    config = CONFIGS[name][0]
    if dtype != "bfloat16":
        return config
    layers = []
    for entry in config["layers"]:
        mlp = entry["mlp"]
        if mlp and mlp["kind"] == "moe":
            entry = dict(entry, mlp=dict(mlp, router=dict(mlp["router"], top=mlp["router"]["experts"])))
        layers.append(entry)
    return dict(config, layers=layers)


SHARPENED = (".mix.q.norm", ".mix.dq.norm")       # the scales whose size sets how sharply a query picks its keys


def weights_for(name, sharpen=1.0):
    """float32 weights as a load will see them (rounded to bfloat16).  ``sharpen`` multiplies the scales of the
    queries' norms, so that attention puts its weight on few keys and a lost key shows."""
    key = (name, sharpen)
    if key not in _weights:
        config, seed = CONFIGS[name]
        _, tensors = bt.random_tensors(config, seed)
        if sharpen != 1.0:
            tensors = {k: (v * sharpen if k.endswith(SHARPENED) else v) for k, v in tensors.items()}
        _weights[key] = {k: v.to(torch.bfloat16).float() for k, v in tensors.items()}
    return _weights[key]


def model_for(name, dtype, sharpen=1.0):
    key = (name, dtype, sharpen)
    if key not in _models:
        stored = {k: v.to(torch.bfloat16) for k, v in weights_for(name, sharpen).items()}
        _models[key] = bt.model_from_tensors(config_for(name, dtype), stored, dtype, "cuda:0")
    return _models[key]


def engine_for(name, dtype, max_tokens=4096, sharpen=1.0, **options):
    return bt.Engine(model_for(name, dtype, sharpen), max_tokens=max_tokens, **options)


def plain_logits(name, ids, sharpen=1.0, dtype="float32"):
    return plain.forward(ids, weights_for(name, sharpen), config_for(name, dtype))


def prompts_for(name, lengths, seed=0):
    gen = torch.Generator().manual_seed(seed)
    return [torch.randint(0, CONFIGS[name][0]["vocab"], (n,), generator=gen).tolist() for n in lengths]


def tolerance(dtype, reference):
    """Largest allowed absolute error of logits: float32 differs from float64 by the rounding of sums;
    bfloat16 rounds the operands of every product to 8 bits."""
    scale = float(reference.abs().max())
    return 2e-5 + 3e-5 * scale if dtype == "float32" else 3e-2 * scale


def random_config(seed):
    """A configuration drawn from a seed: two to five layers of any kind in any order, with any feed-forward or none,
    a loop or none, sizes, chunks, windows, taps and constants from short lists."""
    import random
    rng = random.Random(seed)
    width = rng.choice([64, 96, 128, 160, 256])

    def scaling():
        return (rng.choice([2.0, 4.0, 16.0]), rng.choice([32, 256, 2048]), rng.choice([8.0, 32.0]), rng.choice([0.5, 1.0, 2.0])) \
            if rng.random() < 0.7 else None

    layers = []
    for _ in range(rng.randint(2, 5)):
        kind = rng.random()
        if kind < 0.35:
            kv, dim = rng.choice([1, 2, 4]), rng.choice([16, 32, 48, 64, 80, 128])
            mixer = attention(kv * rng.choice([1, 2, 3, 4]), kv, dim, rng.choice([16, 32, 48, 64, 128]),
                              dim ** -0.5 * rng.choice([0.7, 1.0, 1.5]), taps=rng.choice([None, 1, 2, 3, 4, 5]),
                              rot=rotation(rng.choice([0, dim // 4 * 2, dim]), rng.choice([100.0, 10000.0, 500000.0]), scaling()),
                              chunk=rng.choice([5, 32, 64, 96, 100, 160]) if rng.random() < 0.85 else None)
        elif kind < 0.7:
            dim, rot_dim = rng.choice([16, 32, 64, 96]), rng.choice([0, 8, 16, 32, 64])
            mixer = latent(rng.choice([1, 2, 4, 8]), dim, rot_dim, rng.choice([16, 32, 48, 80]), rng.choice([24, 64, 96]),
                           rng.choice([32, 64, 96, 128, 192]), (dim + rot_dim) ** -0.5 * rng.choice([0.7, 1.0, 1.5]),
                           base=rng.choice([100.0, 30000.0]), scaling=scaling(),
                           window=rng.choice([5, 32, 64, 96, 100, 160]) if rng.random() < 0.85 else None)
        else:
            shared = rng.choice([1, 2, 4])
            mixer = delta(shared * rng.choice([1, 2]), shared, rng.choice([16, 32, 64, 128]), rng.choice([16, 32, 64]),
                          rng.choice([1, 2, 3, 4, 5]))
        kind = rng.random()
        if kind < 0.15:
            mlp = None
        elif kind < 0.45:
            mlp = dense(rng.choice([64, 200, 256]))
        else:
            count = rng.choice([2, 4, 8, 12])
            mlp = moe(count, rng.choice([32, 64]), rng.randint(1, count), shared=rng.choice([None, 32, 100]))
        layers.append(layer(mixer, mlp))
    loop = None
    if rng.random() < 0.7:
        start = rng.randrange(len(layers))
        loop = (start, rng.randint(start + 1, len(layers)), rng.randint(1, 3))
    return model_config(layers, width=width, vocab=rng.choice([97, 320, 1000]), eps=rng.choice([1e-5, 1e-6]),
                        scale=rng.choice([1.0, 3.0, 8.0]), loop=loop)
