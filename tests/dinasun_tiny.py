"""Small Dinasun configurations for the tests, each with sizes and constants of its own.

Between them they differ in everything config.json gives: width, vocabulary, the order of the
mixers, heads and head sizes of both mixers (multiples of 16 and not), key/value heads (as many as
query heads, fewer, one), the score scale, the query temperature (every few positions so that short
prompts cross several steps of it, every position, absent), the experts (one, some and all chosen; with
and without a shared expert; a layer without a feed-forward), the looped span (a part, the whole model,
once, none, a single layer many times), the factor on what a sublayer adds (below one, one, above),
the embedding's scale (given, one, absent), eps.
"""


def wkv(heads, dim):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim}}


def attention(heads, kv_heads, dim, scale, coef=None, every=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if every is not None:
        m["q_temp"] = {"coef": coef, "every": every}
    return {"type": "attention", "mixer": m}


def moe(ff, experts, top, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared is not None:
        m["shared"] = {"ff": shared}
    return m


def with_ff(layer, mlp):
    out = dict(layer)
    out["mlp"] = mlp
    return out


# attention first; the middle two layers three times; head sizes the matrix cores take in bfloat16;
# a temperature step every 5 positions; a layer without a feed-forward; experts without a shared one
TINY_D1 = {
    "architecture": "Dinasun", "vocab": 200, "width": 64, "norm": {"eps": 1e-5}, "residual_mult": 0.6,
    "embedding": {"scale": 1.7},
    "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        with_ff(attention(4, 2, 16, 0.3, coef=0.4, every=5), moe(40, 6, 2, shared=24)),
        with_ff(wkv(2, 32), moe(24, 5, 3)),
        with_ff(attention(6, 6, 32, 0.2), None),
        with_ff(wkv(4, 16), moe(32, 4, 1, shared=48)),
    ],
}

# no loop, no embedding scale, a factor of one; sizes that are multiples of nothing; one key head for
# all query heads; a temperature step at every position; all experts chosen
TINY_D2 = {
    "architecture": "Dinasun", "vocab": 97, "width": 40, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
    "layers": [
        with_ff(wkv(3, 10), moe(20, 3, 3, shared=12)),
        with_ff(attention(3, 1, 10, 0.45, coef=0.25, every=1), moe(12, 2, 1)),
        with_ff(wkv(1, 12), None),
        with_ff(attention(2, 2, 6, 0.6), moe(16, 4, 2, shared=8)),
    ],
}

# the whole model looped twice; heads of 64 channels for the matrix-core attention and the wide
# recurrence; a temperature step of a page; a factor above one; one expert in all
TINY_D3 = {
    "architecture": "Dinasun", "vocab": 256, "width": 96, "norm": {"eps": 1e-5}, "residual_mult": 1.2,
    "embedding": {"scale": 1.0},
    "loop": {"start": 0, "stop": 3, "times": 2},
    "layers": [
        with_ff(wkv(2, 64), moe(48, 1, 1, shared=32)),
        with_ff(attention(8, 4, 64, 0.11, coef=0.3, every=64), moe(32, 6, 2, shared=64)),
        with_ff(wkv(6, 16), moe(32, 4, 4)),
    ],
}

# a span looped once (as good as none) and a last layer alone behind it; sixteen heads whose slopes
# go from near one to 1/256; a temperature that steps once in the tests' sequences
TINY_D4 = {
    "architecture": "Dinasun", "vocab": 128, "width": 64, "norm": {"eps": 1e-6}, "residual_mult": 0.8,
    "embedding": {"scale": 0.4},
    "loop": {"start": 1, "stop": 2, "times": 1},
    "layers": [
        with_ff(attention(16, 4, 16, 0.25, coef=1.0, every=100), moe(32, 4, 2, shared=32)),
        with_ff(wkv(4, 16), moe(32, 4, 2, shared=32)),
        with_ff(attention(2, 1, 48, 0.15), moe(16, 3, 2)),
    ],
}

# a single time-mixing layer run five times, each pass with a state of its own; no attention at all
TINY_D5 = {
    "architecture": "Dinasun", "vocab": 64, "width": 48, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
    "loop": {"start": 0, "stop": 1, "times": 5},
    "layers": [
        with_ff(wkv(3, 8), moe(16, 2, 1, shared=16)),
    ],
}

# attention only, one head, no temperature; a head size beyond what the matrix-core kernel takes in
# one register block (the 32-bit attention on bfloat16 storage)
TINY_D6 = {
    "architecture": "Dinasun", "vocab": 50, "width": 32, "norm": {"eps": 1e-6}, "residual_mult": 0.9,
    "embedding": {"scale": 2.0},
    "layers": [
        with_ff(attention(1, 1, 24, 0.2), moe(8, 2, 1)),
        with_ff(attention(4, 2, 8, 0.35, coef=0.1, every=3), None),
    ],
}

# (configuration, seed, deviation of the matrices: smaller where a factor above one and two passes over the
# whole model would otherwise make single rows pass a rounding on a hundredfold, in 32 bits as in 16)
# a width that is a multiple of nothing the kernels like (no 16-byte rows, no matrix cores), every head count odd
TINY_D7 = {
    "architecture": "Dinasun", "vocab": 61, "width": 30, "norm": {"eps": 1e-5}, "residual_mult": 0.75,
    "embedding": {"scale": 1.3},
    "loop": {"start": 1, "stop": 2, "times": 2},
    "layers": [
        with_ff(wkv(3, 6), moe(10, 3, 2, shared=7)),
        with_ff(attention(3, 3, 10, 0.3, coef=0.2, every=7), moe(9, 2, 2)),
    ],
}

CONFIGS = {"D1": (TINY_D1, 31, 0.2), "D2": (TINY_D2, 32, 0.2), "D3": (TINY_D3, 33, 0.1), "D4": (TINY_D4, 34, 0.2),
           "D5": (TINY_D5, 35, 0.2), "D6": (TINY_D6, 36, 0.2), "D7": (TINY_D7, 37, 0.2)}


def make_model(which: str, folder: str, std: float = 0.0) -> str:
    from xyntetik_runner_amd.weights import write_random_model
    config, seed, own = CONFIGS[which]
    std = std or own
    return write_random_model(config, folder, seed=seed, std=std, norm_jitter=0.1, dtype="bfloat16")
