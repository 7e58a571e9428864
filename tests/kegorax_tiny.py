"""Small Kegorax configurations for the tests, each with sizes and constants of its own.

Between them they differ in everything config.json gives: width, vocabulary, the order of the layers,
heads and head sizes of every mixer (multiples of 16 and of nothing; values as long as keys and not),
key/value heads (as many as query heads, fewer, one), scales, chunk and window lengths (one position,
a few, a page, longer than the tests' prompts), kept first tokens (none, absent, fewer and more than a
window or a page), the rotated part of a head (none, absent, a part, all of it, multiples of 16 and not),
tau, retention decays (with 0 and 1), convolution taps (1 to 4), the experts (groups absent, of one
expert, some kept, all kept; one, some and all experts chosen), dense and no feed-forward, the looped
span (a part, the whole model, once, none, a single layer many times), the embedding's scale, eps, and
the sides' weights.
"""


def attn(heads, kv_heads, dim, vdim, scale, size, keep_first=None, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": size}}
    if keep_first is not None:
        m["mask"]["keep_first"] = keep_first
    if rot is not None:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
    return m


def parallel(left, heads, dim, vdim, tau, mlp):
    return {"type": "parallel", "mixer": {"left": left, "right": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}},
            "mlp": mlp}


def parallel_2(left, heads, dim, vdim, decay, left_scale, right_scale, mlp):
    return {"type": "parallel_2", "mixer": {"left": left, "right": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay},
                                            "left_scale": left_scale, "right_scale": right_scale}, "mlp": mlp}


def delta(heads, kv_heads, dim, vdim, conv, mlp):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, scale, groups=None):
    r = {"experts": experts, "top": top, "scale": scale}
    if groups is not None:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": r}


# the middle two layers three times; head sizes the matrix cores take in bfloat16; a chunk and a window that the
# tests' prompts cross several times, neither a multiple of a key tile; three kept tokens; a layer without a feed-forward
TINY_K1 = {
    "architecture": "Kegorax", "vocab": 200, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.7},
    "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        delta(4, 2, 16, 32, 4, dense(96)),
        parallel(attn(4, 2, 32, 32, 0.2, 24, rot=(10000.0, 8)), 2, 16, 32, 4.0, moe(24, 8, 2, 2.0, groups=(4, 2))),
        parallel_2(attn(6, 3, 16, 16, 0.3, 20, keep_first=3), 2, 32, 16, [0.9, 0.97], 0.7, 1.2, None),
        delta(2, 2, 32, 16, 2, moe(32, 4, 1, 0.8)),
    ],
}

# no loop, no embedding scale; sizes that are multiples of nothing; values of another size than keys; one key head for
# all query heads; the whole head rotated; a chunk of five and a window of seven; all experts chosen; taps of one
TINY_K2 = {
    "architecture": "Kegorax", "vocab": 97, "width": 40, "norm": {"eps": 1e-6},
    "layers": [
        parallel(attn(3, 1, 10, 6, 0.45, 5, rot=(500.0, 10)), 3, 6, 10, 1.0, moe(12, 3, 3, 1.0)),
        delta(3, 1, 10, 6, 1, None),
        parallel_2(attn(2, 2, 6, 14, 0.6, 7, keep_first=0), 1, 12, 6, [1.0], 1.0, 0.5, dense(20)),
        delta(2, 2, 6, 12, 3, dense(24)),
    ],
}

# the whole model twice; heads of 64 for the matrix-core attention and the wide recurrence; a chunk of a page;
# more kept tokens than a window or a page holds; the whole head rotated in the paired order
TINY_K3 = {
    "architecture": "Kegorax", "vocab": 256, "width": 96, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.0},
    "loop": {"start": 0, "stop": 3, "times": 2},
    "layers": [
        parallel_2(attn(4, 4, 64, 64, 0.11, 48, keep_first=70), 2, 64, 64, [0.99, 0.9], 0.5, 0.8, dense(128)),
        parallel(attn(8, 4, 64, 64, 0.08, 64, rot=(500000.0, 64)), 2, 64, 32, 12.0, moe(32, 6, 2, 1.25, groups=(3, 3))),
        delta(2, 1, 64, 64, 3, moe(48, 4, 4, 0.5, groups=(2, 2))),
    ],
}

# a width no kernel likes (no 16-byte rows, no matrix cores), odd head counts; no rotation at all; a chunk and a
# window of one position; kept tokens without the key; a span looped once; groups of one expert each
TINY_K4 = {
    "architecture": "Kegorax", "vocab": 61, "width": 30, "norm": {"eps": 1e-5}, "embedding": {"scale": 0.4},
    "loop": {"start": 1, "stop": 2, "times": 1},
    "layers": [
        parallel(attn(3, 3, 10, 10, 0.3, 1), 1, 8, 6, 2.5, moe(10, 4, 2, 3.0, groups=(4, 3))),
        parallel_2(attn(3, 1, 8, 8, 0.35, 1, keep_first=2), 3, 6, 10, [0.0, 0.5, 1.0], -0.5, 1.5, moe(9, 2, 2, 1.0)),
        delta(3, 3, 6, 10, 2, dense(16)),
    ],
}

# keys of 48 with values of 32 (the 32-bit attention on bfloat16 storage), heads of 16 whose rotated part is all of
# the head; a chunk and a window longer than most prompts; a wide and a narrow recurrence; one delta key head
TINY_K5 = {
    "architecture": "Kegorax", "vocab": 128, "width": 64, "norm": {"eps": 1e-6}, "embedding": {"scale": 8.0},
    "layers": [
        parallel_2(attn(4, 2, 48, 32, 0.14, 100, keep_first=5), 2, 16, 80, [0.999, 0.5], 1.0, 1.0, dense(64)),
        parallel(attn(8, 8, 16, 16, 0.25, 130, rot=(100.0, 16)), 1, 64, 16, 8.0, dense(40)),
        delta(4, 1, 64, 16, 4, moe(16, 8, 3, 1.0, groups=(2, 1))),
    ],
}

# a single layer of two mixers run four times, each pass with pages and a state of its own; 16 heads whose slopes go
# from near one to 1/256
TINY_K6 = {
    "architecture": "Kegorax", "vocab": 64, "width": 48, "norm": {"eps": 1e-5},
    "loop": {"start": 0, "stop": 1, "times": 4},
    "layers": [
        parallel_2(attn(16, 4, 16, 16, 0.25, 33, keep_first=1), 3, 8, 16, [0.8, 0.9, 0.95], 0.5, 0.5, dense(32)),
    ],
}

# sizes nearer a real model's: heads of 128 and 96 for the matrix-core attention, recurrences of 128 key channels,
# dense feed-forwards only (no choice of experts that a rounding could change: every row is compared in bfloat16),
# the first two layers twice
TINY_K7 = {
    "architecture": "Kegorax", "vocab": 512, "width": 256, "norm": {"eps": 1e-5}, "embedding": {"scale": 12.0},
    "loop": {"start": 0, "stop": 2, "times": 2},
    "layers": [
        parallel(attn(4, 1, 128, 128, 0.088, 200, rot=(250000.0, 32)), 2, 128, 64, 10.0, dense(192)),
        parallel_2(attn(2, 2, 96, 96, 0.1, 150, keep_first=9), 4, 32, 32, [0.95, 0.98, 0.99, 0.999], 0.55, 0.95, dense(288)),
        delta(2, 1, 128, 128, 4, dense(256)),
    ],
}

# (configuration, seed, deviation of the matrices)
CONFIGS = {"K1": (TINY_K1, 41, 0.2), "K2": (TINY_K2, 42, 0.2), "K3": (TINY_K3, 43, 0.1), "K4": (TINY_K4, 44, 0.2),
           "K5": (TINY_K5, 45, 0.15), "K6": (TINY_K6, 46, 0.2), "K7": (TINY_K7, 47, 0.06)}


def make_model(which: str, folder: str, std: float = 0.0) -> str:
    from xyntetik_runner_amd.weights import write_random_model
    config, seed, own = CONFIGS[which]
    std = std or own
    return write_random_model(config, folder, seed=seed, std=std, norm_jitter=0.1, dtype="bfloat16")
