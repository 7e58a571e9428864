"""Kegorax without a GPU: the config's refusals by key, the spec it builds, the caches and states of its layer
runs, the pages a window keeps for the first tokens, the plan of a chunked mask, the random-weights writer, and
the plain mechanisms against closed forms."""
import copy

import numpy as np
import pytest

import plain_kegorax as P
from kegorax_tiny import TINY_K1, TINY_K2, TINY_K3, TINY_K4, TINY_K6, make_model


def parse(raw):
    from xyntetik_runner_amd.config import config_from_dict
    return config_from_dict(raw)


def test_config_reads_every_size_and_constant():
    arch, cfg = parse(TINY_K1)
    assert arch.name == "Kegorax" and cfg.vocab == 200 and cfg.width == 64 and cfg.eps == 1e-5
    assert cfg.embedding_scale == 1.7 and cfg.loop == (1, 3, 3)
    assert cfg.run_order() == ((0, None), (1, 0), (2, None), (1, 1), (2, None), (1, 2), (2, None), (3, None))
    d, p, p2 = cfg.layers[0].mixer, cfg.layers[1].mixer, cfg.layers[2].mixer
    assert (d.kind, d.right.heads, d.right.kv_heads, d.right.dim, d.right.vdim, d.right.conv) == ("channel_delta", 4, 2, 16, 32, 4)
    a = p.left
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.mask_size, a.keep_first, a.rot_base, a.rot_dims) == (4, 2, 32, 32, 0.2, 24, 0, 10000.0, 8)
    assert (p.right.heads, p.right.dim, p.right.vdim, p.right.tau) == (2, 16, 32, 4.0)
    b = p2.left
    assert (b.heads, b.kv_heads, b.dim, b.mask_size, b.keep_first, b.rot_dims) == (6, 3, 16, 20, 3, 0)
    assert p2.right.decay == (0.9, 0.97) and (p2.left_scale, p2.right_scale) == (0.7, 1.2)
    m = cfg.layers[1].mlp
    assert (m.kind, m.ff, m.experts, m.top, m.groups, m.keep_groups, m.scale) == ("moe", 24, 8, 2, 4, 2, 2.0)
    assert cfg.layers[2].mlp is None and cfg.layers[0].mlp.kind == "dense" and cfg.layers[0].mlp.ff == 96
    assert cfg.layers[3].mlp.groups == 1 and cfg.layers[3].mlp.keep_groups == 1
    _, c2 = parse(TINY_K2)
    assert c2.loop is None and c2.embedding_scale == 1.0 and c2.layers[2].mixer.left.keep_first == 0
    _, c4 = parse(TINY_K4)       # a span that runs once is still entered; a mixer without "rot" does not rotate
    assert c4.run_order() == ((0, None), (1, 0), (2, None)) and c4.layers[0].mixer.left.rot_dims == 0
    _, c6 = parse(TINY_K6)
    assert c6.run_order() == ((0, 0), (0, 1), (0, 2), (0, 3))
    empty = copy.deepcopy(TINY_K1)
    empty["loop"] = {"start": 2, "stop": 2, "times": 4}
    assert parse(empty)[1].loop is None


def put(raw, path, value):
    raw = copy.deepcopy(raw)
    node = raw
    for key in path[:-1]:
        node = node[key]
    if value is KeyError:
        del node[path[-1]]
    else:
        node[path[-1]] = value
    return raw


@pytest.mark.parametrize("path,value,word", [
    (("vocab",), 0, "vocab"), (("norm",), None, "norm"), (("norm", "eps"), -1.0, "eps"),
    (("layers", 0, "type"), "attention", "type"), (("layers", 1, "mixer", "left"), None, "left"),
    (("layers", 1, "mixer", "left", "kv_heads"), 3, "kv_heads"), (("layers", 1, "mixer", "left", "mask"), None, "mask"),
    (("layers", 1, "mixer", "left", "rot", "dims"), 7, "dims"), (("layers", 1, "mixer", "left", "rot", "dims"), 40, "dims"),
    (("layers", 1, "mixer", "right", "tau"), 0.0, "tau"), (("layers", 2, "mixer", "right", "decay"), [0.5], "decay"),
    (("layers", 2, "mixer", "right", "decay"), [0.5, 1.5], "decay"), (("layers", 0, "mixer", "conv"), 0, "conv"),
    (("layers", 0, "mixer", "kv_heads"), 3, "kv_heads"), (("layers", 1, "mlp", "router", "groups", "count"), 3, "groups"),
    (("layers", 1, "mlp", "router", "groups", "keep"), 5, "keep"), (("layers", 1, "mlp", "router", "top"), 5, "choices"),
    (("layers", 1, "mlp", "router", "scale"), 0.0, "scale"), (("layers", 1, "mlp", "kind"), "shared", "kind"),
    (("loop", "stop"), 9, "stop"), (("loop", "times"), 0, "times"),
])
def test_config_refuses_by_key(path, value, word):
    from xyntetik_runner_amd.config import ConfigError
    with pytest.raises(ConfigError) as e:
        parse(put(TINY_K1, path, value))
    assert word in str(e.value)


def test_spec_caches_and_states_of_every_run():
    from xyntetik_runner_amd.engine.model import Model
    arch, cfg = parse(TINY_K1)
    spec = arch.build_spec(cfg)
    assert [(s.layer, s.enters, s.pass_index) for s in spec.order] == [
        (0, False, 0), (1, True, 0), (2, False, 0), (1, True, 1), (2, False, 0), (1, True, 2), (2, False, 0), (3, False, 0)]
    assert spec.injection.kind == "step_addition" and spec.injection.params["passes"] == 3
    model = Model(spec)
    kv, st, of = model.cache_needs()
    assert all(o is None for o in of)           # every run owns what it keeps
    assert kv[0] is None and set(st[0]) == {"mixer.S", "mixer.conv"} and tuple(st[0]["mixer.conv"].shape) == (3, 2 * 32 + 128)
    # a chunk's pages are kept as a window's of its length; the windowed side keeps its first tokens' pages
    assert (kv[1].num_kv_heads, kv[1].head_dim, kv[1].window, kv[1].keep_first) == (2, 32, 24, 0)
    assert (kv[2].num_kv_heads, kv[2].head_dim, kv[2].window, kv[2].keep_first) == (3, 16, 20, 3)
    assert kv[1] == kv[3] == kv[5] and list(st[1]) == ["mixer.right"] and list(st[2]) == ["mixer.right"]
    names = model.expected()
    for name in ("embed", "loop.step", "l1.mix.left.sink", "l1.mix.left.g", "l1.mix.left.out", "l1.mix.right.out", "l1.mix.right.a2.b",
                 "l2.mix.left.q.b", "l2.mix.left.k.norm", "l0.mix.a1", "l0.mix.g2", "l0.mix.dt_bias", "l0.mix.q.conv",
                 "l1.mlp.e7.gate", "l1.mlp.correction", "l0.mlp.gate", "final.norm"):
        assert name in names, name
    assert tuple(names["loop.step"].shape) == (3, 64) and tuple(names["l0.mix.dt_bias"].shape) == (4 * 16,)
    assert "l2.mix.left.out" not in names and "l2.mlp.gate" not in names and "l1.mix.left.q.b" not in names
    # values of another size than the keys: said to the cache, and to the output projection
    arch2, cfg2 = parse(TINY_K2)
    m2 = Model(arch2.build_spec(cfg2))
    kv2 = m2.cache_needs()[0]
    assert kv2[0].value_dim == 6 and kv2[0].head_dim == 10 and tuple(m2.expected()["l0.mix.left.o"].shape) == (40, 3 * 6)
    assert m2.spec.injection is None


def test_a_window_keeps_the_pages_of_its_first_tokens():
    from xyntetik_runner_amd.cache import CacheManager
    from xyntetik_runner_amd.cache.manager import pages_for_spec
    from xyntetik_runner_amd.parts.base import KVSpec
    plain, kept = KVSpec(2, 16, window=20), KVSpec(2, 16, window=20, keep_first=6)
    assert plain != kept                        # groups of their own
    mgr = CacheManager([plain, kept], 4, [64, 64], 2)
    mgr.admit("a")
    mgr.reserve("a", 90)
    mgr.advance("a", 90)
    t0, t1 = mgr.get("a").tables
    assert all(p < 0 for p in t0[:17]) and all(p >= 0 for p in t0[17:])         # position 71 is the first the next token reads
    assert all(p >= 0 for p in t1[:2]) and all(p < 0 for p in t1[2:17]) and all(p >= 0 for p in t1[17:])
    mgr.check()
    mgr.reserve("a", 200)                       # a portion far on: nothing below its window is taken, the kept pages stay
    assert mgr.get("a").tables[1][0] >= 0 and mgr.get("a").tables[1][20] >= 0
    mgr.advance("a", 200)
    mgr.check()
    assert sum(1 for p in mgr.get("a").tables[1] if p >= 0) == 2 + 5          # positions 181 to 199 and the first 6
    mgr.release("a")
    assert mgr.all_free()
    assert pages_for_spec(kept, 4, 4096, 3, 64) == pages_for_spec(plain, 4, 4096, 3, 64) + 3 * 2


def test_plan_of_a_chunked_mask():
    from xyntetik_runner_amd.engine.batch import Chunked, first_key, mask_reach, plan_attention
    assert [first_key(Chunked(24), p) for p in (0, 23, 24, 47, 100)] == [0, 0, 24, 24, 96]
    assert [first_key(20, p) for p in (0, 19, 20, 100)] == [0, 0, 1, 81] and first_key(None, 500) == 0
    assert mask_reach(Chunked(24)) == 24 and mask_reach(7) == 7 and mask_reach(None) is None
    # a decoded token at position 100 of chunks of 24 reads from key 96 (its tile begins at 96); one at 95 from 72 (tile 64)
    cta, items, jobs, slots = plan_attention([100, 95], [1, 1], 2, Chunked(24), 2, 16)
    assert sorted((it[2], it[3]) for it in items) == [(64, 96), (96, 101)] and not cta and not jobs
    # with a slot more a row block, every item leaves a partial result and every block has a merge job
    cta, items, jobs, slots, extras = plan_attention([100], [1], 2, Chunked(24), 2, 16, extra_slot=True)
    assert len(items) == 1 and items[0][4] == 0 and jobs == [(0, 0, 0, 2, 1, 0, 1)] and extras == [(0, 0, 1, 0, 1, 100, 0, 0)] and slots == 2


def test_random_model_round_trip(tmp_path):
    from plain_llama import load_folder
    d = make_model("K4", str(tmp_path))
    cfg, w = load_folder(d)
    assert cfg["architecture"] == "Kegorax" and w["loop.step"].shape == (1, 30) and w["l0.mix.left.sink"].shape == (3,)
    logits = P.forward(cfg, w, [1, 2, 3, 4, 5])
    assert logits.shape == (5, 61) and np.isfinite(logits).all()


def test_plain_mechanisms_against_closed_forms():
    rng = np.random.default_rng(0)
    # masks
    see = P.visible(7, {"size": 3, "chunked": True})
    assert [list(np.nonzero(r)[0]) for r in see] == [[0], [0, 1], [0, 1, 2], [3], [3, 4], [3, 4, 5], [6]]
    see = P.visible(7, {"size": 2, "keep_first": 1})
    assert [list(np.nonzero(r)[0]) for r in see] == [[0], [0, 1], [0, 1, 2], [0, 2, 3], [0, 3, 4], [0, 4, 5], [0, 5, 6]]
    # a sink: one key of score s and a sink of score s share the weight
    q, k, v = np.ones((1, 1, 2)), np.ones((1, 1, 2)), np.full((1, 1, 3), 4.0)
    o = P.attention_heads(q, k, v, 0.5, np.ones((1, 1), bool), sink=np.array([1.0]))
    assert np.allclose(o, 2.0)
    o = P.attention_heads(q, k, v, 0.5, np.ones((1, 1), bool), sink=np.array([0.0]))        # one added to the denominator
    assert np.allclose(o, 4.0 * np.e / (1.0 + np.e))
    # rotation: a part of the head, pairs (i, i + dims/2), position 0 unchanged
    x = rng.normal(size=(3, 1, 6))
    y = P.rotate_half(x, 100.0, 4)
    assert np.allclose(y[0], x[0]) and np.allclose(y[..., 4:], x[..., 4:])
    a = 2 * 100.0 ** (-2 * 1 / 4)
    assert np.allclose(y[2, 0, 1], x[2, 0, 1] * np.cos(a) - x[2, 0, 3] * np.sin(a))
    assert np.allclose(y[2, 0, 3], x[2, 0, 3] * np.cos(a) + x[2, 0, 1] * np.sin(a))
    # a decay of one keeps every write, a decay of zero only the token's own
    q, k, v = rng.normal(size=(5, 3)), rng.normal(size=(5, 3)), rng.normal(size=(5, 2))
    o = P.decay_recurrence(q, k, v, np.ones((5, 1)))
    assert np.allclose(o[4], sum(np.outer(k[t], v[t]) for t in range(5)).T @ q[4])
    o = P.decay_recurrence(q, k, v, np.zeros((5, 3)))
    assert np.allclose(o[4], np.outer(k[4], v[4]).T @ q[4])
    # the delta rule with a unit key and beta = 1 stores the value exactly: reading with the key gives it back
    kk = np.zeros((1, 4)); kk[0, 2] = 1.0
    o = P.delta_recurrence(kk, kk, np.array([[3.0, -1.0]]), np.array([1.0]), np.full((1, 4), 0.5))
    assert np.allclose(o, [[3.0, -1.0]])
    # the convolution's last tap is the token's own
    y = P.causal_conv_silu(np.array([[1.0], [2.0], [3.0]]), np.array([[10.0, 1.0]]))
    assert np.allclose(y[:, 0], P.silu(np.array([1.0, 12.0, 23.0])))
    # routing: the group left out counts as minus infinity though its scores are the highest above zero
    z = np.array([5.0, 5.0, -5.0, -5.0])
    chosen, wts = P.route(z, np.array([-3.0, -3.0, 0.0, 0.0]), 1, 2, 1, 2.0)
    assert list(chosen) == [2] and np.allclose(wts, 2.0 * P.sigmoid(-5.0))
    assert P.route_margin(z, np.array([-3.0, -3.0, 0.0, 0.0]), 1, 2, 1) == 0.0           # experts 2 and 3 tie
    assert np.allclose(P.gelu_tanh(np.array([0.0, 10.0, -10.0])), [0.0, 10.0, 0.0])
