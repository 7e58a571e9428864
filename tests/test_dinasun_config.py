"""Dinasun without a GPU: the config's refusals by key, the spec it builds, the caches and states
of its layer runs, the random-weights writer, and the plain mechanisms against closed forms."""
import copy
import math

import numpy as np
import pytest

import plain_dinasun as P
from dinasun_tiny import TINY_D1, TINY_D2, TINY_D3, TINY_D4, TINY_D5, TINY_D6, make_model


def parse(raw):
    from xyntetik_runner_amd.config import config_from_dict
    arch, cfg = config_from_dict(raw)
    return arch, cfg


def test_config_reads_every_size_and_constant():
    arch, cfg = parse(TINY_D1)
    assert arch.name == "Dinasun" and cfg.vocab == 200 and cfg.width == 64 and cfg.eps == 1e-5
    assert cfg.residual_mult == 0.6 and cfg.embedding_scale == 1.7 and cfg.loop == (1, 3, 3)
    assert [i for i, _ in cfg.run_order()] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert [enters for _, enters in cfg.run_order()] == [False, True, False, True, False, True, False, False]
    a, t = cfg.layers[0].mixer, cfg.layers[1].mixer
    assert (a.kind, a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.temp_coef, a.temp_every) == ("attention", 4, 2, 16, 16, 0.3, 0.4, 5)
    assert (t.kind, t.heads, t.dim) == ("wkv", 2, 32)
    assert cfg.layers[2].mlp is None and cfg.layers[2].mixer.temp_every == 0
    m = cfg.layers[0].mlp
    assert (m.kind, m.ff, m.experts, m.top, m.shared_ff) == ("moe", 40, 6, 2, 24)
    assert cfg.layers[1].mlp.shared_ff == 0
    _, c2 = parse(TINY_D2)
    assert c2.loop is None and c2.embedding_scale == 1.0 and c2.residual_mult == 1.0
    assert all(not enters for _, enters in c2.run_order())
    _, c4 = parse(TINY_D4)       # a span that runs once is still entered through the injection
    assert c4.run_order() == ((0, False), (1, True), (2, False))
    _, c5 = parse(TINY_D5)
    assert c5.run_order() == ((0, True),) * 5
    empty = copy.deepcopy(TINY_D1)
    empty["loop"] = {"start": 2, "stop": 2, "times": 4}
    assert parse(empty)[1].loop is None


@pytest.mark.parametrize("path,value,word", [
    (("layers", 0, "type"), "lightning", "type"),
    (("layers", 0, "mixer", "heads"), 0, "heads"),
    (("layers", 0, "mixer", "kv_heads"), 3, "kv_heads"),
    (("layers", 0, "mixer", "kv_heads"), 8, "kv_heads"),
    (("layers", 0, "mixer", "vdim"), 24, "vdim"),
    (("layers", 0, "mixer", "scale"), "big", "scale"),
    (("layers", 0, "mixer", "q_temp", "every"), 0, "every"),
    (("layers", 1, "mixer", "dim"), -4, "dim"),
    (("layers", 0, "mlp", "router", "top"), 7, "top"),
    (("layers", 0, "mlp", "kind"), "dense", "kind"),
    (("layers", 0, "mlp", "expert"), None, "expert"),
    (("loop", "stop"), 0, "stop"),
    (("loop", "stop"), 5, "stop"),
    (("loop", "times"), 0, "times"),
    (("norm", "eps"), -1.0, "eps"),
    (("norm",), None, "norm"),
    (("vocab",), None, "vocab"),
])
def test_config_refuses_by_key(path, value, word):
    from xyntetik_runner_amd.config import ConfigError
    raw = copy.deepcopy(TINY_D1)
    at = raw
    for p in path[:-1]:
        at = at[p]
    at[path[-1]] = value
    with pytest.raises(ConfigError) as e:
        parse(raw)
    assert word in str(e.value)


def test_spec_caches_and_states_of_every_run():
    from xyntetik_runner_amd.architectures.dinasun import distance_slopes
    from xyntetik_runner_amd.engine.model import Model
    arch, cfg = parse(TINY_D1)
    spec = arch.build_spec(cfg)
    assert len(spec.order) == 8 and all(st.cache_of is None for st in spec.order)      # every pass owns what it keeps
    assert [st.enters for st in spec.order] == [False, True, False, True, False, True, False, False]
    assert spec.injection is not None and spec.embedding.params["scale"] == 1.7
    att = spec.layers[0].mixer.params
    assert att["values"] == "keys" and att["slopes"] == distance_slopes(4) and att["scale"] == 0.3
    assert np.allclose(distance_slopes(4), [0.25, 0.0625, 0.015625, 0.00390625])
    assert np.allclose(distance_slopes(3), [2 ** (-8 / 3), 2 ** (-16 / 3), 2 ** -8])
    model = Model(spec)
    exp = model.expected()
    assert exp["embed"].shape == (200, 64) and exp["loop.in"].shape == (64, 128) and "l0.mix.v" not in exp
    assert exp["l0.mix.q"].shape == (64, 64) and exp["l0.mix.k"].shape == (32, 64) and exp["l0.mix.k.b"].shape == (32,)
    assert exp["l0.mix.q.norm"].shape == (16,) and exp["l0.mlp.table"].shape == (200, 2)
    assert exp["l0.mlp.e5.gate"].shape == (40, 64) and exp["l0.mlp.shared.down"].shape == (64, 24)
    assert exp["l1.mix.mu.w"].shape == (64,) and exp["l1.mix.u"].shape == (2, 32) and exp["l1.mix.w0"].shape == (64,)
    assert exp["l1.norm1b.alpha"].shape == () or exp["l1.norm1b.alpha"].shape == (1,)
    assert exp["l2.norm2"].optional and exp["l2.norm2b"].optional and not exp["l1.norm2"].optional    # (a layer without a feed-forward)
    assert "l2.mlp.table" not in exp and "l1.mlp.shared.up" not in exp
    assert exp["final.norm.b"].shape == (64,)
    _, c2 = parse(TINY_D2)
    assert arch.build_spec(c2).injection is None


def test_random_model_round_trip(tmp_path):
    from plain_llama import load_folder
    d = make_model("D1", str(tmp_path / "m"))
    cfg, w = load_folder(d)
    table = np.asarray(w["l0.mlp.table"])
    assert table.shape == (200, 2) and table.min() >= 0 and table.max() < 6
    assert (table[:, 0] != table[:, 1]).all()           # the experts of a row differ
    assert np.asarray(w["l3.mlp.table"]).shape == (200, 1)
    logits = P.forward(cfg, w, [3, 9, 9, 150, 1])
    assert logits.shape == (5, 200) and np.isfinite(logits).all()


def test_plain_mechanisms_against_closed_forms():
    rng = np.random.default_rng(0)
    # dynamic tanh: no statistic of the row enters, so two rows do not know of each other
    w = {"n": rng.normal(size=5), "n.b": rng.normal(size=5), "n.alpha": np.float64(0.7)}
    x = rng.normal(size=(2, 5))
    assert np.allclose(P.dyt(x, w, "n")[0], P.dyt(x[:1], w, "n")[0])
    assert np.allclose(P.dyt(np.zeros((1, 5)), w, "n"), w["n.b"])
    assert np.allclose(P.dyt(np.full((1, 5), 1e6), w, "n"), w["n"] + w["n.b"])
    # the query temperature steps where floor((p + 1) / every) does
    t = P.query_temperature([0, 3, 4, 8, 9, 14], 0.5, 5)
    assert np.allclose(t, [1, 1, 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(3), 1 + 0.5 * math.log(4)])
    assert np.allclose(P.query_temperature([0, 1], 0.25, 1), [1 + 0.25 * math.log(2), 1 + 0.25 * math.log(3)])
    # the recurrence with decay 1 and no bonus is a causal sum over strictly earlier tokens
    T, D = 6, 4
    r, k, v = rng.normal(size=(T, D)), rng.normal(size=(T, D)), rng.normal(size=(T, D))
    o = P.wkv_recurrence(r, k, v, np.ones((T, D)), np.zeros(D))
    want = np.stack([sum(((r[i] @ k[j]) * v[j] for j in range(i)), np.zeros(D)) for i in range(T)])
    assert np.allclose(o, want)
    # the bonus weighs the token's own key channel by channel, and only in its own read-out
    u = rng.normal(size=D)
    o2 = P.wkv_recurrence(r, k, v, np.ones((T, D)), u)
    assert np.allclose(o2 - o, np.stack([((r[i] * u) @ k[i]) * v[i] for i in range(T)]))
    # a decay of zero on every channel forgets all but the last token
    o3 = P.wkv_recurrence(r, k, v, np.zeros((T, D)), np.zeros(D))
    assert np.allclose(o3[1:], np.stack([(r[i] @ k[i - 1]) * v[i - 1] for i in range(1, T)])) and np.allclose(o3[0], 0)
    # attention: one head, no temperature, keys that all score alike: the weights fall off with the distance by the slope
    E, Dh = 4, 4
    m = {"heads": 1, "kv_heads": 1, "dim": Dh, "vdim": Dh, "scale": 1.0}
    aw = {"q": np.zeros((Dh, E)), "q.b": np.ones(Dh), "k": np.eye(Dh, E), "k.b": np.zeros(Dh), "q.norm": np.ones(Dh),
          "k.norm": np.zeros(Dh), "o": np.eye(E, Dh)}
    h = rng.normal(size=(5, E))
    out = P.attention(h, aw, m, 1e-6, "")
    slope = 2.0 ** -8
    wts = np.exp(-slope * (4 - np.arange(5)))
    assert np.allclose(out[4], (wts / wts.sum()) @ h)          # the values are the keys as projected: h itself here
    # table experts: the weights are 1 / top, the shared expert is added whole
    F = 3
    ew = {"table": np.array([[0, 1], [1, 0], [1, 2]])}
    for e in range(3):
        ew.update({f"e{e}.gate": rng.normal(size=(F, E)), f"e{e}.up": rng.normal(size=(F, E)), f"e{e}.down": rng.normal(size=(E, F))})
    mlp = {"router": {"experts": 3, "top": 2}}
    hh = rng.normal(size=(3, E))
    got = P.table_experts(hh, [0, 1, 2], ew, mlp, "")
    assert np.allclose(got[0], got[1] - P.table_experts(hh[1:2], [1], ew, mlp, "")[0] + got[0])     # (rows are independent)
    assert np.allclose(P.table_experts(hh[:1], [0], ew, mlp, ""), P.table_experts(hh[:1], [1], ew, mlp, ""))   # the order in a row does not matter
    assert np.allclose(got[2], 0.5 * (P.expert(hh[2], ew, "e1.") + P.expert(hh[2], ew, "e2.")))
