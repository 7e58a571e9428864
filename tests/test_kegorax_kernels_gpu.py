"""Every mechanism of the Kegorax parts alone: the kernel against the plain function of ``plain_kegorax``
(or a few lines of float64 written here), with rows cut into requests and steps the way an engine cuts them,
and with inputs made so that a fault shows: pages handed out in shuffled order, one key whose score stands
out just inside and just outside a chunk, a window and the kept first tokens, at a page's first and last
place, a sink that outweighs every key beside one that none feels, state rows of other requests that are
garbage, a channel that never decays beside one that forgets at once, choice scores below zero."""
import math

import numpy as np
import pytest
import torch

import plain_kegorax as P
from test_dinasun_kernels_gpu import close, dev, step_ctx
from test_kernels_gpu import FakeCtx, scatter_pages

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def ops():
    from xyntetik_runner_amd.csrc.ops import load_ops
    return load_ops()


def fill_pages(k_seq, v_seq, tables, n_pages, ps, dt):
    """Keys ``[n, Hk, D]`` and values ``[n, Hk, Dv]`` of every request into pages that start as NaN."""
    Hk, D = k_seq[0].shape[1:]
    Dv = v_seq[0].shape[2]
    kc = torch.full((n_pages, Hk, ps, D), float("nan"), dtype=dt)
    vc = torch.full((n_pages, Hk, Dv, ps), float("nan"), dtype=dt)
    for b, (k, v) in enumerate(zip(k_seq, v_seq)):
        for p in range(k.shape[0]):
            kc[tables[b][p // ps], :, p % ps, :] = k[p].to(dt)
            vc[tables[b][p // ps], :, :, p % ps] = v[p].to(dt)
    return kc.to(DEV), vc.to(DEV)


def plain_attention(q, k, v, start, scale, mask, sink, slopes):
    """Rows ``start ..`` of a request whose keys are all of ``k``: the plain function over the whole sequence,
    with the queries put where they belong."""
    n = k.shape[0]
    full = np.zeros((n, q.shape[1], q.shape[2]))
    full[start:start + q.shape[0]] = q
    see = P.visible(n, mask)
    return P.attention_heads(full, k, v, scale, see, sink=sink, slopes=slopes)[start:start + q.shape[0]]


MASKS = [
    # chunk, window, keep_first
    (None, None, 0), (24, None, 0), (64, None, 0), (1, None, 0), (None, 20, 0), (None, 20, 3), (None, 7, 70), (None, 1, 2),
    (100, None, 0), (None, 64, 1),
]
SHAPES = [
    # H, Hk, D, Dv, page
    (4, 2, 32, 32, 16), (8, 2, 64, 64, 64), (3, 1, 10, 6, 8), (6, 3, 48, 32, 32), (2, 2, 16, 16, 4), (5, 5, 80, 80, 16),
]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("mask", MASKS)
@pytest.mark.parametrize("shape", SHAPES)
def test_attention_with_masks_sinks_and_kept_keys(ops, dt, mask, shape):
    """A long portion from 0, a portion behind 150 keys, decoded tokens behind 37, 129 and 300 keys, in one batch:
    chunks counted from position 0, windows, kept first keys at their true distances, a sink a head, slopes."""
    H, Hk, D, Dv, ps = shape
    chunk, window, keep = mask
    rng = np.random.default_rng(H * 1000 + D + (chunk or 0) + 7 * (window or 0) + keep)
    starts, q_lens = [0, 150, 37, 129, 300], [140, 45, 1, 1, 1]
    lens = [s + n for s, n in zip(starts, q_lens)]
    tables, n_pages = scatter_pages(lens, ps, D + keep)
    ctx = FakeCtx(starts, q_lens, tables, ps)
    ks = [torch.tensor(rng.normal(size=(n, Hk, D))).to(DT[dt]) for n in lens]
    vs = [torch.tensor(rng.normal(size=(n, Hk, Dv))).to(DT[dt]) for n in lens]
    qs = [torch.tensor(rng.normal(size=(n, H, D)) * 2).to(DT[dt]) for n in q_lens]
    kc, vc = fill_pages(ks, vs, tables, n_pages, ps, DT[dt])
    # a window gives pages back: what lies wholly below every row's range, the kept pages aside, is gone
    reach = chunk or window
    if reach:
        tab = ctx._table.cpu()
        for b, s in enumerate(starts):
            for i in range(-(-keep // ps) if window else 0, max(0, s - reach + 1) // ps):
                tab[b, i] = -1
        ctx._table = tab.to(DEV)
    sinks = rng.normal(size=H) * 2
    sinks[0], sinks[-1] = 30.0, -30.0           # one that outweighs every key, one that none feels
    slopes = P.distance_slopes(H) if window else None
    scale = 0.7 / math.sqrt(D)
    q = torch.cat(qs).reshape(-1, H * D).contiguous().to(DEV)
    got = ops.attention(q, kc, vc, ctx, 0, H, Hk, D, ps, scale, window, slopes=dev(slopes) if slopes is not None else None,
                        chunk=chunk, keep_first=keep, sinks=dev(sinks), v_head_dim=Dv).float().cpu().numpy()
    m = {"size": chunk, "chunked": True} if chunk else ({"size": window, "keep_first": keep} if window else {})
    want = np.concatenate([plain_attention(qs[b].double().numpy(), ks[b].double().numpy(), vs[b].double().numpy(), starts[b],
                                           scale, m, sinks, slopes) for b in range(len(starts))]).reshape(-1, H * Dv)
    close(got, want, 2e-5 if dt == "float32" else 2e-2, f"{shape} {mask}")


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("ps", [16, 64])
@pytest.mark.parametrize("kind", ["chunk", "window", "kept"])
def test_one_key_stands_out_at_every_distance_over_an_edge(ops, dt, ps, kind):
    """One key whose score outweighs all others, and whose value is its own mark: a decoded token and the last row
    of a portion read it exactly when the mask lets them, for every place of the key from a few inside the edge
    to a few outside it, over page borders, far behind hundreds of fillers."""
    H, Hk, D = 4, 2, 32
    size, keep = 70, 5
    n = 420
    rng = np.random.default_rng(ps)
    for pos in (n - 1, 209, 280):                   # the reading position: not on a chunk's edge, on its last place, on its first
        for back in list(range(pos % size - 3, pos % size + 4)) if kind == "chunk" else \
                (list(range(size - 4, size + 4)) if kind == "window" else list(range(pos - keep - 3, pos - keep + 4)) + [pos, pos - 1]):
            j = pos - back
            if not (0 <= j <= pos):
                continue
            k = rng.normal(size=(pos + 1, Hk, D)) * 0.1
            v = rng.normal(size=(pos + 1, Hk, D)) * 0.1
            e = np.zeros(D); e[3] = 1.0
            k[j] = 40.0 * e
            v[j] = 9.0
            q = np.tile(2.0 * e, (H, 1))[None]
            if kind == "chunk":
                sees = j // size == pos // size
                m = {"size": size, "chunked": True}
            elif kind == "window":
                sees = pos - j < size
                m = {"size": size, "keep_first": 0}
            else:
                sees = pos - j < size or j < keep
                m = {"size": size, "keep_first": keep}
            for q_len in (1, 30):
                start = pos + 1 - q_len
                tables, n_pages = scatter_pages([pos + 1], ps, pos + j)
                ctx = FakeCtx([start], [q_len], tables, ps)
                kt, vt = torch.tensor(k).to(DT[dt]), torch.tensor(v).to(DT[dt])
                kc, vc = fill_pages([kt], [vt], tables, n_pages, ps, DT[dt])
                qq = np.concatenate([rng.normal(size=(q_len - 1, H, D)) * 0.1, q]) if q_len > 1 else q
                qd = torch.tensor(qq).to(DT[dt]).reshape(q_len, H * D).to(DEV)
                out = ops.attention(qd, kc, vc, ctx, 0, H, Hk, D, ps, 1.0, size if kind != "chunk" else None,
                                    chunk=size if kind == "chunk" else None, keep_first=keep if kind == "kept" else 0,
                                    sinks=dev(np.zeros(H))).float().cpu().numpy()[-1]
                assert (out.min() > 8.5) == sees and (sees or np.abs(out).max() < 1.0), \
                    f"{kind}: the key at {j} read from {pos} (portion of {q_len}): {out.min():.3g}..{out.max():.3g}, should see: {sees}"


def test_head_gate(ops):
    rng = np.random.default_rng(1)
    T, H, Dv = 9, 5, 12
    o, g = rng.normal(size=(T, H * Dv)), rng.normal(size=(T, H + 3)) * 3
    for dt, tol in (("float32", 2e-6), ("bfloat16", 8e-3)):
        od = dev(o, DT[dt])
        ops.head_gate_(od, dev(g)[:, 1:1 + H], H, Dv)
        want = dev(o, DT[dt]).double().cpu().numpy().reshape(T, H, Dv) * P.sigmoid(g[:, 1:1 + H])[:, :, None]
        close(od.float().cpu().numpy(), want.reshape(T, H * Dv), tol, "head gate")


def test_decays_from_their_projections(ops):
    rng = np.random.default_rng(2)
    T, H, D = 11, 3, 10
    z = rng.normal(size=(T, H * D + 5)) * 6
    for tau in (1.0, 12.0, 0.5):
        x = dev(z)
        ops.decay_prepare_(x[:, 2:2 + H * D], H, D, "sigmoid_root", tau=tau)
        close(x[:, 2:2 + H * D].cpu().numpy(), P.sigmoid(z[:, 2:2 + H * D]) ** (1.0 / tau), 3e-6, f"tau {tau}")
        assert np.array_equal(x[:, :2].cpu().numpy(), z[:, :2].astype(np.float32))
    a_log, bias = rng.normal(size=H), rng.normal(size=H * D)
    x = dev(z)
    ops.decay_prepare_(x[:, :H * D], H, D, "exp_softplus", a_log=dev(a_log), dt_bias=dev(bias))
    want = np.exp(-np.exp(a_log)[None, :, None] * P.softplus((z[:, :H * D] + bias).reshape(T, H, D))).reshape(T, H * D)
    close(x[:, :H * D].cpu().numpy(), want, 3e-6, "exp softplus")


def run_in_steps(ops, plan, lens, slots, rows, call):
    got = [None] * len(lens)
    at = [0] * len(lens)
    for takes in plan:
        take = [min(t, lens[r] - at[r]) for r, t in enumerate(takes)]
        live = [r for r in range(len(lens)) if take[r] > 0]
        if not live:
            continue
        ctx = step_ctx([at[r] for r in live], [take[r] for r in live], [slots[r] for r in live])
        o = call(ctx, dev(np.concatenate([rows[r][at[r]:at[r] + take[r]] for r in live]))).cpu().numpy()
        k = 0
        for r in live:
            if got[r] is None:
                got[r] = np.zeros((lens[r], o.shape[1]))
            got[r][at[r]:at[r] + take[r]] = o[k:k + take[r]]
            k += take[r]
            at[r] += take[r]
    assert at == list(lens)
    return got


@pytest.mark.parametrize("H,D,Dv", [(2, 8, 12), (3, 16, 16), (1, 48, 20), (2, 64, 64), (3, 10, 6), (1, 128, 32)])
def test_gated_linear_attention_in_portions(ops, H, D, Dv):
    """A decay a token and key channel, read out after the update; two requests in one batch, portions down to one
    row, the neighbours' state rows garbage.  One channel never decays and one forgets at once."""
    from xyntetik_runner_amd.csrc.ops import Ops
    rng = np.random.default_rng(H * 100 + D)
    lens = [70, 31]
    QK, V = H * D, H * Dv
    rows = [np.concatenate([rng.normal(size=(L, 2 * QK + V)), rng.uniform(0.3, 1.0, size=(L, QK))], axis=1) for L in lens]
    for x in rows:
        x[:, 2 * QK + V] = 1.0
        x[:, 2 * QK + V + 1] = 0.0
    want = []
    for x in rows:
        L = x.shape[0]
        q, k = x[:, :QK].reshape(L, H, D), x[:, QK:2 * QK].reshape(L, H, D)
        v, a = x[:, 2 * QK:2 * QK + V].reshape(L, H, Dv), x[:, 2 * QK + V:].reshape(L, H, D)
        want.append(np.stack([P.decay_recurrence(q[:, i], k[:, i], v[:, i], a[:, i]) for i in range(H)], axis=1).reshape(L, V))
    state = torch.full((4,) + Ops.recurrence_state_shape(H, D, Dv), float("nan"), device=DEV)
    state[0] = 0.0
    state[2] = 0.0
    call = lambda ctx, row: ops.linear_recurrence("gla", row[:, :QK], row[:, QK:2 * QK], row[:, 2 * QK:2 * QK + V], state, ctx,
                                                  H, H, D, Dv, gate=row[:, 2 * QK + V:])
    got = run_in_steps(ops, [(33, 2), (1, 1), (1, 1), (2, 20), (30, 1), (1, 1), (1, 1), (1, 1), (1, 4)], lens, [0, 2], rows, call)
    for r in (0, 1):
        close(got[r], want[r], 5e-6, f"request {r}")
    assert torch.isnan(state[1]).all() and torch.isnan(state[3]).all()


@pytest.mark.parametrize("H,D,Dv", [(2, 64, 32), (3, 16, 24)])
def test_gated_linear_attention_over_long_portions(ops, H, D, Dv):
    """Portions from 1,024 rows on run as chunks side by side; a write far back is kept by a channel that never decays."""
    from xyntetik_runner_amd.csrc.ops import Ops
    rng = np.random.default_rng(H + D)
    lens = [1300, 40, 2100]
    QK, V = H * D, H * Dv
    rows = [np.concatenate([rng.normal(size=(L, 2 * QK + V)) * 0.5, rng.uniform(0.9, 0.999, size=(L, QK))], axis=1) for L in lens]
    for x in rows:
        x[:, 2 * QK + V] = 1.0
        x[3, QK] = 50.0            # a write at token 3 into the channel that keeps everything
    want = []
    for x in rows:
        L = x.shape[0]
        q, k = x[:, :QK].reshape(L, H, D), x[:, QK:2 * QK].reshape(L, H, D)
        v, a = x[:, 2 * QK:2 * QK + V].reshape(L, H, Dv), x[:, 2 * QK + V:].reshape(L, H, D)
        want.append(np.stack([P.decay_recurrence(q[:, i], k[:, i], v[:, i], a[:, i]) for i in range(H)], axis=1).reshape(L, V))
    state = torch.full((5,) + Ops.recurrence_state_shape(H, D, Dv), float("nan"), device=DEV)
    slots = [4, 0, 2]
    for sl in slots:
        state[sl] = 0.0
    call = lambda ctx, row: ops.linear_recurrence("gla", row[:, :QK], row[:, QK:2 * QK], row[:, 2 * QK:2 * QK + V], state, ctx,
                                                  H, H, D, Dv, gate=row[:, 2 * QK + V:])
    got = run_in_steps(ops, [(1100, 40, 1024), (200, 0, 1076)], lens, slots, rows, call)
    for r in range(3):
        close(got[r], want[r], 3e-5, f"request {r}")


@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 16, 32), (2, 2, 32, 16), (3, 1, 10, 6), (4, 1, 64, 16), (2, 2, 128, 8)])
def test_delta_rule_with_a_decay_a_key_channel(ops, H, G, D, Dv):
    """``S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q`` with unit keys; head h reads key head
    h // (H / G); portions down to one row; beta and the decays in views of other row strides than q, k and v."""
    from xyntetik_runner_amd.csrc.ops import Ops
    rng = np.random.default_rng(H * 10 + D)
    lens = [61, 29]
    QK, V = G * D, H * Dv
    rows = []
    for L in lens:
        k = rng.normal(size=(L, G, D))
        k /= np.sqrt((k * k).sum(-1, keepdims=True))
        g = rng.uniform(0.5, 1.0, size=(L, H * D))
        g[:, 0], g[:, 1] = 1.0, 0.0
        rows.append(np.concatenate([rng.normal(size=(L, QK)), k.reshape(L, QK), rng.normal(size=(L, V)),
                                    rng.uniform(0.0, 1.0, size=(L, H)), g], axis=1))
    want = []
    for x in rows:
        L = x.shape[0]
        q, k = x[:, :QK].reshape(L, G, D), x[:, QK:2 * QK].reshape(L, G, D)
        v = x[:, 2 * QK:2 * QK + V].reshape(L, H, Dv)
        beta, g = x[:, 2 * QK + V:2 * QK + V + H], x[:, 2 * QK + V + H:].reshape(L, H, D)
        want.append(np.stack([P.delta_recurrence(q[:, i // (H // G)], k[:, i // (H // G)], v[:, i], beta[:, i], g[:, i])
                              for i in range(H)], axis=1).reshape(L, V))
    state = torch.full((3,) + Ops.recurrence_state_shape(H, D, Dv), float("nan"), device=DEV)
    state[0] = 0.0
    state[2] = 0.0
    b0 = 2 * QK + V
    call = lambda ctx, row: ops.linear_recurrence("delta_channel", row[:, :QK], row[:, QK:2 * QK], row[:, 2 * QK:b0], state, ctx,
                                                  H, G, D, Dv, beta=row[:, b0:b0 + H], gate=row[:, b0 + H:].contiguous())
    got = run_in_steps(ops, [(17, 2), (1, 1), (1, 1), (2, 20), (30, 1), (1, 1), (9, 1), (1, 2)], lens, [2, 0], rows, call)
    for r in (0, 1):
        close(got[r], want[r], 2e-5, f"request {r}")
    assert torch.isnan(state[1]).all()


def test_two_results_meet_in_one_sum(ops):
    rng = np.random.default_rng(4)
    for T, E in ((1, 30), (9, 64), (5, 1000)):
        x, yl, yr = rng.normal(size=(T, E)), rng.normal(size=(T, E)) * 3, rng.normal(size=(T, E)) * 0.2
        wl, wr = rng.normal(size=E), rng.normal(size=E)
        xd = dev(x)
        ops.pair_combine_(xd, dev(yl), dev(yr), 0.6, -0.9)
        close(xd.cpu().numpy(), x + 0.6 * yl - 0.9 * yr, 2e-6, "weighted sum")
        xd = dev(x)
        ops.pair_combine_(xd, dev(yl), dev(yr), 0.5, 0.5, dev(wl), dev(wr), 1e-5)
        close(xd.cpu().numpy(), x + 0.5 * (P.rms_div(yl, 1e-5) * wl + P.rms_div(yr, 1e-5) * wr), 3e-6, "normed sides")
        for dt, tol in (("float32", 3e-6), ("bfloat16", 8e-3)):      # and the norm that the next sublayer reads through, in the same pass
            xd, wn = dev(x), rng.normal(size=E)
            h = ops.pair_combine_(xd, dev(yl), dev(yr), 0.5, 0.5, dev(wl), dev(wr), 1e-5, then_norm=(dev(wn), 1e-6), out_dtype=DT[dt])
            upd = x + 0.5 * (P.rms_div(yl, 1e-5) * wl + P.rms_div(yr, 1e-5) * wr)
            close(xd.cpu().numpy(), upd, 3e-6, "normed sides, then a norm")
            close(h.float().cpu().numpy(), P.rms_div(upd, 1e-6) * wn, tol, f"the following norm in {dt}")
        xd, v = dev(x), rng.normal(size=E)
        ops.add_rows_(xd, dev(v))
        close(xd.cpu().numpy(), x + v, 1e-6, "a vector a row")
        ops.add_rows_(xd, dev(v), y=dev(yl))
        close(xd.cpu().numpy(), x + 2 * v + yl, 2e-6, "a vector and rows")


@pytest.mark.parametrize("n,top,groups,keep", [(16, 4, 4, 3), (8, 2, 4, 2), (6, 2, 3, 3), (4, 2, 4, 3), (8, 3, 2, 1), (5, 5, 1, 1),
                                               (12, 1, 1, 1), (64, 6, 8, 4), (130, 7, 13, 5)])
def test_choice_by_sigmoid_scores_within_the_best_groups(ops, n, top, groups, keep):
    """Scores are sigmoids, the choice adds the correction and is limited to the groups whose two best add up
    highest; corrections far below zero make choice scores negative, where a group left out must count as minus
    infinity and not as zero; the weights are the scores times a number, not their shares."""
    rng = np.random.default_rng(n + top)
    T = 200
    z = rng.normal(size=(T, n + 2)) * 2
    corr = rng.normal(size=n) * 0.3 - (3.0 if n % 2 == 0 else 0.0)
    idx, wts = ops.route_logits(dev(z)[:, 1:1 + n], dev(corr), top, scores="sigmoid", groups=groups, keep_groups=keep,
                                weight_scale=1.7)
    idx, wts = idx.cpu().numpy(), wts.cpu().numpy()
    checked = 0
    for t in range(T):
        if P.route_margin(z[t, 1:1 + n], corr, top, groups, keep) < 1e-5:
            continue                # (decided within the rounding of 32 bits)
        chosen, w = P.route(z[t, 1:1 + n], corr, top, groups, keep, 1.7)
        assert list(idx[t]) == list(chosen), f"row {t}"
        close(wts[t], w, 3e-6, f"weights of row {t}")
        checked += 1
    assert checked > T * 0.9


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_gate_of_the_tanh_form_of_gelu(ops, dt):
    rng = np.random.default_rng(5)
    T, E, F = 7, 64, 96
    h, w = dev(rng.normal(size=(T, E)), DT[dt]), dev(rng.normal(size=(2 * F, E)) * 0.3, DT[dt])
    gu = h.double().cpu().numpy() @ w.double().cpu().numpy().T
    want = P.gelu_tanh(gu[:, :F]) * gu[:, F:]
    got = ops.linear_gated(h, ops.pack_weight(w, gated=True), activation="gelu_tanh").float().cpu().numpy()
    close(got, want, 3e-6 if dt == "float32" else 1e-2, "gelu gate in the product")
    z = rng.normal(size=(T, 2 * F)) * 4
    close(ops.gate_mul(dev(z), "gelu_tanh").cpu().numpy(), P.gelu_tanh(z[:, :F]) * z[:, F:], 3e-6, "gelu gate alone")


# ----------------------------------------------------------------------------- a one-layer model with made weights
def needle_model(keep, window):
    """One layer of windowed attention beside retention (whose weight in the sum is zero), two heads on one key head,
    no feed-forward.  Token 1 (the needle) has a key along channel 0, where every query lies (through the query's bias,
    whatever the token), with a score of 36 before the bias of the distance; token 0 (the filler) has a key along
    channel 1, with a score around 0.  The needle's value lies along channel 0 too; the output matrix brings head 0's
    there to stream channel 5 and head 1's to channel 4, which rows 3 and 2 of the embedding read as logits."""
    E, V, H, D = 8, 4, 2, 4
    rng = np.random.default_rng(4)
    cfg = {"architecture": "Kegorax", "vocab": V, "width": E, "norm": {"eps": 1e-6},
           "layers": [{"type": "parallel_2", "mlp": None, "mixer": {
               "left": {"heads": H, "kv_heads": 1, "dim": D, "vdim": D, "scale": 1.0, "mask": {"size": window, "keep_first": keep}},
               "right": {"heads": 1, "dim": 4, "vdim": 4, "decay": [0.5]}, "left_scale": 1.0, "right_scale": 0.0}}]}
    emb = np.zeros((V, E)); emb[0, 1] = 1.0; emb[1, 0] = 1.0; emb[2, 4] = 1.0; emb[3, 5] = 1.0
    w = {"embed": emb, "l0.norm1": np.ones(E), "final.norm": np.ones(E)}
    bq = np.zeros(H * D); bq[0] = bq[D] = 1.0                        # channel 0 of both heads
    wk = rng.normal(size=(D, E)) * 0.01
    wk[0, 0] = 1.0                                                    # the needle's key: channel 0
    wk[1, 1] = 1.0                                                    # a filler's: channel 1
    wv = rng.normal(size=(D, E)) * 0.01
    wv[0, 0] = 1.0
    qn, kn = np.ones(D), np.ones(D)
    qn[0] = kn[0] = 3.0                                               # a unit vector of 4 channels has 2 in its one channel: 6 x 6
    o = rng.normal(size=(E, H * D)) * 0.01
    o[5, 0] = 2.0
    o[4, D] = 2.0
    p = "l0.mix.left."
    w.update({p + "q": rng.normal(size=(H * D, E)) * 0.01, p + "q.b": bq, p + "k": wk, p + "k.b": np.zeros(D), p + "v": wv,
              p + "v.b": np.zeros(D), p + "q.norm": qn, p + "k.norm": kn, p + "o": o})
    p = "l0.mix.right."
    w.update({p + n: rng.normal(size=(4, E)) * 0.1 for n in ("q", "k", "v", "g")})
    w[p + "o"] = rng.normal(size=(E, 4)) * 0.1
    return cfg, w


@pytest.mark.parametrize("page", [16, 64])
@pytest.mark.parametrize("decode_from", [None, 30])
@pytest.mark.parametrize("keep,window", [(3, 50), (20, 33)])
def test_a_kept_token_that_stands_out_through_the_engine(tmp_path, page, decode_from, keep, window):
    """The needle as the last kept token and as the first that is not kept: the first is read for as long as the request
    lives (by the head of the flat slope; the steep one loses it to the distance), the second until the window has passed
    it, to the position.  The window gives its pages back on the way, but for the kept ones.  In a prompt's portions and
    with all but 30 positions decoded one by one, in pools of a few pages."""
    import io
    import traces
    from xyntetik_runner_amd.config import config_from_dict
    from xyntetik_runner_amd.engine.runner import ModelRunner
    from xyntetik_runner_amd.trace import replay
    cfg, w = needle_model(keep, window)
    n = 700
    for jstar in (keep - 1, keep):
        toks = [0] * n
        toks[jstar] = 1
        want = P.forward(cfg, w, toks)
        assert (want[-1, 2] > 1.0) == (jstar < keep) and (want[-1, 2] < 0.5) == (jstar >= keep), "the made weights do not show the kept needle"
        assert want[jstar + window - 1, 2] > 1.0 and (jstar < keep or want[jstar + window, 2] < 0.5), "nor the window's edge"
        assert want[-1, 3] < 0.5 and want[jstar + 20, 3] > 1.0, "nor the steep head's loss"
        if decode_from is None:
            steps = traces.portions({"a": toks}, sizes=(17, 2, 40, 3, 400, 64))
        else:
            steps = traces.tail_one_by_one({"a": toks}, tail=n - decode_from)
        arch, typed = config_from_dict(cfg)
        tensors = {k: torch.tensor(v, dtype=torch.float32) for k, v in w.items()}
        runner = ModelRunner(arch.build_spec(typed), tensors, "float32", max_tokens=n + 64, page_size=page, max_requests=2,
                             max_step_tokens=400)
        for lc in runner.storage.layers:
            if lc.owns and lc.k is not None:
                lc.k.fill_(float("nan")); lc.v.fill_(float("nan"))
        if page == 16:      # the pool holds a window, a step and the kept pages, not the request
            assert runner.manager.groups[0].pool.size < n // page
        out = str(tmp_path / f"out{jstar}")
        replay(runner, traces.to_lines(steps), out, report=io.StringIO())
        runner.manager.check()
        got = traces.collect(steps, out, cfg["vocab"])
        close(got["a"], want, 1e-5, f"needle at {jstar}")


# ----------------------------------------------------------------------------- whole models at a sequence's start
def test_first_tokens_of_a_sequence(tmp_path):
    """Sequences of one, two and three tokens beside a longer one in a mixed batch: the states and the convolutions'
    inputs start at zero, position 0 reads itself and the sink alone, a chunk and a window begin at 0, and the step
    vector of every pass is added to a single row."""
    import io
    import traces
    from kegorax_tiny import make_model
    from plain_llama import load_folder
    from xyntetik_runner_amd.engine.runner import ModelRunner
    from xyntetik_runner_amd.trace import replay
    for which in ("K1", "K2", "K4"):
        d = make_model(which, str(tmp_path / which))
        cfg, w = load_folder(d)
        reqs = {f"r{n}": [int(t) for t in np.random.default_rng(n).integers(0, cfg["vocab"], size=n)] for n in (1, 2, 3, 30)}
        steps = traces.mixed(reqs, {k: min(2, len(v)) for k, v in reqs.items()}, max_live=4, seed=1)
        runner = ModelRunner.from_folder(d, dtype="float32", max_tokens=256, page_size=16, max_requests=4)
        out = str(tmp_path / (which + "out"))
        replay(runner, traces.to_lines(steps), out, report=io.StringIO())
        got = traces.collect(steps, out, cfg["vocab"])
        for rid, toks in reqs.items():
            close(got[rid], P.forward(cfg, w, toks), 2e-5, f"{which} {rid}")
