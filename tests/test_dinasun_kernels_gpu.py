"""Every mechanism of the Dinasun parts alone: the kernel against the plain function of
``plain_dinasun`` (or a few lines of float64 written here), with rows cut into requests and steps
the way an engine cuts them, and with inputs made so that a fault shows: state rows of other
requests that are garbage, a channel that never decays beside one that forgets at once, one key
whose score stands out thousands of positions back and at a page's border, a head whose slope hides
that key and a head whose slope does not, temperature steps at a portion's first and last row."""
import io
import math

import numpy as np
import pytest
import torch

import plain_dinasun as P
import traces
from test_kernels_gpu import FakeCtx, fill_cache, scatter_pages

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def ops():
    from xyntetik_runner_amd.csrc.ops import load_ops
    return load_ops()


def dev(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV)


def step_ctx(starts, q_lens, slots, tokens=None):
    """A step's context as the engine makes it: rows of the requests one after another."""
    from xyntetik_runner_amd.cache import RequestCache
    from xyntetik_runner_amd.csrc.ops import load_ops
    from xyntetik_runner_amd.engine.batch import StepContext, StepEntry
    tokens = tokens or [[0] * n for n in q_lens]
    entries = [StepEntry(b, list(tokens[b]), []) for b in range(len(q_lens))]
    rcs = [RequestCache(b, int(slots[b]), int(starts[b]), [], fresh=False) for b in range(len(q_lens))]
    return StepContext(load_ops(), torch.device(DEV), entries, rcs, 0)


def cuts(total, sizes):
    out, i, k = [], 0, 0
    while i < total:
        n = min(sizes[k % len(sizes)], total - i)
        out.append((i, n))
        i += n
        k += 1
    return out


def close(got, want, tol, what=""):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert np.isfinite(got).all(), f"{what}: not finite"
    err = np.abs(got - want).max() / max(1e-30, np.abs(want).max())
    assert err <= tol, f"{what}: {err:.3g} > {tol}"


# ----------------------------------------------------------------------------- dynamic tanh and the sandwich step
@pytest.mark.parametrize("T,E", [(1, 5), (7, 64), (33, 1030)])
@pytest.mark.parametrize("out", ["float32", "bfloat16"])
def test_dynamic_tanh(ops, T, E, out):
    rng = np.random.default_rng(E)
    x = rng.normal(size=(T, E)) * 2
    w = {"n": rng.normal(size=E), "n.b": rng.normal(size=E), "n.alpha": np.float64(0.37)}
    got = ops.dyt(dev(x), 0.37, dev(w["n"]), dev(w["n.b"]), DT[out])
    assert got.dtype == DT[out]
    close(got.float().cpu().numpy(), P.dyt(x, w, "n"), 2e-6 if out == "float32" else 5e-3, "dyt")
    rows = [T - 1, 0] if T > 1 else [0]
    sel = ops.dyt(dev(x), 0.37, dev(w["n"]), dev(w["n.b"]), torch.float32, rows=dev(rows, torch.int32))
    close(sel.cpu().numpy(), P.dyt(x[rows], w, "n"), 2e-6, "dyt of chosen rows")


@pytest.mark.parametrize("mult", [1.0, 0.6, 1.3])
@pytest.mark.parametrize("ydt", ["float32", "bfloat16"])
def test_sandwich_step_adds_the_normed_result_and_norms_for_the_next(ops, mult, ydt):
    """``x += m (tanh(a y) w + b)`` and the next sublayer's ``tanh(a' x) w' + b'`` in one pass, each half alone too."""
    rng = np.random.default_rng(3)
    T, E = 19, 72
    x, y = rng.normal(size=(T, E)), rng.normal(size=(T, E)) * 3
    yd = dev(y, DT[ydt])
    y = yd.float().cpu().numpy().astype(np.float64)
    post = {"n": rng.normal(size=E), "n.b": rng.normal(size=E) * 0.1, "n.alpha": np.float64(0.8)}
    nxt = {"n": rng.normal(size=E), "n.b": rng.normal(size=E) * 0.1, "n.alpha": np.float64(1.9)}
    want_x = x + mult * P.dyt(y, post, "n")
    want_h = P.dyt(want_x, nxt, "n")
    tup = lambda w: (float(w["n.alpha"]), dev(w["n"]), dev(w["n.b"]))
    xd = dev(x)
    h = ops.dyt_step(xd, yd, post=tup(post), mult=mult, norm=tup(nxt), out_dtype=torch.float32)
    close(xd.cpu().numpy(), want_x, 2e-6, "residual")
    close(h.cpu().numpy(), want_h, 3e-6, "next norm")
    xd = dev(x)
    assert ops.dyt_step(xd, yd, post=tup(post), mult=mult) is None
    close(xd.cpu().numpy(), want_x, 2e-6, "residual alone")


# ----------------------------------------------------------------------------- time mixing: the mixes
@pytest.mark.parametrize("E,n", [(40, 5), (64, 1), (130, 3)])
def test_mixes_with_the_row_before(ops, E, n):
    """Two requests side by side, cut into portions and single rows: the row before a portion's first is the
    state's, the row before a sequence's first is zero, and a neighbour's garbage row is never read."""
    rng = np.random.default_rng(E)
    lens = [57, 23]
    h = [rng.normal(size=(L, E)) for L in lens]
    mu = rng.uniform(-0.5, 1.5, size=(n, E))
    want = [np.concatenate([x + (P.shifted(x) - x) * mu[s] for s in range(n)], axis=1) for x in h]
    state = torch.full((4, E), float("nan"), device=DEV)
    state[1] = 0.0
    state[3] = 0.0
    got = [np.zeros_like(w) for w in want]
    at = [0, 0]
    plan = [(20, 1), (1, 1), (1, 2), (2, 0), (30, 5), (1, 1), (1, 1), (1, 12)]
    for a, b in plan:
        take = [min(a, lens[0] - at[0]), min(b, lens[1] - at[1])]
        live = [r for r in (0, 1) if take[r] > 0]
        ctx = step_ctx([at[r] for r in live], [take[r] for r in live], [1 if r == 0 else 3 for r in live])
        rows = np.concatenate([h[r][at[r]:at[r] + take[r]] for r in live])
        out = ops.token_shift(dev(rows), dev(mu), state, ctx, torch.float32).cpu().numpy()
        k = 0
        for r in live:
            got[r][at[r]:at[r] + take[r]] = out[k:k + take[r]]
            k += take[r]
            at[r] += take[r]
    assert at == lens
    for r in (0, 1):
        close(got[r], want[r], 2e-6, f"request {r}")
    assert torch.isnan(state[0]).all() and torch.isnan(state[2]).all()


# ----------------------------------------------------------------------------- time mixing: the recurrence
@pytest.mark.parametrize("H,D", [(2, 8), (3, 16), (1, 48), (2, 64), (3, 10), (1, 128)])
def test_wkv_recurrence_in_portions(ops, H, D):
    """Read-out before the update with the bonus for the token itself, a decay a token and key channel
    from its double logarithm; two requests in one batch, portions down to one row."""
    from xyntetik_runner_amd.csrc.ops import Ops
    rng = np.random.default_rng(H * 100 + D)
    lens = [70, 31]
    N = H * D
    rows = [rng.normal(size=(L, 4 * N)) for L in lens]          # r, k, v, x
    for x in rows:
        x[:, N:2 * N] *= 0.5
        x[:, 3 * N:] = rng.uniform(-4.0, 0.5, size=(x.shape[0], N))
    u = rng.normal(size=(H, D)) * 0.5
    want = []
    for x in rows:
        L = x.shape[0]
        r, k, v = (x[:, i * N:(i + 1) * N].reshape(L, H, D) for i in range(3))
        decay = np.exp(-np.exp(x[:, 3 * N:])).reshape(L, H, D)
        want.append(np.stack([P.wkv_recurrence(r[:, i], k[:, i], v[:, i], decay[:, i], u[i]) for i in range(H)], axis=1).reshape(L, N))
    state = torch.full((4,) + Ops.recurrence_state_shape(H, D, D), float("nan"), device=DEV)
    state[0] = 0.0
    state[2] = 0.0
    got = [np.zeros_like(w) for w in want]
    at = [0, 0]
    for a, b in [(33, 2), (1, 1), (1, 1), (2, 20), (30, 1), (1, 1), (1, 1), (1, 1), (1, 4)]:
        take = [min(a, lens[0] - at[0]), min(b, lens[1] - at[1])]
        live = [r for r in (0, 1) if take[r] > 0]
        ctx = step_ctx([at[r] for r in live], [take[r] for r in live], [0 if r == 0 else 2 for r in live])
        row = dev(np.concatenate([rows[r][at[r]:at[r] + take[r]] for r in live]))
        o = ops.linear_recurrence("wkv", row[:, :N], row[:, N:2 * N], row[:, 2 * N:3 * N], state, ctx, H, H, D, D,
                                  gate=row[:, 3 * N:].contiguous(), decay=dev(u)).cpu().numpy()
        k = 0
        for r in live:
            got[r][at[r]:at[r] + take[r]] = o[k:k + take[r]]
            k += take[r]
            at[r] += take[r]
    assert at == lens
    for r in (0, 1):
        close(got[r], want[r], 5e-6, f"request {r}")


@pytest.mark.parametrize("H,D", [(2, 64), (3, 16), (1, 40)])
def test_wkv_recurrence_over_long_portions(ops, H, D):
    """Portions from 1,024 rows on run as chunks side by side: a chunk's last state from zero plus the state
    before it times the product of the chunk's decays, channel by channel.  Three requests in one step (a long
    portion that ends inside a chunk, a short one, one of exactly four chunks), then their rest from the
    states that the chunks left; decays from 0.69 to 0.9975, so that a chunk's first state still counts at its end."""
    from xyntetik_runner_amd.csrc.ops import Ops
    rng = np.random.default_rng(H + D)
    lens = [1300, 40, 2100]
    N = H * D
    rows = [rng.normal(size=(L, 4 * N)) for L in lens]
    for x in rows:
        x[:, N:2 * N] *= 0.3
        x[:, 3 * N:] = rng.uniform(-6.0, -1.0, size=(x.shape[0], N))
    u = rng.normal(size=(H, D)) * 0.5
    want = []
    for x in rows:
        L = x.shape[0]
        r, k, v = (x[:, i * N:(i + 1) * N].reshape(L, H, D) for i in range(3))
        decay = np.exp(-np.exp(x[:, 3 * N:])).reshape(L, H, D)
        want.append(np.stack([P.wkv_recurrence(r[:, i], k[:, i], v[:, i], decay[:, i], u[i]) for i in range(H)], axis=1).reshape(L, N))
    state = torch.full((5,) + Ops.recurrence_state_shape(H, D, D), float("nan"), device=DEV)
    slots = [4, 0, 2]
    for sl in slots:
        state[sl] = 0.0
    got = [np.zeros_like(w) for w in want]
    at = [0, 0, 0]
    for takes in ([1100, 40, 1024], [200, 0, 1076]):
        live = [r for r in range(3) if takes[r] > 0]
        ctx = step_ctx([at[r] for r in live], [takes[r] for r in live], [slots[r] for r in live])
        row = dev(np.concatenate([rows[r][at[r]:at[r] + takes[r]] for r in live]))
        o = ops.linear_recurrence("wkv", row[:, :N], row[:, N:2 * N], row[:, 2 * N:3 * N], state, ctx, H, H, D, D,
                                  gate=row[:, 3 * N:].contiguous(), decay=dev(u)).cpu().numpy()
        k = 0
        for r in live:
            got[r][at[r]:at[r] + takes[r]] = o[k:k + takes[r]]
            k += takes[r]
            at[r] += takes[r]
    assert at == lens
    for r in range(3):
        close(got[r], want[r], 2e-5, f"request {r}")
    assert torch.isnan(state[1]).all() and torch.isnan(state[3]).all()


@pytest.mark.parametrize("n,sizes", [(610, [40, 1, 1, 300, 2, 1]), (2700, [1500, 1, 1100, 2])])
def test_a_far_write_is_kept_by_a_channel_that_does_not_decay(ops, n, sizes):
    """Token 2 writes a value along key channel 0 (decay exp(-exp(-30)) = 1) and another along channel 1
    (decay exp(-exp(1)) = 0.07): 600 tokens later (or 2,700, across chunks) a query on channel 0 returns the
    first whole, a query on channel 1 nothing.  The bonus enters the token's own read-out and is not written into the state."""
    from xyntetik_runner_amd.csrc.ops import Ops
    H, D = 2, 12
    N = H * D
    rng = np.random.default_rng(8)
    r = np.zeros((n, H, D)); k = rng.normal(size=(n, H, D)) * 0.01; v = rng.normal(size=(n, H, D))
    x = np.full((n, H, D), -1.0)
    x[:, :, 0], x[:, :, 1] = -30.0, 1.0
    r[:, 0, 0] = 1.0                 # head 0 asks channel 0, head 1 channel 1
    r[:, 1, 1] = 1.0
    k[:, :, :2] = 0.0
    k[2, :, :2] = 1.0
    v[2] = 100.0
    u = np.zeros((H, D)); u[:, :2] = 7.0
    decay = np.exp(-np.exp(x))
    want = np.stack([P.wkv_recurrence(r[:, i], k[:, i], v[:, i], decay[:, i], u[i]) for i in range(H)], axis=1)
    assert want[-1, 0, 0] > 99 and abs(want[-1, 1, 0]) < 1e-6
    assert want[2, 0, 0] > 690 and want[3, 0, 0] < 101          # the bonus: 7 x at the token itself, gone at the next
    state = torch.full((3,) + Ops.recurrence_state_shape(H, D, D), float("nan"), device=DEV)
    state[1] = 0.0
    got = np.zeros((n, H, D))
    for i, m in cuts(n, sizes):
        ctx = step_ctx([i], [m], [1])
        row = dev(np.concatenate([a[i:i + m].reshape(m, -1) for a in (r, k, v, x)], axis=1))
        o = ops.linear_recurrence("wkv", row[:, :N], row[:, N:2 * N], row[:, 2 * N:3 * N], state, ctx, H, H, D, D,
                                  gate=row[:, 3 * N:].contiguous(), decay=dev(u))
        got[i:i + m] = o.cpu().numpy().reshape(m, H, D)
    close(got, want, 5e-6, "far write")


# ----------------------------------------------------------------------------- attention: head norms and the temperature
@pytest.mark.parametrize("H,Hk,D", [(4, 2, 16), (3, 1, 10), (8, 8, 64), (2, 1, 48), (1, 1, 128)])
@pytest.mark.parametrize("coef,every", [(0.4, 5), (0.25, 1), (1.0, 64), (0.0, 0)])
def test_head_norms_and_query_temperature(ops, H, Hk, D, coef, every):
    """Positions on both sides of several steps of the temperature, also as a portion's first and last row."""
    rng = np.random.default_rng(H * D + every)
    pos = list(range(0, 12)) + [62, 63, 64, 126, 127, 128, 4999, 5000] + [every * 3 - 1, every * 3] * (every > 1)
    T = len(pos)
    row = rng.normal(size=(T, (H + 2 * Hk) * D)) * 3
    wq, wk = rng.normal(size=D), rng.normal(size=D)
    eps = 1e-5
    q = row[:, :H * D].reshape(T, H, D)
    k = row[:, H * D:(H + Hk) * D].reshape(T, Hk, D)
    want_q = P.rms_div(q, eps) * wq
    if every:
        want_q = want_q * P.query_temperature(pos, coef, every)[:, None, None]
    want_k = P.rms_div(k, eps) * wk
    rd = dev(row)
    ops.head_rmsnorm_(rd[:, :H * D].view(T, H, D), rd[:, H * D:(H + Hk) * D].view(T, Hk, D), dev(wq), dev(wk), eps,
                      positions=dev(pos, torch.int32), temp_coef=coef, temp_every=every)
    got = rd.cpu().numpy()
    close(got[:, :H * D].reshape(T, H, D), want_q, 3e-6, "queries")
    close(got[:, H * D:(H + Hk) * D].reshape(T, Hk, D), want_k, 3e-6, "keys")
    assert np.array_equal(got[:, (H + Hk) * D:], row[:, (H + Hk) * D:].astype(np.float32)), "the values (the keys as projected) changed"


# ----------------------------------------------------------------------------- attention: distance slopes
def slopes_of(H):
    return np.asarray([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)])


def ref_attention_slopes(q, k_seq, v_seq, starts, q_lens, scale, slopes):
    """float64, request by request and row by row: softmax over keys 0 .. p of ``q . k scale - slope_h (p - j)``."""
    outs, t = [], 0
    for b, (s, n) in enumerate(zip(starts, q_lens)):
        k, v = k_seq[b].double().numpy(), v_seq[b].double().numpy()
        H, Hk = q.shape[1], k.shape[1]
        for i in range(n):
            p = s + i
            o = np.zeros((H, v.shape[2]))
            for h in range(H):
                g = h // (H // Hk)
                sc = (k[:p + 1, g] @ q[t, h].double().numpy()) * scale - slopes[h] * (p - np.arange(p + 1))
                o[h] = P.softmax(sc) @ v[:p + 1, g]
            outs.append(o)
            t += 1
    return np.stack(outs)


SLOPE_CASES = [
    # H, Hk, D, page, starts, q_lens
    (4, 2, 16, 16, [0, 5, 100], [33, 1, 1]),
    (8, 2, 64, 64, [0, 63, 900], [150, 2, 1]),          # whole tiles of a prompt beside two short rows and a decoded one
    (16, 4, 128, 64, [37, 0, 1500], [16, 200, 1]),      # sixteen slopes from 0.7 to 1 / 256
    (3, 1, 48, 32, [0, 200], [70, 1]),                  # a head count that is no power of two: slopes that are no powers of two
    (2, 2, 24, 8, [0, 30], [12, 1]),                    # small pages, a head size no multiple of 16: the 32-bit kernel
    (1, 1, 64, 16, [0, 300], [65, 3]),                  # one head: its slope is 1 / 256
    (8, 2, 128, 64, [20001], [1]),                      # a decoded token behind 20,000 keys: key ranges that are merged
    (8, 8, 64, 64, [17000], [40]),                      # a portion behind 17,000 keys
]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", SLOPE_CASES)
def test_attention_with_distance_slopes(ops, dt, case):
    H, Hk, D, ps, starts, q_lens = case
    torch.manual_seed(H * 100 + D)
    lens = [s + n for s, n in zip(starts, q_lens)]
    tables, n_pages = scatter_pages(lens, ps, D)
    ctx = FakeCtx(starts, q_lens, tables, ps)
    T = sum(q_lens)
    q = (torch.randn(T, H, D) * 1.5).to(DT[dt])
    k_seq = [torch.randn(n, Hk, D).to(DT[dt]) for n in lens]
    v_seq = [torch.randn(n, Hk, D).to(DT[dt]) for n in lens]
    kc, vc = fill_cache(k_seq, v_seq, tables, n_pages, ps, DT[dt])
    scale = 0.7 / math.sqrt(D)
    sl = slopes_of(H)
    want = ref_attention_slopes(q.float(), [k.float() for k in k_seq], [v.float() for v in v_seq], starts, q_lens, scale, sl)
    got = ops.attention(q.to(DEV).reshape(T, H * D).contiguous(), kc, vc, ctx, 0, H, Hk, D, ps, scale, None, slopes=dev(sl))
    got = got.float().cpu().numpy().reshape(T, H, D)
    assert np.isfinite(got).all(), "read a slot no request owns"
    close(got, want, 5e-6 if dt == "float32" else 1.2e-2, "slopes")
    plain = ops.attention(q.to(DEV).reshape(T, H * D).contiguous(), kc, vc, ctx, 0, H, Hk, D, ps, scale, None)
    assert np.abs(plain.float().cpu().numpy().reshape(T, H, D) - want).max() > 0.05, "the slopes made no difference"


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("ps,needle", [(64, 0), (64, 63), (64, 64), (16, 4111), (32, 1023)])
@pytest.mark.parametrize("q_len", [1, 2, 70])
def test_one_key_that_stands_out_far_back(ops, dt, ps, needle, q_len):
    """Every query lies along channel 0, and so does one key, 5,000 positions back (or less), at a page's
    first or last place, with a score of 40 before the bias; the other keys score around 0.  The head with
    slope 1/256 still reads the needle's value (the bias is 20 at most), the head with slope 1/16 does not
    (its bias is 300): a slope of the wrong head, a bias from the key's place alone, or a lost far page
    would show."""
    H, Hk, D = 2, 1, 16
    n = 5000 + q_len
    start = n - q_len
    rng = np.random.default_rng(needle + q_len)
    k = rng.normal(size=(n, Hk, D)) * 0.05
    v = rng.normal(size=(n, Hk, D))
    k[:, 0, 0] = 0.0
    k[needle, 0, 0] = 10.0
    v[needle] = 0.0
    v[needle, 0, 1] = 64.0
    q = rng.normal(size=(q_len, H, D)) * 0.05
    q[:, :, 0] = 4.0
    scale = 1.0
    sl = slopes_of(H)
    tables, n_pages = scatter_pages([n], ps, needle)
    ctx = FakeCtx([start], [q_len], tables, ps)
    kt, vt, qt = (torch.tensor(a, dtype=torch.float32).to(DT[dt]) for a in (k, v, q))
    kc, vc = fill_cache([kt], [vt], tables, n_pages, ps, DT[dt])
    want = ref_attention_slopes(qt.float(), [kt.float()], [vt.float()], [start], [q_len], scale, sl)
    assert want[:, 1, 1].min() > 60 and np.abs(want[:, 0, 1]).max() < 5, "the made inputs do not show the needle"
    got = ops.attention(qt.to(DEV).reshape(q_len, H * D).contiguous(), kc, vc, ctx, 0, H, Hk, D, ps, scale, None, slopes=dev(sl))
    close(got.float().cpu().numpy().reshape(q_len, H, D), want, 1e-5 if dt == "float32" else 1.2e-2, "needle")


# ----------------------------------------------------------------------------- experts by a table
@pytest.mark.parametrize("n,top,V", [(6, 2, 50), (3, 1, 17), (4, 4, 9), (1, 1, 5)])
def test_table_choice(ops, n, top, V):
    rng = np.random.default_rng(V)
    table = np.stack([rng.permutation(n)[:top] for _ in range(V)]).astype(np.int32)
    ids = rng.integers(0, V, size=41)
    idx, wts = ops.table_route(dev(table, torch.int32), dev(ids, torch.int32), n)
    assert np.array_equal(idx.cpu().numpy(), table[ids])
    assert np.array_equal(wts.cpu().numpy(), np.full((41, top), np.float32(1.0 / top)))


@pytest.mark.parametrize("dt,tol", [("float32", 5e-6), ("bfloat16", 2e-2)])
@pytest.mark.parametrize("n,top,E,F,T", [(6, 2, 40, 24, 5), (3, 1, 17, 5, 9), (4, 4, 64, 96, 3), (1, 1, 32, 16, 4),
                                         (6, 2, 64, 24, 70), (8, 3, 128, 80, 300), (5, 5, 32, 8, 33), (1, 1, 64, 40, 100)])
def test_gated_experts_chosen_by_token_id(ops, n, top, E, F, T, dt, tol):
    """A few rows (the experts' weights are streamed) and many (sorted by expert, on the matrix cores in
    bfloat16): the sum of the chosen gated experts, each with the weight 1 / top."""
    rng = np.random.default_rng(n * 1000 + T)
    V = 37
    w = {"table": np.stack([rng.permutation(n)[:top] for _ in range(V)])}
    for e in range(n):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = rng.normal(size=(F, E)) * 0.3, rng.normal(size=(F, E)) * 0.3, rng.normal(size=(E, F)) * 0.3
    rnd = lambda a: torch.tensor(a, dtype=torch.float32).to(DT[dt]).double().numpy()       # the plain side reads what the kernel reads
    w = {k: (rnd(a) if k != "table" else a) for k, a in w.items()}
    h = rnd(rng.normal(size=(T, E)))
    ids = rng.integers(0, V, size=T)
    want = P.table_experts(h, ids, w, {"router": {"experts": n, "top": top}}, "")
    w_up = torch.stack([torch.cat([dev(w[f"e{e}.gate"], DT[dt]), dev(w[f"e{e}.up"], DT[dt])]) for e in range(n)]).contiguous()
    w_down = torch.stack([dev(w[f"e{e}.down"], DT[dt]) for e in range(n)]).contiguous()
    idx, wts = ops.table_route(dev(w["table"], torch.int32), dev(ids, torch.int32), n)
    got = ops.moe_experts(dev(h, DT[dt]), w_up, w_down, idx, wts, activation="swiglu")
    close(got.cpu().numpy(), want, tol, "experts")
    base = torch.ones_like(got)
    ops.moe_experts(dev(h, DT[dt]), w_up, w_down, idx, wts, out=base, accumulate=True, activation="swiglu")
    close(base.cpu().numpy(), want + 1.0, tol, "experts added to what is there")


# ----------------------------------------------------------------------------- a one-layer model with made weights
def needle_model():
    """One attention layer, two heads on one key head, no feed-forward.  Token 1 (the needle) has a key along
    channel 0, where every query lies (through the query's bias, whatever the token), with a score of 36 before the
    bias of the distance; token 0 (the filler) has a key along channel 1, with a score around 0.  The value is the
    key as projected, so the needle's lands in channel 0 of a head's output; the output matrix brings head 0's
    there to stream channel 5 and head 1's to channel 4, which rows 3 and 2 of the embedding read as logits."""
    E, V, H, D = 8, 4, 2, 4
    rng = np.random.default_rng(4)
    cfg = {"architecture": "Dinasun", "vocab": V, "width": E, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
           "layers": [{"type": "attention", "mixer": {"heads": H, "kv_heads": 1, "dim": D, "vdim": D, "scale": 1.0}, "mlp": None}]}
    emb = np.zeros((V, E)); emb[0, 1] = 1.0; emb[1, 0] = 1.0; emb[2, 4] = 1.0; emb[3, 5] = 1.0
    w = {"embed": emb}
    for n in ("l0.norm1", "l0.norm1b", "final.norm"):
        w[n], w[n + ".b"], w[n + ".alpha"] = np.ones(E), np.zeros(E), np.asarray(1.0)
    wq = rng.normal(size=(H * D, E)) * 0.01
    bq = np.zeros(H * D); bq[0] = bq[D] = 1.0                        # channel 0 of both heads
    wk = rng.normal(size=(D, E)) * 0.01
    wk[0, 0] = 1.0                                                    # the needle's key: channel 0
    wk[1, 1] = 1.0                                                    # a filler's: channel 1
    qn, kn = np.ones(D), np.ones(D)
    qn[0] = kn[0] = 3.0                                               # a unit vector of 4 channels has 2 in its one channel: 6 x 6
    o = rng.normal(size=(E, H * D)) * 0.01
    o[5, 0] = 2.0
    o[4, D] = 2.0
    w.update({"l0.mix.q": wq, "l0.mix.q.b": bq, "l0.mix.k": wk, "l0.mix.k.b": np.zeros(D), "l0.mix.q.norm": qn, "l0.mix.k.norm": kn,
              "l0.mix.o": o})
    return cfg, w


def engine_logits(cfg, w, steps, dtype, page, max_tokens, tmp_path):
    from xyntetik_runner_amd.config import config_from_dict
    from xyntetik_runner_amd.engine.runner import ModelRunner
    from xyntetik_runner_amd.trace import replay
    arch, typed = config_from_dict(cfg)
    tensors = {k: torch.tensor(v, dtype=torch.float32) for k, v in w.items()}
    runner = ModelRunner(arch.build_spec(typed), tensors, dtype, max_tokens=max_tokens, page_size=page, max_requests=2)
    for lc in runner.storage.layers:
        if lc.owns and lc.k is not None:
            lc.k.fill_(float("nan")); lc.v.fill_(float("nan"))
    out = str(tmp_path / "out")
    replay(runner, traces.to_lines(steps), out, report=io.StringIO())
    return traces.collect(steps, out, cfg["vocab"])


@pytest.mark.parametrize("page", [16, 64])
@pytest.mark.parametrize("decode_from", [None, 30])
def test_one_key_that_stands_out_through_the_engine(tmp_path, page, decode_from):
    """The needle at the start, at a page's last and first place: 1,500 (decoded: 800) tokens later, among the fillers, the
    head of slope 1/256 still reads it (logit 2), the head of slope 1/16 has lost it since some 500 tokens
    (logit 3) and had it before.  In a prompt's portions and with all but 30 positions decoded one by one."""
    cfg, w = needle_model()
    n = 1560 if decode_from is None else 900
    for jstar in (3, 63, 64):
        toks = [0] * n
        toks[jstar] = 1
        want = P.forward(cfg, w, toks)
        assert want[-1, 2] > 0.5 and want[-1, 3] < 0.05 and want[jstar + 100, 3] > 0.5, "the made weights do not show the needle"
        assert want[jstar - 1, 2] < 0.05, "the needle shows before it is there"
        if decode_from is None:
            steps = traces.portions({"a": toks}, sizes=(17, 2, 40, 3, 1100, 64))
        else:
            steps = traces.tail_one_by_one({"a": toks}, tail=n - decode_from)
        got = engine_logits(cfg, w, steps, "float32", page, -(-n // 64) * 64 + 64, tmp_path / f"{jstar}")
        close(got["a"], want, 1e-5, f"needle at {jstar}")


# ----------------------------------------------------------------------------- whole models at a sequence's start
def test_first_tokens_of_a_sequence(tmp_path):
    """Sequences of one, two and three tokens beside a longer one in a mixed batch: the row before the
    first is zero, the state starts at zero, position 0 has a temperature of its own when the step is 1,
    and the injection runs for a single row."""
    from dinasun_tiny import make_model
    from plain_llama import load_folder
    from xyntetik_runner_amd.engine.runner import ModelRunner
    from xyntetik_runner_amd.trace import replay
    for which in ("D1", "D2"):
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
