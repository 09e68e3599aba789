"""The Melizen decoder on the GPU against the plain implementation (``plain_melizen.py``): each mechanism's
kernels alone, with inputs made so that a fault shows, then whole models through the engine's step function, its
cache and state, its batching and its generation loop."""
import numpy as np
import pytest
import torch

import plain_melizen as P
from melizen_models import CONFIGS, TOL, close, model, row_errors, tokens

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
TD = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.ascontiguousarray(a)).to(dtype).to(DEV)


def i32(a):
    return torch.as_tensor(np.asarray(a, np.int32)).to(DEV)


def engine(name, dtype, **kw):
    from gpullama3_java_amd.engine import Engine
    folder, cfg, W = model(name)
    kw.setdefault("max_tokens", 2048)
    kw.setdefault("n_slots", 6)
    return Engine.from_folder(folder, dtype=dtype, **kw), cfg, W


# ----------------------------------------------------------------- the attention's kernel
def paged(k, v, page, dtype):
    """One sequence's keys [S, G, D] and values [S, G, Dv] as a paged cache in the kernels' order; the sequence's
    pages are 1, 2, ... (page 0 is nobody's). Returns (k_cache, v_cache, block table [1, pages])."""
    from gpullama3_java_amd.cache.layout import tile_keys, tile_values
    S, G, D = k.shape
    Dv = v.shape[2]
    n = -(-S // page)
    kc = np.zeros((n + 1, G, page, D), np.float32)
    vc = np.zeros((n + 1, G, Dv, page), np.float32)
    for j in range(S):
        kc[1 + j // page, :, j % page] = k[j]
        vc[1 + j // page, :, :, j % page] = v[j]
    return (dev(tile_keys(kc), TD[dtype]), dev(tile_values(vc), TD[dtype]), i32(np.arange(1, n + 1)[None]))


def run_attention(q, k, v, positions, dtype, window, scale, slopes, sink, page=64):
    from gpullama3_java_amd.csrc import lib as K
    T, H, D = q.shape
    G, Dv = k.shape[1], v.shape[2]
    kc, vc, table = paged(k, v, page, dtype)
    out = torch.zeros(T, H * Dv, dtype=TD[dtype], device=DEV)
    K.attention_generic(dev(q.reshape(T, H * D), TD[dtype]), kc, vc, i32(positions), i32([0] * T), table, out, H, G, D,
                        page, window, scale, v_head_dim=Dv, slopes=None if slopes is None else dev(slopes), sink=sink)
    return out.float().cpu().numpy().reshape(T, H, Dv)


def plain_attention_at(q, k, v, positions, window, scale, slopes, sink):
    return np.concatenate([P.sink_attention(q[t:t + 1], k, v, scale, window, slopes, sink, first=p)
                           for t, p in enumerate(positions)])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, D, Dv, window", [(4, 2, 32, 48, 37), (3, 3, 16, 16, 64), (8, 1, 48, 32, 130)])
def test_attention_keys_just_inside_and_just_outside_the_window(dtype, H, G, D, Dv, window):
    """One key's score stands out, and its value is like no other: at distance window - 1 the output is that
    value, at distance window it must not appear. Queries in the first tokens, at page borders, far on."""
    rng = np.random.default_rng(window)
    S = 400
    k = 0.05 * rng.standard_normal((S, G, D))
    v = 0.1 * rng.standard_normal((S, G, Dv))
    positions = [1, window - 1, window, 64, 127, 200, 399]         # (two queries each: fewer than the smallest head has columns)
    qs, edge, used = [], [], set()
    for n, p in enumerate(positions):
        for dist in (window - 1, window):
            j = p - dist
            q = 0.05 * rng.standard_normal((H, D))
            if j in used:
                j = -1                       # (that key is another query's already)
            used.add(j)
            c = len(qs)                      # the query's own column: no other query or marked key has anything there
            q[:, :len(positions) * 2] = 0.0
            if j >= 0:
                k[j] = 0.0
                k[j, :, c] = 6.0
                v[j] = 0.0
                v[j, :, c] = 3.0
                q[:, c] = 6.0
            qs.append(q)
            edge.append((p, j, dist))
    # (two queries a position share nothing: each marked key is its own)
    pos2 = [p for p, _, _ in edge]
    k, v = k.astype(np.float32), v.astype(np.float32)
    bf = lambda a: torch.tensor(a).to(TD[dtype]).float().numpy()
    q, k, v = bf(np.array(qs, np.float32)), bf(k), bf(v)
    slopes = P.head_slopes(H)
    got = run_attention(q, k, v, pos2, dtype, window, 1.0, slopes, 0.0)
    ref = plain_attention_at(q, k, v, pos2, window, 1.0, slopes, 0.0)
    tol = 2e-5 if dtype == "float32" else 2e-2
    np.testing.assert_allclose(got, ref, atol=tol * 3.0)
    for t, (p, j, dist) in enumerate(edge):
        if j >= 0 and dist == window - 1 and 6.0 * 6.0 - slopes[0] * dist > 20:
            assert got[t, 0, t] > 2.0, (p, j)               # the key just inside is seen
        if j >= 0 and dist == window:
            assert abs(got[t, :, t]).max() < 0.5, (p, j)    # the key just outside is not


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_sink_takes_its_share_and_the_bias_grows_with_the_distance(dtype):
    rng = np.random.default_rng(5)
    H, G, D, Dv, S = 4, 2, 16, 32, 150
    bf = lambda a: torch.tensor(np.asarray(a, np.float32)).to(TD[dtype]).float().numpy()
    k = bf(rng.standard_normal((S, G, D)))
    v = bf(1.0 + 0.1 * rng.standard_normal((S, G, Dv)))
    positions = [0, 3, 70, 149]
    # every score far below the sink's: the weights of the real keys sum to almost nothing
    q = bf(np.stack([-8.0 * k[p, [0, 0, 1, 1]] for p in positions]))
    got = run_attention(q, k, v, positions, dtype, None, 1.0, None, 0.0)
    ref = plain_attention_at(q, k, v, positions, None, 1.0, None, 0.0)
    np.testing.assert_allclose(got, ref, atol=1e-5 if dtype == "float32" else 1e-2)
    assert abs(got[0]).max() < 0.05                       # the first token: one key, and the sink takes the rest
    without = run_attention(q, k, v, positions, dtype, None, 1.0, None, None)
    assert without[0].min() > 0.5                         # an ordinary softmax gives the one key everything
    np.testing.assert_allclose(without, plain_attention_at(q, k, v, positions, None, 1.0, None, None),
                               atol=1e-5 if dtype == "float32" else 2e-2)
    # equal scores everywhere: only the bias tells the keys apart, and another sink score moves the share
    q0 = np.zeros((len(positions), H, D), np.float32)
    slopes = np.array([1.0, 0.25, 0.05, 0.0])
    got = run_attention(q0, k, v, positions, dtype, 50, 0.7, slopes, -1.5)
    ref = plain_attention_at(q0, k, v, positions, 50, 0.7, slopes, -1.5)
    np.testing.assert_allclose(got, ref, atol=1e-5 if dtype == "float32" else 2e-2)


@pytest.mark.parametrize("splits", [1, 3])
@pytest.mark.parametrize("H, G, D, window", [(8, 1, 64, None), (4, 2, 32, 300), (2, 2, 96, 77), (3, 1, 128, 1000)])
def test_decode_attention_on_the_matrix_cores_with_bias_and_sink(H, G, D, window, splits):
    """One token per sequence against a long cache, the key range cut into splits or not: the sink joins the sums
    once, wherever they are completed."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(D + splits)
    S = 1100
    bf = lambda a: torch.tensor(np.asarray(a, np.float32)).to(torch.bfloat16).float().numpy()
    k, v = bf(rng.standard_normal((S, G, D))), bf(rng.standard_normal((S, G, D)))
    positions = [0, 1, 31, 32, 63, 64, 500, S - 1]
    q = bf(rng.standard_normal((len(positions), H, D)))
    q[2] = bf(-8.0 * k[31, [h // (H // G) for h in range(H)]])        # scores far below the sink's on a short row
    slopes = P.head_slopes(H)
    kc, vc, table = paged(k, v, 64, "bfloat16")
    T = len(positions)
    out = torch.zeros(T, H * D, dtype=torch.bfloat16, device=DEV)
    part_o = torch.empty(T, H, splits, D, device=DEV) if splits > 1 else None
    part_ml = torch.empty(T, H, splits, 2, device=DEV) if splits > 1 else None
    K.attention_decode(dev(q.reshape(T, H * D), torch.bfloat16), kc, vc, i32(positions), i32([0] * T), table, out, H, G, D,
                       64, window, 0.2, splits, part_o, part_ml, slopes=dev(slopes), sink=0.0)
    ref = plain_attention_at(q, k, v, positions, window, 0.2, slopes, 0.0)
    np.testing.assert_allclose(out.float().cpu().numpy().reshape(T, H, D), ref, atol=2e-2)
    K.attention_decode(dev(q.reshape(T, H * D), torch.bfloat16), kc, vc, i32(positions), i32([0] * T), table, out, H, G, D,
                       64, window, 0.2, splits, part_o, part_ml, slopes=None, sink=-2.0)
    ref = plain_attention_at(q, k, v, positions, window, 0.2, None, -2.0)
    np.testing.assert_allclose(out.float().cpu().numpy().reshape(T, H, D), ref, atol=2e-2)


@pytest.mark.parametrize("wide_from", [1, 10 ** 6])
@pytest.mark.parametrize("H, G, D, window", [(8, 1, 64, 100), (4, 4, 32, None), (2, 1, 96, 70), (2, 2, 128, 130)])
def test_prompt_attention_on_the_matrix_cores_with_bias_and_sink(H, G, D, window, wide_from):
    """Both kernels for prompts (64 and 128 queries a block) over two sequences, one of which goes on from keys it
    holds already; a marked key just inside the window of the last query, one just outside."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(D)
    bf = lambda a: torch.tensor(np.asarray(a, np.float32)).to(torch.bfloat16).float().numpy()
    S0, S1, before1 = 200, 330, 150                 # sequence 1 brings 180 tokens after 150 that it holds
    ks = [bf(0.3 * rng.standard_normal((S, G, D))) for S in (S0, S1)]
    vs = [bf(rng.standard_normal((S, G, D))) for S in (S0, S1)]
    qs = [bf(rng.standard_normal((S0, H, D))), bf(rng.standard_normal((S1 - before1, H, D)))]
    if window:
        for kk, vv, qq, last in ((ks[0], vs[0], qs[0], S0 - 1), (ks[1], vs[1], qs[1], S1 - 1)):
            for col, j in ((0, last - window + 1), (1, last - window)):
                if j >= 0:
                    kk[j] = 0.0
                    kk[j, :, col] = 8.0
                    vv[j] = 0.0
                    vv[j, :, col] = 5.0
            qq[-1, :, :2] = 8.0
    page = 64
    n0, n1 = -(-S0 // page), -(-S1 // page)
    from gpullama3_java_amd.cache.layout import tile_keys, tile_values
    kc = np.zeros((1 + n0 + n1, G, page, D), np.float32)
    vc = np.zeros((1 + n0 + n1, G, D, page), np.float32)
    table = np.zeros((2, max(n0, n1)), np.int32)
    table[0, :n0] = np.arange(1, 1 + n0)
    table[1, :n1] = np.arange(1 + n0, 1 + n0 + n1)[::-1]          # (pages in another order than the positions)
    for b, (kk, vv) in enumerate(zip(ks, vs)):
        for j in range(len(kk)):
            kc[table[b, j // page], :, j % page] = kk[j]
            vc[table[b, j // page], :, :, j % page] = vv[j]
    T = S0 + S1 - before1
    out = torch.zeros(T, H * D, dtype=torch.bfloat16, device=DEV)
    slopes = P.head_slopes(H)
    K.attention_prefill(dev(np.concatenate(qs).reshape(T, H * D), torch.bfloat16), dev(tile_keys(kc), torch.bfloat16),
                        dev(tile_values(vc), torch.bfloat16), i32([0, S0, T]), i32([0, before1]), i32(table), out,
                        max(S0, S1 - before1), H, G, D, page, window, 0.2, wide_from=wide_from, slopes=dev(slopes), sink=0.0)
    ref = np.concatenate([P.sink_attention(qs[0], ks[0], vs[0], 0.2, window, slopes, 0.0, 0),
                          P.sink_attention(qs[1], ks[1], vs[1], 0.2, window, slopes, 0.0, before1)])
    got = out.float().cpu().numpy().reshape(T, H, D)
    np.testing.assert_allclose(got, ref, atol=3e-2)
    if window:
        assert got[-1, H - 1, 0] > 2.0 and abs(got[-1, :, 1]).max() < 1.0      # (the last head: the smallest slope)


# ----------------------------------------------------------------- the delta rule's kernels
def delta_kernels(proj, shape, conv_w, A_log, dt_bias, norm_w, state, cuts, slot, eps, dtype="float32"):
    """The kernels' launches over one sequence cut at ``cuts``; returns the normalised, gated read-outs [T, H Dv]."""
    from gpullama3_java_amd.csrc import lib as K
    H, G, D, Dv, taps = shape
    GD, HV = G * D, H * Dv
    offs = (0, GD, 2 * GD, 2 * GD + 2 * HV, 2 * GD + 2 * HV + H)
    outs, lo = [], 0
    for hi in cuts:
        T = hi - lo
        p = dev(proj[lo:hi])
        act = torch.empty(T, 2 * GD + HV, device=DEV)
        gates = torch.empty(T, 2 * H, device=DEV)
        cu, seq, slots = i32([0, T]), i32([0] * T), i32([slot])
        K.delta_prep(p, offs, dev(conv_w), dev(A_log), dev(dt_bias), state, cu, seq, slots, act, gates, H, G, D, Dv, taps,
                     1e-6, D ** -0.5)
        o = torch.empty(T, HV, device=DEV)
        y = torch.empty(T, HV, dtype=TD[dtype], device=DEV)
        K.delta_recurrence(act, gates, state, cu, slots, o, p, 2 * GD + HV, dev(norm_w), y, H, G, D, Dv, taps, eps)
        outs.append(y.float().cpu().numpy())
        lo = hi
    return np.concatenate(outs)


def plain_delta(proj, shape, conv_w, A_log, dt_bias, norm_w, eps):
    H, G, D, Dv, taps = shape
    GD, HV = G * D, H * Dv
    T = len(proj)
    cols = np.split(proj.astype(np.float64), np.cumsum([GD, GD, HV, HV, H]), axis=1)
    cw = np.split(conv_w.astype(np.float64), [GD, 2 * GD])
    q = P.unit_length(P.short_conv_silu(cols[0], cw[0])[0].reshape(T, G, D)) * D ** -0.5
    k = P.unit_length(P.short_conv_silu(cols[1], cw[1])[0].reshape(T, G, D))
    v = P.short_conv_silu(cols[2], cw[2])[0].reshape(T, H, Dv)
    beta = P.sigmoid(cols[4])
    g = np.exp(-np.exp(A_log) * P.softplus(cols[5] + dt_bias))
    o = np.stack([P.delta_rule(q[:, h // (H // G)], k[:, h // (H // G)], v[:, h], g[:, h], beta[:, h])[0] for h in range(H)], 1)
    return (P.rms_unit(o, eps) * norm_w * P.silu(cols[3].reshape(T, H, Dv))).reshape(T, HV)


@pytest.mark.parametrize("shape", [(4, 2, 32, 48, 3), (1, 1, 40, 20, 1), (6, 3, 16, 32, 5), (2, 2, 100, 17, 2),
                                   (3, 1, 256, 64, 4)])
def test_delta_rule_kernels_whole_and_in_pieces(shape):
    from gpullama3_java_amd.csrc import lib as K
    H, G, D, Dv, taps = shape
    rng = np.random.default_rng(D + Dv)
    T = 90
    N = 2 * G * D + 2 * H * Dv + 2 * H
    proj = rng.standard_normal((T, N)).astype(np.float32)
    conv_w = (0.6 * rng.standard_normal((2 * G * D + H * Dv, taps))).astype(np.float32)
    A_log = rng.uniform(-4, 0.5, H).astype(np.float32)
    dt_bias = rng.uniform(-2, 1, H).astype(np.float32)
    norm_w = (1 + 0.2 * rng.standard_normal(Dv)).astype(np.float32)
    ref = plain_delta(proj, shape, conv_w, A_log, dt_bias, norm_w, 1e-5)
    n = K.delta_state_floats(H, G, D, Dv, taps)
    state = torch.zeros(4, n + 3, device=DEV)                  # (rows longer than needed: the stride is the tensor's)
    state[3] = 7.0                                               # another sequence's state must not be touched
    for slot, cuts in ((0, [T]), (1, [40, 41, 43, 44, 45, 46, 47, 48, T]), (2, list(range(1, T + 1)))):
        got = delta_kernels(proj, shape, conv_w, A_log, dt_bias, norm_w, state, cuts, slot, 1e-5)
        np.testing.assert_allclose(got, ref, atol=3e-5 * np.abs(ref).max(), err_msg=f"cuts {cuts[:3]}")
    assert float((state[3] - 7.0).abs().max()) == 0.0
    # the three ways of cutting leave the same state (the matrices, and the convolution's held inputs)
    np.testing.assert_allclose(state[1, :n].cpu().numpy(), state[0, :n].cpu().numpy(), atol=1e-5)
    np.testing.assert_allclose(state[2, :n].cpu().numpy(), state[0, :n].cpu().numpy(), atol=1e-5)


def test_delta_rule_reads_what_was_written_hundreds_of_tokens_ago():
    """The first token writes under a key that no later token touches, nothing decays; the last token's query is
    that key, and its read-out is the first token's value."""
    H, G, D, Dv, taps = 2, 1, 32, 16, 1
    T = 500
    GD, HV = G * D, H * Dv
    proj = np.zeros((T, 2 * GD + 2 * HV + 2 * H), np.float32)
    rng = np.random.default_rng(1)
    for t in range(T):
        proj[t, GD + (0 if t == 0 else 1 + t % (D - 1))] = 30.0          # the key
        proj[t, 1 + t % (D - 1)] = 30.0                                    # queries that do not read key 0
    proj[T - 1, :GD] = 0.0
    proj[T - 1, 0] = 30.0
    proj[:, 2 * GD:2 * GD + HV] = rng.standard_normal((T, HV)) + 3.0      # values
    proj[:, 2 * GD + HV:2 * GD + 2 * HV] = 2.0                             # gate
    proj[:, 2 * GD + 2 * HV:2 * GD + 2 * HV + H] = 30.0                    # beta = 1
    conv_w = np.ones((2 * GD + HV, 1), np.float32)
    A_log = np.full(H, -30.0, np.float32)                                  # no decay
    norm_w = np.ones(Dv, np.float32)
    ref = plain_delta(proj, (H, G, D, Dv, taps), conv_w, A_log, np.zeros(H, np.float32), norm_w, 1e-5)
    v0 = P.silu(proj[0, 2 * GD:2 * GD + HV].astype(np.float64)).reshape(H, Dv)
    want = (P.rms_unit(v0 * D ** -0.5, 1e-5) * P.silu(2.0)).reshape(HV)
    np.testing.assert_allclose(ref[-1], want, atol=1e-4)                   # the plain implementation agrees with the story
    from gpullama3_java_amd.csrc import lib as K
    state = torch.zeros(2, K.delta_state_floats(H, G, D, Dv, taps), device=DEV)
    for slot, cuts in ((0, [T]), (1, [300] + list(range(301, T + 1)))):
        got = delta_kernels(proj, (H, G, D, Dv, taps), conv_w, A_log, np.zeros(H, np.float32), norm_w, state, cuts, slot, 1e-5)
        np.testing.assert_allclose(got, ref, atol=2e-4)


# ----------------------------------------------------------------- the products' epilogues
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M", [1, 7, 40, 300])
def test_bounded_gate_and_scaled_columns(dtype, M):
    from gpullama3_java_amd.parts import ops
    rng = np.random.default_rng(M)
    d, F = 96, 160
    bf = lambda a: torch.tensor(np.asarray(a, np.float32)).to(TD[dtype]).float().numpy()
    h = bf(rng.standard_normal((M, d)))
    wg, wu, wd = bf(rng.standard_normal((F, d)) * 0.3), bf(rng.standard_normal((F, d)) * 0.3), bf(rng.standard_normal((d, F)) * 0.1)
    ls = (0.5 + rng.random(d)).astype(np.float32)
    x0 = rng.standard_normal((M, d)).astype(np.float32)
    limit = 1.25                                           # with these weights a third of the values are bounded
    g = np.minimum(h.astype(np.float64) @ wg.T, limit)
    u = np.clip(h.astype(np.float64) @ wu.T, -limit, limit)
    assert (np.abs(h @ wu.T) > limit).mean() > 0.1
    y = g * P.sigmoid(1.702 * g) * (u + 1.0)
    act = torch.empty(M, F, dtype=TD[dtype], device=DEV)
    ops.linear(dev(h, TD[dtype]), dev(np.concatenate([wg, wu]), TD[dtype]), act, ops.EPI_GATED, act="quick_gelu",
               act_limit=limit, act_shift=1.0)
    tol = 1e-5 if dtype == "float32" else 1.5e-2
    np.testing.assert_allclose(act.float().cpu().numpy(), y, atol=tol * np.abs(y).max())
    yb = act.float().cpu().numpy().astype(np.float64)
    x = dev(x0)
    ops.linear(act, dev(wd, TD[dtype]), x, ops.EPI_ADD, col_scale=dev(ls))
    ref = x0 + (yb @ wd.T.astype(np.float64)) * ls
    np.testing.assert_allclose(x.cpu().numpy(), ref, atol=tol * np.abs(ref).max())


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_with_a_weight_stored_around_zero(dtype):
    from gpullama3_java_amd.config import NormSpec
    from gpullama3_java_amd.parts import build_part
    from gpullama3_java_amd.engine.context import Workspace
    rng = np.random.default_rng(2)
    part = build_part("norm", NormSpec(dim=72, eps=1e-3, names={"weight": "w"}, weight_offset=1.0), dtype=TD[dtype])
    w = torch.tensor(0.01 * rng.standard_normal(72), dtype=torch.float32).to(torch.bfloat16)   # small: 1 + w must not be rounded to 16 bits
    part.load({"w": w.to(TD[dtype]).to(DEV)})
    x = (0.02 * rng.standard_normal((5, 72))).astype(np.float32)
    ctx = type("Ctx", (), {})()
    ws = Workspace(torch.device(DEV))
    ctx.buffer = ws.get
    out = part(ctx, dev(x)).float().cpu().numpy()
    ref = P.norm_around_zero(x, w.float().numpy(), 1e-3)
    np.testing.assert_allclose(out, ref, atol=(2e-6 if dtype == "float32" else 8e-3) * np.abs(ref).max())
    if dtype == "float32":
        assert np.abs(out - P.rms_unit(x, 1e-3)).max() > 1e-3 * np.abs(ref).max()      # the weight matters


# ----------------------------------------------------------------- whole models through the engine
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompt_and_every_layer(name, dtype):
    eng, cfg, W = engine(name, dtype)
    toks = tokens(name, 1, 210)                       # beyond every window, over four pages
    trace, seen = [], []
    ref = P.Sequence(cfg, W).feed(toks, trace)
    eng.after_block = lambda i, x: seen.append(x.float().cpu().numpy())
    s = eng.take_slot()
    got = eng.step([(s, toks)], want="all").cpu().numpy()
    eng.after_block = None
    assert len(seen) == len(trace) == len(P.run_order(cfg))
    for r, (a, b) in enumerate(zip(seen, trace)):     # the first entry of the run order that differs names the mechanism
        np.testing.assert_allclose(a, b, atol=(3e-5 if dtype == "float32" else 4e-2) * np.abs(b).max(), err_msg=f"run {r}")
    close(got, ref, dtype, name)
    # the first tokens of a sequence, each alone from an empty slot
    for n in (1, 2, 3):
        s2 = eng.take_slot()
        close(eng.step([(s2, toks[:n])], want="all").cpu().numpy(), ref[:n], dtype, f"first {n}")
        eng.give_back_slot(s2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_prompt_then_token_by_token(name, dtype):
    """Decoding passes every window's edge and two page borders; the decoded rows are those of the whole prompt."""
    eng, cfg, W = engine(name, dtype)
    toks = tokens(name, 2, 200)
    ref = P.forward(cfg, W, toks)
    s = eng.take_slot()
    rows = [eng.step([(s, toks[:50])], want="all").cpu().numpy()]
    for t in toks[50:]:
        rows.append(eng.step([(s, [t])]).cpu().numpy())
    close(np.concatenate(rows), ref, dtype, name)
    assert eng.cache.length(s) == 200


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name, cuts", [("looped", [2, 4, 7, 64, 66, 128, 129, 131, 190]),
                                        ("straight", [63, 65, 67, 100, 102, 190]),
                                        ("loop_at_end", [1, 3, 5, 9, 10, 12, 33, 35, 70, 190])])
def test_portions_of_a_prompt(name, cuts, dtype):
    eng, cfg, W = engine(name, dtype)
    toks = tokens(name, 3, 190)
    ref = P.forward(cfg, W, toks)
    s = eng.take_slot()
    rows, lo = [], 0
    for hi in cuts:
        rows.append(eng.step([(s, toks[lo:hi])], want="all").cpu().numpy())
        lo = hi
    close(np.concatenate(rows), ref, dtype, name)
    if dtype == "float32":
        # nothing but rounding hangs on the cut: against the same prompt in one step
        s2 = eng.take_slot()
        whole = eng.step([(s2, toks)], want="all").cpu().numpy()
        assert row_errors(np.concatenate(rows), whole).max() < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["looped", "straight"])
def test_unequal_requests_in_one_batch_and_slots_used_again(name, dtype):
    eng, cfg, W = engine(name, dtype, n_slots=4, max_tokens=1024)
    lens = [1, 70, 131, 9]
    prompts = [tokens(name, 10 + i, n + 12) for i, n in enumerate(lens)]
    refs = [P.forward(cfg, W, p) for p in prompts]
    for round_ in range(2):                           # the second round takes the slots and pages that the first gave back
        slots = [eng.take_slot() for _ in lens]
        order = list(range(4)) if round_ == 0 else [2, 0, 3, 1]
        got = eng.step([(slots[i], prompts[i][:lens[i]]) for i in order], want="all").cpu().numpy()
        lo = 0
        for i in order:
            close(got[lo:lo + lens[i]], refs[i][:lens[i]], dtype, f"{name} prompt {i} round {round_}")
            lo += lens[i]
        live = list(order)
        for step in range(12):
            if step == 5:                             # the shortest request ends earlier
                eng.give_back_slot(slots[live.pop(0)])
            got = eng.step([(slots[i], [prompts[i][lens[i] + step]]) for i in live]).cpu().numpy()
            for r, i in enumerate(live):
                close(got[r:r + 1], refs[i][lens[i] + step:lens[i] + step + 1], dtype, f"{name} request {i} step {step}")
        for i in live:
            eng.give_back_slot(slots[i])
    assert eng.slots_free() == 4


def test_long_decoding_in_32_bit():
    eng, cfg, W = engine("loop_at_end", "float32")
    toks = tokens("loop_at_end", 4, 300)
    ref = P.forward(cfg, W, toks)
    s = eng.take_slot()
    rows = [eng.step([(s, toks[:2])], want="all").cpu().numpy()]
    for t in toks[2:]:
        rows.append(eng.step([(s, [t])]).cpu().numpy())
    close(np.concatenate(rows), ref, "float32")


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_scheduler(dtype):
    eng, cfg, W = engine("looped", dtype)
    prompts = [tokens("looped", 20, 5), tokens("looped", 21, 45), tokens("looped", 22, 1)]
    out = eng.generate(prompts, max_new_tokens=20, temperature=0.0)
    tie = 1e-4 if dtype == "float32" else 0.15
    for p, r in zip(prompts, out):
        assert len(r.tokens) == 20
        seq = list(p)
        for t in r.tokens:
            logits = P.forward(cfg, W, seq)[-1]
            best = int(np.argmax(logits))
            assert t == best or logits[best] - logits[t] < tie * np.abs(logits).max(), (dtype, len(seq), t, best)
            seq.append(t)
    assert eng.slots_free() == eng.n_slots


def test_the_command_line_takes_the_model(tmp_path, capsys):
    from gpullama3_java_amd import cli
    folder, cfg, W = model("straight")
    prompt = tokens("straight", 30, 6)
    rc = cli.main(["--model", folder, "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "12", "--temperature", "0",
                   "--dtype", "float32", "--stream", "false"])
    assert not rc
    words = capsys.readouterr().out.split()
    got = [int(w) for w in words if w.lstrip("-").isdigit()]
    seq = list(prompt)
    for t in got[:3]:
        assert t == int(np.argmax(P.forward(cfg, W, seq)[-1]))
        seq.append(t)
    assert len(got) >= 3


def test_a_folder_may_hold_tensors_that_nothing_reads(tmp_path):
    """The scale of a feed-forward that a layer does not have is tolerated; any other unknown tensor is reported."""
    import json
    import os
    from safetensors.torch import save_file
    from gpullama3_java_amd.engine import Engine
    from gpullama3_java_amd.weights import WeightsError
    folder, cfg, W = model("looped")                    # its layer 2 has no feed-forward
    for extra, ok in (("l2.ls2", True), ("l2.ls3", False)):
        d = tmp_path / extra
        os.makedirs(d)
        tensors = {k: torch.tensor(v).to(torch.bfloat16) for k, v in W.items()}
        tensors[extra] = torch.ones(cfg["width"], dtype=torch.bfloat16)
        save_file(tensors, str(d / "model.safetensors"))
        (d / "config.json").write_text(json.dumps(cfg))
        if ok:
            eng = Engine.from_folder(str(d), dtype="float32", max_tokens=256, n_slots=2)
            toks = tokens("looped", 40, 12)
            close(eng.step([(eng.take_slot(), toks)], want="all").cpu().numpy(), P.forward(cfg, W, toks), "float32")
        else:
            with pytest.raises(WeightsError, match="l2.ls3"):
                Engine.from_folder(str(d), dtype="float32", max_tokens=256, n_slots=2)
