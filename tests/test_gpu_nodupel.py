"""The Nodupel decoder on the GPU against the plain implementation (``plain_nodupel.py``): each mechanism's kernels
alone, with inputs made so that a fault shows, then whole models through the engine's step function, its cache and
state, its batching and its generation loop."""
import numpy as np
import pytest
import torch

import plain_nodupel as P
from nodupel_models import CONFIGS, TOL, close, model, row_errors, tokens

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


def bf16_exact(a):
    return torch.tensor(np.asarray(a), dtype=torch.float32).to(torch.bfloat16).float().numpy()


# ----------------------------------------------------------------- the window that keeps the first keys
def paged(k, v, page, dtype):
    """One sequence's keys [S, G, D] and values [S, G, Dv] as a paged cache in the kernels' order; its pages are
    1, 2, ... Returns (k_cache, v_cache, block table [1, pages])."""
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


def attention_on_gpu(q, k, v, positions, dtype, window, keep, scale, page=64, kernel="generic"):
    from gpullama3_java_amd.csrc import lib as K
    T, H, D = q.shape
    G, Dv = k.shape[1], v.shape[2]
    kc, vc, table = paged(k, v, page, dtype)
    out = torch.zeros(T, H * Dv, dtype=TD[dtype], device=DEV)
    qd = dev(q.reshape(T, H * D), TD[dtype])
    if kernel == "generic":
        K.attention_generic(qd, kc, vc, i32(positions), i32([0] * T), table, out, H, G, D, page, window, scale,
                            v_head_dim=Dv, keep_first=keep)
    elif kernel[0] == "decode":
        n = kernel[1]
        part_o = torch.zeros((T, H, n, D), dtype=torch.float32, device=DEV) if n > 1 else None
        part_ml = torch.zeros((T, H, n, 2), dtype=torch.float32, device=DEV) if n > 1 else None
        K.attention_decode(qd, kc, vc, i32(positions), i32([0] * T), table, out, H, G, D, page, window, scale, n, part_o,
                           part_ml, keep_first=keep)
    else:
        # the tokens of one sequence, the first of them at positions[0]
        K.attention_prefill(qd, kc, vc, i32([0, T]), i32([positions[0]]), table, out, T, H, G, D, page, window, scale,
                            wide_from=kernel[1], keep_first=keep)
    return out.float().cpu().numpy().reshape(T, H, Dv)


def plain_attention_at(q, k, v, positions, window, keep, scale):
    return np.concatenate([P.masked_attention(q[t:t + 1], k[:p + 1], v[:p + 1], scale, window, keep, first=p)
                           for t, p in enumerate(positions)])


def marked_case(H, G, D, Dv, S, marked, rng):
    """Random keys and values whose one key ``marked`` answers every query strongly and carries a value far from
    the others: whether a query sees it decides its output."""
    q, k = bf16_exact(rng.standard_normal((S, H, D)) * 0.3), bf16_exact(rng.standard_normal((S, G, D)) * 0.3)
    v = bf16_exact(rng.standard_normal((S, G, Dv)))
    k[marked] = 0.0
    k[marked, :, 0] = 6.0
    q[:, :, 0] = 6.0
    v[marked] = 30.0
    return q, k, v


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H, G, D, Dv, window, keep", [(4, 2, 32, 48, 37, 5), (3, 3, 16, 16, 64, 1), (2, 1, 48, 32, 20, 70),
                                                      (2, 2, 64, 64, 130, 64)])
def test_kept_first_keys_and_the_window_edges(dtype, H, G, D, Dv, window, keep):
    """A marked key just inside and just outside the kept first keys, and just inside and just outside the window,
    for queries near and far, at page borders (64) and beyond."""
    rng = np.random.default_rng([H, D, window, keep])
    S = 330
    for marked in (keep - 1, keep, 200 - window, 200 - window + 1, 63, 64):
        if marked < 0:
            continue
        q, k, v = marked_case(H, G, D, Dv, S, marked, rng)
        positions = sorted({p for p in (marked, marked + 1, marked + window - 1, marked + window, marked + window + 1, 63,
                                        64, 65, 127, 128, 199, 200, 201, 329) if marked <= p < S} | {0, 1, keep, keep + 1, max(0, marked - 1)})
        ref = plain_attention_at(q[positions], k, v, positions, window, keep, 0.25)
        got = attention_on_gpu(q[positions], k, v, positions, dtype, window, keep, 0.25)
        sees = [P.visible(p, marked, window, keep) for p in positions]
        assert any(sees) and (marked == 0 or not all(sees))
        np.testing.assert_allclose(got, ref, atol=2e-4 if dtype == "float32" else 0.25, err_msg=f"marked {marked}")
        for t, see in enumerate(sees):      # the marked value dominates exactly where the key is visible
            assert (np.abs(got[t]).mean() > 10.0) == see, (marked, positions[t])


MATRIX_CORE_CASES = [(8, 1, 64, 37, 5), (4, 2, 32, 64, 33), (2, 2, 96, 20, 70), (3, 1, 128, 130, 64), (4, 4, 64, 100, 0)]


@pytest.mark.parametrize("splits", [1, 3])
@pytest.mark.parametrize("H, G, D, window, keep", MATRIX_CORE_CASES)
def test_decode_attention_on_the_matrix_cores_keeps_the_first_keys(H, G, D, window, keep, splits):
    rng = np.random.default_rng([H, D, window, keep, splits])
    S = 330
    for marked in (max(keep - 1, 0), keep, 200 - window, 200 - window + 1, 64):
        q, k, v = marked_case(H, G, D, D, S, marked, rng)
        positions = sorted({p for p in (marked, marked + 1, marked + window - 1, marked + window, marked + window + 1, 63,
                                        64, 65, 127, 128, 199, 200, 201, 329) if marked <= p < S} | {0, 1, keep, keep + 1, max(0, marked - 1)})
        ref = plain_attention_at(q[positions], k, v, positions, window, keep, 0.25)
        got = attention_on_gpu(q[positions], k, v, positions, "bfloat16", window, keep, 0.25, kernel=("decode", splits))
        np.testing.assert_allclose(got, ref, atol=0.25, err_msg=f"marked {marked}")
        for t, p in enumerate(positions):
            assert (np.abs(got[t]).mean() > 10.0) == P.visible(p, marked, window, keep), (marked, p)


@pytest.mark.parametrize("wide_from", [1, 10 ** 6])
@pytest.mark.parametrize("H, G, D, window, keep", MATRIX_CORE_CASES)
def test_prompt_attention_on_the_matrix_cores_keeps_the_first_keys(H, G, D, window, keep, wide_from):
    """Both prompt kernels, a prompt from its start and a portion that follows 150 cached tokens."""
    rng = np.random.default_rng([H, D, window, keep, 77])
    S = 330
    for marked in (max(keep - 1, 0), keep, 200 - window, 64):
        for first in (0, 150):
            q, k, v = marked_case(H, G, D, D, S, marked, rng)
            positions = list(range(first, S))
            ref = plain_attention_at(q[positions], k, v, positions, window, keep, 0.25)
            got = attention_on_gpu(q[positions], k, v, positions, "bfloat16", window, keep, 0.25, kernel=("prompt", wide_from))
            np.testing.assert_allclose(got, ref, atol=0.25, err_msg=f"marked {marked}, from {first}")
            for t, p in enumerate(positions):
                assert (np.abs(got[t]).mean() > 10.0) == P.visible(p, marked, window, keep), (marked, first, p)


# ----------------------------------------------------------------- rotations of heads, the gate per head
@pytest.mark.parametrize("dtype", DTYPES)
def test_heads_turned_in_place_and_back_with_a_gate(dtype):
    from gpullama3_java_amd.config.specs import LinearRopeScaling, RotarySpec
    from gpullama3_java_amd.csrc import lib as K
    from gpullama3_java_amd.parts.rotary import Rotary
    rng = np.random.default_rng(5)
    T, H, G, D, Dv, dims = 9, 3, 2, 32, 24, 12
    positions = [0, 1, 2, 63, 64, 65, 500, 1023, 7]
    qk = Rotary(RotarySpec(head_dim=dims, theta=500.0, scaling=LinearRopeScaling(4.0), max_positions=1024), DEV)
    val = Rotary(RotarySpec(head_dim=Dv, theta=500.0, max_positions=1024), DEV)
    ld = H * D + G * D + G * Dv + 16
    rows = bf16_exact(rng.standard_normal((T, ld)))
    buf = dev(rows, TD[dtype])
    K.rotate_heads(buf, i32(positions), [(0, H, D, dims, qk.cos, qk.sin), (H * D, G, D, dims, qk.cos, qk.sin),
                                         ((H + G) * D, G, Dv, Dv, val.cos, val.sin)])
    got = buf.float().cpu().numpy()
    # (32-bit: an angle of a thousand radians is known to 6e-5)
    tol = 5e-5 if dtype == "float32" else 2e-2
    q = P.turn_halves(rows[:, :H * D].reshape(T, H, D), positions, 500.0, dims, 4.0)
    k = P.turn_halves(rows[:, H * D:(H + G) * D].reshape(T, G, D), positions, 500.0, dims, 4.0)
    v = P.turn_halves(rows[:, (H + G) * D:(H + G) * D + G * Dv].reshape(T, G, Dv), positions, 500.0, Dv)
    np.testing.assert_allclose(got[:, :H * D], q.reshape(T, -1), atol=tol * 4)
    np.testing.assert_allclose(got[:, H * D:(H + G) * D], k.reshape(T, -1), atol=tol * 4)
    np.testing.assert_allclose(got[:, (H + G) * D:(H + G) * D + G * Dv], v.reshape(T, -1), atol=tol * 4)
    np.testing.assert_array_equal(got[:, -16:], rows[:, -16:])                       # what lies behind the runs is not touched
    np.testing.assert_array_equal(got[:, dims:D], rows[:, dims:D])                   # nor a head's elements behind the rotated ones
    # back by the same positions, times sigmoid of a gate per head that stands in other rows
    out = bf16_exact(rng.standard_normal((T, G * Dv)))
    gates = bf16_exact(rng.standard_normal((T, 8)) * 2)
    obuf = dev(out, TD[dtype])
    K.rotate_heads(obuf, i32(positions), [(0, G, Dv, Dv, val.cos, val.sin)], back=True, gate=dev(gates, TD[dtype]), gate_col=3)
    ref = P.turn_halves(out.reshape(T, G, Dv), positions, 500.0, Dv, back=True) * P.sigmoid(gates[:, 3:3 + G])[:, :, None]
    np.testing.assert_allclose(obuf.float().cpu().numpy(), ref.reshape(T, -1), atol=tol * 4)


# ----------------------------------------------------------------- the table of token pairs
def test_pair_rows_in_pieces_with_large_multipliers():
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(2)
    for buckets, mp, mc in ((211, 7, 13), (97, 2000000011, 1999999973), (1, 3, 5)):
        seqs = [rng.integers(0, 50000, size=n).tolist() for n in (1, 9, 30)]
        state = torch.full((5, 1), -7, dtype=torch.int32, device=DEV)
        slots = [3, 0, 2]
        done = [0, 0, 0]
        got = [[], [], []]
        for counts in ([1, 4, 10], [0, 1, 1], [0, 4, 19]):
            live = [b for b in range(3) if counts[b]]
            toks = sum((seqs[b][done[b]:done[b] + counts[b]] for b in live), [])
            pos = sum((list(range(done[b], done[b] + counts[b])) for b in live), [])
            seq_of = sum(([i] * counts[b] for i, b in enumerate(live)), [])
            cu = np.cumsum([0] + [counts[b] for b in live])
            rows = torch.zeros(len(toks), dtype=torch.int32, device=DEV)
            K.pair_rows(i32(toks), i32(pos), i32(seq_of), i32(cu), i32([slots[b] for b in live]), state, mp, mc, buckets, rows)
            r = rows.cpu().tolist()
            for i, b in enumerate(live):
                got[b] += r[cu[i]:cu[i + 1]]
                done[b] += counts[b]
        for b in range(3):
            assert got[b] == P.bigram_rows(seqs[b], None, buckets, mp, mc)
        assert state[1, 0].item() == -7 and state[4, 0].item() == -7              # other slots' rows are not touched


# ----------------------------------------------------------------- minGRU
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [40, 256, 700])
def test_mingru_scan_whole_and_in_pieces(W, dtype):
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(W)
    lens = [1, 33, 150]
    T = sum(lens)
    ld = 3 * W + 16
    proj = (rng.standard_normal((T, ld)) * 2).astype(np.float32)
    cu = np.cumsum([0] + lens)
    refs = [P.mingru_scan(P.sigmoid(proj[a:b, :W].astype(np.float64)), proj[a:b, W:2 * W], np.zeros(W))[0]
            * P.silu(proj[a:b, 2 * W:3 * W].astype(np.float64)) for a, b in zip(cu[:-1], cu[1:])]
    tol = 2e-5 if dtype == "float32" else 2e-2
    for cuts in ([1.0], [0.3, 0.31, 1.0]):
        state = torch.zeros((6, W + 8), dtype=torch.float32, device=DEV)
        state[5] = 3.0                                          # another sequence's state
        out = [np.zeros((n, W)) for n in lens]
        lo = [0, 0, 0]
        for c in cuts:
            hi = [max(l, min(n, int(np.ceil(c * n)))) for l, n in zip(lo, lens)]
            live = [b for b in range(3) if hi[b] > lo[b]]
            rows = np.concatenate([proj[cu[b] + lo[b]:cu[b] + hi[b]] for b in live])
            y = torch.zeros((rows.shape[0], W), dtype=TD[dtype], device=DEV)
            longest = max(hi[b] - lo[b] for b in live)
            # (steps whose longest sequence has more than 32 tokens take the scan in three passes over runs of 32)
            runs = torch.zeros(2 * len(live) * -(-longest // 32) * W, dtype=torch.float32, device=DEV)
            K.mingru_scan(dev(rows), W, state, i32(np.cumsum([0] + [hi[b] - lo[b] for b in live])), i32([b + 1 for b in live]), y,
                          longest, runs)
            y = y.float().cpu().numpy()
            at = 0
            for b in live:
                out[b][lo[b]:hi[b]] = y[at:at + hi[b] - lo[b]]
                at += hi[b] - lo[b]
            lo = hi
        for b in range(3):
            np.testing.assert_allclose(out[b], refs[b], atol=tol * max(1.0, np.abs(refs[b]).max()))
        assert (state[5] == 3.0).all() and (state[0] == 0.0).all()


# ----------------------------------------------------------------- the blends with the previous token
@pytest.mark.parametrize("dtype", DTYPES)
def test_blends_read_the_previous_token_across_steps(dtype):
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(9)
    d, n = 72, 5
    mu = rng.uniform(0, 1, (n, d)).astype(np.float32)
    seqs = [bf16_exact(rng.standard_normal((m, d))) for m in (7, 1, 20)]
    state = torch.zeros((4, d + 12), dtype=torch.float32, device=DEV)
    got = [[], [], []]
    done = [0, 0, 0]
    for counts in ([3, 1, 1], [1, 0, 1], [3, 0, 18]):
        live = [b for b in range(3) if counts[b]]
        h = np.concatenate([seqs[b][done[b]:done[b] + counts[b]] for b in live])
        T = h.shape[0]
        out = torch.zeros((n, T, d), dtype=TD[dtype], device=DEV)
        seq_of = sum(([i] * counts[b] for i, b in enumerate(live)), [])
        cu = np.cumsum([0] + [counts[b] for b in live])
        K.shift_mix(dev(h, TD[dtype]), dev(mu), state, i32(cu), i32(seq_of), i32([b for b in live]), out,
                    one_token_each=all(counts[b] == 1 for b in live))
        o = out.float().cpu().numpy()
        for i, b in enumerate(live):
            got[b].append(o[:, cu[i]:cu[i + 1]])
            done[b] += counts[b]
    for b in range(3):
        h = seqs[b]
        ref = np.stack([h + (P.shifted(h, None) - h) * mu[s] for s in range(n)])
        np.testing.assert_allclose(np.concatenate(got[b], 1), ref, atol=1e-6 if dtype == "float32" else 3e-2)


# ----------------------------------------------------------------- the decayed matrix per head
@pytest.mark.parametrize("H, D", [(3, 24), (2, 48), (1, 64), (2, 100), (1, 128), (1, 200), (2, 8), (1, 256)])
def test_decayed_matrix_whole_and_in_pieces(H, D):
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng([H, D])
    lens = [1, 2, 61]
    T = sum(lens)
    r, k, v = (rng.standard_normal((T, H * D)).astype(np.float32) * 0.5 for _ in range(3))
    wl = rng.uniform(-5.0, 0.5, (T, H * D)).astype(np.float32)
    bonus = rng.standard_normal((H, D)).astype(np.float32)
    gate = rng.standard_normal((T, H * D)).astype(np.float32)
    norm_w = rng.standard_normal(H * D).astype(np.float32)
    cu = np.cumsum([0] + lens)
    refs = [P.decayed_outer_scan(*(a[lo:hi].reshape(-1, H, D) for a in (r, k, v)),
                                 np.exp(-np.exp(wl[lo:hi].astype(np.float64))).reshape(-1, H, D), bonus,
                                 np.zeros((H, D, D))) for lo, hi in zip(cu[:-1], cu[1:])]
    off = 20
    for cuts in ([1.0], [0.2, 0.22, 0.5, 1.0]):
        state = torch.zeros((5, off + H * D * D + 4), dtype=torch.float32, device=DEV)
        state[4] = 2.0
        out = [np.zeros((n, H * D)) for n in lens]
        lo = [0, 0, 0]
        for c in cuts:
            hi = [max(l, min(n, int(np.ceil(c * n)))) for l, n in zip(lo, lens)]
            live = [b for b in range(3) if hi[b] > lo[b]]
            pick = lambda a: dev(np.concatenate([a[cu[b] + lo[b]:cu[b] + hi[b]] for b in live]))
            n_rows = sum(hi[b] - lo[b] for b in live)
            o = torch.zeros((n_rows, H * D), dtype=torch.float32, device=DEV)
            # (r, k, v as columns of wider rows, as the stacked product of a short step leaves them; with the read-outs'
            # norm, weight and gate at the end of every round)
            wide = torch.zeros((n_rows, 3 * H * D + 8), dtype=torch.float32, device=DEV)
            for i, a in enumerate((r, k, v)):
                wide[:, i * H * D:(i + 1) * H * D] = pick(a)
            normed = torch.zeros((n_rows, H * D), dtype=torch.float32, device=DEV)
            K.timemix(wide[:, :H * D], wide[:, H * D:2 * H * D], wide[:, 2 * H * D:3 * H * D], pick(wl), dev(bonus), state, off,
                      i32(np.cumsum([0] + [hi[b] - lo[b] for b in live])), i32([b for b in live]), o, H, D,
                      gate=pick(gate), norm_w=dev(norm_w), eps=1e-4, normed=normed)
            o = o.cpu().numpy()
            ref_n = (P.rms_unit(o.reshape(-1, H, D), 1e-4).reshape(-1, H * D) * norm_w
                     * P.silu(np.concatenate([gate[cu[b] + lo[b]:cu[b] + hi[b]] for b in live]).astype(np.float64)))
            np.testing.assert_allclose(normed.cpu().numpy(), ref_n, atol=1e-4 * max(1.0, np.abs(ref_n).max()))
            at = 0
            for b in live:
                out[b][lo[b]:hi[b]] = o[at:at + hi[b] - lo[b]]
                at += hi[b] - lo[b]
            lo = hi
        for b in range(3):
            ref = refs[b][0].reshape(-1, H * D)
            np.testing.assert_allclose(out[b], ref, atol=3e-5 * max(1.0, np.abs(ref).max()))
            np.testing.assert_allclose(state[b, off:off + H * D * D].cpu().numpy(), refs[b][1].reshape(-1),
                                       atol=3e-5 * max(1.0, np.abs(refs[b][1]).max()))
        assert (state[4] == 2.0).all() and (state[:4, :off] == 0.0).all() and (state[3] == 0.0).all()


def test_decayed_matrix_reads_what_was_written_hundreds_of_tokens_ago():
    """One channel hardly decays; what token 3 wrote there is read by a query 500 tokens later and by no other."""
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(11)
    H, D, T = 2, 32, 520
    r = np.zeros((T, H * D), np.float32)
    k = (rng.standard_normal((T, H * D)) * 0.01).astype(np.float32)
    v = rng.standard_normal((T, H * D)).astype(np.float32)
    wl = np.full((T, H * D), 1.0, np.float32)              # exp(-e): everything else is gone after a few tokens
    ch = D + 7                                             # head 1, channel 7
    wl[:, ch] = -12.0
    k[:, ch] = 0.0
    k[3, ch] = 5.0
    v[3, D:] = 9.0
    r[503, ch] = 1.0
    r[100, ch - 1] = 1.0
    bonus = np.zeros((H, D), np.float32)
    state = torch.zeros((2, H * D * D), dtype=torch.float32, device=DEV)
    o = torch.zeros((T, H * D), dtype=torch.float32, device=DEV)
    K.timemix(dev(r), dev(k), dev(v), dev(wl), dev(bonus), state, 0, i32([0, T]), i32([1]), o, H, D)
    o = o.cpu().numpy()
    ref = P.decayed_outer_scan(r.reshape(T, H, D), k.reshape(T, H, D), v.reshape(T, H, D),
                               np.exp(-np.exp(wl.astype(np.float64))).reshape(T, H, D), bonus, np.zeros((H, D, D)))[0]
    # (a decay so close to one is known to 3e-8 in 32-bit: 500 of them in a row to 2e-5)
    np.testing.assert_allclose(o, ref.reshape(T, -1), atol=1e-4, rtol=1e-4)
    assert np.abs(o[503, D:] - 45.0).max() < 0.2 and np.abs(o[100]).max() < 1.0


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_per_head_with_gate_and_the_average_of_two_sides(dtype):
    from gpullama3_java_amd.csrc import lib as K
    rng = np.random.default_rng(3)
    T, H, D, d = 11, 3, 40, 72
    o = rng.standard_normal((T, H * D)).astype(np.float32) * 3
    gate = rng.standard_normal((T, H * D)).astype(np.float32)
    w = rng.standard_normal(H * D).astype(np.float32)
    out = torch.zeros((T, H * D), dtype=TD[dtype], device=DEV)
    K.head_norm_gate(dev(o), dev(w), dev(gate), 1e-3, out, H, D)
    ref = P.rms_unit(o.reshape(T, H, D), 1e-3).reshape(T, -1) * w * P.silu(gate.astype(np.float64))
    np.testing.assert_allclose(out.float().cpu().numpy(), ref, atol=1e-5 if dtype == "float32" else 3e-2)
    x = rng.standard_normal((T, d)).astype(np.float32)
    a, b = rng.standard_normal((T, d)).astype(np.float32) * 5, rng.standard_normal((T, d)).astype(np.float32) * 0.01
    wa, wb = rng.standard_normal(d).astype(np.float32), rng.standard_normal(d).astype(np.float32)
    xd = dev(x)
    K.sides_norm_add(xd, dev(a), dev(b), dev(wa), dev(wb), 1e-6, 0.35)
    ref = x + 0.35 * (P.rms_norm(a, wa, 1e-6) + P.rms_norm(b, wb, 1e-6))
    np.testing.assert_allclose(xd.cpu().numpy(), ref, atol=1e-5)
    # with what a folded norm reads: the completed rows' sums of squares, and the rows times the next norm's weight
    xd, ssq, xg = dev(x), torch.zeros(64, dtype=torch.float32, device=DEV), torch.zeros((T, d), dtype=torch.bfloat16, device=DEV)
    nw = rng.standard_normal(d).astype(np.float32)
    K.sides_norm_add(xd, dev(a), dev(b), dev(wa), dev(wb), 1e-6, 0.35, ssq, dev(nw), xg)
    np.testing.assert_allclose(xd.cpu().numpy(), ref, atol=1e-5)
    np.testing.assert_allclose(ssq[:T].cpu().numpy(), (ref * ref).sum(1), rtol=1e-5)
    np.testing.assert_allclose(xg.float().cpu().numpy(), ref * nw, atol=2e-2 * np.abs(ref * nw).max())


# ----------------------------------------------------------------- whole models through the engine
def plain_trace(cfg, W, toks):
    s = P.Sequence(cfg, W)
    return s.feed(toks), s.layers


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompt_and_every_layer(name, dtype):
    eng, cfg, W = engine(name, dtype)
    toks = tokens(name, 1, 210)                       # beyond every window, over four pages
    ref, trace = plain_trace(cfg, W, toks)
    seen = []
    eng.after_block = lambda i, x: seen.append(x.float().cpu().numpy())
    s = eng.take_slot()
    got = eng.step([(s, toks)], want="all").cpu().numpy()
    eng.after_block = None
    assert len(seen) == len(trace) == len(P.Sequence.run_order(cfg))
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
    """Decoding passes every window's edge, the kept first keys and two page borders; the decoded rows are those of
    the whole prompt."""
    eng, cfg, W = engine(name, dtype)
    toks = tokens(name, 2, 200)
    ref = P.forward(cfg, W, toks)
    s = eng.take_slot()
    rows = [eng.step([(s, toks[:3])], want="all").cpu().numpy()]
    for t in toks[3:]:
        rows.append(eng.step([(s, [t])]).cpu().numpy())
    close(np.concatenate(rows), ref, dtype, name)
    assert eng.cache.length(s) == 200


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name, cuts", [("looped", [2, 4, 7, 64, 66, 128, 129, 131, 190]),
                                        ("straight", [63, 65, 67, 100, 102, 190]),
                                        ("loop_at_end", [1, 3, 5, 9, 10, 12, 33, 35, 70, 72, 190])])
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
@pytest.mark.parametrize("name", ["looped", "loop_at_end", "tiled"])
def test_unequal_requests_in_one_batch_and_slots_used_again(name, dtype):
    eng, cfg, W = engine(name, dtype, n_slots=4, max_tokens=1024)
    lens = [1, 70, 131, 9]
    prompts = [tokens(name, 10 + i, n + 12) for i, n in enumerate(lens)]
    refs = [P.forward(cfg, W, p) for p in prompts]
    for round_ in range(2):                           # the second time takes the slots and pages that the first gave back
        slots = [eng.take_slot() for _ in lens]
        order = list(range(4)) if round_ == 0 else [2, 0, 3, 1]
        got = eng.step([(slots[i], prompts[i][:lens[i]]) for i in order], want="all").cpu().numpy()
        lo = 0
        for i in order:
            close(got[lo:lo + lens[i]], refs[i][:lens[i]], dtype, f"{name} prompt {i} time {round_}")
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


def test_the_command_line_takes_the_model(capsys):
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


def test_the_trace_runner_replays_a_model_of_this_design(tmp_path):
    """bin/trace_run as a user drives it: a request whole, one with its last tokens one by one, two of unequal lengths
    in one batch that end at different times; the model class comes from the folder's config.json."""
    from test_gpu_replay import Replay
    name = "loop_at_end"
    folder, cfg, W = model(name)
    V = cfg["vocab"]
    reqs = {"a": tokens(name, 50, 90), "b": tokens(name, 51, 140), "c": tokens(name, 52, 7)}
    ref = {k: P.forward(cfg, W, t) for k, t in reqs.items()}
    rp = Replay(folder, "float32", tmp_path, max_tokens=400)
    t = reqs["a"]
    close(rp.step([("a", t, list(range(len(t))))], end=["a"]).reshape(-1, V), ref["a"], "float32", "whole")
    t = reqs["b"]
    rows = [rp.step([("b", t[:100], [0, 50, 99])]).reshape(-1, V)]
    for j in range(100, len(t)):
        rows.append(rp.step([("b", [t[j]], [0])], end=["b"] if j == len(t) - 1 else []).reshape(-1, V))
    close(np.concatenate(rows), ref["b"][[0, 50, 99] + list(range(100, len(t)))], "float32", "decoded")
    got = {"a": [], "c": []}
    out = rp.step([("c", reqs["c"][:3], [0, 1, 2]), ("a", reqs["a"][:70], [69])]).reshape(-1, V)
    got["c"].append(out[:3]); got["a"].append(out[3:])
    for j in range(20):
        live = [k for k in ("c", "a") if (3 if k == "c" else 70) + j < len(reqs[k])]
        at = {k: (3 if k == "c" else 70) + j for k in live}
        out = rp.step([(k, [reqs[k][at[k]]], [0]) for k in live], end=[k for k in live if at[k] + 1 == len(reqs[k])]).reshape(-1, V)
        for r, k in enumerate(live):
            got[k].append(out[r:r + 1])
    close(np.concatenate(got["c"]), ref["c"], "float32", "the shorter of a batch")
    close(np.concatenate(got["a"]), ref["a"][69:90], "float32", "the longer of a batch")
    rp.close()


# ----------------------------------------------------------------- seeded random configurations
def random_config(seed):
    """Sizes, counts, order of layers, windows and constants drawn from a seed: what no hand-made configuration
    happened to combine."""
    rng = np.random.default_rng([seed, 99])
    pick = lambda xs: xs[int(rng.integers(len(xs)))]
    width = pick([40, 64, 72, 90, 128, 200])
    n_layers = int(rng.integers(2, 6))
    layers = []
    for i in range(n_layers):
        ff = pick([None, 48, 100, 192, 256])
        mlp = None if ff is None else {"kind": "dense", "ff": ff}
        if rng.random() < 0.35:
            layers.append({"type": "mingru", "mixer": {"width": pick([16, 50, 64, 136, 200])}, "mlp": mlp})
            continue
        heads = pick([1, 2, 3, 4, 6, 8])
        kv = pick([k for k in (1, 2, 3, 4, 6, 8) if heads % k == 0])
        dim, vdim = pick([8, 16, 24, 32, 40, 64, 96, 128]), pick([8, 16, 24, 32, 48, 64, 96, 128])
        dims = pick([d for d in (2, 4, 8, 16, 24, 32, 64, 96, 128) if d <= dim])
        rot = {"base": pick([100.0, 10000.0, 500000.0]), "dims": dims}
        if rng.random() < 0.5:
            rot["scaling"] = {"factor": pick([1.5, 2.0, 8.0])}
        left = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": float(pick([0.1, 0.2, dim ** -0.5])), "rot": rot}
        if rng.random() < 0.8:
            left["mask"] = {"size": pick([1, 2, 7, 31, 32, 64, 65, 100, 150]), "keep_first": pick([0, 1, 3, 16, 64, 65, 80])}
        layers.append({"type": "parallel", "mlp": mlp,
                       "mixer": {"left": left, "right": {"heads": pick([1, 2, 3, 4]), "dim": pick([8, 16, 20, 32, 48, 64, 80])}}})
    if not any(l["type"] == "parallel" for l in layers):
        layers[0], layers[-1] = layers[-1], layers[0]
    cfg = {"architecture": "Nodupel", "vocab": int(rng.integers(50, 700)), "width": width, "norm": {"eps": pick([1e-5, 1e-6])},
           "residual_mult": float(pick([0.25, 0.5, 0.9, 1.0, 1.2])),
           "embedding": {"scale": float(pick([1.0, 3.0, width ** 0.5])),
                         "bigram": {"buckets": int(rng.integers(1, 2000)), "mul_prev": int(rng.integers(1, 10 ** 6)),
                                    "mul_cur": int(rng.integers(1, 10 ** 6))}},
           "layers": layers}
    if rng.random() < 0.7:
        cfg["logit_softcap"] = float(pick([5.0, 30.0, 50.0]))
    if rng.random() < 0.7:
        start = int(rng.integers(0, n_layers))
        cfg["loop"] = {"start": start, "stop": int(rng.integers(start + 1, n_layers + 1)), "times": int(rng.integers(1, 4))}
    return cfg, int(rng.integers(1, 40))


def close_mostly(got, ref, dtype, what):
    """32-bit: every row within the bound. bfloat16: a drawn configuration may run nine layers over a width of 40, where
    single rows gather more rounding than the hand-made models' bound allows for: at most one row in fifty beyond the
    bound, none beyond twice the bound (a fault moves whole runs of rows by many times that)."""
    if dtype == "float32":
        return close(got, ref, dtype, what)
    e = row_errors(got, ref)
    assert (e > 2 * TOL[dtype]).sum() == 0 and (e > TOL[dtype]).sum() <= max(1, len(e) // 50), \
        f"{what}: {int((e > TOL[dtype]).sum())} of {len(e)} rows over {TOL[dtype]}, the worst {e.max():.3e}"


@pytest.mark.parametrize("seed", range(10))
def test_seeded_random_configurations(seed, tmp_path):
    import json
    import os
    from safetensors.torch import save_file
    from gpullama3_java_amd.engine import Engine
    cfg, rank = random_config(seed)
    W = P.make_weights(cfg, seed, rank)
    save_file({k: torch.tensor(v).to(torch.bfloat16).contiguous() for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    rng = np.random.default_rng([seed, 7])
    prompts = [rng.integers(0, cfg["vocab"], size=n).tolist() for n in (172, 1, 40)]
    refs = [P.forward(cfg, W, p) for p in prompts]
    for dtype in DTYPES:
        eng = Engine.from_folder(str(tmp_path), dtype=dtype, max_tokens=1024, n_slots=4)
        # whole; the last 40 tokens one by one; three unequal requests in one batch, then together token by token
        s = eng.take_slot()
        close_mostly(eng.step([(s, prompts[0])], want="all").cpu().numpy(), refs[0], dtype, f"seed {seed} whole")
        eng.give_back_slot(s)
        s = eng.take_slot()
        rows = [eng.step([(s, prompts[0][:132])], want="all").cpu().numpy()]
        for t in prompts[0][132:]:
            rows.append(eng.step([(s, [t])]).cpu().numpy())
        close_mostly(np.concatenate(rows), refs[0], dtype, f"seed {seed} decoded")
        eng.give_back_slot(s)
        slots = [eng.take_slot() for _ in prompts]
        cut = [150, 1, 20]
        got = eng.step([(slots[i], prompts[i][:cut[i]]) for i in range(3)], want="all").cpu().numpy()
        lo = 0
        for i in range(3):
            close_mostly(got[lo:lo + cut[i]], refs[i][:cut[i]], dtype, f"seed {seed} batch prompt {i}")
            lo += cut[i]
        for step in range(20):
            live = [i for i in range(3) if cut[i] + step < len(prompts[i])]
            got = eng.step([(slots[i], [prompts[i][cut[i] + step]]) for i in live]).cpu().numpy()
            for r, i in enumerate(live):
                close_mostly(got[r:r + 1], refs[i][cut[i] + step:cut[i] + step + 1], dtype, f"seed {seed} batch step {step} request {i}")
        del eng
