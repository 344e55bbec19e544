"""The mechanisms of the Lokedra design one at a time, each op of the
package against the plain functions of tests/lokedra_oracle.py or a closed
form: token shift with its slot state, the per-channel scaled residual
step, the generalized delta rule and HGRN2 (portions, stale slots, batches
with a padding chunk, every row tiling of the kernel, slow decays that keep
a far token), the interleaved rotation with interpolated frequencies, the
chunked mask with a unit sink (edges made visible by one dominant score, in
prompts and decoding, at page borders), the convolved attention mixer with
keys as values, routing with a choice correction, and clamped experts. CPU
runs check the reference ops; `-m gpu` runs the HIP kernels in f32 and
bf16."""
import math
import os
import sys
from types import SimpleNamespace

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import lokedra_oracle as L  # noqa: E402

from kaito_amd import ops  # noqa: E402

MODES = [("cpu", torch.float32),
         pytest.param(("cuda", torch.float32), marks=pytest.mark.gpu),
         pytest.param(("cuda", torch.bfloat16), marks=pytest.mark.gpu)]
BS = 16      # page size used here


def i32(x, dev):
    return torch.tensor(x, dtype=torch.int32, device=dev)


def close(got, want, dtype, scale=None, f32=1e-5, bf16=2e-2):
    want = torch.as_tensor(np.asarray(want), dtype=torch.float64)
    scale = scale if scale is not None else want.abs().max().item() + 1e-9
    err = (got.double().cpu() - want).abs().max().item() / scale
    assert err < (f32 if dtype == torch.float32 else bf16), err


def act(a, mode):
    """Values as the activation dtype holds them: (device tensor, float64
    copy of what it holds)."""
    dev, dt = mode
    t = torch.tensor(np.asarray(a), dtype=torch.float32).to(dt).to(dev)
    return t, t.double().cpu().numpy()


def layout(chunks, dev):
    """chunks: [(rows, slot, start)] -> cu, slots, starts, token_seq."""
    cu, seq = [0], []
    for i, (n, _, _) in enumerate(chunks):
        cu.append(cu[-1] + n)
        seq += [i] * n
    return (i32(cu, dev), i32([c[1] for c in chunks], dev),
            i32([c[2] for c in chunks], dev), i32(seq, dev))


# ---- token shift ----------------------------------------------------------------

@pytest.mark.parametrize("mode", MODES)
def test_token_shift_portions_batches_and_stale_slots(mode):
    dev, dt = mode
    rng = np.random.default_rng(0)
    width = 40
    mu = rng.uniform(0, 1, width)
    mu_t = torch.tensor(mu, dtype=torch.float32, device=dev)
    ha, a = act(rng.normal(0, 1, (9, width)), mode)
    hb, b = act(rng.normal(0, 1, (4, width)), mode)
    want_a, want_b = L.token_shift(a, mu), L.token_shift(b, mu)
    # slots hold rows of earlier sequences
    state = torch.full((3, width), 7.0, dtype=dt, device=dev)

    def step(parts):
        h = torch.cat([p[0] for p in parts], 0)
        cu, sl, st, seq = layout([(p[0].size(0), p[1], p[2]) for p in parts],
                                 dev)
        return ops.token_shift(h.contiguous(), mu_t, state, cu, sl, st, seq)
    pad = torch.ones(1, width, dtype=dt, device=dev)
    x1 = step([(ha[:3], 2, 0), (pad, -1, 0), (hb[:1], 0, 0)])
    x2 = step([(hb[1:4], 0, 1), (ha[3:4], 2, 3)])
    x3 = step([(ha[4:9], 2, 4)])
    close(torch.cat([x1[:3], x2[3:4], x3]), want_a, dt)
    close(torch.cat([x1[4:5], x2[:3]]), want_b, dt)
    assert torch.equal(state[2], ha[8]) and torch.equal(state[0], hb[3])
    assert state[1].eq(7.0).all()
    # a new sequence in a used slot starts from zeros, not from the slot
    x4 = step([(hb, 2, 0)])
    close(x4, want_b, dt)


# ---- residual step ---------------------------------------------------------------

@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("terms", [1, 2, 3])
def test_scaled_residual_step(mode, terms):
    dev, dt = mode
    rng = np.random.default_rng(terms)
    T, width, eps = 6, 72, 1e-5
    x = rng.normal(0, 2, (T, width))
    x0 = rng.normal(0, 2, (T, width))
    w = rng.uniform(0.5, 1.5, width)
    ys = [act(rng.normal(0, 1, (T, width)), mode) for _ in range(terms)]
    vs = [rng.uniform(0.2, 1.2, width) for _ in range(terms)]
    f32 = dict(dtype=torch.float32, device=dev)
    for with_x0 in (False, True):
        x32 = torch.tensor(x, **f32)
        want = np.float32(x).astype(np.float64) + sum(
            y[1] * np.float32(v) for y, v in zip(ys, vs))
        if with_x0:
            want = want + np.float32(x0)
        h = ops.scaled_residual_add_norm(
            x32, [(y[0], torch.tensor(v, **f32)) for y, v in zip(ys, vs)],
            torch.tensor(w, **f32), eps, dt,
            x_add=torch.tensor(x0, **f32) if with_x0 else None)
        close(x32, want, torch.float32, f32=1e-6)
        close(h, L.rms(want, eps) * np.float32(w), dt)
    # the last layer: no norm follows
    x32 = torch.tensor(x, **f32)
    assert ops.scaled_residual_add_norm(
        x32, [(ys[0][0], torch.tensor(vs[0], **f32))], None, eps, dt) is None
    close(x32, np.float32(x).astype(np.float64)
          + ys[0][1] * np.float32(vs[0]), torch.float32, f32=1e-6)


# ---- generalized delta rule --------------------------------------------------------

def delta_inputs(rng, T, H, D, mode, slow=False):
    n = H * D
    r, rf = act(rng.normal(0, 1, (T, n)), mode)
    k, kf = act(rng.normal(0, 1, (T, n)), mode)
    v, vf = act(rng.normal(0, 1, (T, n)), mode)
    g, gf = act(rng.normal(0, 1, (T, n)), mode)
    w_pre = np.float32(rng.normal(-8.0 if slow else -1.0, 1.0, (T, n)))
    a_pre = np.float32(rng.normal(-6.0 if slow else 0.0, 1.0, (T, n)))
    return (r, k, v, g), (rf, kf, vf, gf), w_pre, a_pre


def delta_oracle(parts, w_pre, a_pre, norm_w, H, D, eps, rate=math.exp(-0.5),
                 k_eps=1e-6):
    """The recurrence written out from its definition (float64)."""
    rf, kf, vf, gf = (p.reshape(-1, H, D) for p in parts)
    T = rf.shape[0]
    w = np.exp(-rate * L.sigmoid(w_pre.astype(np.float64))).reshape(T, H, D)
    a = L.sigmoid(a_pre.astype(np.float64)).reshape(T, H, D)
    out = np.zeros((T, H, D))
    for h in range(H):
        S = np.zeros((D, D))
        for t in range(T):
            u = kf[t, h] / math.sqrt(kf[t, h] @ kf[t, h] + k_eps)
            S = w[t, h][:, None] * S - np.outer(a[t, h] * u, u @ S) \
                + np.outer(kf[t, h], vf[t, h])
            out[t, h] = S.T @ rf[t, h]
    out = L.rms(out, eps).reshape(T, H * D) * norm_w
    return out * L.sigmoid(gf.reshape(T, H * D))


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("rows_per_lane", ["16", "32"])
@pytest.mark.parametrize("sizes", [(3, 8), (2, 48), (1, 100), (1, 200)])
def test_delta_rule_portions_and_batches(mode, sizes, rows_per_lane,
                                         monkeypatch):
    """Head sizes for every row tiling of the kernel (32, 64, 128 and 256
    padded rows, at 16 and at 32 state rows per lane: the kernel picks by
    the step's shape, the test pins it); two sequences cut differently in
    shared steps, a padding chunk, slots that hold another sequence's
    state."""
    monkeypatch.setenv("KAITO_DIAG_ROWS_PER_LANE", rows_per_lane)
    dev, dt = mode
    if dev == "cpu" and rows_per_lane == "32":
        pytest.skip("the reference op has no tiling")
    H, D = sizes
    rng = np.random.default_rng(D)
    eps = 1e-5
    Ta, Tb = 21, 11
    norm_w = rng.uniform(0.5, 1.5, H * D)
    nw = torch.tensor(norm_w, dtype=torch.float32, device=dev)
    A = delta_inputs(rng, Ta, H, D, mode)
    B = delta_inputs(rng, Tb, H, D, mode)
    want_a = delta_oracle(A[1], A[2], A[3], np.float32(norm_w), H, D, eps)
    want_b = delta_oracle(B[1], B[2], B[3], np.float32(norm_w), H, D, eps)
    state = torch.full((3, H, D, D), 3.0, dtype=torch.float32, device=dev)

    def step(parts):
        """parts: (inputs, lo, hi, slot) or None for a padding chunk."""
        cols, wp, ap, chunks = [[], [], [], []], [], [], []
        for p in parts:
            if p is None:
                for c in cols:
                    c.append(torch.ones(2, H * D, dtype=dt, device=dev))
                wp.append(np.zeros((2, H * D), np.float32))
                ap.append(np.zeros((2, H * D), np.float32))
                chunks.append((2, -1, 0))
                continue
            X, lo, hi, slot = p
            for c, t in zip(cols, X[0]):
                c.append(t[lo:hi])
            wp.append(X[2][lo:hi])
            ap.append(X[3][lo:hi])
            chunks.append((hi - lo, slot, lo))
        cu, sl, st, _ = layout(chunks, dev)
        # r, k, v, gate are column ranges of one projection output
        packed = torch.cat([torch.cat(c, 0) for c in cols], 1)
        n = H * D
        views = [packed[:, i * n:(i + 1) * n].unflatten(-1, (H, D))
                 for i in range(4)]
        return ops.diag_delta_rule(
            views[0], views[1], views[2],
            torch.tensor(np.concatenate(wp), device=dev),
            torch.tensor(np.concatenate(ap), device=dev), views[3], nw,
            state, cu, sl, st, math.exp(-0.5), 1e-6, eps)
    y1 = step([(A, 0, 9, 2), None, (B, 0, 1, 0)])
    y2 = step([(B, 1, 3, 0), (A, 9, 10, 2)])
    y3 = step([(A, 10, 21, 2), (B, 3, 11, 0)])
    got_a = torch.cat([y1[:9], y2[2:3], y3[:11]])
    got_b = torch.cat([y1[11:12], y2[:2], y3[11:]])
    close(got_a, want_a, dt, f32=5e-5, bf16=3e-2)
    close(got_b, want_b, dt, f32=5e-5, bf16=3e-2)
    assert state[1].eq(3.0).all()             # nobody's slot


@pytest.mark.parametrize("mode", MODES)
def test_delta_rule_keeps_a_far_token(mode):
    """Decays near one and removal rates near zero: the first token's
    write is still read 300 tokens later, through portions and single
    tokens; changing that token changes the last output."""
    dev, dt = mode
    H, D, T, eps = 2, 16, 300, 1e-5
    rng = np.random.default_rng(5)
    X = delta_inputs(rng, T, H, D, mode, slow=True)
    norm_w = np.ones(H * D, np.float32)
    nw = torch.tensor(norm_w, device=dev)

    def run(inputs):
        state = torch.zeros(1, H, D, D, dtype=torch.float32, device=dev)
        out, at = [], 0
        for n in [1, 120, 2, 150] + [1] * 27:
            cu, sl, st, _ = layout([(n, 0, at)], dev)
            hd = (H, D)
            out.append(ops.diag_delta_rule(
                *(t[at:at + n].unflatten(-1, hd) for t in inputs[0][:3]),
                torch.tensor(inputs[2][at:at + n], device=dev),
                torch.tensor(inputs[3][at:at + n], device=dev),
                inputs[0][3][at:at + n].unflatten(-1, hd), nw, state, cu, sl,
                st, math.exp(-0.5), 1e-6, eps))
            at += n
        return torch.cat(out)
    want = delta_oracle(X[1], X[2], X[3], norm_w, H, D, eps)
    close(run(X), want, dt, f32=1e-4, bf16=4e-2)
    v2 = X[0][2].clone()
    v2[0] = -3.0 * v2[0]
    other = ((X[0][0], X[0][1], v2, X[0][3]),
             (X[1][0], X[1][1], v2.double().cpu().numpy(), X[1][3]),
             X[2], X[3])
    want2 = delta_oracle(other[1], X[2], X[3], norm_w, H, D, eps)
    assert np.abs(want2[-1] - want[-1]).max() > 0.05
    close(run(other)[-5:], want2[-5:], dt, f32=1e-4, bf16=4e-2)


# ---- HGRN2 ---------------------------------------------------------------------

@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("rows_per_lane", ["16", "32"])
@pytest.mark.parametrize("sizes", [(3, 8, 20), (2, 32, 64), (1, 72, 9),
                                   (1, 130, 70)])
def test_hgrn2_portions_and_batches(mode, sizes, rows_per_lane, monkeypatch):
    monkeypatch.setenv("KAITO_DIAG_ROWS_PER_LANE", rows_per_lane)
    dev, dt = mode
    if dev == "cpu" and rows_per_lane == "32":
        pytest.skip("the reference op has no tiling")
    H, D, V = sizes
    rng = np.random.default_rng(V)
    eps, width = 1e-5, 24
    T = 19
    W = {"q": L._bf16_round(rng.normal(0, 0.3, (H * D, width))),
         "v": L._bf16_round(rng.normal(0, 0.3, (H * V, width))),
         "f": L._bf16_round(rng.normal(0, 0.5, (H * D, width))),
         "f.b": L._bf16_round(rng.normal(2, 2, H * D)),
         "lower": L._bf16_round(rng.uniform(0, 0.95, H * D)),
         "norm": L._bf16_round(rng.uniform(0.5, 1.5, V)),
         "o": np.eye(H * V)}
    hx, hf = act(rng.normal(0, 1, (T, width)), mode)
    want = L.hgrn2(hf, W, "", {"heads": H, "dim": D, "vdim": V}, eps)
    q, qf = act(hf @ W["q"].T, mode)
    v, vf = act(hf @ W["v"].T, mode)
    if dt == torch.bfloat16:      # the oracle sees the rounded projections
        f = W["lower"] + (1 - W["lower"]) * L.sigmoid(hf @ W["f"].T
                                                      + W["f.b"])
        want = np.zeros((T, H, V))
        qs = L.silu(qf).reshape(T, H, D)
        for h in range(H):
            S = np.zeros((D, V))
            for t in range(T):
                ft = f[t].reshape(H, D)[h]
                S = ft[:, None] * S + np.outer(1 - ft,
                                               vf[t].reshape(H, V)[h])
                want[t, h] = S.T @ qs[t, h]
        want = (L.rms(want, eps) * W["norm"]).reshape(T, H * V)
    f_pre = torch.tensor(np.float32(hf @ W["f"].T + W["f.b"]), device=dev)
    lower = torch.tensor(np.float32(W["lower"]), device=dev)
    nw = torch.tensor(np.float32(W["norm"]), device=dev)
    state = torch.full((2, H, D, V), -2.0, dtype=torch.float32, device=dev)
    packed = torch.cat([q, v], 1)
    out, at = [], 0
    for n in (1, 6, 2, 10):
        cu, sl, st, _ = layout([(n, 1, at), (1, -1, 0)], dev)
        rows = torch.cat([packed[at:at + n], packed[:1]], 0)
        fp = torch.cat([f_pre[at:at + n], f_pre[:1]], 0)
        y = ops.hgrn2_scan(rows[:, :H * D].unflatten(-1, (H, D)),
                           rows[:, H * D:].unflatten(-1, (H, V)), fp, lower,
                           nw, state, cu, sl, st, eps)
        out.append(y[:n])
        at += n
    close(torch.cat(out), want, dt, f32=5e-5, bf16=3e-2)
    assert state[0].eq(-2.0).all()


# ---- rotation ---------------------------------------------------------------------

@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("scaling", [None, {"factor": 4.0, "original": 64,
                                            "fast": 8.0, "slow": 1.0}])
def test_interleaved_rotation_and_latent_cache_write(mode, scaling):
    from kaito_amd.models.hybrid_config import _rotary_spec
    dev, dt = mode
    rng = np.random.default_rng(2)
    H, D, R2, rank, T, eps = 3, 6, 8, 10, 7, 1e-5
    rot = {"base": 40.0, "dims": R2}
    if scaling:
        rot["scaling"] = scaling
    pos = [0, 1, 2, 40, 41, 500, 7]
    cos, sin = L.rotary_tables(rot, pos)
    if scaling:
        # the interpolation changes some frequencies and the magnitude
        plain = L.rotary_tables({"base": 40.0, "dims": R2}, pos)[0]
        assert np.abs(plain - cos).max() > 0.05
    freq, mag = _rotary_spec(rot).frequencies()
    inv = torch.tensor(freq, dtype=torch.float64).float().to(dev)
    q, qf = act(rng.normal(0, 1, (T, H, D + R2)), mode)
    dkv, df = act(rng.normal(0, 1, (T, rank + R2)), mode)
    nw = rng.uniform(0.5, 1.5, rank)
    q_want = qf.copy()
    q_want[..., D:] = L.rotate_pairs(qf[..., D:], cos, sin, R2)
    row_want = np.concatenate(
        [L.rms(df[:, :rank], eps) * np.float32(nw),
         L.rotate_pairs(df[:, rank:], cos, sin, R2)], 1)
    cache = torch.zeros(40, BS, rank + R2, dtype=dt, device=dev)
    slots = torch.tensor([5, 16, 17, 31, 32, 639, -1], dtype=torch.long,
                         device=dev)
    got = ops.latent_rope_cache_write(
        q, dkv, torch.tensor(nw, dtype=torch.float32, device=dev), eps, cache,
        slots, torch.tensor(pos, dtype=torch.long, device=dev), inv, D,
        interleaved=True, rot_mag=mag)
    close(got, q_want, dt)
    flat = cache.view(-1, rank + R2)
    close(flat[slots[:6]], row_want[:6], dt)


# ---- chunked mask, unit sink -------------------------------------------------------

def paged(keys, vals, mode, extra_pages=3, perm_seed=0):
    """Scatter [n, G, D] rows into shuffled pages; returns caches + table."""
    dev, dt = mode
    n, G, D = keys.shape
    pages = -(-n // BS)
    order = np.random.default_rng(perm_seed).permutation(pages + extra_pages)
    kc = torch.zeros(pages + extra_pages, G, BS, D, dtype=dt, device=dev)
    vc = torch.zeros(pages + extra_pages, G, BS, vals.shape[2], dtype=dt,
                     device=dev)
    for j in range(n):
        p = int(order[j // BS])
        kc[p, :, j % BS] = torch.tensor(keys[j], dtype=dt)
        vc[p, :, j % BS] = torch.tensor(vals[j], dtype=dt)
    return kc, vc, i32([list(order[:pages])], dev)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("chunk", [1, 7, 16, 24, 64])
def test_chunked_mask_against_closed_form(mode, chunk):
    """Random rows of one sequence (prompt rows and single rows), keys as
    values, unit sink: p_j = e^{s_j} / (1 + sum)."""
    dev, dt = mode
    rng = np.random.default_rng(chunk)
    H, G, D, n = 4, 2, 16, 75
    k = L._bf16_round(rng.normal(0, 1, (n, G, D)))
    q = L._bf16_round(rng.normal(0, 1, (n, H, D)))
    kc, _, table = paged(k, k, mode)
    rows = [0, 1, chunk - 1, chunk, min(chunk + 1, n - 1), 31, 32, 47, 48,
            63, 64, n - 1]
    rows = sorted(set(r for r in rows if 0 <= r < n))
    want = np.zeros((len(rows), H, D))
    for a, i in enumerate(rows):
        lo = i // chunk * chunk
        for h in range(H):
            e = np.exp(k[lo:i + 1, h // 2] @ q[i, h] * 0.3)
            want[a, h] = (e / (1 + e.sum())) @ k[lo:i + 1, h // 2]
    got = ops.window_attention(
        torch.tensor(q[rows], dtype=dt, device=dev), kc, kc, table,
        i32([0] * len(rows), dev),
        torch.tensor(rows, dtype=torch.long, device=dev), 0.3,
        sinks=torch.zeros(H, dtype=torch.float32, device=dev), chunk=chunk)
    close(got, want, dt)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("kernel", ["rows", "tiles"])
def test_chunk_edges_show_in_the_output(mode, kernel):
    """One key per chunk edge is made to dominate every query's scores (a
    large key along a direction all queries share). A query whose chunk
    holds that key returns it; the query one position before the edge's
    chunk, or one chunk later, must not see it at all. Edges at, before
    and after page borders; prompt tiles (bf16 on the GPU: the matrix-core
    kernel with head size 64) and single rows."""
    dev, dt = mode
    if kernel == "tiles" and (dev == "cpu" or dt != torch.bfloat16):
        pytest.skip("the tiled prompt kernel is the GPU's, in bf16")
    H = G = 1
    D, n = 64, 200
    for chunk in (16, 17, 31, 48, 96):
        rng = np.random.default_rng(chunk)
        k = L._bf16_round(rng.normal(0, 0.1, (n, G, D)))
        q = L._bf16_round(rng.normal(0, 0.1, (n, H, D)))
        q[:, :, 0] = 4.0
        marks = list(range(0, n, chunk))           # first key of each chunk
        for m in marks:
            k[m, 0, 0] = 8.0                       # score 32 against noise
        kc, _, table = paged(k, k, mode, perm_seed=chunk)
        qt = torch.tensor(q, dtype=dt, device=dev)
        pos = torch.arange(n, dtype=torch.long, device=dev)
        sinks = torch.zeros(H, dtype=torch.float32, device=dev)
        tiles = None
        if kernel == "tiles":
            ts, tb = ops.build_query_tiles([n], dev)
            tiles = (ts, tb, i32([0, n], dev), i32([0], dev))
        got = ops.window_attention(qt, kc, kc, table, i32([0] * n, dev), pos,
                                   1.0, sinks=sinks, chunk=chunk,
                                   tiles=tiles).double().cpu()
        for i in range(n):
            # every query's own chunk starts with a marked key, so it
            # returns that key, never the one of a neighbouring chunk
            m = i // chunk * chunk
            assert abs(got[i, 0, 0].item() - 8.0) < 0.2, (chunk, i)
            assert (got[i, 0] - torch.tensor(k[m, 0])).abs().max() < 0.1
        # take a chunk's first key away: its queries fall back to their
        # own noise keys and the sink, and nobody else notices
        m = marks[2]
        k2 = k.copy()
        k2[m, 0, 0] = 0.0
        kc2, _, _ = paged(k2, k2, mode, perm_seed=chunk)
        got2 = ops.window_attention(qt, kc2, kc2, table, i32([0] * n, dev),
                                    pos, 1.0, sinks=sinks, chunk=chunk,
                                    tiles=tiles).double().cpu()
        inside = range(m, min(m + chunk, n))
        for i in range(n):
            if i in inside:
                assert got2[i, 0, 0].abs().item() < 1.0, (chunk, i)
            else:
                assert torch.equal(got2[i], got[i]), (chunk, i)


@pytest.mark.gpu
def test_tiled_chunk_kernel_matches_rows_kernel():
    """bf16: the matrix-core prompt kernel against the one-row kernel, two
    sequences of unequal length, portions that start inside a chunk."""
    dev, dt = "cuda", torch.bfloat16
    rng = np.random.default_rng(9)
    H, G, D = 4, 2, 64
    lens, starts = [150, 70], [37, 0]
    for chunk in (20, 64, 100):
        qs, tables, kcs = [], [], []
        total = [s + n for s, n in zip(starts, lens)]
        k = [L._bf16_round(rng.normal(0, 0.5, (t, G, D))) for t in total]
        allk = np.concatenate(k, 0)
        # one pool: sequence 1's pages follow sequence 0's
        pages0 = -(-total[0] // BS)
        kc = torch.zeros(pages0 + -(-total[1] // BS), G, BS, D, dtype=dt,
                         device=dev)
        for s, ks in enumerate(k):
            base = 0 if s == 0 else pages0
            for j in range(ks.shape[0]):
                kc[base + j // BS, :, j % BS] = torch.tensor(ks[j], dtype=dt)
        mb = max(pages0, -(-total[1] // BS))
        table = torch.zeros(2, mb, dtype=torch.int32, device=dev)
        table[0, :pages0] = torch.arange(pages0)
        table[1, :-(-total[1] // BS)] = torch.arange(
            pages0, pages0 + -(-total[1] // BS))
        q = torch.tensor(L._bf16_round(rng.normal(0, 0.5, (sum(lens), H, D))),
                         dtype=dt, device=dev)
        pos = torch.tensor([starts[0] + i for i in range(lens[0])]
                           + [starts[1] + i for i in range(lens[1])],
                           dtype=torch.long, device=dev)
        seq = i32([0] * lens[0] + [1] * lens[1], dev)
        sinks = torch.zeros(H, dtype=torch.float32, device=dev)
        ts, tb = ops.build_query_tiles(lens, dev)
        tiles = (ts, tb, i32([0, lens[0], sum(lens)], dev), i32(starts, dev))
        a = ops.window_attention(q, kc, kc, table, seq, pos, 0.2, sinks=sinks,
                                 chunk=chunk)
        b = ops.window_attention(q, kc, kc, table, seq, pos, 0.2, sinks=sinks,
                                 chunk=chunk, tiles=tiles)
        assert (a.float() - b.float()).abs().max().item() < 2e-2
        del allk


# ---- the convolved attention mixer with keys as values -----------------------------

@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("taps", [1, 4])
def test_chunk_attention_mixer_in_portions(mode, taps):
    from kaito_amd.models.hybrid_config import RotaryAttnSpec
    from kaito_amd.models.mixers import RotaryWindowAttention
    dev, dt = mode
    rng = np.random.default_rng(taps)
    width, H, G, D, chunk, T = 32, 4, 2, 8, 10, 37
    mx = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "conv": taps,
          "mask": {"size": chunk}, "scale": 0.4}
    cfg = L.make_config([{"type": "parallel", "mixer": {
        "left": mx, "right": {"heads": 1, "dim": 4, "vdim": 4},
        "left_scale": 1.0, "right_scale": 1.0}, "mlp": None}], width, 8)
    W = L.random_weights(cfg, seed=taps)
    pre = "l0.mix.left."
    hx, hf = act(rng.normal(0, 1, (T, width)), mode)
    want = L.chunk_attention(hf, W, pre, mx)
    spec = RotaryAttnSpec(heads=H, kv_heads=G, dim=D, vdim=D, scale=0.4,
                          conv_taps=taps, chunk=chunk, qk_norm=False,
                          bias=True, tied_values=True, unit_sink=True)
    m = RotaryWindowAttention(width, spec, dt, 1e-5).to(dev)

    def put(p, a):
        p.data.copy_(torch.tensor(np.asarray(a)).to(p.dtype))
    put(m.qkv_proj, np.concatenate([W[pre + "q"], W[pre + "k"]], 0))
    put(m.qkv_bias, np.concatenate([W[pre + "q.b"], W[pre + "k.b"]], 0))
    put(m.conv_weight, np.concatenate([W[pre + "q.conv"],
                                       W[pre + "k.conv"]], 0))
    put(m.o_proj, W[pre + "o"])
    put(m.o_bias, W[pre + "o.b"])
    cache = m.alloc_cache(8, BS, 2, dev)
    assert set(cache) == {"k", "conv"}          # one tensor for keys = values
    table = i32([[5, 2, 7]], dev)
    out, at = [], 0
    for n in (3, 1, 2, 14, 1, 16):
        pos = torch.arange(at, at + n, dtype=torch.long, device=dev)
        cu, sl, st, seq = layout([(n, 1, at)], dev)
        slots = torch.tensor([int(table[0, p // BS]) * BS + p % BS
                              for p in range(at, at + n)], dtype=torch.long,
                             device=dev)
        meta = SimpleNamespace(cu_seqlens=cu, state_slots=sl, seq_starts=st,
                               token_seq=seq, slot_mapping=slots,
                               block_tables=table, tile_seq=None,
                               tile_qbase=None, layer_shared={})
        out.append(m(hx[at:at + n], pos, cache, meta))
        at += n
    close(torch.cat(out), want, dt, f32=2e-5, bf16=4e-2)


# ---- feed-forward ---------------------------------------------------------------------

def test_routing_choice_uses_the_correction_and_weights_do_not():
    z = np.array([2.0, 1.9, 0.5, -1.0])
    s = L.softmax(z)
    # without a correction: experts 0 and 1
    assert [e for e, _ in L.route(z, np.zeros(4), 2)] == [0, 1]
    # the correction lifts expert 3 over everyone; its weight stays its
    # small score, and nothing is renormalised
    got = L.route(z, np.array([0.0, 0.0, 0.0, 1.0]), 2)
    assert [e for e, _ in got] == [3, 0]
    assert abs(got[0][1] - s[3]) < 1e-12 and abs(got[1][1] - s[0]) < 1e-12
    assert sum(w for _, w in got) < 0.9


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("sizes", [(5, 2, 24, 40, 0.75), (8, 3, 64, 64, 2.0),
                                   (3, 1, 16, 72, 1.0)])
def test_routed_clamped_experts(mode, sizes):
    from kaito_amd.engine.config import ModelConfig
    from kaito_amd.models.hybrid_config import MoESpec, layer_moe_config
    from kaito_amd.models.moe import MoEMLP
    from kaito_amd.parallel.state import init_parallel
    init_parallel(1)
    dev, dt = mode
    E, top, ff, width, limit = sizes
    rng = np.random.default_rng(E)
    mlp = L.moe(E, top, ff, limit)
    cfg = L.make_config([L.delta_layer(1, 4, mlp)], width, 8)
    W = L.random_weights(cfg, seed=E)
    fp = "l0.mlp."
    # corrections large enough to change the choice for most rows
    W[fp + "correction"] = L._bf16_round(rng.normal(0, 0.3, E))
    T = 23
    hx, hf = act(rng.normal(0, 1.5, (T, width)), mode)
    want = L.moe_ff(hf, W, fp, mlp)
    changed = sum(
        [e for e, _ in L.route(z, W[fp + "correction"], top)]
        != [e for e, _ in L.route(z, np.zeros(E), top)]
        for z in hf @ W[fp + "router"].T)
    assert changed > 0
    base = ModelConfig(name="t", hidden_size=width, num_layers=1,
                       num_heads=1, num_kv_heads=1, head_dim=width,
                       intermediate_size=ff, vocab_size=8, dtype=dt)
    spec = MoESpec(experts=E, top=top, ff=ff, routing="softmax_bias",
                   act="clamped_glu", limit=limit)
    m = MoEMLP(layer_moe_config(base, spec)).to(dev)
    ie = m.ie_local
    with torch.no_grad():
        m.gate.copy_(torch.tensor(W[fp + "router"]))
        m.e_score_correction_bias.copy_(torch.tensor(W[fp + "correction"]))
        m.w_gate_up.zero_()
        m.w_down.zero_()
        for e in range(E):
            m.w_gate_up[e, :ff] = torch.tensor(W[f"{fp}e{e}.gate"])
            m.w_gate_up[e, ie:ie + ff] = torch.tensor(W[f"{fp}e{e}.up"])
            m.w_down[e, :, :ff] = torch.tensor(W[f"{fp}e{e}.down"])
    got = m(hx)
    if dt == torch.float32:
        close(got, want, dt, f32=2e-5)
    else:
        # a rounded score may pick another expert on a near-tie: rows
        err = (got.double().cpu() - torch.tensor(want)).abs().amax(-1) \
            / np.abs(want).max()
        assert err.median().item() < 2e-2
        assert (err < 4e-2).float().mean() > 0.8


# ---- projections whose result stays f32 ---------------------------------------------

@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("shape", [(37, 96, 50), (5, 72, 33), (128, 256, 192)])
def test_gate_projection_keeps_f32(mode, shape):
    """bf16 operands multiply exactly; the sum must not be rounded back to
    bf16 (a sigmoid near 0 or 1 would lose its tail)."""
    dev, dt = mode
    T, K, N = shape
    rng = np.random.default_rng(T)
    x, xf = act(rng.normal(0, 1, (T, K)), mode)
    w, wf = act(rng.normal(0, 1, (N, K)), mode)
    b = rng.normal(0, 1, N)
    got = ops.linear_f32(x, w, torch.tensor(b, dtype=torch.float32,
                                            device=dev))
    assert got.dtype == torch.float32
    close(got, xf @ wf.T + np.float32(b), torch.float32, f32=2e-6)
