"""The mechanisms of the Munerax design one at a time, each op of the
package against the plain functions of tests/munerax_oracle.py or a
closed form: hashed bigram embedding with its previous-token state,
rotation + latent norm + paged cache write, latent-space attention (sink,
far keys, page borders, more heads than a kernel tile, padding rows; sizes
for the simple and for the matrix-core kernel, which also splits the keys
of a row over workgroups), the
expanded prompt path against the latent path, group-limited sigmoid
routing, squared-relu experts with a shared expert, and the element-wise
gates. CPU runs check the reference ops; `-m gpu` runs the HIP kernels in
f32 and bf16."""
import math
import os
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import munerax_oracle as M  # noqa: E402

from kaito_amd import ops  # noqa: E402

MODES = [("cpu", torch.float32),
         pytest.param(("cuda", torch.float32), marks=pytest.mark.gpu),
         pytest.param(("cuda", torch.bfloat16), marks=pytest.mark.gpu)]
BS = 16      # page size used here


def i32(x, dev):
    return torch.tensor(x, dtype=torch.int32, device=dev)


def close(got, want, dtype, scale=None):
    want = torch.as_tensor(np.asarray(want), dtype=torch.float64)
    scale = scale if scale is not None else want.abs().max().item() + 1e-9
    err = (got.double().cpu() - want).abs().max().item() / scale
    assert err < (1e-5 if dtype == torch.float32 else 2e-2), err


# ---- embedding ----------------------------------------------------------------

@pytest.mark.parametrize("mode", MODES)
def test_bigram_embedding_rows_and_state(mode):
    dev, dt = mode
    rng = np.random.default_rng(0)
    vocab, width, bg = 40, 24, {"buckets": 17, "mul_prev": 5, "mul_cur": 3}
    E = M._bf16_round(rng.normal(0, 1, (vocab, width)))
    B = M._bf16_round(rng.normal(0, 1, (18, width)))
    cfg = {"embedding": {"scale": 2.5, "bigram": bg}}
    seq_a = [int(t) for t in rng.integers(0, vocab, 9)]
    seq_b = [int(t) for t in rng.integers(0, vocab, 4)]
    want_a = M.embed(cfg, {"embed": E, "bigram": B}, seq_a)
    want_b = M.embed(cfg, {"embed": E, "bigram": B}, seq_b)
    Et = torch.tensor(E, dtype=dt, device=dev)
    Bt = torch.tensor(B, dtype=dt, device=dev)
    # slots hold stale tokens of earlier sequences
    state = torch.tensor([33, 7, 21], dtype=torch.long, device=dev)

    def step(chunks):
        """chunks: (tokens, slot, start) in one batch."""
        ids, cu, seq_of = [], [0], []
        for i, (tk, _, _) in enumerate(chunks):
            ids += tk
            cu.append(len(ids))
            seq_of += [i] * len(tk)
        return ops.bigram_embed(
            torch.tensor(ids, dtype=torch.long, device=dev), Et, 2.5, Bt,
            17, 5, 3, state, i32(cu, dev),
            i32([c[1] for c in chunks], dev), i32([c[2] for c in chunks], dev),
            i32(seq_of, dev))
    # a in slot 2, b in slot 0, cut differently, in shared steps; a
    # padding chunk (slot -1) between them
    x1 = step([(seq_a[:3], 2, 0), ([0], -1, 0), (seq_b[:1], 0, 0)])
    x2 = step([(seq_b[1:4], 0, 1), (seq_a[3:4], 2, 3)])
    x3 = step([(seq_a[4:9], 2, 4)])
    got_a = torch.cat([x1[:3], x2[3:4], x3])
    got_b = torch.cat([x1[4:5], x2[:3]])
    close(got_a, want_a, torch.float32)       # the sum itself is f32
    close(got_b, want_b, torch.float32)
    assert x1[3].abs().max().item() == 0.0    # padding row
    assert state.tolist() == [seq_b[3], 7, seq_a[8]]
    # without a table: the scaled embedding alone
    x = ops.bigram_embed(torch.tensor(seq_b, dtype=torch.long, device=dev),
                         Et, 2.5, None, 0, 0, 0, None, i32([0, 4], dev),
                         i32([1], dev), i32([0], dev), i32([0] * 4, dev))
    close(x, E[seq_b] * 2.5, torch.float32)


# ---- rotation, latent norm, cache write -----------------------------------------

@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("sizes", [(3, 6, 4, 10, 3), (5, 16, 8, 24, 8)])
def test_rotation_norm_and_cache_write(mode, sizes):
    """Sizes with odd offsets (element-wise moves) and with 16-byte
    aligned heads and rows (vector moves)."""
    dev, dt = mode
    rng = np.random.default_rng(1)
    H, D, R2, rank, gap = sizes
    T, eps, base = 7, 1e-5, 50.0
    pos = [0, 1, 2, 40, 41, 500, 7]
    width = 12
    h = M._bf16_round(rng.normal(0, 1, (T, width)))
    W = {"m.dkv": M._bf16_round(rng.normal(0, 1, (rank + R2, width))),
         "m.dkv.norm": M._bf16_round(rng.uniform(0.5, 1.5, rank))}
    d = h @ W["m.dkv"].T
    c_want = M.rms(d[:, :rank], eps) * W["m.dkv.norm"]
    kr_want = M.rotate_half(d[:, rank:], pos, base, R2)
    q = M._bf16_round(rng.normal(0, 1, (T, H, D + R2)))
    q_want = q.copy()
    q_want[..., D:] = M.rotate_half(q[..., D:], pos, base, R2)
    inv = torch.tensor([base ** (-2.0 * i / R2) for i in range(R2 // 2)],
                       dtype=torch.float64).float().to(dev)
    cache = torch.zeros(40, BS, rank + R2, dtype=dt, device=dev)
    slots = torch.tensor([5, 16, 17, 31, 32, 639, -1], dtype=torch.long,
                         device=dev)
    # q and the latent row are column ranges of one projection output
    packed = torch.zeros(T, H * (D + R2) + gap + rank + R2, dtype=dt,
                         device=dev)
    packed[:, :H * (D + R2)] = torch.tensor(q.reshape(T, -1), dtype=dt)
    packed[:, H * (D + R2) + gap:] = torch.tensor(d, dtype=dt)
    got_q = ops.latent_rope_cache_write(
        packed[:, :H * (D + R2)].unflatten(-1, (H, D + R2)),
        packed[:, H * (D + R2) + gap:],
        torch.tensor(W["m.dkv.norm"], dtype=torch.float32, device=dev), eps,
        cache, slots, torch.tensor(pos, dtype=torch.long, device=dev), inv, D)
    close(got_q, q_want, dt)
    flat = cache.view(-1, rank + R2)
    for t, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        close(flat[s, :rank], c_want[t], dt)
        close(flat[s, rank:], kr_want[t], dt)
    written = {s for s in slots.tolist() if s >= 0}
    rest = [i for i in range(flat.size(0)) if i not in written]
    assert flat[rest].abs().max().item() == 0.0
    # a layer that reads another layer's cache only rotates its queries
    got_q2 = ops.latent_rope_cache_write(
        packed[:, :H * (D + R2)].unflatten(-1, (H, D + R2)), None, None, eps,
        cache, slots, torch.tensor(pos, dtype=torch.long, device=dev), inv, D)
    assert torch.equal(got_q, got_q2)
    # zero-padded heads for a kernel that takes fixed key sizes
    got_q3 = ops.latent_rope_cache_write(
        packed[:, :H * (D + R2)].unflatten(-1, (H, D + R2)), None, None, eps,
        cache, slots, torch.tensor(pos, dtype=torch.long, device=dev), inv, D,
        pad_to=32)
    assert got_q3.shape == (T, H, 32)
    assert torch.equal(got_q3[..., :D + R2], got_q)
    assert got_q3[..., D + R2:].abs().max().item() == 0.0


# ---- latent-space attention ---------------------------------------------------------

def plain_attention(q, rows, scale, rank, sink):
    """q [H, DT], rows [n, DT] float64 → [H, rank]."""
    s = q @ rows.T * scale
    out = np.zeros((q.shape[0], rank))
    for h in range(q.shape[0]):
        m = max(s[h].max(), sink[h]) if sink is not None else s[h].max()
        e = np.exp(s[h] - m)
        den = e.sum() + (math.exp(sink[h] - m) if sink is not None else 0.0)
        out[h] = (e / den) @ rows[:, :rank]
    return out


def paged(rows_per_seq, DT, dt, dev, pages=64, seed=0):
    """Scatter sequences' rows into shuffled pages; returns cache, tables."""
    rng = np.random.default_rng(seed)
    order = list(rng.permutation(pages))
    cache = torch.zeros(pages, BS, DT, dtype=dt, device=dev)
    # unused pages hold junk, not zeros
    cache.normal_(0, 3.0)
    tables = []
    for rows in rows_per_seq:
        n = -(-len(rows) // BS)
        tab = [int(order.pop()) for _ in range(n)]
        for j, r in enumerate(rows):
            cache[tab[j // BS], j % BS] = torch.tensor(r, dtype=dt)
        tables.append(tab)
    width = max(len(t) for t in tables)
    bt = i32([t + [0] * (width - len(t)) for t in tables], dev)
    return cache, bt


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("shape", [(3, 20, 4), (11, 33, 2), (16, 64, 16),
                                   (20, 160, 32)])
def test_latent_attention_rows_of_mixed_steps(mode, shape):
    """Rows of several sequences at unequal positions (first tokens, page
    borders, mid-page) in one call, heads beyond one tile of 8, a padding
    row; with and without sinks."""
    dev, dt = mode
    H, rank, P = shape
    DT = rank + P
    rng = np.random.default_rng(H)
    lens = [1, 16, 17, 70]
    seqs = [M._bf16_round(rng.normal(0, 1, (n, DT))) for n in lens]
    cache, bt = paged(seqs, DT, dt, dev, seed=H)
    rows = [(0, 0), (1, 15), (2, 15), (2, 16), (3, 0), (3, 31), (3, 32),
            (3, 69), (-1, 0), (3, 47)]
    q = M._bf16_round(rng.normal(0, 1, (len(rows), H, DT)))
    sink = M._bf16_round(rng.normal(0, 1, H))
    for use_sink in (True, False):
        got = ops.latent_attention(
            torch.tensor(q, dtype=dt, device=dev), cache, bt,
            i32([r[0] for r in rows], dev),
            torch.tensor([r[1] for r in rows], dtype=torch.long, device=dev),
            0.3, rank,
            torch.tensor(sink, dtype=torch.float32, device=dev)
            if use_sink else None)
        for t, (b, p) in enumerate(rows):
            if b < 0:
                assert got[t].abs().max().item() == 0.0
                continue
            want = plain_attention(q[t], seqs[b][:p + 1], 0.3, rank,
                                   sink if use_sink else None)
            close(got[t], want, dt, scale=1.0)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("far", [0, 15, 16, 31, 32, 299])
def test_far_key_found_among_hundreds(mode, far):
    """One key is made to match the query (all others nearly orthogonal),
    so the output must be that key's latent: at the first position, at
    page borders, and at the query's own position."""
    dev, dt = mode
    H, rank, P, n = 2, 16, 8, 300
    DT = rank + P
    rng = np.random.default_rng(far)
    rows = M._bf16_round(rng.normal(0, 0.05, (n, DT)))
    rows[far, :] = 0.0
    rows[far, 3] = 4.0
    rows[far, rank + 1] = 4.0
    q = np.zeros((1, H, DT))
    q[0, :, 3] = 4.0
    q[0, :, rank + 1] = 4.0
    cache, bt = paged([rows], DT, dt, dev, seed=far)
    got = ops.latent_attention(
        torch.tensor(q, dtype=dt, device=dev), cache, bt, i32([0], dev),
        torch.tensor([n - 1], dtype=torch.long, device=dev), 1.0, rank,
        torch.full((H,), -5.0, device=dev))
    want = plain_attention(q[0], rows, 1.0, rank, np.full(H, -5.0))
    assert abs(want[0, 3] - 4.0) < 1e-3, "the key must dominate the oracle"
    close(got[0], want, dt, scale=4.0)
    # one position earlier than the far key at the end: it is not seen
    if far == n - 1:
        got = ops.latent_attention(
            torch.tensor(q, dtype=dt, device=dev), cache, bt, i32([0], dev),
            torch.tensor([n - 2], dtype=torch.long, device=dev), 1.0, rank,
            torch.full((H,), -5.0, device=dev))
        assert got[0, 0, 3].abs().item() < 0.5


@pytest.mark.parametrize("mode", MODES)
def test_sink_takes_its_share(mode):
    """With every score zero and n keys, the weights are 1 / (n + e^sink):
    the sink counts once, unscaled, and has no value."""
    dev, dt = mode
    H, rank, P, n = 3, 8, 8, 5
    rows = np.zeros((n, rank + P))
    rows[:, :rank] = 1.0
    rows[:, rank:] = 0.0
    q = np.zeros((1, H, rank + P))
    sink = np.array([0.0, math.log(3.0), -40.0])
    cache, bt = paged([rows], rank + P, dt, dev)
    got = ops.latent_attention(
        torch.tensor(q, dtype=dt, device=dev), cache, bt, i32([0], dev),
        torch.tensor([n - 1], dtype=torch.long, device=dev), 7.0, rank,
        torch.tensor(sink, dtype=torch.float32, device=dev))
    want = np.array([n / (n + 1.0), n / (n + 3.0), 1.0])
    close(got[0, :, 0], want, dt, scale=1.0)


# ---- the whole mixer, and the expanded prompt path -----------------------------------

def mixer_setup(dev, dt, H, D, R2, V, rank, width, seed, kv_from=None):
    from kaito_amd.models.hybrid_config import LatentAttnSpec, RotarySpec
    from kaito_amd.models.mixers import LatentAttention
    mx = M.latent_layer(H, D, R2, V, rank, scale=0.4, base=300.0,
                        kv_from=kv_from)["mixer"]
    cfg = M.make_config([{"type": "latent_attention", "mixer": mx,
                          "mlp": None}], width=width, vocab=8, bigram=None)
    cfg["layers"][0]["mixer"].pop("kv_from", None)
    W = M.random_weights(cfg, seed=seed)
    spec = LatentAttnSpec(heads=H, dim=D, rot_dim=R2, vdim=V, kv_rank=rank,
                          scale=0.4, rot=RotarySpec(dims=R2, base=300.0),
                          sink=True, gate=True)
    m = LatentAttention(width, spec, dt, 1e-5).to(dev)
    with torch.no_grad():
        def t(name):
            return torch.tensor(W["l0.mix." + name])
        m.in_proj.zero_()
        m.in_proj[:m.in_rows].copy_(
            torch.cat([t("q"), t("g"), t("dkv")], 0).to(dt))
        m.kv_norm.copy_(t("dkv.norm").float())
        m.w_uk.copy_(t("uk").to(dt))
        m.w_uv.copy_(t("uv").to(dt))
        m.sinks.copy_(t("sink").float())
        m.o_proj.copy_(t("o").to(dt))
    return m, mx, W


def step_meta(dev, chunks, tables, tiles):
    """chunks: (start, length) per sequence, block tables given."""
    from kaito_amd.models.llama import AttnMetadata
    pos, slots, cu, seq_of = [], [], [0], []
    for i, (s, n) in enumerate(chunks):
        for p in range(s, s + n):
            pos.append(p)
            slots.append(tables[i][p // BS] * BS + p % BS)
            seq_of.append(i)
        cu.append(cu[-1] + n)
    width = max(len(t) for t in tables)
    meta = AttnMetadata(
        is_prefill=True,
        slot_mapping=torch.tensor(slots, dtype=torch.long, device=dev),
        cu_seqlens=i32(cu, dev), max_seqlen=max(n for _, n in chunks),
        block_tables=i32([t + [0] * (width - len(t)) for t in tables], dev))
    meta.state_slots = i32(list(range(len(chunks))), dev)
    meta.seq_starts = i32([s for s, _ in chunks], dev)
    meta.token_seq = i32(seq_of, dev)
    meta.ctx_lens = [s + n for s, n in chunks]
    if tiles:
        meta.tile_seq, meta.tile_qbase = ops.build_query_tiles(
            [n for _, n in chunks], dev)
    return meta, torch.tensor(pos, dtype=torch.long, device=dev)


@pytest.mark.parametrize("mode", MODES)
def test_mixer_in_portions_against_oracle(mode):
    """The mixer alone on a sequence fed in portions (cache carried in
    pages) against the oracle's attention on the whole sequence."""
    dev, dt = mode
    H, D, R2, V, rank, width, T = 3, 10, 6, 7, 18, 40, 50
    m, mx, W = mixer_setup(dev, dt, H, D, R2, V, rank, width, seed=4)
    rng = np.random.default_rng(4)
    h = M._bf16_round(rng.normal(0, 1, (T, width)))
    want = M.latent_attention(h, W, "l0.mix.", mx, 1e-5,
                              M.latent_kv(h, W, "l0.mix.", mx, 1e-5))
    cache = m.alloc_cache(8, BS, 1, dev)
    tab = [[5, 2, 7, 0]]
    out, at = [], 0
    for n in (1, 2, 14, 3, 17, 1, 12):
        meta, pos = step_meta(dev, [(at, n)], tab, tiles=False)
        out.append(m(torch.tensor(h[at:at + n], dtype=dt, device=dev), pos,
                     cache, meta))
        at += n
    close(torch.cat(out), want, dt)


@pytest.mark.gpu
@pytest.mark.parametrize("sizes", [(4, 48, 16, 32, 64), (2, 20, 12, 24, 40),
                                   (9, 100, 28, 64, 96)])
def test_expanded_prompt_path_matches_latent_path(sizes):
    """bf16 prompt portions take the expanded form (per-head keys and
    values in a step-local scratch, MFMA kernel); the same step through
    the latent form must agree: two sequences, one continuing at an
    uneven start with keys behind it, key sizes with and without
    padding."""
    dev, dt = "cuda", torch.bfloat16
    H, D, R2, V, rank = sizes
    width = 64
    m, mx, W = mixer_setup(dev, dt, H, D, R2, V, rank, width, seed=H)
    rng = np.random.default_rng(H)
    h = torch.tensor(rng.normal(0, 1, (120, width)), dtype=dt, device=dev)
    tabs = [[3, 9, 1, 12, 6], [4, 10, 2, 8, 11]]
    caches = [m.alloc_cache(16, BS, 2, dev) for _ in range(2)]
    outs = []
    for tiles, cache in zip((True, False), caches):
        # first portions (latent form both times, fills the cache)
        meta, pos = step_meta(dev, [(0, 21), (0, 3)], tabs, tiles=False)
        m(h[:24], pos, cache, meta)
        meta, pos = step_meta(dev, [(21, 50), (3, 45)], tabs, tiles=tiles)
        assert m._expanded_ok(h, meta) == tiles
        outs.append(m(h[24:119], pos, cache, meta))
    err = (outs[0].float() - outs[1].float()).abs().max().item()
    assert err < 0.03 * outs[1].float().abs().max().item(), err


# ---- feed-forward ------------------------------------------------------------------

def moe_module(dev, dt, width, mlp, W, pre):
    import dataclasses
    from kaito_amd.engine.config import ModelConfig
    from kaito_amd.models.hybrid_config import (_munerax_ff,
                                                layer_moe_config)
    from kaito_amd.models.moe import MoEMLP
    from kaito_amd.parallel.state import init_parallel
    init_parallel(1)
    _, spec = _munerax_ff(mlp)
    base = ModelConfig(name="t", hidden_size=width, dtype=dt)
    m = MoEMLP(layer_moe_config(base, spec)).to(dev)
    with torch.no_grad():
        m.gate.copy_(torch.tensor(W[pre + "router"]).float())
        m.w_gate_up.zero_()
        m.w_down.zero_()
        for e in range(spec.experts):
            u = torch.tensor(W[f"{pre}e{e}.up"]).to(dt)
            d = torch.tensor(W[f"{pre}e{e}.down"]).to(dt)
            m.w_gate_up[e, :u.shape[0]].copy_(u)
            m.w_down[e, :, :u.shape[0]].copy_(d)
        if spec.shared_ff:
            m.w_shared_gate_up.copy_(torch.tensor(W[pre + "shared.up"]).to(dt))
            m.w_shared_down.copy_(torch.tensor(W[pre + "shared.down"]).to(dt))
    return m


def test_group_limited_routing_choices():
    """Crafted scores: the best single expert sits in a group whose pair
    sum loses, so it must not be chosen; weights are the sigmoid scores
    times the scale, not renormalised."""
    router = {"experts": 6, "top": 2, "scale": 1.5,
              "groups": {"count": 3, "keep": 1}}
    z = np.array([4.0, -6.0, 2.0, 2.5, -1.0, -2.0])
    chosen, w = M.route(z, router)
    assert sorted(chosen.tolist()) == [2, 3]
    W = {"r.router": np.eye(6)}
    for e in range(6):
        W[f"r.e{e}.up"] = np.zeros((4, 6))
        W[f"r.e{e}.down"] = np.zeros((6, 4))
    mlp = M.moe(6, 2, 4, scale=1.5, groups=(3, 1))
    m = moe_module("cpu", torch.float32, 6, mlp, W, "r.")
    tok, gates, offsets = m._route(torch.tensor(z, dtype=torch.float32)[None])
    counts = (offsets[1:] - offsets[:-1]).tolist()
    assert counts == [0, 0, 1, 1, 0, 0]
    assert torch.allclose(gates.double(), torch.tensor(
        [M.sigmoid(2.0) * 1.5, M.sigmoid(2.5) * 1.5]), atol=1e-6)
    # groups of one expert: a group's score is its only expert's
    router = {"experts": 4, "top": 2, "scale": 1.0,
              "groups": {"count": 4, "keep": 3}}
    chosen, _ = M.route(np.array([0.1, 0.9, 0.5, 0.7]), router)
    assert sorted(chosen.tolist()) == [1, 3]


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("shape", [(6, 2, 24, (3, 2), 20, 64),
                                   (5, 1, 12, (5, 2), 0, 96),
                                   (8, 3, 64, None, 40, 128)])
def test_routed_feed_forward(mode, shape):
    dev, dt = mode
    experts, top, ff, groups, shared, width = shape
    mlp = M.moe(experts, top, ff, scale=1.7, groups=groups,
                shared_ff=shared or None)
    cfg = M.make_config([M.latent_layer(1, 4, 2, 4, 4, mlp=mlp)],
                        width=width, vocab=8, bigram=None)
    W = M.random_weights(cfg, seed=experts)
    m = moe_module(dev, dt, width, mlp, W, "l0.mlp.")
    rng = np.random.default_rng(experts)
    h = M._bf16_round(rng.normal(0, 1, (37, width)))
    want = M.moe_ff(h, W, "l0.mlp.", mlp)
    got = m(torch.tensor(h, dtype=dt, device=dev))
    if dt == torch.float32:
        close(got, want, dt)
    else:
        # a rounded score may pick another expert for a rare token
        err = (got.double().cpu() - torch.tensor(want)).abs().amax(-1)
        assert torch.quantile(err, 0.8).item() < 0.03 * np.abs(want).max()


@pytest.mark.parametrize("mode", MODES)
def test_element_wise_gates(mode):
    dev, dt = mode
    rng = np.random.default_rng(3)
    for T, F_ in ((5, 24), (3, 7)):
        gu = M._bf16_round(rng.normal(0, 2, (T, 2 * F_)))
        g = torch.tensor(gu, dtype=dt, device=dev)
        close(ops.gelu_glu(g), M.gelu_tanh(gu[:, :F_]) * gu[:, F_:], dt)
        close(ops.relu2(g), np.maximum(gu, 0) ** 2, dt)
        # a column range of a wider buffer
        wide = torch.zeros(T, 2 * F_ + 5, dtype=dt, device=dev)
        wide[:, 3:3 + 2 * F_] = g
        close(ops.relu2(wide[:, 3:3 + 2 * F_]), np.maximum(gu, 0) ** 2, dt)
    x = M._bf16_round(rng.normal(0, 1, (4, 12)))
    gate = M._bf16_round(rng.normal(0, 2, (4, 3)))
    want = x * np.repeat(M.sigmoid(gate), 4, axis=1)
    close(ops.sigmoid_mul(torch.tensor(x, dtype=dt, device=dev),
                          torch.tensor(gate, dtype=dt, device=dev)), want, dt)


@pytest.mark.parametrize("mode", MODES)
def test_dense_feed_forward(mode):
    from kaito_amd.models.hybrid_config import GeluGLUSpec
    from kaito_amd.models.mixers import GeluGLU
    dev, dt = mode
    cfg = M.make_config([M.latent_layer(1, 4, 2, 4, 4, mlp=M.dense(36))],
                        width=20, vocab=8, bigram=None)
    W = M.random_weights(cfg, seed=8)
    m = GeluGLU(20, GeluGLUSpec(36), dt).to(dev)
    with torch.no_grad():
        m.gate_up.copy_(torch.cat([torch.tensor(W["l0.mlp.gate"]),
                                   torch.tensor(W["l0.mlp.up"])], 0).to(dt))
        m.down.copy_(torch.tensor(W["l0.mlp.down"]).to(dt))
    h = M._bf16_round(np.random.default_rng(8).normal(0, 1, (9, 20)))
    close(m(torch.tensor(h, dtype=dt, device=dev)),
          M.dense_ff(h, W, "l0.mlp."), dt)
