"""The Lokedra model served by the engine against the plain oracle in
tests/lokedra_oracle.py: whole prompts, the residual stream after every
layer run, token-by-token decoding, portions down to two tokens, unequal
batches, reuse of pages and state slots, far-away tokens, chunk edges,
loops of several shapes, other sizes, greedy generation through the
scheduler. CPU runs use the engine's reference ops; the same tests run on
the HIP kernels under `-m gpu` (f32 and bf16)."""
import os
import random
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import lokedra_oracle as L  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
MODES = [("cpu", "float32"),
         pytest.param(("cuda", "float32"), marks=pytest.mark.gpu),
         pytest.param(("cuda", "bfloat16"), marks=pytest.mark.gpu)]

YARN = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}


def config_a():
    # a parallel layer first, a loop over the middle run three times, a
    # layer without feed-forward, chunk 10 (inside pages), four taps
    return L.make_config([
        L.parallel_layer(heads=4, kv_heads=2, dim=8, chunk=10, taps=4,
                         r_heads=2, r_dim=8, r_vdim=12, scales=(1.3, 0.6),
                         mlp=L.moe(5, 2, 24, limit=1.5)),
        L.delta_layer(heads=3, dim=8, mlp=None),
        L.latent_layer(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=20,
                       q_rank=14, base=100.0, scaling=YARN,
                       mlp=L.moe(4, 3, 16, limit=0.5)),
        L.delta_layer(heads=1, dim=24, mlp=L.moe(6, 1, 8, limit=3.0)),
    ], width=64, vocab=50, embed_scale=3.0, loop=(1, 3, 3))


def config_b():
    # no loop; width not a multiple of 64; kv_heads = heads; one tap;
    # chunk 1 (a query sees itself only) and a chunk longer than any
    # prompt here; top-1; plain rotation; nine latent heads; embedding
    # scale 1; a head of 72 state rows
    return L.make_config([
        L.latent_layer(heads=9, dim=6, rot_dim=2, vdim=10, kv_rank=33,
                       q_rank=20, base=50.0, mlp=L.moe(5, 1, 12)),
        L.parallel_layer(heads=3, kv_heads=3, dim=12, chunk=1, taps=1,
                         r_heads=1, r_dim=20, r_vdim=6, scales=(0.7, 1.0),
                         mlp=None),
        L.parallel_layer(heads=2, kv_heads=1, dim=16, chunk=4096, taps=2,
                         r_heads=3, r_dim=4, r_vdim=8, scales=(1.0, 1.0),
                         mlp=L.moe(3, 3, 20, limit=2.0)),
        L.delta_layer(heads=1, dim=72, mlp=L.moe(4, 2, 8)),
    ], width=96, vocab=70, eps=1e-6, embed_scale=1.0)


def config_c():
    # sizes the matrix-core prompt kernels and the fused expert kernels
    # take in bf16 (head 64, latent key 48 + 16, widths multiples of 64);
    # a loop that covers the whole stack once more; chunk 48
    return L.make_config([
        L.latent_layer(heads=4, dim=48, rot_dim=16, vdim=32, kv_rank=64,
                       q_rank=48, scaling=YARN, mlp=L.moe(8, 2, 64)),
        L.delta_layer(heads=2, dim=64, mlp=L.moe(4, 2, 64, limit=2.0)),
        L.parallel_layer(heads=4, kv_heads=2, dim=64, chunk=48, taps=3,
                         r_heads=2, r_dim=32, r_vdim=64, scales=(1.2, 0.9),
                         mlp=L.moe(8, 3, 128)),
    ], width=128, vocab=96, embed_scale=8.0, loop=(0, 3, 2))


CONFIGS = {"a": config_a, "b": config_b, "c": config_c}
_CKPT = {}


def checkpoint(tmp_path_factory, name):
    if name not in _CKPT:
        cfg = CONFIGS[name]()
        W = L.random_weights(cfg, seed=len(_CKPT) + 3)
        folder = L.write_checkpoint(
            str(tmp_path_factory.mktemp(f"lk_{name}")), cfg, W)
        _CKPT[name] = (cfg, W, folder)
    return _CKPT[name]


def engine(folder, mode, max_tokens=512, max_live=4):
    from kaito_amd.engine.trace_replay import build_engine
    device, dtype = mode
    return build_engine(folder, dtype, max_tokens, device, max_live)


def tokens(cfg, n, seed):
    rng = random.Random(seed)
    return [rng.randrange(cfg["vocab"]) for _ in range(n)]


def row_err(got, want, quantile=1.0):
    """Mean-free RMS difference per row relative to the oracle's logit
    spread; the worst row, or the given quantile of the rows."""
    d = got.double().cpu() - want
    d = d - d.mean(-1, keepdim=True)
    spread = (want - want.mean(-1, keepdim=True)).pow(2).mean().sqrt()
    e = d.pow(2).mean(-1).sqrt() / spread
    return torch.quantile(e, quantile).item()


def tol(mode):
    return 2e-4 if mode[1] == "float32" else 0.1


def check(got, want, mode):
    """f32 runs must match on every row; under bf16 rounding the typical
    row must match and the worst nearly (narrow random layers are noisy,
    and a rounded router score can pick another expert); the f32 run of
    the same templated kernels holds the line on single rows."""
    if mode[1] == "float32":
        assert row_err(got, want) < tol(mode)
    else:
        assert row_err(got, want, 0.5) < tol(mode)
        assert row_err(got, want, 0.9) < 4 * tol(mode)


def run_portions(eng, sid, toks, sizes):
    """Feed toks to request sid in portions; returns all-row logits."""
    out, at = [], 0
    for n in sizes:
        eng.extend_request(sid, toks[at:at + n])
        out.append(eng.step_explicit([(sid, n)], [(0, i) for i in range(n)]))
        at += n
    assert at == len(toks)
    return torch.cat(out, 0)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("name", ["a", "b"])
def test_whole_prompt(tmp_path_factory, name, mode):
    cfg, W, folder = checkpoint(tmp_path_factory, name)
    toks = tokens(cfg, 45, 1)
    want = L.model_logits(cfg, W, toks)
    eng = engine(folder, mode)
    check(run_portions(eng, 0, toks, [45]), want, mode)
    # a one-token prompt: nothing before it anywhere (zero shift row,
    # zero states, empty convolution tail)
    check(run_portions(eng, 1, toks[:1], [1]), want[:1], mode)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("name", ["a", "c"])
def test_residual_stream_per_layer_run(tmp_path_factory, name, mode):
    """One stream per RUN of a layer (a looped layer counts every time),
    taken before the next pass adds the embedding output."""
    cfg, W, folder = checkpoint(tmp_path_factory, name)
    toks = tokens(cfg, 20, 2)
    streams = []
    L.model_logits(cfg, W, toks, streams)
    assert len(streams) == len(L.layer_runs(cfg))
    eng = engine(folder, mode)
    seen = []
    eng.runner.model.layer_hook = lambda i, x: seen.append(x.clone())
    with_hook = run_portions(eng, 0, toks, [20])
    assert len(seen) == len(streams)
    lim = 1e-4 if mode[1] == "float32" else 0.1
    for got, want in zip(seen, streams):
        err = (got.double().cpu() - want).abs().max() / want.abs().max()
        assert err < lim
    # the observer's unfused path and the fused one agree
    eng.runner.model.layer_hook = None
    plain = run_portions(eng, 1, toks, [20])
    assert row_err(with_hook, plain.double().cpu()) < \
        (1e-5 if mode[1] == "float32" else 0.05)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_decode_and_portions_match_whole(tmp_path_factory, name, mode):
    cfg, W, folder = checkpoint(tmp_path_factory, name)
    toks = tokens(cfg, 70, 3)
    want = L.model_logits(cfg, W, toks)
    eng = engine(folder, mode)
    # prompt then one by one, over page and chunk borders
    check(run_portions(eng, 0, toks, [9] + [1] * 61), want, mode)
    # all one by one from the very first token
    check(run_portions(eng, 1, toks, [1] * 70), want, mode)
    # uneven portions: 2-token ones, cuts at and beside page borders
    check(run_portions(eng, 2, toks, [2, 1, 2, 11, 2, 14, 2, 3, 11, 10, 2,
                                      10]), want, mode)
    eng.release(0)
    eng.release(1)
    eng.release(2)
    # a long portion after a short one: the tiled prompt kernels start in
    # the middle of a page and of a chunk with keys behind them
    check(run_portions(eng, 3, toks, [5, 65]), want, mode)


@pytest.mark.parametrize("mode", MODES)
def test_unequal_batches_and_reuse(tmp_path_factory, mode):
    """Requests of different lengths share steps (portions beside single
    tokens); the page pool and the four state slots are too small for all
    of them at once, so both are freed and used again — a reused slot
    still holds the previous request's states, shift rows and
    convolution tails, in every run of every layer."""
    cfg, W, folder = checkpoint(tmp_path_factory, "a")
    lens = [37, 5, 50, 18, 1, 33, 26]
    reqs = [tokens(cfg, n, 10 + i) for i, n in enumerate(lens)]
    want = [L.model_logits(cfg, W, t) for t in reqs]
    eng = engine(folder, mode, max_tokens=192, max_live=4)
    rng = random.Random(5)
    at = [0] * len(reqs)
    got = [[] for _ in reqs]
    live, nxt = [], 0
    while nxt < len(reqs) or live:
        while nxt < len(reqs) and len(live) < 4 and \
                sum(-(-lens[i] // 64) * 64 for i in live + [nxt]) <= 192:
            live.append(nxt)
            nxt += 1
        portions, want_rows, owners = [], [], []
        for i in list(live):
            if rng.random() < 0.25 and len(live) > 1:
                continue                      # sits this step out
            left = lens[i] - at[i]
            n = min(left, rng.choice([1, 1, 2, 3, 8, 17]))
            eng.extend_request(i, reqs[i][at[i]:at[i] + n])
            want_rows += [(len(portions), k) for k in range(n)]
            owners += [i] * n
            portions.append((i, n))
            at[i] += n
        if not portions:
            continue
        lg = eng.step_explicit(portions, want_rows)
        for row, i in zip(lg, owners):
            got[i].append(row)
        for i in list(live):
            if at[i] == lens[i]:
                eng.release(i)
                live.remove(i)
    assert eng.pool.num_free == eng.pool.num_blocks
    assert eng.state_pool.num_free == 4
    for g, w in zip(got, want):
        check(torch.stack(g), w, mode)


def far_config(kind):
    if kind == "delta":
        layer = L.delta_layer(heads=2, dim=8, mlp=None)
    elif kind == "hgrn":
        layer = L.parallel_layer(heads=1, kv_heads=1, dim=4, chunk=4, taps=1,
                                 r_heads=2, r_dim=8, r_vdim=8,
                                 scales=(0.0, 1.0), mlp=None)
    else:
        layer = L.latent_layer(heads=2, dim=8, rot_dim=2, vdim=16,
                               kv_rank=12, q_rank=10, base=1e6, scale=1.5,
                               mlp=None)
    return L.make_config([layer], width=32, vocab=24, embed_scale=2.0)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("kind", ["delta", "hgrn", "latent"])
def test_far_token_decides_late(tmp_path_factory, kind, mode):
    """One layer whose memory is long (decays near one and no removal; a
    forget gate near one; a sharp softmax): a swapped token near the start
    of a 200-token prompt moves the last logits. The engine must follow
    the oracle for both prompts, through portions and decoding."""
    cfg = far_config(kind)
    W = L.random_weights(cfg, seed=11)
    W["l0.shift"][:] = 0.0
    if kind == "delta":
        W["l0.mix.w0"][:] = -9.0
        W["l0.mix.w2"][:] = 0.0
        W["l0.mix.a.b"][:] = -9.0
        W["l0.mix.a"][:] = 0.0
    elif kind == "hgrn":
        W["l0.mix.right.lower"][:] = 0.984375    # a value bfloat16 holds
    folder = L.write_checkpoint(
        str(tmp_path_factory.mktemp(f"lk_far_{kind}")), cfg, W)
    base = tokens(cfg, 200, 9)
    want = L.model_logits(cfg, W, base)[-3:]
    # a recurrence sums two hundred writes, so one of them moves the
    # logits by a percent: fifty times what an f32 run may differ by
    felt = 0.05 if kind == "latent" else 0.01
    for pos in range(2, 12):
        other = list(base)
        other[pos] = (other[pos] + 7) % cfg["vocab"]
        want_other = L.model_logits(cfg, W, other)[-3:]
        if row_err(want_other.float(), want) > felt:
            break
    else:
        pytest.fail("the oracle itself must depend on a far token")
    sizes = [3, 60, 2, 100] + [1] * 35
    for toks, w in ((base, want), (other, want_other)):
        eng = engine(folder, mode)
        check(run_portions(eng, 0, toks, sizes)[-3:], w, mode)


@pytest.mark.parametrize("mode", MODES)
def test_chunk_edge_decides(tmp_path_factory, mode):
    """An attention-only layer (the recurrent branch weighted zero, no
    shift, one tap) with a sharp softmax: swapping the token at a chunk's
    first position changes the logits of that chunk's rows and of no row
    before or after the chunk. Chunk 24 over 16-token pages, through
    portions cut inside the chunk and single tokens."""
    cfg = L.make_config([
        L.parallel_layer(heads=2, kv_heads=1, dim=16, chunk=24, taps=1,
                         r_heads=1, r_dim=4, r_vdim=4, scales=(1.0, 0.0),
                         scale=2.0, mlp=None)], width=32, vocab=24,
        embed_scale=2.0)
    W = L.random_weights(cfg, seed=4)
    W["l0.shift"][:] = 0.0
    folder = L.write_checkpoint(str(tmp_path_factory.mktemp("lk_edge")),
                                cfg, W)
    base = tokens(cfg, 80, 6)
    other = list(base)
    other[48] = (other[48] + 5) % cfg["vocab"]       # first key of chunk 2
    wa, wb = L.model_logits(cfg, W, base), L.model_logits(cfg, W, other)
    changed = (wa - wb).abs().amax(-1) > 1e-9
    assert changed[48:72].all() and not changed[:48].any() \
        and not changed[72:].any()
    assert row_err(wb[49:72].float(), wa[49:72]) > 0.02
    sizes = [20, 27, 2, 1, 1, 20, 2, 1, 1, 5]        # cuts at 47, 49, 71, 73
    for toks, w in ((base, wa), (other, wb)):
        eng = engine(folder, mode)
        check(run_portions(eng, 0, toks, sizes), w, mode)
        check(run_portions(eng, 1, toks, [45] + [1] * 35), w, mode)


@pytest.mark.parametrize("mode", MODES[:2])
def test_loop_shapes(tmp_path_factory, mode):
    """Loops that cover nothing, one layer, a tail, and run once: each
    against the oracle, and each run of a layer has state of its own (a
    loop run twice differs from the same stack run once)."""
    layers = [L.delta_layer(heads=2, dim=8, mlp=L.moe(3, 2, 8)),
              L.parallel_layer(heads=2, kv_heads=2, dim=8, chunk=6, taps=2,
                               r_heads=1, r_dim=8, r_vdim=8, mlp=None),
              L.latent_layer(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=12,
                             q_rank=12, mlp=None)]
    toks = None
    seen = []
    for loop in (None, (0, 3, 1), (1, 1, 4), (1, 2, 3), (1, 3, 2),
                 (0, 1, 2)):
        cfg = L.make_config(layers, width=32, vocab=30, embed_scale=2.0,
                            loop=loop)
        W = L.random_weights(cfg, seed=8)
        folder = L.write_checkpoint(
            str(tmp_path_factory.mktemp("lk_loop")), cfg, W)
        toks = toks or tokens(cfg, 33, 4)
        want = L.model_logits(cfg, W, toks)
        eng = engine(folder, mode)
        assert len(eng.runner.model.runs) == len(L.layer_runs(cfg))
        check(run_portions(eng, 0, toks, [7, 2, 1, 1, 22]), want, mode)
        seen.append(want)
    assert row_err(seen[0], seen[1]) < 1e-12      # times 1 = no loop
    assert row_err(seen[0], seen[2]) < 1e-12      # an empty loop
    assert row_err(seen[3], seen[0]) > 0.01


@pytest.mark.parametrize("mode", MODES)
def test_greedy_generation_through_scheduler(tmp_path_factory, mode):
    """LLMEngine.generate (scheduler admission, prefill, batched decode,
    sampler) against greedy decoding with the oracle."""
    from kaito_amd.engine import SamplingParams
    cfg, W, folder = checkpoint(tmp_path_factory, "a")
    prompts = [tokens(cfg, n, 20 + n) for n in (5, 23, 1)]
    eng = engine(folder, mode, max_tokens=512, max_live=4)
    outs = eng.generate(prompts, SamplingParams(max_tokens=14,
                                                ignore_eos=True))
    for p, o in zip(prompts, outs):
        seq = list(p)
        assert len(o.output_token_ids) == 14
        for tok in o.output_token_ids:
            lg = L.model_logits(cfg, W, seq)[-1]
            top2 = torch.topk(lg, 2).values
            if mode[1] == "bfloat16" and top2[0] - top2[1] < 0.5:
                break            # a near-tie may flip under bf16 rounding
            assert tok == int(lg.argmax())
            seq.append(tok)
    assert eng.state_pool.num_free == 4


@pytest.mark.gpu
def test_graph_replayed_decode_matches_eager(tmp_path_factory):
    """Decode steps captured into hipGraphs (token shift and recurrent
    states in slots, latent attention, chunked attention, fused routed
    experts) replayed many times, with eager prefills and host bookkeeping
    between the replays, against the eager engine; two rounds so that
    slots and pages are reused under the same graphs."""
    from kaito_amd.engine import SamplingParams
    cfg, W, folder = checkpoint(tmp_path_factory, "c")
    mode = ("cuda", "bfloat16")
    eager = engine(folder, mode)
    graphed = engine(folder, mode)
    assert graphed.runner.model.decode_graph_capturable()
    graphed.cfg.enforce_eager = False
    graphed.capture_graphs()
    assert graphed.runner._graphs, "no decode graph was captured"
    sp = SamplingParams(max_tokens=24, ignore_eos=True)
    for rnd in range(2):
        prompts = [tokens(cfg, n, 40 + 10 * rnd + n) for n in (7, 30, 2)]
        a = eager.generate(prompts, sp)
        b = graphed.generate(prompts, sp)
        for x, y in zip(a, b):
            assert x.output_token_ids == y.output_token_ids


def test_catalog_resolves_checkpoint_folder(tmp_path_factory):
    """The server's way in: an unknown model name plus a weights folder
    whose config.json names the design."""
    from kaito_amd.models import get_model_config, resolve_model_class
    cfg, W, folder = checkpoint(tmp_path_factory, "b")
    mc = get_model_config("some-looped-stack", weights_path=folder)
    assert mc.arch == "lokedra" and mc.runtime == "native"
    assert mc.layer_loop is None and mc.embed_scale == 1.0
    assert len(mc.layer_specs) == len(cfg["layers"])
    s0, s1, s2, s3 = mc.layer_specs
    assert s0.latent.heads == 9 and s0.latent.q_rank == 20
    assert s0.latent.rot.interleaved and s0.latent.rot.factor == 0
    assert s1.rattn.chunk == 1 and s1.rattn.tied_values and s1.moe is None
    assert s1.rattn.conv_taps == 1 and s1.hgrn.dim == 20
    assert s1.branch_scales == (0.7, 1.0)
    assert s2.moe.routing == "softmax_bias" and s2.moe.act == "clamped_glu"
    assert s2.moe.limit == 2.0 and s2.moe.top == 3
    assert s3.ddelta.dim == 72 and s3.ddelta.heads == 1
    assert resolve_model_class(mc).__name__ == "LokedraForCausalLM"
    ca = checkpoint(tmp_path_factory, "a")[2]
    lp = get_model_config("another-looped-stack", weights_path=ca).layer_loop
    assert (lp.start, lp.stop, lp.times) == (1, 3, 3)


def test_config_reader_rejects_bad_files():
    from kaito_amd.models.hybrid_config import lokedra_model_config
    cfg = config_a()
    cfg["loop"]["stop"] = 9                       # beyond the last layer
    with pytest.raises(ValueError):
        lokedra_model_config(cfg)
    cfg = config_a()
    cfg["layers"][0]["mixer"]["left"]["vdim"] = 4   # keys double as values
    with pytest.raises(ValueError):
        lokedra_model_config(cfg)
    cfg = config_a()
    cfg["layers"][1]["type"] = "delta"
    with pytest.raises(ValueError):
        lokedra_model_config(cfg)


@pytest.mark.parametrize("device", DEVICES)
def test_random_init_preset_generates(device):
    """The registered tiny preset with random weights through the normal
    engine entry point (no checkpoint): batched sampling requests."""
    import dataclasses
    from kaito_amd.engine import EngineConfig, LLMEngine, SamplingParams
    from kaito_amd.models import get_model_config
    from kaito_amd.parallel.state import init_parallel
    init_parallel(1)
    mc = get_model_config("tiny-lokedra-test")
    if device == "cpu":
        mc = dataclasses.replace(mc, dtype=torch.float32)
    eng = LLMEngine(EngineConfig(model=mc, device=device, max_num_seqs=4,
                                 max_model_len=256, num_gpu_blocks=64,
                                 enforce_eager=True))
    prompts = [list(range(3, 3 + n)) for n in (40, 7, 19, 64, 5)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=9, temperature=0.8,
                                                top_p=0.9, seed=1,
                                                ignore_eos=True))
    assert [len(o.output_token_ids) for o in outs] == [9] * 5
    assert eng.state_pool.num_free == 4
    assert eng.pool.num_free == eng.pool.num_blocks


def test_trace_replay_command_line(tmp_path_factory, tmp_path):
    """bin/trace_run as a user starts it: steps on standard input, logits
    files and `done` lines out (CPU reference ops, f32)."""
    import json
    import subprocess
    cfg, W, folder = checkpoint(tmp_path_factory, "b")
    a, b = tokens(cfg, 21, 31), tokens(cfg, 6, 32)
    steps = [
        {"step": 0, "entries": [{"id": "x", "tokens": a[:9], "want": [0, 8]}],
         "end": []},
        {"step": 1, "entries": [{"id": "x", "tokens": a[9:20], "want": []},
                                {"id": "y", "tokens": b[:5], "want": [4]}],
         "end": []},
        {"step": 2, "entries": [{"id": "y", "tokens": b[5:], "want": [0]},
                                {"id": "x", "tokens": a[20:], "want": [0]}],
         "end": ["x", "y"]},
    ]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    r = subprocess.run(
        [sys.executable, os.path.join(root, "bin", "trace_run"), "--model",
         folder, "--dtype", "float32", "--out", str(out), "--max-tokens",
         "128", "--device", "cpu"],
        input="".join(json.dumps(s) + "\n" for s in steps), text=True,
        capture_output=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.split("\n") if ln.startswith("done")] == \
        ["done 0", "done 1", "done 2"]
    wa, wb = L.model_logits(cfg, W, a), L.model_logits(cfg, W, b)
    V = cfg["vocab"]
    got = [torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4")
                            .reshape(-1, V)) for i in range(3)]
    mode = ("cpu", "float32")
    check(got[0], wa[[0, 8]], mode)
    check(got[1], wb[[4]], mode)
    check(got[2], torch.stack([wb[5], wa[20]]), mode)
