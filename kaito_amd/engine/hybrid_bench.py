"""Prefill and decode throughput of the hybrid stacks (Gurapel, Pokulorn,
Munerax, Lokedra) beside each other and beside the engine's closest homogeneous
model at equal size: a sliding-window GQA transformer with the same MoE
feed-forward (the gpt-oss class without sinks) for the recurrent hybrids,
the latent-attention MoE transformer (deepseek class) for Munerax. Random
weights, synthetic tokens; all models run through the same LLMEngine
(scheduler, paged cache, hipGraph decode).

Used by `bench.py --hybrid-compare`; prints one JSON line per
(size, model).
"""
from __future__ import annotations

import json
import time
from typing import Dict, List

import torch

# layers of a size: the hybrid pattern is delta, parallel, parallel
SIZES: Dict[str, dict] = {
    "w1024": dict(width=1024, layers=6, heads=8, kv_heads=2, dim=128,
                  window=512, experts=8, top=2, ff=1024, vocab=32000,
                  lru_blocks=8),
    "w2048": dict(width=2048, layers=6, heads=16, kv_heads=4, dim=128,
                  window=1024, experts=8, top=2, ff=2048, vocab=32000,
                  lru_blocks=16),
    "w4096": dict(width=4096, layers=6, heads=32, kv_heads=8, dim=128,
                  window=1024, experts=8, top=2, ff=4096, vocab=32000,
                  lru_blocks=16),
}


def hybrid_config(name: str, z: dict, max_pos: int):
    from ..models.hybrid_config import gurapel_model_config
    moe = {"kind": "moe", "expert": {"ff": z["ff"]},
           "router": {"experts": z["experts"], "top": z["top"]}}
    delta = {"type": "delta", "mlp": moe, "mixer": {
        "heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"],
        "vdim": z["dim"], "conv": 4}}
    par = {"type": "parallel", "mlp": moe, "mixer": {
        "left": {"heads": z["heads"], "kv_heads": z["kv_heads"],
                 "dim": z["dim"], "vdim": z["dim"],
                 "mask": {"size": z["window"]}, "scale": z["dim"] ** -0.5,
                 "softcap": 30.0},
        "right": {"width": z["width"], "blocks": z["lru_blocks"],
                  "conv": 4}}}
    layers = [(delta if i % 3 == 0 else par) for i in range(z["layers"])]
    return gurapel_model_config({
        "architecture": "Gurapel", "embedding": {"scale": 1.0},
        "layers": layers, "max_positions": max_pos, "norm": {"eps": 1e-5},
        "vocab": z["vocab"], "width": z["width"]}, name=f"gurapel-{name}")


def pokulorn_config(name: str, z: dict, max_pos: int):
    """The pre-norm hybrid at the sizes of `z`: layers cycle matrix
    memory, windowed attention, attention beside a state-space mixer. The
    recurrent states match the Gurapel stack's (one dim x dim matrix per
    head); the dense feed-forward is as wide as the MoE's active experts
    together."""
    from ..models.hybrid_config import pokulorn_model_config
    ff = {"kind": "dense", "ff": z["ff"] * z["top"], "limit": 7.0}
    rot = {"base": 10000.0, "dims": z["dim"] // 2,
           "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0,
                       "slow": 1.0}}
    mem = {"type": "mlstm", "mlp": ff, "mixer": {
        "heads": z["heads"], "dim": z["dim"], "vdim": z["dim"],
        "gate_cap": 15.0}}
    att = {"type": "attention", "mlp": ff, "mixer": {
        "heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"],
        "vdim": z["dim"], "conv": 4, "rot": rot, "scale": z["dim"] ** -0.5,
        "mask": {"size": z["window"], "keep_first": 64}, "v_mix": True}}
    par = {"type": "parallel", "mlp": ff, "mixer": {
        "left": {"heads": z["heads"], "kv_heads": z["kv_heads"],
                 "dim": z["dim"], "vdim": z["dim"], "conv": 4, "rot": rot,
                 "scale": z["dim"] ** -0.5,
                 "mask": {"size": z["window"], "keep_first": 0}},
        "right": {"heads": z["width"] // 64, "vdim": 64, "state": 128,
                  "groups": z["kv_heads"], "norm_groups": z["kv_heads"],
                  "conv": 4},
        "left_scale": 0.5, "right_scale": 0.5}}
    layers = [(mem, att, par)[i % 3] for i in range(z["layers"])]
    return pokulorn_model_config({
        "architecture": "Pokulorn", "layers": layers,
        "max_positions": max_pos, "norm": {"eps": 1e-5},
        "vocab": z["vocab"], "width": z["width"]}, name=f"pokulorn-{name}")


def transformer_config(name: str, z: dict, max_pos: int):
    from .config import ModelConfig
    return ModelConfig(
        name=f"swa-moe-{name}", hidden_size=z["width"],
        num_layers=z["layers"], num_heads=z["heads"],
        num_kv_heads=z["kv_heads"], head_dim=z["dim"],
        intermediate_size=z["ff"], vocab_size=z["vocab"],
        max_position=max_pos, num_experts=z["experts"],
        num_experts_per_tok=z["top"], moe_intermediate_size=z["ff"],
        moe_routing="topk_softmax", sliding_window=z["window"],
        sliding_window_pattern="all")


# latent attention at the sizes of `z`: the head layout of the public
# deepseek-v2-lite class (128 unrotated + 64 rotated key dims, 128 value
# dims, latent rank 512), four expert groups of which two are eligible,
# one shared expert as wide as a routed one
LATENT = dict(dim=128, rot_dim=64, vdim=128, kv_rank=512, groups=4, keep=2,
              scale=1.0)


def munerax_config(name: str, z: dict, max_pos: int):
    """The latent-attention stack: a dense first layer, then routed
    layers, every third of which reads the latents of the layer before
    it."""
    from ..models.hybrid_config import munerax_model_config
    a = LATENT
    moe = {"kind": "moe", "expert": {"ff": z["ff"]},
           "router": {"experts": z["experts"], "top": z["top"],
                      "scale": a["scale"],
                      "groups": {"count": a["groups"], "keep": a["keep"]}},
           "shared": {"ff": z["ff"]}}

    def layer(i):
        mx = {"heads": z["heads"], "dim": a["dim"], "rot_dim": a["rot_dim"],
              "vdim": a["vdim"], "kv_rank": a["kv_rank"],
              "rot": {"base": 10000.0, "dims": a["rot_dim"]},
              "scale": (a["dim"] + a["rot_dim"]) ** -0.5}
        if i % 3 == 2:
            mx["kv_from"] = i - 1
        return {"type": "latent_attention", "mixer": mx,
                "mlp": {"kind": "dense", "ff": z["ff"] * (z["top"] + 1)}
                if i == 0 else moe}
    return munerax_model_config({
        "architecture": "Munerax",
        "embedding": {"scale": 1.0, "bigram": {
            "buckets": 65521, "mul_prev": 31, "mul_cur": 17}},
        "layers": [layer(i) for i in range(z["layers"])],
        "max_positions": max_pos, "norm": {"eps": 1e-5},
        "vocab": z["vocab"], "width": z["width"]}, name=f"munerax-{name}")


def lokedra_config(name: str, z: dict, max_pos: int):
    """The looped parallel-layer stack at the sizes of `z`: three layers
    (generalized delta rule, latent attention with low-rank queries,
    chunked attention beside HGRN2) run twice, so as many layer runs as
    the other stacks have layers. Recurrent states match the Gurapel
    stack's (one dim x dim matrix per head), the latent layer has the
    Munerax head layout, the chunk is the other stacks' window, the
    experts are the same count and width."""
    from ..models.hybrid_config import lokedra_model_config
    a = LATENT
    moe = {"kind": "moe", "expert": {"ff": z["ff"], "limit": 7.0},
           "router": {"experts": z["experts"], "top": z["top"]}}
    layers = [
        {"type": "general_delta", "mlp": moe,
         "mixer": {"heads": z["heads"], "dim": z["dim"]}},
        {"type": "latent_attention", "mlp": moe, "mixer": {
            "heads": z["heads"], "dim": a["dim"], "rot_dim": a["rot_dim"],
            "vdim": a["vdim"], "kv_rank": a["kv_rank"],
            "q_rank": 3 * a["kv_rank"] // 2,
            "scale": (a["dim"] + a["rot_dim"]) ** -0.5,
            "rot": {"base": 10000.0, "dims": a["rot_dim"], "scaling": {
                "factor": 4.0, "original": 4096, "fast": 32.0,
                "slow": 1.0}}}},
        {"type": "parallel", "mlp": moe, "mixer": {
            "left": {"heads": z["heads"], "kv_heads": z["kv_heads"],
                     "dim": z["dim"], "vdim": z["dim"], "conv": 4,
                     "mask": {"size": z["window"]},
                     "scale": z["dim"] ** -0.5},
            "right": {"heads": z["heads"], "dim": z["dim"],
                      "vdim": z["dim"]},
            "left_scale": 0.5, "right_scale": 0.5}},
    ]
    return lokedra_model_config({
        "architecture": "Lokedra", "embedding": {"scale": 1.0},
        "layers": layers,
        "loop": {"start": 0, "stop": 3, "times": z["layers"] // 3},
        "max_positions": max_pos, "norm": {"eps": 1e-5},
        "vocab": z["vocab"], "width": z["width"]}, name=f"lokedra-{name}")


def latent_transformer_config(name: str, z: dict, max_pos: int):
    """The engine's latent-attention MoE transformer (deepseek class) with
    the same head layout, latent rank, experts, groups and shared
    expert."""
    from .config import ModelConfig
    a = LATENT
    return ModelConfig(
        name=f"mla-moe-{name}", hidden_size=z["width"],
        num_layers=z["layers"], num_heads=z["heads"],
        num_kv_heads=z["heads"], head_dim=a["dim"] + a["rot_dim"],
        intermediate_size=z["ff"] * (z["top"] + 1), vocab_size=z["vocab"],
        max_position=max_pos, kv_lora_rank=a["kv_rank"], q_lora_rank=0,
        qk_nope_head_dim=a["dim"], qk_rope_head_dim=a["rot_dim"],
        v_head_dim=a["vdim"], num_experts=z["experts"],
        num_experts_per_tok=z["top"], moe_intermediate_size=z["ff"],
        moe_routing="noaux_tc", moe_norm_topk=False,
        routed_scaling_factor=a["scale"], n_group=a["groups"],
        topk_group=a["keep"], n_shared_experts=1, first_k_dense=1)


def _measure(mcfg, batch: int, prompt: int, out_tokens: int, eager: bool):
    from .config import EngineConfig
    from .engine import LLMEngine
    from .sequence import SamplingParams
    cfg = EngineConfig(
        model=mcfg, device="cuda", max_num_seqs=batch,
        max_model_len=prompt + out_tokens + 16,
        max_num_batched_tokens=max(8192, prompt),
        enforce_eager=eager, enable_prefix_caching=False,
        graph_batch_sizes=(batch,), gpu_memory_utilization=0.5)
    eng = LLMEngine(cfg)
    if not eager:
        eng.capture_graphs()
    gen = torch.Generator().manual_seed(0)

    def prompts():
        return [torch.randint(10, mcfg.vocab_size - 10, (prompt,),
                              generator=gen).tolist() for _ in range(batch)]

    def one_round():
        sp = SamplingParams(max_tokens=out_tokens, ignore_eos=True)
        ids = [eng.add_request(p, sp) for p in prompts()]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while eng.scheduler.waiting or eng.scheduler.prefilling:
            eng.step()
        eng.flush()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        n0 = eng.num_generation_tokens
        while eng.has_unfinished():
            eng.step()
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        n1 = eng.num_generation_tokens
        for i in ids:
            eng.seqs.pop(i, None)
        return batch * prompt / (t1 - t0), (n1 - n0) / (t2 - t1)

    one_round()                              # warm-up (allocator, GEMM pick)
    pre, dec = zip(*(one_round() for _ in range(2)))
    del eng
    torch.cuda.empty_cache()
    return max(pre), max(dec)


def run(sizes: List[str], batch: int, prompt: int, out_tokens: int,
        eager: bool = False, models=("gurapel", "swa-moe")) -> List[dict]:
    from ..parallel import state as ps
    ps.init_parallel(1)
    results = []
    for name in sizes:
        z = SIZES[name]
        max_pos = prompt + out_tokens + 16
        for kind in models:
            mcfg = {"gurapel": hybrid_config, "pokulorn": pokulorn_config,
                    "swa-moe": transformer_config,
                    "munerax": munerax_config,
                    "lokedra": lokedra_config,
                    "mla-moe": latent_transformer_config}[kind](
                        name, z, max_pos)
            pre, dec = _measure(mcfg, batch, prompt, out_tokens, eager)
            row = {"bench": "hybrid-compare", "size": name, "model": kind,
                   "batch": batch, "prompt_tokens": prompt,
                   "out_tokens": out_tokens,
                   "prefill_tokens_per_s": round(pre, 1),
                   "decode_tokens_per_s": round(dec, 1),
                   "decode_graphs": not eager, "dtype": "bf16",
                   "data": "synthetic"}
            print(json.dumps(row), flush=True)
            results.append(row)
    return results
