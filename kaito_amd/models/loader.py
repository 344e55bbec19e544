"""Weight loading: HF-layout safetensors → our module tree.

Handles the fused projections (q/k/v → qkv_proj, gate/up → gate_up_proj)
and TP sharding. Random-init path lives on the model (bench contract:
no network, synthetic weights).
"""
from __future__ import annotations

from pathlib import Path
from typing import Dict

import torch

from ..parallel.state import get_state


def _shard(t: torch.Tensor, dim: int) -> torch.Tensor:
    st = get_state()
    if st.tp_size == 1:
        return t
    n = t.size(dim) // st.tp_size
    return t.narrow(dim, st.tp_rank * n, n).contiguous()


def load_safetensors_weights(model, path: str,
                             skip_projections: bool = False) -> None:
    if getattr(model.cfg, "arch", "llama") == "gurapel":
        return load_gurapel_weights(model, path)
    if getattr(model.cfg, "arch", "llama") == "pokulorn":
        return load_pokulorn_weights(model, path)
    if getattr(model.cfg, "arch", "llama") == "munerax":
        return load_munerax_weights(model, path)
    if getattr(model.cfg, "arch", "llama") == "lokedra":
        return load_lokedra_weights(model, path)
    from safetensors.torch import safe_open

    cfg = model.cfg
    files = sorted(Path(path).glob("*.safetensors"))
    if not files:
        raise FileNotFoundError(f"no safetensors under {path}")
    tensors: Dict[str, torch.Tensor] = {}
    for f in files:
        with safe_open(str(f), framework="pt", device="cpu") as sf:
            for k in sf.keys():
                tensors[k] = sf.get_tensor(k)

    def get(name):
        for prefix in ("model.", ""):
            if prefix + name in tensors:
                return tensors[prefix + name]
        raise KeyError(name)

    params = dict(model.named_parameters())

    def setp(name, value):
        with torch.no_grad():
            params[name].copy_(value.to(params[name].dtype))

    def has(name):
        return any(p + name in tensors for p in ("model.", ""))

    # norm weights: gemma stores w with y = x*(1+w); we fold to (1+w) at
    # load so the RMSNorm kernel is unchanged (cfg.rms_norm_offset)
    def norm_w(name):
        t = get(name)
        return t.float() + 1.0 if cfg.rms_norm_offset else t

    # head-dim padding (phi-2: checkpoint heads are 80-dim, the engine
    # runs the D∈{64,128,256} kernels on zero-padded 128-dim heads —
    # exact numerics, cfg.attn_scale keeps the 80^-0.5 scaling)
    def pad_heads(t, n_heads):
        d_ckpt = t.shape[0] // n_heads
        if d_ckpt == cfg.head_dim:
            return t
        x = t.reshape(n_heads, d_ckpt, -1)
        pad = torch.zeros(n_heads, cfg.head_dim - d_ckpt, x.shape[-1],
                          dtype=t.dtype)
        return torch.cat([x, pad], dim=1).reshape(n_heads * cfg.head_dim, -1)

    def pad_heads_cols(t, n_heads):
        d_ckpt = t.shape[1] // n_heads
        if d_ckpt == cfg.head_dim:
            return t
        x = t.reshape(t.shape[0], n_heads, d_ckpt)
        pad = torch.zeros(t.shape[0], n_heads, cfg.head_dim - d_ckpt,
                          dtype=t.dtype)
        return torch.cat([x, pad], dim=2).reshape(t.shape[0], -1)

    setp("embed_tokens.weight", _shard(get("embed_tokens.weight"), 0))
    # final norm (phi-2 checkpoints call it final_layernorm, with bias)
    final = "final_layernorm" if has("final_layernorm.weight") else "norm"
    setp("norm", norm_w(final + ".weight"))
    if getattr(model, "norm_bias", None) is not None and             has(final + ".bias"):
        setp("norm_bias", get(final + ".bias"))
    if model.lm_head is not None:
        setp("lm_head.weight", _shard(get("lm_head.weight"), 0))

    def attn_name(base, i):
        # phi-2 calls o_proj `dense`
        pre = f"layers.{i}.self_attn."
        if base == "o_proj" and not has(pre + "o_proj.weight") and                 has(pre + "dense.weight"):
            return pre + "dense"
        return pre + base

    # deepseek stores rope dims INTERLEAVED (HF apply_rotary permutes
    # inside the model); our rotate-half kernel wants the half-split
    # layout, so permute those output ROWS once at load — exact
    def deinterleave_pe(t, n_heads=1):
        d = t.shape[0] // n_heads
        x = t.reshape(n_heads, d // 2, 2, -1)
        return torch.cat([x[:, :, 0], x[:, :, 1]],
                         dim=1).reshape(t.shape[0], -1)

    def load_mla_attn(pre):
        a = pre + "self_attn."
        nope, rope, r = (cfg.qk_nope_head_dim, cfg.qk_rope_head_dim,
                         cfg.kv_lora_rank)
        if cfg.q_lora_rank > 0:
            setp(a + "q_a_proj", get(a + "q_a_proj.weight"))
            setp(a + "q_a_layernorm", get(a + "q_a_layernorm.weight"))
            qb = get(a + "q_b_proj.weight")
        else:
            qb = get(a + "q_proj.weight")
        # per-head [nope | rope] rows; de-interleave the rope part
        qb = qb.reshape(cfg.num_heads, nope + rope, -1)
        qb = torch.cat([qb[:, :nope],
                        deinterleave_pe(
                            qb[:, nope:].reshape(-1, qb.shape[-1]),
                            cfg.num_heads).reshape(cfg.num_heads, rope, -1)],
                       dim=1).reshape(cfg.num_heads * (nope + rope), -1)
        tgt = "q_b_proj" if cfg.q_lora_rank > 0 else "q_proj"
        setp(a + tgt + ".weight", _shard(qb, 0))
        kva = get(a + "kv_a_proj_with_mqa.weight")
        kva = torch.cat([kva[:r], deinterleave_pe(kva[r:])], 0)
        setp(a + "kv_a_proj_with_mqa", kva)
        setp(a + "kv_a_layernorm", get(a + "kv_a_layernorm.weight"))
        kvb = get(a + "kv_b_proj.weight").reshape(
            cfg.num_heads, nope + cfg.v_head_dim, r)
        setp(a + "w_kc", _shard(kvb[:, :nope], 0))
        setp(a + "w_vc", _shard(kvb[:, nope:].transpose(1, 2), 0))
        setp(a + "o_proj.weight", _shard(get(a + "o_proj.weight"), 1))

    # deepseek MoE: mlp.gate (+ e_score_correction_bias), per-expert
    # gate/up/down, optional shared_experts
    def load_deepseek_moe(pre, i):
        setp(pre + "mlp.gate", get(pre + "mlp.gate.weight"))
        if has(pre + "mlp.gate.e_score_correction_bias"):
            setp(pre + "mlp.e_score_correction_bias",
                 get(pre + "mlp.gate.e_score_correction_bias"))
        moe = params[pre + "mlp.w_gate_up"]
        e_base = getattr(model.layers[i].mlp, "e_base", 0)
        with torch.no_grad():
            for le in range(moe.shape[0]):
                ex = f"{pre}mlp.experts.{e_base + le}."
                params[pre + "mlp.w_gate_up"][le].copy_(torch.cat(
                    [get(ex + "gate_proj.weight"),
                     get(ex + "up_proj.weight")], 0).to(moe.dtype))
                params[pre + "mlp.w_down"][le].copy_(
                    get(ex + "down_proj.weight").to(moe.dtype))
        if cfg.n_shared_experts > 0:
            sh = pre + "mlp.shared_experts."
            setp(pre + "mlp.w_shared_gate_up", _shard(torch.cat(
                [get(sh + "gate_proj.weight"),
                 get(sh + "up_proj.weight")], 0), 0))
            setp(pre + "mlp.w_shared_down",
                 _shard(get(sh + "down_proj.weight"), 1))

    for i in range(cfg.num_layers):
        pre = f"layers.{i}."
        if cfg.is_mla and not skip_projections:
            load_mla_attn(pre)
            if i < cfg.first_k_dense or cfg.num_experts == 0:
                g = _shard(get(pre + "mlp.gate_proj.weight"), 0)
                u = _shard(get(pre + "mlp.up_proj.weight"), 0)
                setp(pre + "mlp.gate_up_proj.weight", torch.cat([g, u], 0))
                setp(pre + "mlp.down_proj.weight",
                     _shard(get(pre + "mlp.down_proj.weight"), 1))
            else:
                load_deepseek_moe(pre, i)
            setp(pre + "input_layernorm",
                 norm_w(pre + "input_layernorm.weight"))
            setp(pre + "post_attention_layernorm",
                 norm_w(pre + "post_attention_layernorm.weight"))
            continue
        if not skip_projections:   # AWQ checkpoints carry qweight instead
            q = pad_heads(get(attn_name("q_proj", i) + ".weight"),
                          cfg.num_heads)
            k = pad_heads(get(attn_name("k_proj", i) + ".weight"),
                          cfg.num_kv_heads)
            v = pad_heads(get(attn_name("v_proj", i) + ".weight"),
                          cfg.num_kv_heads)
            setp(pre + "self_attn.qkv_proj.weight", torch.cat(
                [_shard(q, 0), _shard(k, 0), _shard(v, 0)], 0))
            if cfg.attention_bias and has(attn_name("q_proj", i) + ".bias"):
                qb = pad_heads(get(attn_name("q_proj", i) + ".bias")
                               .unsqueeze(-1), cfg.num_heads).squeeze(-1)
                kb = pad_heads(get(attn_name("k_proj", i) + ".bias")
                               .unsqueeze(-1), cfg.num_kv_heads).squeeze(-1)
                vb = pad_heads(get(attn_name("v_proj", i) + ".bias")
                               .unsqueeze(-1), cfg.num_kv_heads).squeeze(-1)
                setp(pre + "self_attn.qkv_proj.bias", torch.cat(
                    [_shard(qb, 0), _shard(kb, 0), _shard(vb, 0)], 0))
            o = pad_heads_cols(get(attn_name("o_proj", i) + ".weight"),
                               cfg.num_heads)
            setp(pre + "self_attn.o_proj.weight", _shard(o, 1))
            if cfg.gated_mlp:
                g = _shard(get(pre + "mlp.gate_proj.weight"), 0)
                u = _shard(get(pre + "mlp.up_proj.weight"), 0)
                setp(pre + "mlp.gate_up_proj.weight", torch.cat([g, u], 0))
                setp(pre + "mlp.down_proj.weight",
                     _shard(get(pre + "mlp.down_proj.weight"), 1))
            else:   # phi-2/falcon ungated fc1/fc2
                fc1 = "mlp.fc1" if has(pre + "mlp.fc1.weight") else                     "mlp.up_proj"
                fc2 = "mlp.fc2" if has(pre + "mlp.fc2.weight") else                     "mlp.down_proj"
                setp(pre + "mlp.up_proj.weight",
                     _shard(get(pre + fc1 + ".weight"), 0))
                setp(pre + "mlp.down_proj.weight",
                     _shard(get(pre + fc2 + ".weight"), 1))
                if cfg.attention_bias and has(pre + fc1 + ".bias"):
                    setp(pre + "mlp.up_proj.bias",
                         _shard(get(pre + fc1 + ".bias"), 0))
                    setp(pre + "mlp.down_proj.bias",
                         get(pre + fc2 + ".bias"))
        if cfg.qk_norm:
            setp(pre + "self_attn.q_norm",
                 norm_w(pre + "self_attn.q_norm.weight"))
            setp(pre + "self_attn.k_norm",
                 norm_w(pre + "self_attn.k_norm.weight"))
        setp(pre + "input_layernorm", norm_w(pre + "input_layernorm.weight"))
        if cfg.norm_type == "layernorm" and                 has(pre + "input_layernorm.bias"):
            setp(pre + "input_layernorm_bias",
                 get(pre + "input_layernorm.bias"))
        if not cfg.parallel_block:
            setp(pre + "post_attention_layernorm",
                 norm_w(pre + "post_attention_layernorm.weight"))
        if cfg.sandwich_norms:
            setp(pre + "pre_feedforward_layernorm",
                 norm_w(pre + "pre_feedforward_layernorm.weight"))
            setp(pre + "post_feedforward_layernorm",
                 norm_w(pre + "post_feedforward_layernorm.weight"))
        # Mixtral-style MoE experts: block_sparse_moe.experts.N.w1/w3/w2
        if cfg.num_experts > 0 and                 has(pre + "block_sparse_moe.gate.weight"):
            setp(pre + "mlp.gate", get(pre + "block_sparse_moe.gate.weight"))
            moe = params[pre + "mlp.w_gate_up"]
            e_base = getattr(model.layers[i].mlp, "e_base", 0)
            for le in range(moe.shape[0]):
                ex = f"{pre}block_sparse_moe.experts.{e_base + le}."
                w1 = get(ex + "w1.weight")   # gate
                w3 = get(ex + "w3.weight")   # up
                with torch.no_grad():
                    params[pre + "mlp.w_gate_up"][le].copy_(
                        torch.cat([w1, w3], 0).to(moe.dtype))
                    params[pre + "mlp.w_down"][le].copy_(
                        get(ex + "w2.weight").to(moe.dtype))


# ---- hybrid stacks ------------------------------------------------------

class _FlatCheckpoint:
    """All tensors of a folder's safetensors files by name, with
    shape-checked copies into parameters and a record of what was read."""

    def __init__(self, path: str):
        from safetensors.torch import safe_open
        self.tensors: Dict[str, torch.Tensor] = {}
        for f in sorted(Path(path).glob("*.safetensors")):
            with safe_open(str(f), framework="pt", device="cpu") as sf:
                for k in sf.keys():
                    self.tensors[k] = sf.get_tensor(k)
        if not self.tensors:
            raise FileNotFoundError(f"no safetensors under {path}")
        self.used = set()

    def get(self, name):
        self.used.add(name)
        return self.tensors[name]

    @staticmethod
    def put(param, value):
        if tuple(param.shape) != tuple(value.shape):
            raise ValueError(f"shape mismatch: parameter {tuple(param.shape)}"
                             f" vs checkpoint {tuple(value.shape)}")
        with torch.no_grad():
            param.copy_(value.to(param.dtype))

    def warn_unused(self):
        extra = set(self.tensors) - self.used
        if extra:
            import logging
            logging.getLogger(__name__).warning(
                "checkpoint tensors not used by the model: %s",
                sorted(extra)[:8])


def load_gurapel_weights(model, path: str) -> None:
    """Gurapel checkpoint (flat tensor names, `l<i>.` per layer, linear
    weights [out, in]) → GurapelForCausalLM. Fuses the per-mixer input
    projections, folds the one-plus norm weights and the recurrence's
    decay constant, and widens every small per-channel tensor to f32."""
    ck = _FlatCheckpoint(path)
    get, put = ck.get, ck.put

    def one_plus(name):
        return get(name).float() + 1.0

    put(model.embed_tokens.weight, get("embed"))
    put(model.pos_embed, get("pos"))
    put(model.norm, one_plus("final.norm"))
    put(model.lm_head, get("head"))
    for i, layer in enumerate(model.layers):
        pre = f"l{i}."
        spec = layer.spec
        put(layer.norm1, one_plus(pre + "norm1"))
        if spec.kind == "delta":
            m, mp = layer.mixer, pre + "mix."
            put(m.in_proj, torch.cat(
                [get(mp + n) for n in ("q", "k", "v", "g", "a", "b")], 0))
            put(m.conv_weight, torch.cat(
                [get(mp + n + ".conv") for n in ("q", "k", "v")], 0).float())
            put(m.a_log, get(mp + "A_log").float())
            put(m.dt_bias, get(mp + "dt_bias").float())
            put(m.out_norm, get(mp + "norm").float())
            put(m.o_proj, get(mp + "o"))
        else:
            a, ap = layer.attn, pre + "mix.left."
            put(a.qkv_proj, torch.cat(
                [get(ap + n) for n in ("q", "k", "v")], 0))
            put(a.q_norm, get(ap + "q.norm").float())
            put(a.k_norm, get(ap + "k.norm").float())
            put(a.r1, get(ap + "r1").float())
            put(a.r2, get(ap + "r2").float())
            put(a.o_proj, get(ap + "o"))
            r, rp = layer.rglru, pre + "mix.right."
            put(r.in_proj, torch.cat([get(rp + "y"), get(rp + "x")], 0))
            put(r.in_bias, torch.cat([get(rp + "y.b"), get(rp + "x.b")], 0))
            put(r.conv_weight, get(rp + "conv").float())
            put(r.conv_bias, get(rp + "conv.b").float())
            # [blocks, out, in] ×2 → [blocks, in, 2·out]
            put(r.gate_w, torch.cat(
                [get(rp + "ra").float().transpose(1, 2),
                 get(rp + "ri").float().transpose(1, 2)], 2))
            put(r.gate_b, torch.cat(
                [get(rp + "ra.b").float(), get(rp + "ri.b").float()],
                1).unsqueeze(1))
            put(r.decay_rate, r.spec.decay_scale *
                torch.nn.functional.softplus(get(rp + "lam").float()))
            put(r.o_proj, get(rp + "o"))
            put(layer.attn_out_norm, get(pre + "mix.left.out").float())
            put(layer.rglru_out_norm, get(pre + "mix.right.out").float())
        if layer.mlp is not None:
            mlp, fp = layer.mlp, pre + "mlp."
            put(layer.norm2, one_plus(pre + "norm2"))
            put(mlp.gate, get(fp + "router").float())
            ie = mlp.ie_local
            with torch.no_grad():
                mlp.w_gate_up.zero_()
                mlp.w_down.zero_()
                for e in range(mlp.num_experts):
                    g, u, d = (get(f"{fp}e{e}.{n}")
                               for n in ("gate", "up", "down"))
                    ff = g.shape[0]
                    mlp.w_gate_up[e, :ff].copy_(g.to(mlp.w_gate_up.dtype))
                    mlp.w_gate_up[e, ie:ie + ff].copy_(
                        u.to(mlp.w_gate_up.dtype))
                    mlp.w_down[e, :, :ff].copy_(d.to(mlp.w_down.dtype))
    ck.warn_unused()


def load_pokulorn_weights(model, path: str) -> None:
    """Pokulorn checkpoint (flat tensor names, `l<i>.` per layer, mixer
    tensors under `.mix.`, feed-forward under `.mlp.`, linear weights
    [out, in]) → PokulornForCausalLM. Fuses each mixer's input
    projections, splits off the small projections that feed recurrences
    (kept f32) and widens every per-channel tensor to f32."""
    ck = _FlatCheckpoint(path)
    get, put = ck.get, ck.put

    def load_attention(a, ap, first_mixer):
        s = a.spec
        names = ("q", "k", "v") + (("g",) if s.gate else ())
        put(a.qkv_proj, torch.cat([get(ap + n) for n in names], 0))
        if s.conv_taps > 0:
            put(a.conv_weight, torch.cat(
                [get(ap + n + ".conv") for n in ("q", "k", "v")], 0).float())
        if s.qk_norm:
            put(a.q_norm, get(ap + "q.norm").float())
            put(a.k_norm, get(ap + "k.norm").float())
        if s.sink:
            put(a.sinks, get(ap + "sink").float())
        if s.mix_values:
            lam = float(get(ap + "vmix").float())
            a.v_lambda = 0.0 if first_mixer else lam
        put(a.o_proj, get(ap + "o"))

    put(model.embed_tokens.weight, get("embed"))
    put(model.norm, get("final.norm").float())
    put(model.lm_head, get("head"))
    seen_mixing = False
    for i, layer in enumerate(model.layers):
        pre = f"l{i}."
        spec = layer.spec
        put(layer.norm1, get(pre + "norm1").float())
        if spec.kind == "mlstm":
            m, mp = layer.mixer, pre + "mix."
            put(m.in_proj, torch.cat(
                [get(mp + n) for n in ("q", "k", "v", "g")], 0))
            put(m.gate_proj, torch.cat(
                [get(mp + "i"), get(mp + "f")], 0).float())
            put(m.gate_bias, torch.cat(
                [get(mp + "i.b"), get(mp + "f.b")], 0).float())
            put(m.out_norm, get(mp + "norm").float())
            put(m.o_proj, get(mp + "o"))
        elif spec.kind == "attention":
            load_attention(layer.attn, pre + "mix.", not seen_mixing)
            seen_mixing = seen_mixing or spec.rattn.mix_values
        else:
            load_attention(layer.attn, pre + "mix.left.", not seen_mixing)
            seen_mixing = seen_mixing or spec.rattn.mix_values
            r, rp = layer.ssd, pre + "mix.right."
            w_in = get(rp + "in")
            main = r.inner + r.conv_ch          # rows [z | x | B | C], then dt
            put(r.in_proj, w_in[:main])
            put(r.dt_proj, w_in[main:].float())
            put(r.conv_weight, get(rp + "conv").float())
            put(r.conv_bias, get(rp + "conv.b").float())
            put(r.a_log, get(rp + "A_log").float())
            put(r.dt_bias, get(rp + "dt_bias").float())
            put(r.d_skip, get(rp + "D").float())
            put(r.out_norm, get(rp + "norm").float())
            put(r.o_proj, get(rp + "o"))
        if layer.mlp is not None:
            fp = pre + "mlp."
            put(layer.norm2, get(pre + "norm2").float())
            put(layer.mlp.gate_up, torch.cat(
                [get(fp + "gate"), get(fp + "up")], 0))
            put(layer.mlp.down, get(fp + "down"))
    ck.warn_unused()


def load_munerax_weights(model, path: str) -> None:
    """Munerax checkpoint (flat tensor names, `l<i>.` per layer, mixer
    tensors under `.mix.`, feed-forward under `.mlp.`, linear weights
    [out, in]) → MuneraxForCausalLM. Fuses each mixer's input projections
    (query, gate, latent down-projection), stacks the experts (zero-filled
    up to the kernels' tile width) and widens per-channel tensors to f32."""
    ck = _FlatCheckpoint(path)
    get, put = ck.get, ck.put
    put(model.embed_tokens.weight, get("embed"))
    if model.bigram is not None:
        put(model.bigram, get("bigram"))
    put(model.norm, get("final.norm").float())
    for i, layer in enumerate(model.layers):
        pre = f"l{i}."
        a, ap = layer.attn, pre + "mix."
        s = a.spec
        put(layer.norm1, get(pre + "norm1").float())
        names = ("q",) + (("g",) if s.gate else ()) \
            + (("dkv",) if a.own_kv else ())
        w_in = torch.cat([get(ap + n) for n in names], 0)
        if w_in.shape[0] != a.in_rows:
            raise ValueError(f"{ap}: projection rows {w_in.shape[0]} vs "
                             f"{a.in_rows} from the config")
        put(a.in_proj, torch.nn.functional.pad(
            w_in, (0, 0, 0, a.in_proj.shape[0] - a.in_rows)))
        if a.own_kv:
            put(a.kv_norm, get(ap + "dkv.norm").float())
        put(a.w_uk, get(ap + "uk"))
        put(a.w_uv, get(ap + "uv"))
        if s.sink:
            put(a.sinks, get(ap + "sink").float())
        put(a.o_proj, get(ap + "o"))
        if layer.mlp is None:
            continue
        fp = pre + "mlp."
        put(layer.norm2, get(pre + "norm2").float())
        if layer.spec.glu is not None:
            put(layer.mlp.gate_up, torch.cat(
                [get(fp + "gate"), get(fp + "up")], 0))
            put(layer.mlp.down, get(fp + "down"))
            continue
        mlp = layer.mlp
        put(mlp.gate, get(fp + "router").float())
        with torch.no_grad():
            mlp.w_gate_up.zero_()
            mlp.w_down.zero_()
            for e in range(mlp.num_experts):
                u, d = get(f"{fp}e{e}.up"), get(f"{fp}e{e}.down")
                ff = u.shape[0]
                mlp.w_gate_up[e, :ff].copy_(u.to(mlp.w_gate_up.dtype))
                mlp.w_down[e, :, :ff].copy_(d.to(mlp.w_down.dtype))
        if mlp.w_shared_gate_up is not None:
            put(mlp.w_shared_gate_up, get(fp + "shared.up"))
            put(mlp.w_shared_down, get(fp + "shared.down"))
    ck.warn_unused()


def load_lokedra_weights(model, path: str) -> None:
    """Lokedra checkpoint (flat tensor names, `l<i>.` per layer, mixer
    tensors under `.mix.`, feed-forward under `.mlp.`, linear weights
    [out, in]) → LokedraForCausalLM. Fuses each mixer's input
    projections, folds the one-plus norm weights and the branch weights
    into the layer scales, sizes the decay bottleneck by the checkpoint's
    tensors, stacks the experts (zero-filled up to the kernels' tile
    width) and widens per-channel tensors to f32."""
    ck = _FlatCheckpoint(path)
    get, put = ck.get, ck.put
    cat = torch.cat

    def one_plus(name):
        return get(name).float() + 1.0

    put(model.embed_tokens.weight, get("embed"))
    put(model.norm, one_plus("final.norm"))
    for i, layer in enumerate(model.layers):
        pre, mp = f"l{i}.", f"l{i}.mix."
        spec = layer.spec
        put(layer.norm1, one_plus(pre + "norm1"))
        put(layer.shift, get(pre + "shift").float())
        ls1 = get(pre + "ls1").float()
        if spec.kind == "general_delta":
            m = layer.mixer
            put(layer.scale_mix, ls1)
            put(m.in_proj, cat([get(mp + n) for n in "rkvg"], 0))
            w1 = get(mp + "w1")
            if w1.shape[0] != m.decay_rank:
                m.set_decay_rank(int(w1.shape[0]))
            put(m.gate_proj, cat([get(mp + "a"), w1], 0))
            put(m.a_bias, get(mp + "a.b").float())
            put(m.w2, get(mp + "w2").float())
            put(m.w0, get(mp + "w0").float())
            put(m.out_norm, get(mp + "norm").float())
            put(m.o_proj, get(mp + "o"))
        elif spec.kind == "latent_attention":
            a = layer.mixer
            put(layer.scale_mix, ls1)
            w_in = cat([get(mp + "dq"), get(mp + "dkv")], 0)
            if w_in.shape[0] != a.in_rows:
                raise ValueError(f"{mp}: projection rows {w_in.shape[0]} vs "
                                 f"{a.in_rows} from the config")
            put(a.in_proj, torch.nn.functional.pad(
                w_in, (0, 0, 0, a.in_proj.shape[0] - a.in_rows)))
            put(a.q_norm, get(mp + "dq.norm").float())
            put(a.w_uq, get(mp + "uq"))
            put(a.kv_norm, get(mp + "dkv.norm").float())
            put(a.w_uk, get(mp + "uk"))
            put(a.w_uv, get(mp + "uv"))
            put(a.o_proj, get(mp + "o"))
        else:
            a, r = layer.attn, layer.hgrn
            lp, rp = mp + "left.", mp + "right."
            left, right = spec.branch_scales
            put(layer.scale_mix, ls1 * left)
            put(layer.scale_mix2, ls1 * right)
            put(a.qkv_proj, cat([get(lp + "q"), get(lp + "k")], 0))
            put(a.qkv_bias, cat([get(lp + "q.b"), get(lp + "k.b")], 0))
            if a.conv_weight is not None:
                put(a.conv_weight, cat([get(lp + "q.conv"),
                                        get(lp + "k.conv")], 0).float())
            put(a.o_proj, get(lp + "o"))
            put(a.o_bias, get(lp + "o.b"))
            put(r.in_proj, cat([get(rp + "q"), get(rp + "v")], 0))
            put(r.f_proj, get(rp + "f"))
            put(r.f_bias, get(rp + "f.b").float())
            put(r.lower, get(rp + "lower").float())
            put(r.out_norm, get(rp + "norm").float())
            put(r.o_proj, get(rp + "o"))
        mlp = layer.mlp
        if mlp is None:
            continue
        fp = pre + "mlp."
        put(layer.scale_ff, get(pre + "ls2").float())
        put(mlp.gate, get(fp + "router").float())
        put(mlp.e_score_correction_bias, get(fp + "correction").float())
        ie = mlp.ie_local
        with torch.no_grad():
            mlp.w_gate_up.zero_()
            mlp.w_down.zero_()
            for e in range(mlp.num_experts):
                g, u, d = (get(f"{fp}e{e}.{n}") for n in ("gate", "up",
                                                          "down"))
                ff = g.shape[0]
                dt = mlp.w_gate_up.dtype
                mlp.w_gate_up[e, :ff].copy_(g.to(dt))
                mlp.w_gate_up[e, ie:ie + ff].copy_(u.to(dt))
                mlp.w_down[e, :, :ff].copy_(d.to(dt))
    ck.warn_unused()
