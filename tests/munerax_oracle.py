"""Plain restatement of the Munerax design for tests: float64 numpy, token
loops, one function per mechanism, operating on checkpoint-named tensors.
Nothing here is shared with the package; it exists to be obviously right,
not fast.

Notation: h is a sub-layer's input row, W[name] a checkpoint tensor
(linear maps stored [out, in]), rms(v) = v / sqrt(mean(v^2) + eps).
"""
from __future__ import annotations

import json
import math
import os

import numpy as np


def rms(v, eps):
    return v / np.sqrt(np.mean(v * v, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi)
                                    * (z + 0.044715 * z ** 3)))


# ---- input ------------------------------------------------------------------

def bigram_rows(tokens, bg):
    """Row of the bigram table per token: a hash of (previous, current);
    the first token of a sequence takes the extra last row."""
    buckets = int(bg["buckets"])
    rows = []
    for t, tok in enumerate(tokens):
        if t == 0:
            rows.append(buckets)
        else:
            rows.append((int(tokens[t - 1]) * int(bg["mul_prev"])
                         + int(tok) * int(bg["mul_cur"])) % buckets)
    return rows


def embed(cfg, W, tokens):
    e = cfg["embedding"]
    x = W["embed"][np.asarray(tokens)] * float(e["scale"])
    if e.get("bigram"):
        x = x + W["bigram"][np.asarray(bigram_rows(tokens, e["bigram"]))]
    return x


# ---- rotation ---------------------------------------------------------------

def rotate_half(x, positions, base, dims):
    """x [T, ..., n]: the first `dims` of the last axis rotate, i paired
    with i + dims/2, angle = position * base^(-2i/dims)."""
    half = dims // 2
    out = x.copy()
    for t, p in enumerate(positions):
        for i in range(half):
            a = p * base ** (-2.0 * i / dims)
            u, v = x[t, ..., i].copy(), x[t, ..., i + half].copy()
            out[t, ..., i] = u * math.cos(a) - v * math.sin(a)
            out[t, ..., i + half] = v * math.cos(a) + u * math.sin(a)
    return out


# ---- latent attention ---------------------------------------------------------

def latent_kv(h, W, pre, mx, eps):
    """What a layer with its own down-projection caches per token: the
    normed latent c [T, kv_rank] and the rotated shared key part
    [T, rot_dim]."""
    T = h.shape[0]
    r, rd = int(mx["kv_rank"]), int(mx["rot_dim"])
    d = h @ W[pre + "dkv"].T
    c = rms(d[:, :r], eps) * W[pre + "dkv.norm"]
    kr = rotate_half(d[:, r:r + rd], range(T), float(mx["rot"]["base"]),
                     int(mx["rot"]["dims"]))
    return c, kr


def latent_attention(h, W, pre, mx, eps, kv):
    """h [T, width] (positions 0..T-1); kv = (c, k_rot) of this layer or
    of the layer it borrows from."""
    T = h.shape[0]
    H, D, rd, V = (int(mx[k]) for k in ("heads", "dim", "rot_dim", "vdim"))
    r = int(mx["kv_rank"])
    c, kr = kv
    q = (h @ W[pre + "q"].T).reshape(T, H, D + rd)
    q_plain = q[:, :, :D]
    q_rot = rotate_half(q[:, :, D:], range(T), float(mx["rot"]["base"]),
                        int(mx["rot"]["dims"]))
    k_plain = (c @ W[pre + "uk"].T).reshape(T, H, D)
    v = (c @ W[pre + "uv"].T).reshape(T, H, V)
    gate = sigmoid(h @ W[pre + "g"].T)                  # [T, H]
    sink = W[pre + "sink"]
    out = np.zeros((T, H, V))
    for i in range(T):
        for hh in range(H):
            # keys 0..i: unrotated part per head, rotated part shared
            s = (k_plain[:i + 1, hh] @ q_plain[i, hh]
                 + kr[:i + 1] @ q_rot[i, hh]) * float(mx["scale"])
            m = max(s.max(), sink[hh])
            e = np.exp(s - m)
            den = e.sum() + math.exp(sink[hh] - m)
            out[i, hh] = (e / den) @ v[:i + 1, hh]
            out[i, hh] *= gate[i, hh]
    return out.reshape(T, H * V) @ W[pre + "o"].T


# ---- feed-forward -------------------------------------------------------------

def dense_ff(h, W, pre):
    g = gelu_tanh(h @ W[pre + "gate"].T)
    return (g * (h @ W[pre + "up"].T)) @ W[pre + "down"].T


def squared_relu_expert(h, W, pre):
    a = np.maximum(h @ W[pre + "up"].T, 0.0) ** 2
    return a @ W[pre + "down"].T


def route(z, router):
    """z [experts] logits of one token -> (chosen experts, weights)."""
    n, top = int(router["experts"]), int(router["top"])
    s = sigmoid(z)
    allowed = np.ones(n, dtype=bool)
    groups = router.get("groups")
    if groups:
        cnt, keep = int(groups["count"]), int(groups["keep"])
        size = n // cnt
        gs = []
        for g in range(cnt):
            part = np.sort(s[g * size:(g + 1) * size])[::-1]
            gs.append(part[:2].sum())
        best = np.argsort(-np.asarray(gs), kind="stable")[:keep]
        allowed[:] = False
        for g in best:
            allowed[g * size:(g + 1) * size] = True
    masked = np.where(allowed, s, -np.inf)
    chosen = np.argsort(-masked, kind="stable")[:top]
    return chosen, s[chosen] * float(router["scale"])


def moe_ff(h, W, pre, mlp):
    out = np.zeros((h.shape[0], W[pre + "e0.down"].shape[0]))
    z = h @ W[pre + "router"].T
    for t in range(h.shape[0]):
        chosen, w = route(z[t], mlp["router"])
        for e, we in zip(chosen, w):
            out[t] += we * squared_relu_expert(h[t:t + 1], W,
                                               f"{pre}e{e}.")[0]
    if mlp.get("shared"):
        out += squared_relu_expert(h, W, pre + "shared.")
    return out


def feed_forward(h, W, pre, mlp):
    if mlp["kind"] == "dense":
        return dense_ff(h, W, pre)
    return moe_ff(h, W, pre, mlp)


# ---- whole model --------------------------------------------------------------

def forward(cfg, W, tokens, streams=None):
    """tokens of ONE sequence → logits [T, vocab]."""
    eps = float(cfg["norm"]["eps"])
    x = embed(cfg, W, tokens)
    kv = {}
    for i, layer in enumerate(cfg["layers"]):
        pre, mx = f"l{i}.", layer["mixer"]
        assert layer["type"] == "latent_attention"
        h = rms(x, eps) * W[pre + "norm1"]
        src = mx.get("kv_from")
        if src is None:
            kv[i] = latent_kv(h, W, pre + "mix.", mx, eps)
            src = i
        x = x + latent_attention(h, W, pre + "mix.", mx, eps, kv[int(src)])
        if layer.get("mlp"):
            h = rms(x, eps) * W[pre + "norm2"]
            x = x + feed_forward(h, W, pre + "mlp.", layer["mlp"])
        if streams is not None:
            streams.append(x.copy())
    return (rms(x, eps) * W["final.norm"]) @ W["embed"].T


# ---- builders for tests -------------------------------------------------------

def latent_layer(heads, dim, rot_dim, vdim, kv_rank, scale=None,
                 base=10000.0, kv_from=None, mlp=None):
    mx = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
          "kv_rank": kv_rank, "rot": {"base": base, "dims": rot_dim},
          "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if kv_from is not None:
        mx["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mx, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, scale=1.0, groups=None, shared_ff=None):
    router = {"experts": experts, "top": top, "scale": scale}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    m = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared_ff:
        m["shared"] = {"ff": shared_ff}
    return m


def make_config(layers, width, vocab, eps=1e-5, embed_scale=1.0,
                bigram=(61, 7, 13)):
    e = {"scale": embed_scale}
    if bigram:
        e["bigram"] = {"buckets": bigram[0], "mul_prev": bigram[1],
                       "mul_cur": bigram[2]}
    return {"architecture": "Munerax", "embedding": e, "layers": layers,
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


def _bf16_round(a):
    """Round float64 values to bfloat16-representable ones (checkpoints
    hold bfloat16)."""
    import torch
    return torch.from_numpy(np.asarray(a, dtype=np.float32)).to(
        torch.bfloat16).float().numpy().astype(np.float64)


def random_weights(cfg, seed=0):
    rng = np.random.default_rng(seed)
    width, vocab = int(cfg["width"]), int(cfg["vocab"])
    W = {}

    def lin(name, out, inp, gain=1.0):
        W[name] = _bf16_round(rng.normal(0, gain / math.sqrt(inp),
                                         (out, inp)))

    def vec(name, n, lo=0.8, hi=1.2):
        W[name] = _bf16_round(rng.uniform(lo, hi, n))

    W["embed"] = _bf16_round(rng.normal(0, 0.5, (vocab, width)))
    bg = cfg["embedding"].get("bigram")
    if bg:
        W["bigram"] = _bf16_round(
            rng.normal(0, 0.5, (int(bg["buckets"]) + 1, width)))
    vec("final.norm", width)
    for i, layer in enumerate(cfg["layers"]):
        pre, mx = f"l{i}.", layer["mixer"]
        H, D, rd, V, r = (int(mx[k]) for k in
                          ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
        vec(pre + "norm1", width)
        lin(pre + "mix.q", H * (D + rd), width, 2.0)
        if mx.get("kv_from") is None:
            lin(pre + "mix.dkv", r + rd, width, 2.0)
            vec(pre + "mix.dkv.norm", r)
        lin(pre + "mix.uk", H * D, r, 2.0)
        lin(pre + "mix.uv", H * V, r)
        W[pre + "mix.sink"] = _bf16_round(rng.normal(0, 1.0, H))
        lin(pre + "mix.g", H, width, 2.0)
        lin(pre + "mix.o", width, H * V)
        mlp = layer.get("mlp")
        if not mlp:
            continue
        vec(pre + "norm2", width)
        fp = pre + "mlp."
        if mlp["kind"] == "dense":
            ff = int(mlp["ff"])
            lin(fp + "gate", ff, width)
            lin(fp + "up", ff, width)
            lin(fp + "down", width, ff)
        else:
            ff = int(mlp["expert"]["ff"])
            for e in range(int(mlp["router"]["experts"])):
                lin(f"{fp}e{e}.up", ff, width, 1.5)
                lin(f"{fp}e{e}.down", width, ff)
            lin(fp + "router", int(mlp["router"]["experts"]), width, 3.0)
            if mlp.get("shared"):
                sf = int(mlp["shared"]["ff"])
                lin(fp + "shared.up", sf, width, 1.5)
                lin(fp + "shared.down", width, sf)
    return W


def write_checkpoint(folder, cfg, W):
    """config.json + model.safetensors (bfloat16) as a served folder."""
    import torch
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: torch.from_numpy(np.asarray(v, dtype=np.float32)).to(
        torch.bfloat16).contiguous() for k, v in W.items()},
        os.path.join(folder, "model.safetensors"))
    return folder


def model_logits(cfg, W, tokens, streams=None):
    """Logits [T, vocab] as a float64 torch tensor; `streams`, if a list,
    receives the residual stream after every layer."""
    import torch
    raw = [] if streams is not None else None
    out = torch.from_numpy(forward(cfg, W, list(tokens), raw))
    if streams is not None:
        streams.extend(torch.from_numpy(x) for x in raw)
    return out
