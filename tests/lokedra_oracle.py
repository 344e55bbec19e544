"""Plain restatement of the Lokedra design for tests: float64 numpy, token
loops, one function per mechanism, operating on checkpoint-named tensors.
Nothing here is shared with the package; it exists to be obviously right,
not fast.

Notation: h is a layer's normed input row, W[name] a checkpoint tensor
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


def silu(z):
    return z * sigmoid(z)


def softmax(z):
    e = np.exp(z - np.max(z, axis=-1, keepdims=True))
    return e / np.sum(e, axis=-1, keepdims=True)


# ---- token shift --------------------------------------------------------------

def token_shift(h, mu):
    """Row t becomes h_t + (h_{t-1} - h_t)·mu; the row before the first is
    zero."""
    prev = np.concatenate([np.zeros_like(h[:1]), h[:-1]], 0)
    return h + (prev - h) * mu


# ---- generalized delta rule -------------------------------------------------

def general_delta(h, W, pre, mx, eps):
    H, D = int(mx["heads"]), int(mx["dim"])
    T = h.shape[0]
    r = (h @ W[pre + "r"].T).reshape(T, H, D)
    k = (h @ W[pre + "k"].T).reshape(T, H, D)
    v = (h @ W[pre + "v"].T).reshape(T, H, D)
    low = np.tanh(h @ W[pre + "w1"].T) @ W[pre + "w2"].T + W[pre + "w0"]
    decay = np.exp(-math.exp(-0.5) * sigmoid(low)).reshape(T, H, D)
    rate = sigmoid(h @ W[pre + "a"].T + W[pre + "a.b"]).reshape(T, H, D)
    out = np.zeros((T, H, D))
    for n in range(H):
        S = np.zeros((D, D))                      # [key channel, value]
        for t in range(T):
            kt = k[t, n]
            u = kt / math.sqrt(float(kt @ kt) + 1e-6)
            S = decay[t, n][:, None] * S \
                - np.outer(rate[t, n] * u, u @ S) + np.outer(kt, v[t, n])
            out[t, n] = S.T @ r[t, n]
    out = rms(out, eps).reshape(T, H * D) * W[pre + "norm"]
    out = out * sigmoid(h @ W[pre + "g"].T)
    return out @ W[pre + "o"].T


# ---- rotation -----------------------------------------------------------------

def rotary_tables(rot, positions):
    """cos, sin [T, dims/2] of the interleaved rotation with the
    by-parts frequency interpolation."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def at(turns):
            return dims * math.log(orig / (2 * math.pi * turns)) \
                / (2 * math.log(base))
        lo = max(math.floor(at(float(sc["fast"]))), 0)
        hi = min(math.ceil(at(float(sc["slow"]))), dims - 1)
        ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001),
                       0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    ang = np.asarray(positions, dtype=np.float64)[:, None] * f[None, :]
    return np.cos(ang) * mag, np.sin(ang) * mag


def rotate_pairs(x, cos, sin, dims):
    """x [T, ..., n]: dimension 2i is paired with 2i+1 for 2i < dims."""
    out = x.copy()
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (dims // 2,)
    c, s = cos.reshape(shape), sin.reshape(shape)
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


# ---- latent attention ---------------------------------------------------------

def latent_attention(h, W, pre, mx, eps, positions=None):
    H, D, R, V, rank = (int(mx[k]) for k in
                        ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
    T = h.shape[0]
    positions = np.arange(T) if positions is None else positions
    cos, sin = rotary_tables(mx["rot"], positions)
    dims = int(mx["rot"]["dims"])
    cq = rms(h @ W[pre + "dq"].T, eps) * W[pre + "dq.norm"]
    q = (cq @ W[pre + "uq"].T).reshape(T, H, D + R)
    down = h @ W[pre + "dkv"].T
    c = rms(down[:, :rank], eps) * W[pre + "dkv.norm"]
    k_rot = rotate_pairs(down[:, rank:], cos, sin, dims)
    q_rot = rotate_pairs(q[..., D:], cos, sin, dims)
    keys = (c @ W[pre + "uk"].T).reshape(T, H, D)
    vals = (c @ W[pre + "uv"].T).reshape(T, H, V)
    out = np.zeros((T, H, V))
    for n in range(H):
        for t in range(T):
            s = (keys[:t + 1, n] @ q[t, n, :D] + k_rot[:t + 1] @ q_rot[t, n]) \
                * float(mx["scale"])
            out[t, n] = softmax(s) @ vals[:t + 1, n]
    return out.reshape(T, H * V) @ W[pre + "o"].T


# ---- chunked attention with convolved keys as values --------------------------

def short_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_{t - taps + 1 + j}."""
    taps = w.shape[1]
    pad = np.concatenate([np.zeros((taps - 1, u.shape[1])), u], 0)
    return sum(pad[j:j + u.shape[0]] * w[:, j] for j in range(taps))


def chunk_attention(h, W, pre, mx):
    H, G, D = int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"])
    T = h.shape[0]
    q = h @ W[pre + "q"].T + W[pre + "q.b"]
    k = h @ W[pre + "k"].T + W[pre + "k.b"]
    if mx.get("conv"):
        q = short_conv(q, W[pre + "q.conv"])
        k = short_conv(k, W[pre + "k.conv"])
    q, k = q.reshape(T, H, D), k.reshape(T, G, D)
    size = int(mx["mask"]["size"]) if mx.get("mask") else 0
    out = np.zeros((T, H, D))
    for n in range(H):
        g = n // (H // G)
        for t in range(T):
            first = (t // size) * size if size else 0
            s = k[first:t + 1, g] @ q[t, n] * float(mx["scale"])
            e = np.exp(s)
            out[t, n] = (e / (1.0 + e.sum())) @ k[first:t + 1, g]
    return out.reshape(T, H * D) @ W[pre + "o"].T + W[pre + "o.b"]


# ---- gated linear attention with a tied write gate ----------------------------

def hgrn2(h, W, pre, mx, eps):
    H, D, V = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"])
    T = h.shape[0]
    q = silu(h @ W[pre + "q"].T).reshape(T, H, D)
    v = (h @ W[pre + "v"].T).reshape(T, H, V)
    low = W[pre + "lower"]
    f = (low + (1.0 - low) * sigmoid(h @ W[pre + "f"].T + W[pre + "f.b"])) \
        .reshape(T, H, D)
    out = np.zeros((T, H, V))
    for n in range(H):
        S = np.zeros((D, V))
        for t in range(T):
            S = f[t, n][:, None] * S + np.outer(1.0 - f[t, n], v[t, n])
            out[t, n] = S.T @ q[t, n]
    out = rms(out, eps) * W[pre + "norm"]
    return out.reshape(T, H * V) @ W[pre + "o"].T


def parallel_mixer(h, W, pre, mx, eps):
    return float(mx["left_scale"]) * chunk_attention(h, W, pre + "left.",
                                                     mx["left"]) \
        + float(mx["right_scale"]) * hgrn2(h, W, pre + "right.", mx["right"],
                                           eps)


# ---- feed-forward ---------------------------------------------------------------

def clamped_expert(h, W, pre, limit):
    g = np.minimum(h @ W[pre + "gate"].T, limit)
    u = np.clip(h @ W[pre + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ W[pre + "down"].T


def route(z, correction, top):
    """Softmax scores; the choice adds the correction, the weights do
    not. Returns [(expert, weight)]."""
    s = softmax(z)
    order = np.argsort(-(s + correction), kind="stable")[:top]
    return [(int(e), float(s[e])) for e in order]


def moe_ff(h, W, pre, mlp):
    top = int(mlp["router"]["top"])
    limit = float(mlp["expert"]["limit"])
    out = np.zeros((h.shape[0], W[pre + "e0.down"].shape[0]))
    z = h @ W[pre + "router"].T
    for t in range(h.shape[0]):
        for e, w in route(z[t], W[pre + "correction"], top):
            out[t] += w * clamped_expert(h[t:t + 1], W, f"{pre}e{e}.",
                                         limit)[0]
    return out


# ---- the stack ------------------------------------------------------------------

def layer_runs(cfg):
    """Layer indices in execution order, with True where the embedding
    output is added first (the opening of the second and later passes)."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, False) for i in range(n)]
    a, b, times = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    runs = [(i, False) for i in range(a)]
    for p in range(times):
        runs += [(i, p > 0 and i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg, W, tokens, streams=None):
    eps = float(cfg["norm"]["eps"])
    x0 = W["embed"][np.asarray(tokens)] * float(cfg["embedding"]["scale"])
    x = x0.copy()
    for i, add_input in layer_runs(cfg):
        layer, pre = cfg["layers"][i], f"l{i}."
        if add_input:
            x = x + x0
        h = rms(x, eps) * (1.0 + W[pre + "norm1"])
        hs = token_shift(h, W[pre + "shift"])
        kind, mx = layer["type"], layer["mixer"]
        if kind == "general_delta":
            y = general_delta(hs, W, pre + "mix.", mx, eps)
        elif kind == "latent_attention":
            y = latent_attention(hs, W, pre + "mix.", mx, eps)
        elif kind == "parallel":
            y = parallel_mixer(hs, W, pre + "mix.", mx, eps)
        else:
            raise ValueError(kind)
        y = y * W[pre + "ls1"]
        if layer.get("mlp"):
            y = y + moe_ff(h, W, pre + "mlp.", layer["mlp"]) * W[pre + "ls2"]
        x = x + y
        if streams is not None:
            streams.append(x.copy())
    x = rms(x, eps) * (1.0 + W["final.norm"])
    return x @ W["embed"].T


# ---- configurations and random checkpoints -----------------------------------

def delta_layer(heads, dim, mlp=None):
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim},
            "mlp": mlp}


def latent_layer(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale=None,
                 base=10000.0, scaling=None, mlp=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = scaling
    return {"type": "latent_attention", "mixer": {
        "heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
        "kv_rank": kv_rank, "q_rank": q_rank, "rot": rot,
        "scale": scale if scale is not None else (dim + rot_dim) ** -0.5},
        "mlp": mlp}


def parallel_layer(heads, kv_heads, dim, chunk, taps, r_heads, r_dim, r_vdim,
                   scales=(1.0, 1.0), scale=None, mlp=None):
    return {"type": "parallel", "mixer": {
        "left": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                 "vdim": dim, "conv": taps, "mask": {"size": chunk},
                 "scale": scale if scale is not None else dim ** -0.5},
        "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim},
        "left_scale": scales[0], "right_scale": scales[1]}, "mlp": mlp}


def moe(experts, top, ff, limit=1.0):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "top": top}}


def make_config(layers, width, vocab, eps=1e-5, embed_scale=1.0, loop=None):
    cfg = {"architecture": "Lokedra", "embedding": {"scale": embed_scale},
           "layers": layers, "norm": {"eps": eps}, "vocab": vocab,
           "width": width}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def _bf16_round(a):
    """Values a bfloat16 checkpoint can hold, as float64."""
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

    def vec(name, n, lo, hi):
        W[name] = _bf16_round(rng.uniform(lo, hi, n))

    W["embed"] = _bf16_round(rng.normal(0, 0.5, (vocab, width)))
    vec("final.norm", width, -0.2, 0.2)
    for i, layer in enumerate(cfg["layers"]):
        pre, mp, mx = f"l{i}.", f"l{i}.mix.", layer["mixer"]
        vec(pre + "norm1", width, -0.2, 0.2)
        vec(pre + "shift", width, 0.0, 1.0)
        vec(pre + "ls1", width, 0.3, 1.0)
        vec(pre + "ls2", width, 0.3, 1.0)
        kind = layer["type"]
        if kind == "general_delta":
            n = int(mx["heads"]) * int(mx["dim"])
            low = max(4, n // 6)
            for t in ("r", "k", "v", "g"):
                lin(mp + t, n, width, 2.0)
            lin(mp + "a", n, width, 2.0)
            W[mp + "a.b"] = _bf16_round(rng.normal(0, 1.0, n))
            lin(mp + "w1", low, width, 2.0)
            lin(mp + "w2", n, low, 2.0)
            W[mp + "w0"] = _bf16_round(rng.normal(-1.0, 2.0, n))
            vec(mp + "norm", n, 0.8, 1.2)
            lin(mp + "o", width, n)
        elif kind == "latent_attention":
            H, D, R, V, r, qr = (int(mx[k]) for k in (
                "heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"))
            lin(mp + "dq", qr, width, 2.0)
            vec(mp + "dq.norm", qr, 0.8, 1.2)
            lin(mp + "uq", H * (D + R), qr, 2.0)
            lin(mp + "dkv", r + R, width, 2.0)
            vec(mp + "dkv.norm", r, 0.8, 1.2)
            lin(mp + "uk", H * D, r, 2.0)
            lin(mp + "uv", H * V, r)
            lin(mp + "o", width, H * V)
        elif kind == "parallel":
            lf, rt = mx["left"], mx["right"]
            H, G, D = int(lf["heads"]), int(lf["kv_heads"]), int(lf["dim"])
            lp, rp = mp + "left.", mp + "right."
            lin(lp + "q", H * D, width, 2.0)
            lin(lp + "k", G * D, width, 2.0)
            W[lp + "q.b"] = _bf16_round(rng.normal(0, 0.3, H * D))
            W[lp + "k.b"] = _bf16_round(rng.normal(0, 0.3, G * D))
            if lf.get("conv"):
                taps = int(lf["conv"])
                W[lp + "q.conv"] = _bf16_round(
                    rng.normal(0, 0.6, (H * D, taps)))
                W[lp + "k.conv"] = _bf16_round(
                    rng.normal(0, 0.6, (G * D, taps)))
            lin(lp + "o", width, H * D)
            W[lp + "o.b"] = _bf16_round(rng.normal(0, 0.3, width))
            Hr, Dr, Vr = int(rt["heads"]), int(rt["dim"]), int(rt["vdim"])
            lin(rp + "q", Hr * Dr, width, 2.0)
            lin(rp + "f", Hr * Dr, width, 2.0)
            W[rp + "f.b"] = _bf16_round(rng.normal(1.0, 1.5, Hr * Dr))
            vec(rp + "lower", Hr * Dr, 0.0, 0.9)
            lin(rp + "v", Hr * Vr, width, 2.0)
            vec(rp + "norm", Vr, 0.8, 1.2)
            lin(rp + "o", width, Hr * Vr)
        else:
            raise ValueError(kind)
        mlp = layer.get("mlp")
        if not mlp:
            continue
        fp = pre + "mlp."
        ff, E = int(mlp["expert"]["ff"]), int(mlp["router"]["experts"])
        for e in range(E):
            lin(f"{fp}e{e}.gate", ff, width, 1.5)
            lin(f"{fp}e{e}.up", ff, width, 1.5)
            lin(f"{fp}e{e}.down", width, ff)
        lin(fp + "router", E, width, 3.0)
        W[fp + "correction"] = _bf16_round(rng.normal(0, 0.1, E))
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
    receives the residual stream after every layer run."""
    import torch
    raw = [] if streams is not None else None
    out = torch.from_numpy(forward(cfg, W, list(tokens), raw))
    if streams is not None:
        streams.extend(torch.from_numpy(x) for x in raw)
    return out
