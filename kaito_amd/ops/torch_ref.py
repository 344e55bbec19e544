"""Pure-PyTorch fp32 reference implementations of every HIP op.

Used (a) on CPU so the engine/scheduler stack is testable without a GPU and
(b) as the numerics oracle for the GPU kernels (tests compare HIP bf16
kernels against these fp32 references).
"""
from __future__ import annotations

import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    var = xf.pow(2).mean(-1, keepdim=True)
    out = xf * torch.rsqrt(var + eps) * weight.float()
    return out.to(x.dtype)


def fused_add_rms_norm(x: torch.Tensor, residual: torch.Tensor,
                       weight: torch.Tensor, eps: float):
    """Returns (normed, new_residual). Residual update happens in bf16 to
    match the kernel's residual-stream precision."""
    new_res = (x.float() + residual.float()).to(x.dtype)
    return rms_norm(new_res, weight, eps), new_res


def rotary_embedding(positions: torch.Tensor, q: torch.Tensor, k: torch.Tensor,
                     head_dim: int, cos_sin_cache: torch.Tensor):
    """Neox/llama rotate-half RoPE. q: [T, QH*D] or [T, QH, D]; in-place-like
    (returns rotated copies). cos_sin_cache: [max_pos, R] = [cos | sin]."""
    rot = cos_sin_cache.size(1)
    half = rot // 2
    cs = cos_sin_cache[positions]          # [T, R]
    cos = cs[:, :half].float()             # [T, half]
    sin = cs[:, half:].float()

    def _apply(t: torch.Tensor) -> torch.Tensor:
        shp = t.shape
        x = t.reshape(shp[0], -1, head_dim).float()
        x1 = x[..., :half]
        x2 = x[..., half:rot]
        c = cos.unsqueeze(1)
        s = sin.unsqueeze(1)
        o1 = x1 * c - x2 * s
        o2 = x2 * c + x1 * s
        out = torch.cat([o1, o2, x[..., rot:]], dim=-1)
        return out.reshape(shp).to(t.dtype)

    return _apply(q), _apply(k)


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    d = x.size(-1) // 2
    gate, up = x[..., :d].float(), x[..., d:].float()
    return (torch.nn.functional.silu(gate) * up).to(x.dtype)


def gelu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """GeGLU (gemma): gelu_tanh(gate) * up."""
    d = x.size(-1) // 2
    gate, up = x[..., :d].float(), x[..., d:].float()
    return (torch.nn.functional.gelu(gate, approximate="tanh") * up
            ).to(x.dtype)


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """Plain tanh-approx GELU (phi-2's ungated MLP activation)."""
    return torch.nn.functional.gelu(x.float(), approximate="tanh").to(x.dtype)


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias, eps: float
               ) -> torch.Tensor:
    """LayerNorm with optional bias (phi-2/falcon norm layers)."""
    xf = x.float()
    mu = xf.mean(-1, keepdim=True)
    var = (xf - mu).pow(2).mean(-1, keepdim=True)
    out = (xf - mu) * torch.rsqrt(var + eps) * weight.float()
    if bias is not None:
        out = out + bias.float()
    return out.to(x.dtype)


def reshape_and_cache(k: torch.Tensor, v: torch.Tensor, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, slot_mapping: torch.Tensor):
    """k/v: [T, KH, D]; caches: [B, KH, BS, D]."""
    bs = k_cache.size(2)
    mask = slot_mapping >= 0
    slots = slot_mapping[mask]
    blocks = torch.div(slots, bs, rounding_mode="floor")
    offs = slots % bs
    k_cache[blocks, :, offs] = k[mask].to(k_cache.dtype)
    v_cache[blocks, :, offs] = v[mask].to(v_cache.dtype)


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    block_tables: torch.Tensor, seq_lens: torch.Tensor,
                    scale: float, window: int = 0,
                    sinks=None) -> torch.Tensor:
    """q: [T, QH, D] (one token/seq). Returns [T, QH, D].
    window>0: sliding-window attention — only the last `window` tokens
    are attended. sinks: [QH] learned attention-sink logits (gpt-oss)
    folded into the softmax denominator."""
    T, QH, D = q.shape
    KH = k_cache.size(1)
    BS = k_cache.size(2)
    G = QH // KH
    out = torch.empty_like(q)
    for i in range(T):
        L = int(seq_lens[i])
        start = max(0, L - window) if window > 0 else 0
        nb = (L + BS - 1) // BS
        blocks = block_tables[i, :nb].long()
        keys = k_cache[blocks].permute(1, 0, 2, 3).reshape(KH, nb * BS, D)[:, start:L]
        vals = v_cache[blocks].permute(1, 0, 2, 3).reshape(KH, nb * BS, D)[:, start:L]
        qh = q[i].float()                                # [QH, D]
        kx = keys.float().repeat_interleave(G, dim=0)    # [QH, Lw, D]
        vx = vals.float().repeat_interleave(G, dim=0)
        s = torch.einsum("hd,hld->hl", qh, kx) * scale
        if sinks is not None:
            s = torch.cat([sinks.float().unsqueeze(1), s], dim=1)
            p = torch.softmax(s, dim=-1)[:, 1:]          # sink absorbs mass
        else:
            p = torch.softmax(s, dim=-1)
        out[i] = torch.einsum("hl,hld->hd", p, vx).to(q.dtype)
    return out


def prefill_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                      cu_seqlens: torch.Tensor, scale: float,
                      window: int = 0, sinks=None) -> torch.Tensor:
    """Varlen causal attention. q: [T, QH, D], k/v: [T, KH, D].
    window>0: sliding window (k in (qpos-window, qpos]); sinks: [QH]."""
    T, QH, D = q.shape
    KH = k.size(1)
    G = QH // KH
    out = torch.empty_like(q)
    cs = cu_seqlens.tolist()
    for b in range(len(cs) - 1):
        s0, s1 = cs[b], cs[b + 1]
        L = s1 - s0
        qs = q[s0:s1].float().transpose(0, 1)                      # [QH, L, D]
        ks = k[s0:s1].float().transpose(0, 1).repeat_interleave(G, 0)
        vs = v[s0:s1].float().transpose(0, 1).repeat_interleave(G, 0)
        att = torch.einsum("hqd,hkd->hqk", qs, ks) * scale
        qpos = torch.arange(L, device=q.device).unsqueeze(1)
        kpos = torch.arange(L, device=q.device).unsqueeze(0)
        mask = kpos > qpos
        if window > 0:
            mask = mask | (kpos <= qpos - window)
        att = att.masked_fill(mask.unsqueeze(0), float("-inf"))
        if sinks is not None:
            att = torch.cat([sinks.float()[:, None, None].expand(QH, L, 1),
                             att], dim=-1)
            p = torch.softmax(att, dim=-1)[..., 1:]
        else:
            p = torch.softmax(att, dim=-1)
        o = torch.einsum("hqk,hkd->hqd", p, vs)
        out[s0:s1] = o.transpose(0, 1).to(q.dtype)
    return out


def context_attention(q: torch.Tensor, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, cu_seqlens_q: torch.Tensor,
                      kv_lens: torch.Tensor, block_tables: torch.Tensor,
                      scale: float, window: int = 0,
                      sinks=None) -> torch.Tensor:
    """Suffix-query causal attention over the paged cache. q: [Tq, QH, D];
    cache holds each sequence's FULL kv_len tokens (suffix included)."""
    Tq, QH, D = q.shape
    KH = k_cache.size(1)
    BS = k_cache.size(2)
    G = QH // KH
    out = torch.empty_like(q)
    cs = cu_seqlens_q.tolist()
    for b in range(len(cs) - 1):
        s0, s1 = cs[b], cs[b + 1]
        q_len = s1 - s0
        L = int(kv_lens[b])
        nb = (L + BS - 1) // BS
        blocks = block_tables[b, :nb].long()
        keys = k_cache[blocks].permute(1, 0, 2, 3).reshape(KH, nb * BS, D)[:, :L]
        vals = v_cache[blocks].permute(1, 0, 2, 3).reshape(KH, nb * BS, D)[:, :L]
        qs = q[s0:s1].float().transpose(0, 1)                  # [QH, q_len, D]
        kx = keys.float().repeat_interleave(G, 0)
        vx = vals.float().repeat_interleave(G, 0)
        att = torch.einsum("hqd,hkd->hqk", qs, kx) * scale
        qpos = torch.arange(L - q_len, L, device=q.device).unsqueeze(1)
        kpos = torch.arange(L, device=q.device).unsqueeze(0)
        mask = kpos > qpos
        if window > 0:
            mask = mask | (kpos <= qpos - window)
        att = att.masked_fill(mask.unsqueeze(0), float("-inf"))
        if sinks is not None:
            att = torch.cat(
                [sinks.float()[:, None, None].expand(QH, q_len, 1), att],
                dim=-1)
            p = torch.softmax(att, dim=-1)[..., 1:]
        else:
            p = torch.softmax(att, dim=-1)
        o = torch.einsum("hqk,hkd->hqd", p, vx)
        out[s0:s1] = o.transpose(0, 1).to(q.dtype)
    return out


def w4a16_unpack(qweight: torch.Tensor, scales: torch.Tensor,
                 zeros: torch.Tensor, group: int) -> torch.Tensor:
    """Dequantize the native W4A16 layout (qweight u32 [N, K/8], 8
    consecutive K nibbles per word; w = s*q - z) to float [N, K]."""
    N, kw = qweight.shape
    K = kw * 8
    shifts = torch.arange(8, device=qweight.device, dtype=torch.long) * 4
    q = (qweight.unsqueeze(-1).long() >> shifts) & 0xF      # [N, K/8, 8]
    q = q.reshape(N, K).float()
    s = scales.repeat_interleave(group, dim=1).float()       # [N, K]
    z = zeros.repeat_interleave(group, dim=1).float()
    return s * q - z


def w4a16_gemv(x: torch.Tensor, qweight: torch.Tensor, scales: torch.Tensor,
               zeros: torch.Tensor, group: int) -> torch.Tensor:
    w = w4a16_unpack(qweight, scales, zeros, group)
    return (x.float() @ w.T).to(x.dtype)


def mla_decode(q: torch.Tensor, cache: torch.Tensor,
               block_tables: torch.Tensor, seq_lens: torch.Tensor,
               scale: float, r: int) -> torch.Tensor:
    """Absorbed MLA decode reference (fp32 math). q: [T, H, r+rope] latent
    queries; cache: [NB, BS, r+rope] (c_kv || k_rope per token). Scores are
    the full latent dot; output is the latent-space V accumulation
    (first r dims). Mirrors ops/csrc/mla_attention.hip."""
    T, H, DT = q.shape
    NB, BS, _ = cache.shape
    out = torch.empty(T, H, r, dtype=q.dtype, device=q.device)
    for i in range(T):
        L = int(seq_lens[i])
        nb = (L + BS - 1) // BS
        rows = cache[block_tables[i, :nb].long()].reshape(-1, DT)[:L].float()
        s = q[i].float() @ rows.t() * scale          # [H, L]
        p = torch.softmax(s, dim=-1)
        out[i] = (p @ rows[:, :r]).to(out.dtype)
    return out


# ---- sequence mixers with per-sequence state (hybrid stacks) -------------
#
# Shared batch layout: rows of all chunks are concatenated; chunk b owns
# rows cu[b]..cu[b+1], continues the sequence held in state slot slots[b]
# and starts at sequence position starts[b] (0 = fresh sequence: the state
# is taken as zero and the slot's old content is ignored). Slots < 0 mark
# padding chunks, which are skipped.

def _chunks(cu_seqlens, state_slots, seq_starts):
    cu = cu_seqlens.tolist()
    sl = state_slots.tolist()
    st = seq_starts.tolist()
    for b in range(len(sl)):
        if sl[b] >= 0 and cu[b + 1] > cu[b]:
            yield cu[b], cu[b + 1], sl[b], st[b]


def causal_conv_update(x, weight, bias, conv_state, cu_seqlens, state_slots,
                       seq_starts, act: int):
    """Depthwise causal convolution over time. x [T, C]; weight [C, taps]
    (last column multiplies the current token); conv_state
    [slots, taps-1, C] holds each sequence's last taps-1 inputs and is
    advanced in place. act: 0 none, 1 silu."""
    taps = weight.size(1)
    out = torch.empty_like(x)
    w = weight.float()
    for r0, r1, slot, start in _chunks(cu_seqlens, state_slots, seq_starts):
        prev = conv_state[slot, :taps - 1].float() if start > 0 else \
            torch.zeros(taps - 1, x.size(1))
        seq = torch.cat([prev, x[r0:r1].float()], 0)
        n = r1 - r0
        acc = torch.zeros(n, x.size(1))
        for j in range(taps):
            acc += seq[j:j + n] * w[:, j]
        if bias is not None:
            acc += bias.float()
        if act == 1:
            acc = torch.nn.functional.silu(acc)
        out[r0:r1] = acc.to(x.dtype)
        if taps > 1:
            conv_state[slot, :taps - 1] = seq[n:].to(conv_state.dtype)
    return out


def gated_delta_rule(q, k, v, gate, a, b, a_log, dt_bias, norm_w, state,
                     cu_seqlens, state_slots, seq_starts, qk_eps: float,
                     norm_eps: float):
    """q/k [T, G, D], v/gate [T, H, V], a/b [T, H]; state [slots, H, D, V]
    f32, advanced in place. Per token and head: decay the state, write the
    beta-scaled prediction error along k, read out along q; the read-out
    is RMS-normed, weighted and gated by silu(gate)."""
    T, G, D = q.shape
    H, V = v.shape[1], v.shape[2]
    rep = H // G
    qf, kf, vf = q.float(), k.float(), v.float()
    qf = qf * torch.rsqrt(qf.pow(2).sum(-1, keepdim=True) + qk_eps) * D ** -0.5
    kf = kf * torch.rsqrt(kf.pow(2).sum(-1, keepdim=True) + qk_eps)
    qf = qf.repeat_interleave(rep, 1)
    kf = kf.repeat_interleave(rep, 1)
    beta = torch.sigmoid(b.float())
    decay = torch.exp(-torch.exp(a_log.float()) *
                      torch.nn.functional.softplus(a.float() + dt_bias.float()))
    o = torch.zeros(T, H, V)
    for r0, r1, slot, start in _chunks(cu_seqlens, state_slots, seq_starts):
        S = state[slot].clone() if start > 0 else torch.zeros(H, D, V)
        for t in range(r0, r1):
            S = S * decay[t, :, None, None]
            pred = torch.einsum("hdv,hd->hv", S, kf[t])
            u = beta[t, :, None] * (vf[t] - pred)
            S = S + kf[t, :, :, None] * u[:, None, :]
            o[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        state[slot] = S
    o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + norm_eps)
    o = o * norm_w.float() * torch.nn.functional.silu(gate.float())
    return o.to(v.dtype)


def rglru_scan(u, gates, y, decay_rate, state, cu_seqlens, state_slots,
               seq_starts):
    """Real-gated linear recurrent unit. u, y [T, W]; gates [B, T, 2*bw]
    f32 pre-activations (recurrence gate | input gate per block of
    bw = W // B channels); decay_rate [W] f32 (already multiplied by the
    design's constant); state [slots, W] f32, advanced in place.
    out = S_t * gelu_tanh(y)."""
    T, W = u.shape
    B = gates.size(0)
    bw = W // B
    g = gates.float().permute(1, 0, 2)                   # [T, B, 2bw]
    r = torch.sigmoid(g[..., :bw]).reshape(T, W)
    i = torch.sigmoid(g[..., bw:]).reshape(T, W)
    log_a = -r * decay_rate.float()
    a = torch.exp(log_a)
    drive = torch.sqrt(1.0 - a * a) * i * u.float()
    out = torch.empty(T, W)
    for r0, r1, slot, start in _chunks(cu_seqlens, state_slots, seq_starts):
        S = state[slot].clone() if start > 0 else torch.zeros(W)
        for t in range(r0, r1):
            S = a[t] * S + drive[t]
            out[t] = S
        state[slot] = S
    return (out * gelu_tanh(y.float())).to(u.dtype)


def qk_norm_cache_write(q, k, v, q_w, k_w, eps: float, k_cache, v_cache,
                        slot_mapping, positions=None, inv_freq=None,
                        rot_mag: float = 1.0, v_first=None,
                        v_lambda: float = 0.0):
    """Per-head RMS norm of q [T, H, D] and k [T, G, D] (weights [D], or
    None for no norm), optional rotation of the first 2*len(inv_freq)
    dims of every head (dim i paired with i + len(inv_freq); angle =
    position * inv_freq[i]; cos and sin times rot_mag), optional blend
    v <- (1 - v_lambda) v + v_lambda v_first, then scatter k and v
    [T, G, V] into the paged caches [blocks, G, block_size, D|V].
    Returns the normed (rotated) q."""
    def norm(t, w):
        tf = t.float()
        if w is not None:
            tf = tf * torch.rsqrt(tf.pow(2).mean(-1, keepdim=True) + eps) \
                * w.float()
        return tf

    def rot(tf):
        if inv_freq is None or inv_freq.numel() == 0:
            return tf
        half = inv_freq.numel()
        ang = positions.float()[:, None] * inv_freq.float()[None, :]
        c = (torch.cos(ang) * rot_mag)[:, None, :]
        s = (torch.sin(ang) * rot_mag)[:, None, :]
        a, b = tf[..., :half], tf[..., half:2 * half]
        return torch.cat([a * c - b * s, b * c + a * s, tf[..., 2 * half:]],
                         -1)
    qn = rot(norm(q, q_w)).to(q.dtype)
    kn = rot(norm(k, k_w)).to(k.dtype)
    if v_first is not None:
        v = ((1.0 - v_lambda) * v.float() + v_lambda * v_first.float()) \
            .to(v.dtype)
    bs = k_cache.size(2)
    for t, slot in enumerate(slot_mapping.tolist()):
        if slot < 0:
            continue
        k_cache[slot // bs, :, slot % bs] = kn[t].to(k_cache.dtype)
        v_cache[slot // bs, :, slot % bs] = v[t].to(v_cache.dtype)
    return qn


def window_attention(q, k_cache, v_cache, block_tables, token_seq, positions,
                     scale: float, softcap: float, r1, r2, window: int,
                     keep_first: int = 0, sinks=None, chunk: int = 0):
    """Causal sliding-window attention of query rows over the paged cache.
    Row t belongs to chunk token_seq[t] (its block table row) at sequence
    position positions[t] and sees keys j <= pos with pos - j < window or
    j < keep_first (window <= 0: all earlier keys). score =
    cap(q.k * scale) - r1 * ln(1 + r2 * (pos - j)). With `sinks` [H] the
    softmax denominator also holds exp(sink_h). With `chunk` > 0 the mask
    is chunked instead: keys j <= pos in pos's block of `chunk` positions
    counted from 0."""
    T, H, D = q.shape
    G, bs, V = k_cache.size(1), k_cache.size(2), v_cache.size(3)
    rep = H // G
    out = torch.zeros(T, H, V)
    pos_l, seq_l = positions.tolist(), token_seq.tolist()
    for t in range(T):
        if seq_l[t] < 0:
            continue
        p = pos_l[t]
        lo = max(0, p - window + 1) if window > 0 else 0
        if chunk > 0:
            lo = p // chunk * chunk
        js = torch.cat([torch.arange(0, min(keep_first, lo)),
                        torch.arange(lo, p + 1)])
        blk = block_tables[seq_l[t]].long()[js // bs]
        kk = k_cache[blk, :, js % bs].float()            # [n, G, D]
        vv = v_cache[blk, :, js % bs].float()
        kk = kk.repeat_interleave(rep, 1)
        vv = vv.repeat_interleave(rep, 1)
        s = torch.einsum("hd,nhd->hn", q[t].float(), kk) * scale
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        if r1 is not None:
            dist = (p - js).float()
            s = s - r1.float()[:, None] * torch.log1p(
                r2.float()[:, None] * dist[None, :])
        if sinks is not None:
            s = torch.cat([s, sinks.float()[:, None]], 1)
            w = torch.softmax(s, -1)[:, :-1]
        else:
            w = torch.softmax(s, -1)
        out[t] = torch.einsum("hn,nhv->hv", w, vv)
    return out.to(q.dtype)


def post_norm_residual(x32, y, w, eps: float, out_dtype, y2=None, w_y=None,
                       w_y2=None):
    """Residual update with the norm on the sub-layer OUTPUT:
    x32 += rms(m) * w, in place, where m = y, or with y2 given
    m = (rms(y) * w_y + rms(y2) * w_y2) / 2. Returns x32 rounded to
    out_dtype (the next sub-layer's input)."""
    def rms(t):
        return t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps)
    m = y.float()
    if y2 is not None:
        m = 0.5 * (rms(m) * w_y.float() + rms(y2.float()) * w_y2.float())
    x32 += rms(m) * w.float()
    return x32.to(out_dtype)


def rms_norm_cast(x, weight, eps: float, out_dtype):
    """RMS norm of rows of any float dtype with an f32 weight, rounded to
    out_dtype."""
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
            * weight.float()).to(out_dtype)


def mlstm_scan(q, k, v, ogate, ipre, fpre, norm_w, state_c, state_n, state_m,
               cu_seqlens, state_slots, seq_starts, cap: float,
               q_scale: float, norm_eps: float, denom_floor: float):
    """Matrix-memory recurrence. q/k [T, H, D], v/ogate [T, H, V], ipre /
    fpre [T, H] f32 gate pre-activations; states C [slots, H, D, V],
    n [slots, H, D], m [slots, H] f32, advanced in place. Log gates
    i = cap*tanh(ipre/cap), f = logsigmoid(cap*tanh(fpre/cap)); running
    maximum m (0 at the start of a sequence):
        m' = max(f + m, i);  C' = e^(f+m-m') C + e^(i-m') k v^T  (n alike)
        o  = C'^T q / (max(|n'.q|, e^(-m')) + denom_floor)
    The read-out is RMS-normed per head, weighted, times sigmoid(ogate)."""
    T, H, D = q.shape
    V = v.shape[2]
    qf, kf, vf = q.float() * q_scale, k.float(), v.float()
    gi = cap * torch.tanh(ipre.float() / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh(fpre.float() / cap))
    o = torch.zeros(T, H, V)
    for r0, r1, slot, start in _chunks(cu_seqlens, state_slots, seq_starts):
        if start > 0:
            C, n, m = (state_c[slot].clone(), state_n[slot].clone(),
                       state_m[slot].clone())
        else:
            C, n, m = torch.zeros(H, D, V), torch.zeros(H, D), torch.zeros(H)
        for t in range(r0, r1):
            m_new = torch.maximum(gf[t] + m, gi[t])
            keep = torch.exp(gf[t] + m - m_new)
            take = torch.exp(gi[t] - m_new)
            C = keep[:, None, None] * C + take[:, None, None] * (
                kf[t, :, :, None] * vf[t, :, None, :])
            n = keep[:, None] * n + take[:, None] * kf[t]
            m = m_new
            den = torch.maximum((n * qf[t]).sum(-1).abs(), torch.exp(-m)) \
                + denom_floor
            o[t] = torch.einsum("hdv,hd->hv", C, qf[t]) / den[:, None]
        state_c[slot], state_n[slot], state_m[slot] = C, n, m
    o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + norm_eps)
    o = o.reshape(T, H * V) * norm_w.float() \
        * torch.sigmoid(ogate.float().reshape(T, H * V))
    return o.to(v.dtype)


def ssd_scan(x, B, C, dt, z, a_log, dt_bias, d_skip, norm_w, state,
             cu_seqlens, state_slots, seq_starts, norm_groups: int,
             norm_eps: float):
    """Selective state space with scalar decay. x [T, H, P], B/C
    [T, G, N], dt [T, H] f32 (before bias and softplus), z [T, H*P];
    state [slots, H, N, P] f32 in place. Per head (group h // (H/G)):
        d = softplus(dt + dt_bias);  S' = e^(-e^(a_log) d) S + d B x^T
        y = S'^T C + d_skip x
    then y * silu(z), RMS norm in norm_groups equal parts, times norm_w."""
    T, H, P = x.shape
    G, N = B.shape[1], B.shape[2]
    rep = H // G
    xf = x.float()
    Bf = B.float().repeat_interleave(rep, 1)
    Cf = C.float().repeat_interleave(rep, 1)
    d = torch.nn.functional.softplus(dt.float() + dt_bias.float())
    decay = torch.exp(-torch.exp(a_log.float()) * d)
    y = torch.zeros(T, H, P)
    for r0, r1, slot, start in _chunks(cu_seqlens, state_slots, seq_starts):
        S = state[slot].clone() if start > 0 else torch.zeros(H, N, P)
        for t in range(r0, r1):
            S = decay[t, :, None, None] * S + d[t, :, None, None] * (
                Bf[t, :, :, None] * xf[t, :, None, :])
            y[t] = torch.einsum("hnp,hn->hp", S, Cf[t]) \
                + d_skip.float()[:, None] * xf[t]
        state[slot] = S
    y = y.reshape(T, H * P) * torch.nn.functional.silu(z.float())
    y = y.reshape(T, norm_groups, -1)
    y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + norm_eps)
    return (y.reshape(T, H * P) * norm_w.float()).to(x.dtype)


def residual_add_norm(x32, y, w, eps: float, out_dtype, y2=None,
                      s1: float = 1.0, s2: float = 1.0):
    """Pre-norm residual step on an f32 stream: x32 += s1*y (+ s2*y2) in
    place; returns rms(x32) * w rounded to out_dtype (None without w)."""
    add = s1 * y.float() if s1 != 1.0 else y.float()
    if y2 is not None:
        add = add + s2 * y2.float()
    x32 += add
    if w is None:
        return None
    return rms_norm_cast(x32, w, eps, out_dtype)


def clamped_glu(gu, limit: float, alpha: float):
    """gu [T, 2F] = [gate | up] -> g*sigmoid(alpha*g)*(u + 1) with
    g = min(gate, limit), u = clamp(up, -limit, limit)."""
    F_ = gu.size(-1) // 2
    g = gu[..., :F_].float().clamp(max=limit)
    u = gu[..., F_:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)


def sigmoid_mul(x, gate):
    """x [T, N] * sigmoid(gate [T, Ng]); with Ng < N each gate column
    serves N/Ng consecutive columns of x."""
    g = torch.sigmoid(gate.float())
    if gate.size(-1) != x.size(-1):
        g = g.repeat_interleave(x.size(-1) // gate.size(-1), -1)
    return (x.float() * g).to(x.dtype)


def gelu_glu(gu):
    """gu [T, 2F] = [gate | up] -> gelu_tanh(gate) * up."""
    F_ = gu.size(-1) // 2
    g = torch.nn.functional.gelu(gu[..., :F_].float(), approximate="tanh")
    return (g * gu[..., F_:].float()).to(gu.dtype)


def relu2(x):
    return torch.relu(x.float()).square().to(x.dtype)


def bigram_embed(ids, embed, scale: float, table, buckets: int,
                 mul_prev: int, mul_cur: int, prev_state, cu_seqlens,
                 state_slots, seq_starts):
    """x[t] = embed[ids[t]] * scale (+ table[row(t)]) as f32 rows. With a
    table, row(t) = (previous * mul_prev + ids[t] * mul_cur) mod buckets,
    the previous token being the row before t in its chunk or, for a
    chunk's first row, prev_state[slot] (a chunk starting at position 0
    takes row `buckets`). prev_state [slots] int64 is advanced to each
    chunk's last token."""
    x = embed[ids].float() * scale
    idl = ids.tolist()
    valid = torch.zeros(len(idl), 1)
    rows = torch.zeros(len(idl), dtype=torch.long)
    for c0, c1, slot, start in _chunks(cu_seqlens, state_slots, seq_starts):
        valid[c0:c1] = 1.0
        if table is None:
            continue
        prev = int(prev_state[slot]) if start > 0 else -1
        for t in range(c0, c1):
            rows[t] = buckets if prev < 0 else \
                (prev * mul_prev + idl[t] * mul_cur) % buckets
            prev = idl[t]
        prev_state[slot] = prev
    if table is not None:
        x = x + table[rows].float()
    return x * valid          # rows of padding chunks are zero


def latent_rope_cache_write(q, dkv, norm_w, eps: float, cache, slot_mapping,
                            positions, inv_freq, dim: int,
                            interleaved: bool = False, rot_mag: float = 1.0):
    """q [T, H, dim + 2R]: the last 2R dims of every head rotate (i paired
    with i + R, or with `interleaved` 2i with 2i + 1; angle = position *
    inv_freq[i], f32; cos and sin times rot_mag). dkv [T, rank + 2R]
    (or None): the first rank dims are RMS-normed with norm_w, the last
    2R rotated, and the row is scattered into cache [blocks, block_size,
    rank + 2R] at slot_mapping (negative: skipped). Returns q rotated."""
    R = inv_freq.numel()
    ang = positions.float()[:, None] * inv_freq.float()[None, :]
    c, s = torch.cos(ang) * rot_mag, torch.sin(ang) * rot_mag

    def rot(t, cc, ss):
        if interleaved:
            a, b = t[..., 0::2], t[..., 1::2]
            return torch.stack([a * cc - b * ss, b * cc + a * ss],
                               -1).flatten(-2)
        a, b = t[..., :R], t[..., R:]
        return torch.cat([a * cc - b * ss, b * cc + a * ss], -1)
    qf = q.float()
    qr = torch.cat([qf[..., :dim],
                    rot(qf[..., dim:], c[:, None], s[:, None])], -1)
    if dkv is not None:
        rank = dkv.size(-1) - 2 * R
        lat = dkv[:, :rank].float()
        lat = lat * torch.rsqrt(lat.pow(2).mean(-1, keepdim=True) + eps) \
            * norm_w.float()
        row = torch.cat([lat, rot(dkv[:, rank:].float(), c, s)], -1)
        flat = cache.view(-1, cache.size(-1))
        for t, slot in enumerate(slot_mapping.tolist()):
            if slot >= 0:
                flat[slot] = row[t].to(cache.dtype)
    return qr.to(q.dtype)


def latent_attention(q, cache, block_tables, token_seq, positions,
                     scale: float, rank: int, sinks=None):
    """Causal attention in the latent space. q [T, H, rank + P] (the
    unrotated query already folded through the key up-projection), cache
    [blocks, block_size, rank + P]; row t belongs to chunk token_seq[t]
    (its block-table row; negative: padding) at position positions[t] and
    sees cached rows 0..position. score = q . row * scale; with `sinks`
    [H] the softmax denominator also holds exp(sink_h). Returns the
    weighted sum of the rows' first `rank` dims, [T, H, rank]."""
    T, H, DT = q.shape
    bs = cache.size(1)
    flat = cache.view(-1, DT)
    out = torch.zeros(T, H, rank)
    pos_l, seq_l = positions.tolist(), token_seq.tolist()
    for t in range(T):
        if seq_l[t] < 0:
            continue
        js = torch.arange(pos_l[t] + 1)
        rows = flat[block_tables[seq_l[t]].long()[js // bs] * bs + js % bs]
        rows = rows.float()
        s = q[t].float() @ rows.t() * scale              # [H, n]
        if sinks is not None:
            s = torch.cat([s, sinks.float()[:, None]], 1)
            w = torch.softmax(s, -1)[:, :-1]
        else:
            w = torch.softmax(s, -1)
        out[t] = w @ rows[:, :rank]
    return out.to(q.dtype)


# ---- looped parallel-layer stacks ------------------------------------------

def scaled_residual_add_norm(x32, terms, w, eps: float, out_dtype,
                             x_add=None):
    """x32 [T, H] f32 += sum of v*y over `terms` = [(y [T, H], v [H] f32)]
    (+ x_add [T, H] f32), in place; returns rms(x32)*w rounded to
    out_dtype (None when w is None)."""
    add = None
    for y, v in terms:
        t = y.float() * v.float()
        add = t if add is None else add + t
    x32 += add
    if x_add is not None:
        x32 += x_add
    if w is None:
        return None
    return (x32 * torch.rsqrt(x32.pow(2).mean(-1, keepdim=True) + eps)
            * w.float()).to(out_dtype)


def token_shift(h, mu, state, cu_seqlens, state_slots, seq_starts):
    """Row t becomes h_t + (h_{t-1} - h_t)*mu, mu [H] f32; the row before a
    chunk's first comes from state [slots, H] (zeros at position 0),
    which is advanced in place to the chunk's last row of h."""
    out = torch.zeros_like(h)
    m = mu.float()
    for r0, r1, slot, start in _chunks(cu_seqlens, state_slots, seq_starts):
        first = state[slot].float()[None] if start > 0 else \
            torch.zeros(1, h.size(1))
        cur = h[r0:r1].float()
        prev = torch.cat([first, cur[:-1]], 0)
        out[r0:r1] = (cur + (prev - cur) * m).to(h.dtype)
        state[slot] = h[r1 - 1].to(state.dtype)
    return out


def diag_delta_rule(r, k, v, w_pre, a_pre, gate, norm_w, state, cu_seqlens,
                    state_slots, seq_starts, decay_rate: float, k_eps: float,
                    norm_eps: float):
    """Generalized delta rule. r/k/v/gate [T, H, D]; w_pre/a_pre [T, H*D]
    f32 pre-activations of the decay w = exp(-decay_rate*sigmoid(w_pre))
    and the removal rate a = sigmoid(a_pre); state [slots, H, D, D] f32 in
    place. Per token and head, with u = k/sqrt(k.k + k_eps):
    S <- diag(w) S - (a*u)(u^T S) + k v^T, o = S^T r; o is divided by its
    root mean square per head, weighted by norm_w [H*D] and gated by
    sigmoid(gate). Returns [T, H*D]."""
    T, H, D = r.shape
    rf, kf, vf = r.float(), k.float(), v.float()
    w = torch.exp(-decay_rate * torch.sigmoid(w_pre.float())).view(T, H, D)
    a = torch.sigmoid(a_pre.float()).view(T, H, D)
    u = kf * torch.rsqrt(kf.pow(2).sum(-1, keepdim=True) + k_eps)
    au = a * u
    out = torch.zeros(T, H, D)
    for r0, r1, slot, start in _chunks(cu_seqlens, state_slots, seq_starts):
        S = state[slot].clone() if start > 0 else torch.zeros(H, D, D)
        for t in range(r0, r1):
            p = torch.einsum("hd,hdv->hv", u[t], S)
            S = w[t][..., None] * S - au[t][..., None] * p[:, None, :] \
                + kf[t][..., None] * vf[t][:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, rf[t])
        state[slot] = S
    out = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + norm_eps)
    out = out.reshape(T, H * D) * norm_w.float() \
        * torch.sigmoid(gate.float().reshape(T, H * D))
    return out.to(r.dtype)


def hgrn2_scan(q, v, f_pre, lower, norm_w, state, cu_seqlens, state_slots,
               seq_starts, norm_eps: float):
    """q [T, H, D] (pre-activation; silu applied here), v [T, H, V], f_pre
    [T, H*D] f32, lower [H*D] f32; state [slots, H, D, V] f32 in place.
    f = lower + (1 - lower) sigmoid(f_pre); S <- diag(f) S + (1 - f) v^T,
    o = S^T silu(q); o is RMS-normed over V with norm_w [V]. Returns
    [T, H*V]."""
    T, H, D = q.shape
    V = v.size(2)
    qf = torch.nn.functional.silu(q.float())
    vf = v.float()
    lo = lower.float()
    f = (lo + (1.0 - lo) * torch.sigmoid(f_pre.float())).view(T, H, D)
    out = torch.zeros(T, H, V)
    for r0, r1, slot, start in _chunks(cu_seqlens, state_slots, seq_starts):
        S = state[slot].clone() if start > 0 else torch.zeros(H, D, V)
        for t in range(r0, r1):
            S = f[t][..., None] * S + (1.0 - f[t])[..., None] * vf[t][:, None]
            out[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        state[slot] = S
    out = out * torch.rsqrt(out.pow(2).mean(-1, keepdim=True) + norm_eps) \
        * norm_w.float()
    return out.reshape(T, H * V).to(q.dtype)
