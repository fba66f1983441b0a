"""Pure-PyTorch reference implementations of the engine's hot ops.

These are the numerics oracle for the HIP/CDNA4 kernels (tests compare the
HIP kernel against these in fp32 — SURVEY.md §4 test strategy (c)) and the
CPU execution path. They are intentionally simple and readable; the GPU path
never runs these (opsagent_amd.ops dispatch raises if the HIP extension is
missing on a GPU box).
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    dtype = x.dtype
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    out = xf * torch.rsqrt(var + eps) * weight.float()
    return out.to(dtype)


def fused_add_rms_norm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns (rmsnorm(x + residual), x + residual)."""
    s = (x.float() + residual.float())
    out = rms_norm(s, weight, eps)
    return out.to(x.dtype), s.to(x.dtype)


def rope_cos_sin(
    max_seq: int, head_dim: int, theta: float = 500000.0, device="cpu", dtype=torch.float32
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Precomputed RoPE tables [max_seq, head_dim/2] (host-side per CDNA guide §B)."""
    inv_freq = 1.0 / (
        theta ** (torch.arange(0, head_dim, 2, device=device, dtype=torch.float32) / head_dim)
    )
    t = torch.arange(max_seq, device=device, dtype=torch.float32)
    freqs = torch.outer(t, inv_freq)
    return freqs.cos().to(dtype), freqs.sin().to(dtype)


def rope_apply(
    q: torch.Tensor,
    k: torch.Tensor,
    cos: torch.Tensor,
    sin: torch.Tensor,
    positions: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Neox-style (rotate-half) RoPE.

    q: [T, Hq, D], k: [T, Hk, D]; cos/sin: [max_seq, D/2]; positions: [T].
    """
    def _rot(x: torch.Tensor) -> torch.Tensor:
        d = x.shape[-1]
        c = cos[positions].to(torch.float32).unsqueeze(1)  # [T,1,D/2]
        s = sin[positions].to(torch.float32).unsqueeze(1)
        x1 = x[..., : d // 2].float()
        x2 = x[..., d // 2 :].float()
        return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1).to(x.dtype)

    return _rot(q), _rot(k)


def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return (torch.nn.functional.silu(gate.float()) * up.float()).to(gate.dtype)


def attention_prefill(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: Optional[float] = None,
    causal: bool = True,
) -> torch.Tensor:
    """Causal attention over contiguous tensors.

    q: [B, Hq, Sq, D]; k, v: [B, Hk, Skv, D] with Skv >= Sq (the causal
    diagonal is offset so that query i attends keys [0 .. Skv-Sq+i]).
    GQA: Hq % Hk == 0 (kv heads broadcast over query-head groups).
    """
    B, Hq, Sq, D = q.shape
    Hk, Skv = k.shape[1], k.shape[2]
    scale = scale if scale is not None else D ** -0.5
    group = Hq // Hk
    kf = k.float().repeat_interleave(group, dim=1)
    vf = v.float().repeat_interleave(group, dim=1)
    s = torch.einsum("bhqd,bhkd->bhqk", q.float(), kf) * scale
    if causal:
        offset = Skv - Sq
        qi = torch.arange(Sq, device=q.device).unsqueeze(1)
        ki = torch.arange(Skv, device=q.device).unsqueeze(0)
        mask = ki > (qi + offset)
        s = s.masked_fill(mask, float("-inf"))
    p = torch.softmax(s, dim=-1)
    out = torch.einsum("bhqk,bhkd->bhqd", p, vf)
    return out.to(q.dtype)


def attention_decode_paged(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_lens: torch.Tensor,
    scale: Optional[float] = None,
) -> torch.Tensor:
    """Single-token decode attention against a paged KV cache.

    q:           [B, Hq, D]         (one new token per sequence)
    k/v_cache:   [num_blocks, block_size, Hk, D]
    block_table: [B, max_blocks] int32 (block ids per sequence, -1 padded)
    seq_lens:    [B] int32 — total tokens in cache per sequence (incl. current)
    """
    B, Hq, D = q.shape
    block_size = k_cache.shape[1]
    Hk = k_cache.shape[2]
    group = Hq // Hk
    scale = scale if scale is not None else D ** -0.5
    outs = []
    for b in range(B):
        n = int(seq_lens[b].item())
        nblocks = (n + block_size - 1) // block_size
        blocks = block_table[b, :nblocks].long()
        k = k_cache[blocks].reshape(-1, Hk, D)[:n].float()  # [n, Hk, D]
        v = v_cache[blocks].reshape(-1, Hk, D)[:n].float()
        kf = k.repeat_interleave(group, dim=1)  # [n, Hq, D]
        vf = v.repeat_interleave(group, dim=1)
        s = torch.einsum("hd,nhd->hn", q[b].float(), kf) * scale
        p = torch.softmax(s, dim=-1)
        outs.append(torch.einsum("hn,nhd->hd", p, vf))
    return torch.stack(outs).to(q.dtype)


def kv_cache_write(
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    """Scatter new K/V rows into the paged cache.

    k/v: [T, Hk, D]; slot_mapping: [T] int64 flat slot = block_id*block_size + offset.
    """
    nb, bs, hk, d = k_cache.shape
    k_cache.view(nb * bs, hk, d)[slot_mapping] = k
    v_cache.view(nb * bs, hk, d)[slot_mapping] = v


def quant_fp8(x: torch.Tensor):
    """Per-row OCP e4m3 quantization reference (torch.float8_e4m3fn)."""
    shape = x.shape
    xf = x.reshape(-1, shape[-1]).float()
    amax = xf.abs().amax(dim=-1, keepdim=True).clamp_min(1e-8)
    scale = (amax / 448.0).squeeze(-1)
    q = (xf / scale.unsqueeze(-1)).to(torch.float8_e4m3fn)
    return q.view(torch.uint8).reshape(shape), scale


def dequant_fp8(q: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    f = q.view(torch.float8_e4m3fn).float()
    return f * scale.unsqueeze(-1)


def linear_fp8(x: torch.Tensor, w8: torch.Tensor, w_scale: torch.Tensor) -> torch.Tensor:
    w = dequant_fp8(w8, w_scale)
    return torch.nn.functional.linear(x.float(), w).to(x.dtype)


def greedy_sample_masked(logits: torch.Tensor, mask: Optional[torch.Tensor]) -> torch.Tensor:
    """argmax over allowed tokens. logits [B, V]; mask [B, V] bool (True = allowed)."""
    lf = logits.float()
    if mask is not None:
        lf = lf.masked_fill(~mask, float("-inf"))
    return lf.argmax(dim=-1)


# ---------------------------------------------------------------------------
# Sequence-mixer ops over a flat multi-sequence batch (CPU path and numerics
# reference of mixers.hip). A batch is T tokens of B sequences laid end to
# end: cu[b]..cu[b+1] are sequence b's new tokens, which continue it from
# position past[b]; slots[b] is its row in the state tensors.


def causal_conv_seq(x, w, state, cu, past, slots, add_input, act_silu, out_dtype):
    """Causal per-channel convolution over time, continued from `state`
    (the last taps-1 inputs of each sequence, float32 [slots, taps-1, C]);
    inputs before position 0 are zero whatever the slot holds. Returns
    (x if add_input) + conv(x), optionally through silu; updates state."""
    taps = w.shape[1]
    wf = w.float()
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    for b in range(len(cu) - 1):
        lo, hi = cu[b], cu[b + 1]
        if hi == lo:
            continue
        xs = x[lo:hi].float()
        if taps > 1:
            prev = state[slots[b]].clone()
            keep = min(past[b], taps - 1)
            prev[: taps - 1 - keep] = 0
            ext = torch.cat([prev, xs], 0)
        else:
            ext = xs
        n = hi - lo
        y = torch.zeros_like(xs)
        for j in range(taps):
            y += ext[j : j + n] * wf[:, j]
        if add_input:
            y += xs
        if act_silu:
            y = torch.nn.functional.silu(y)
        out[lo:hi] = y.to(out_dtype)
        if taps > 1:
            state[slots[b]] = ext[-(taps - 1):]
    return out


def group_rms_norm(y, w, groups, eps, residual, out_dtype):
    """RMS norm over `groups` equal consecutive parts of the last axis, times
    w. With `residual` (float32, updated in place) returns residual + norm."""
    T, C = y.shape
    yf = y.float().view(T, groups, C // groups)
    n = (yf * torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps)).view(T, C) * w.float()
    if residual is not None:
        residual += n
        return residual
    return n.to(out_dtype)


def attn_qkv_prepare(qkv, bias, q_norm_w, k_norm_w, H, G, D, Dv, eps, k_cache, v_cache,
                     slot_mapping):
    """Adds the projection bias (if any), then whole-projection RMS norm of q
    and of k (weighted), per-head RMS norm of v (no weight); k and v go to
    their cache slots, q is returned."""
    T = qkv.shape[0]
    n = H * D + G * D + G * Dv
    x = qkv[:, :n].float()
    if bias is not None:
        x = x + bias[:n].float()
    q, k, v = x[:, : H * D], x[:, H * D : H * D + G * D], x[:, H * D + G * D :]
    q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_norm_w.float()
    k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_norm_w.float()
    v = v.reshape(T, G, Dv)
    v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    nb, bs = k_cache.shape[0], k_cache.shape[1]
    sm = slot_mapping.long()
    k_cache.view(nb * bs, G, D)[sm] = k.reshape(T, G, D).to(k_cache.dtype)
    v_cache.view(nb * bs, G, Dv)[sm] = v.to(v_cache.dtype)
    return q.reshape(T, H, D).to(qkv.dtype)


def attention_biased_paged(q, gate_logits, k_cache, v_cache, cu, past, block_table,
                           scale, slopes):
    """Causal softmax attention of each new token over its sequence's cached
    keys 0..position, score = q.k*scale - slope_h*(i-j), each head's output
    times sigmoid(gate logit). q [T,H,D]; returns [T, H*Dv]."""
    T, H, D = q.shape
    nb, bs, G, Dv = v_cache.shape
    out = torch.empty(T, H, Dv, dtype=q.dtype, device=q.device)
    rep = H // G
    for b in range(len(cu) - 1):
        lo, hi = cu[b], cu[b + 1]
        if hi == lo:
            continue
        total = past[b] + hi - lo
        nblk = (total + bs - 1) // bs
        blocks = block_table[b, :nblk].long()
        kk = k_cache[blocks].reshape(nblk * bs, G, D)[:total].float()
        vv = v_cache[blocks].reshape(nblk * bs, G, Dv)[:total].float()
        kk = kk.repeat_interleave(rep, dim=1)
        vv = vv.repeat_interleave(rep, dim=1)
        qs = q[lo:hi].float()
        s = torch.einsum("ihd,jhd->hij", qs, kk) * scale
        i = torch.arange(past[b], total, dtype=torch.float32).view(1, -1, 1)
        j = torch.arange(total, dtype=torch.float32).view(1, 1, -1)
        s = s - slopes.float().view(H, 1, 1) * (i - j)
        s = s.masked_fill(j > i, float("-inf"))
        p = torch.softmax(s, dim=-1)
        o = torch.einsum("hij,jhd->ihd", p, vv)
        o = o * torch.sigmoid(gate_logits[lo:hi].float()).unsqueeze(-1)
        out[lo:hi] = o.to(q.dtype)
    return out.view(T, H * Dv)


def channel_delta_rule(q, k, v, b_logits, a, dt_bias, a_log, state, cu, past, slots):
    """Gated delta rule with a decay per head and key channel, continued from
    `state` [slots, H, Dv, D] float32 (S stored transposed; zero at position 0
    whatever the slot holds). q,k [T,G,D], v [T,H,Dv] after convolution and silu; b_logits
    [T,H]; a [T,H*D]. Returns the read-out [T,H,Dv] float32; updates state."""
    T, G, D = q.shape
    H, Dv = v.shape[1], v.shape[2]
    rep = H // G
    qf, kf = q.float(), k.float()
    qf = qf * torch.rsqrt(qf.pow(2).sum(-1, keepdim=True) + 1e-6) * (D ** -0.5)
    kf = kf * torch.rsqrt(kf.pow(2).sum(-1, keepdim=True) + 1e-6)
    qf = qf.repeat_interleave(rep, dim=1)
    kf = kf.repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(b_logits.float())
    sp = torch.nn.functional.softplus(a.float() + dt_bias.float())
    g = torch.exp(-torch.exp(a_log.float()).view(1, H, 1) * sp.view(T, H, D))
    vf = v.float()
    out = torch.empty(T, H, Dv, dtype=torch.float32, device=q.device)
    for bi in range(len(cu) - 1):
        lo, hi = cu[bi], cu[bi + 1]
        if hi == lo:
            continue
        S = state[slots[bi]].transpose(-1, -2).clone()
        if past[bi] == 0:
            S.zero_()
        for t in range(lo, hi):
            S = S * g[t].unsqueeze(-1)
            u = beta[t].unsqueeze(-1) * (vf[t] - torch.einsum("hdv,hd->hv", S, kf[t]))
            S = S + kf[t].unsqueeze(-1) * u.unsqueeze(1)
            out[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        state[slots[bi]] = S.transpose(-1, -2)
    return out


def gated_head_rms_norm(o, w, gate_logits, eps, out_dtype):
    """o [T,H,Dv] float32: per-head RMS norm, times w [Dv], times
    sigmoid(gate_logits [T, H*Dv]). Returns [T, H*Dv]."""
    T, H, Dv = o.shape
    n = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    n = n * torch.sigmoid(gate_logits.float()).view(T, H, Dv)
    return n.reshape(T, H * Dv).to(out_dtype)


def softcap(logits, cap):
    return cap * torch.tanh(logits.float() / cap)


# ---------------------------------------------------------------------------
# Blocks of sandwich-norm decoders with rotary window attention and routed
# experts (same flat multi-sequence layout as above).


def dyt_norm(y, post, residual, nxt, out_dtype):
    """Dynamic-tanh norm dyt(x; w, b, a) = tanh(a x) w + b in float32.
    With y and post = (w, b, a): residual += dyt(y; post), in place. With
    nxt = (w, b, a): also returns dyt(residual; nxt) in out_dtype."""
    if y is not None:
        w, b, a = post
        residual += torch.tanh(a.float() * y.float()) * w.float() + b.float()
    if nxt is None:
        return None
    w, b, a = nxt
    return (torch.tanh(a.float() * residual.float()) * w.float() + b.float()).to(out_dtype)


def attn_rope_prepare(qkv, q_norm_w, k_norm_w, inv_freq, H, G, D, Dv, eps, k_cache, v_cache,
                      positions, slot_mapping, v_heads=None):
    """Per-head RMS norm of q and k (weight [D] shared by heads; None: no
    norm), then rotation of channel pairs (2i, 2i+1), i < len(inv_freq), by
    position * inv_freq[i]; k and v (v_heads heads, default G) go to their
    cache slots, q is returned [T, H, D]."""
    T = qkv.shape[0]
    Gv = v_heads or G
    x = qkv[:, : H * D + G * D + Gv * Dv].float()
    q = x[:, : H * D].reshape(T, H, D)
    k = x[:, H * D : H * D + G * D].reshape(T, G, D)
    v = x[:, H * D + G * D :].reshape(T, Gv, Dv)
    if q_norm_w is not None:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_norm_w.float()
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_norm_w.float()
    r = 2 * inv_freq.numel()
    if r:
        ang = positions.float()[:, None] * inv_freq.float()[None, :]
        c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]

        def rot(t):
            a, b = t[..., 0:r:2], t[..., 1:r:2]
            out = t.clone()
            out[..., 0:r:2] = a * c - b * s
            out[..., 1:r:2] = b * c + a * s
            return out

        q, k = rot(q), rot(k)
    nb, bs = k_cache.shape[0], k_cache.shape[1]
    sm = slot_mapping.long()
    k_cache.view(nb * bs, G, D)[sm] = k.to(k_cache.dtype)
    v_cache.view(nb * bs, Gv, Dv)[sm] = v.to(v_cache.dtype)
    return q.to(qkv.dtype)


def attention_paged(q, k_cache, v_cache, cu, past, block_table, scale, slopes=None,
                    gate_logits=None, window=None, sinks=None, softcap=None):
    """Causal softmax attention of each new token over its sequence's cached
    keys. Options: a linear distance penalty slope_h*(i-j), a window (key j
    seen iff i - j < window), a per-head sink term exp(sink_h) in the
    denominator, a sigmoid gate on each head's output, a soft cap
    cap * tanh(score / cap) on the scaled score. The cache may hold fewer
    value heads than key heads: key head g reads value head g mod Gv."""
    T, H, D = q.shape
    nb, bs, Gv, Dv = v_cache.shape
    G = k_cache.shape[2]
    out = torch.empty(T, H, Dv, dtype=q.dtype, device=q.device)
    rep = H // G
    for b in range(len(cu) - 1):
        lo, hi = cu[b], cu[b + 1]
        if hi == lo:
            continue
        total = past[b] + hi - lo
        first = max(0, past[b] - window + 1) if window else 0
        fb = first // bs
        first = fb * bs
        nblk = (total + bs - 1) // bs
        blocks = block_table[b, fb:nblk].long()
        kk = k_cache[blocks].reshape(-1, G, D)[: total - first].float()
        vv = v_cache[blocks].reshape(-1, Gv, Dv)[: total - first].float()
        if Gv != G:
            vv = vv.repeat(1, G // Gv, 1)
        kk = kk.repeat_interleave(rep, dim=1)
        vv = vv.repeat_interleave(rep, dim=1)
        qs = q[lo:hi].float()
        s = torch.einsum("ihd,jhd->hij", qs, kk) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        i = torch.arange(past[b], total, dtype=torch.float32).view(1, -1, 1)
        j = torch.arange(first, total, dtype=torch.float32).view(1, 1, -1)
        if slopes is not None:
            s = s - slopes.float().view(H, 1, 1) * (i - j)
        hide = j > i
        if window:
            hide = hide | (i - j >= window)
        s = s.masked_fill(hide, float("-inf"))
        if sinks is not None:
            s = torch.cat([s, sinks.float().view(H, 1, 1).expand(H, s.shape[1], 1)], -1)
        p = torch.softmax(s, dim=-1)
        if sinks is not None:
            p = p[..., :-1]
        o = torch.einsum("hij,jhd->ihd", p, vv)
        if gate_logits is not None:
            o = o * torch.sigmoid(gate_logits[lo:hi].float()).unsqueeze(-1)
        out[lo:hi] = o.to(q.dtype)
    return out.view(T, H * Dv)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z * z * z)))


def act_mul(gate, up, act):
    """act: "silu" | "gelu_tanh" | ("clamp_swish", limit, alpha):
    g = min(gate, limit), u = clamp(up, -limit, limit), g sigmoid(alpha g) (u + 1)."""
    g = gate.float()
    if isinstance(act, tuple):
        kind, limit, alpha = act
        assert kind == "clamp_swish"
        g = g.clamp(max=limit)
        u = up.float().clamp(-limit, limit)
        return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gate.dtype)
    a = torch.nn.functional.silu(g) if act == "silu" else gelu_tanh(g)
    return (a * up.float()).to(gate.dtype)


def route_topk(logits, correction, top, groups, keep, scale, score, rating="top2",
               renorm=True):
    """logits float32 [T, E] -> (experts int32 [T, top], weights float32
    [T, top]). Scores are sigmoid or softmax of the logits; the choice uses
    c = score + correction inside the `keep` top-rated of `groups` runs of
    neighbouring experts (rating: max1(c) + max2(c), or max(c) with rating
    "max"); weights w_j = scale * s_j / (sum_k s_k + 1e-20) over the picked
    experts, or scale * s_j with renorm off."""
    T, E = logits.shape
    s = torch.sigmoid(logits) if score == "sigmoid" else torch.softmax(logits, -1)
    choice = s + correction.float() if correction is not None else s.clone()
    if groups > 1:
        per = E // groups
        gs = choice.view(T, groups, per).topk(1 if rating == "max" else min(2, per),
                                              dim=-1).values.sum(-1)
        best = gs.topk(keep, dim=-1).indices
        ok = torch.zeros(T, groups, dtype=torch.bool, device=logits.device)
        ok.scatter_(1, best, True)
        choice = choice.masked_fill(~ok.repeat_interleave(per, dim=1), float("-inf"))
    idx = choice.topk(top, dim=-1).indices
    w = s.gather(1, idx)
    w = w / (w.sum(-1, keepdim=True) + 1e-20) * scale if renorm else w * scale
    return idx.to(torch.int32), w


def moe_pairs_mlp(x, w13, w2, idx, wts, act):
    """out[t] = sum_j wts[t, j] * W2[e] (act(Wg[e] x_t) * (Wu[e] x_t)), e =
    idx[t, j]; w13 [E, 2I, K] holds gate rows then up rows, w2 [E, C, I]."""
    T, top = idx.shape
    inter = w13.shape[1] // 2
    out = torch.zeros(T, w2.shape[1], dtype=torch.float32, device=x.device)
    for t in range(T):
        for j in range(top):
            e = int(idx[t, j])
            gu = torch.nn.functional.linear(x[t : t + 1], w13[e])
            a = act_mul(gu[:, :inter], gu[:, inter:], act)
            out[t] += wts[t, j] * torch.nn.functional.linear(a, w2[e])[0].float()
    return out.to(x.dtype)


# ---------------------------------------------------------------------------
# Pre-norm decoders with latent attention and decayed linear attention.


def add_layer_norm(residual, y, w, eps, out_dtype, y2=None, y2_gate=None):
    """residual (float32 [T, C], in place) += y + sigmoid(y2_gate) * y2 (each
    optional; y2_gate [T] scales the rows of y2). With w: returns the layer
    norm (x - mean) / sqrt(mean((x - mean)^2) + eps) * w of the new residual
    in out_dtype."""
    if y is not None:
        residual += y.float()
    if y2 is not None:
        g = torch.sigmoid(y2_gate.float()).unsqueeze(-1) if y2_gate is not None else 1.0
        residual += g * y2.float()
    if w is None:
        return None
    mu = residual.mean(-1, keepdim=True)
    d = residual - mu
    return (d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)


def _rotate_pairs(x, pos, inv_freq):
    """x [T, ..., n] float32: channel pairs (2i, 2i+1), i < len(inv_freq),
    turn by pos * inv_freq[i]; the rest pass."""
    n = 2 * inv_freq.numel()
    ang = pos.float().view(-1, *([1] * (x.dim() - 1))) * inv_freq.float()
    c, s = torch.cos(ang), torch.sin(ang)
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    out = x.clone()
    out[..., 0:n:2] = u * c - v * s
    out[..., 1:n:2] = v * c + u * s
    return out


def latent_kv_prepare(dkv, norm_w, inv_freq, rank, rot, eps, k_cache, pos, slot_mapping):
    """dkv [T, rank + rot]: the first `rank` columns, RMS-normed with norm_w,
    and the last `rot`, rotated by position, go to the token's cache row
    [rank + rot]."""
    x = dkv.float()
    c = x[:, :rank]
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
    kr = _rotate_pairs(x[:, rank:rank + rot], pos, inv_freq)
    nb, bs = k_cache.shape[0], k_cache.shape[1]
    k_cache.view(nb * bs, rank + rot)[slot_mapping.long()] = torch.cat([c, kr], -1).to(k_cache.dtype)


def latent_q_assemble(q, q_lat, inv_freq, H, D, rot, pos):
    """q [T, H*(D+rot)] (per head: D unrotated, rot rotated channels), q_lat
    [H, T, rank] (the unrotated part taken through the key up-projection).
    Returns [T, H, rank + rot]: q_lat beside the rotated part."""
    T = q.shape[0]
    qr = _rotate_pairs(q.float().view(T, H, D + rot)[..., D:], pos, inv_freq)
    return torch.cat([q_lat.float().transpose(0, 1), qr], -1).to(q.dtype).contiguous()


def decay_linear_attention(q, k, v, z, z_bias, inv_tau, head_decay, state, cu, past, slots,
                           H, D, Dv, act, q_scale):
    """S_t = diag(a_t) S_{t-1} + k_t v_t^T, o_t = S_t^T q_t per head, continued
    from `state` [slots, H, Dv, D] float32 (S transposed; zero at position 0
    whatever the slot holds). a_t = head_decay[h] for every channel, or
    sigmoid(z_t + z_bias)^(inv_tau) per key channel when z is given. act
    "silu" is applied to q, k and v first; q is then scaled. Returns the
    read-out [T, H*Dv] float32; updates state."""
    T = q.shape[0]
    f = (lambda t: torch.nn.functional.silu(t.float())) if act == "silu" else (lambda t: t.float())
    qf = (f(q) * q_scale).view(T, H, D)
    kf, vf = f(k).view(T, H, D), f(v).view(T, H, Dv)
    if z is not None:
        zz = z.float() + z_bias.float()
        a = torch.exp(torch.nn.functional.logsigmoid(zz) * inv_tau).view(T, H, D)
    else:
        a = head_decay.float().view(1, H, 1).expand(T, H, D)
    out = torch.empty(T, H, Dv, dtype=torch.float32, device=q.device)
    for bi in range(len(cu) - 1):
        lo, hi = cu[bi], cu[bi + 1]
        if hi == lo:
            continue
        S = state[slots[bi]].transpose(-1, -2).clone()      # [H, D, Dv]
        if past[bi] == 0:
            S.zero_()
        for t in range(lo, hi):
            S = S * a[t].unsqueeze(-1) + kf[t].unsqueeze(-1) * vf[t].unsqueeze(1)
            out[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        state[slots[bi]] = S.transpose(-1, -2)
    return out.view(T, H * Dv)


def gated_rms_norm(o, w, groups, gate_logits, gate_act, eps, out_dtype):
    """o [T, N] float32: RMS norm over each of `groups` equal parts, times w
    ([N/groups], shared by the parts, or [N]), times sigmoid or silu of
    gate_logits [T, N]."""
    T, N = o.shape
    x = o.view(T, groups, N // groups)
    x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    wf = w.float()
    x = (x * wf).view(T, N) if wf.numel() == N // groups else x.reshape(T, N) * wf
    g = gate_logits.float()
    g = torch.sigmoid(g) if gate_act == "sigmoid" else torch.nn.functional.silu(g)
    return (x * g).to(out_dtype)


# ---------------------------------------------------------------------------
# Hyper-connected pre-norm decoders: several residual streams, differential
# attention, retention, ungated experts.


def hyper_norm(streams, y, y2, y2_gate, mix, write, read, w, b, eps, out_dtype):
    """streams float32 [T, S, C], updated in place. With y (and mix [S, S]
    indexed [from, to], write [S]): new_t = sum_s mix[s, t] old_s + write[t] *
    (y + sigmoid(y2_gate) * y2), every stream from the OLD ones. With read
    [S]: returns the layer norm ((u - mean) / sqrt(var + eps) * w + b) of
    u = sum_s read[s] new_s in out_dtype."""
    if y is not None:
        yy = y.float()
        if y2 is not None:
            g = torch.sigmoid(y2_gate.float()).unsqueeze(-1) if y2_gate is not None else 1.0
            yy = yy + g * y2.float()
        new = (torch.einsum("sb,asc->abc", mix.float(), streams)
               + write.float().view(1, -1, 1) * yy.unsqueeze(1))
        streams.copy_(new)
    if read is None:
        return None
    u = torch.einsum("s,tsc->tc", read.float(), streams)
    mu = u.mean(-1, keepdim=True)
    d = u - mu
    out = d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    if b is not None:
        out = out + b.float()
    return out.to(out_dtype)


def rope_rows(x, n_rot, D, inv_freq, pos):
    """x [T, n]: the first n_rot * D columns are heads of D channels whose
    pairs (2i, 2i+1), i < len(inv_freq), turn by pos * inv_freq[i]; the other
    columns are copied. Returns float32 [T, n]."""
    T = x.shape[0]
    out = x.float().clone()
    if inv_freq.numel():
        out[:, : n_rot * D] = _rotate_pairs(out[:, : n_rot * D].reshape(T, n_rot, D), pos,
                                            inv_freq).reshape(T, n_rot * D)
    return out


def combine_norm_gate(a, a2, lam, H, Dv, norm, eps, post_scale, gate_logits, gate_act, out_dtype):
    """a [T, H*Dv] (minus lam * a2 if a2 is given); with norm each head's Dv
    values are divided by their root mean square (eps inside the root) and
    multiplied by post_scale; then times sigmoid or silu of gate_logits
    [T, H*Dv] (None: no gate)."""
    T = a.shape[0]
    o = a.float()
    if a2 is not None:
        o = o - float(lam) * a2.float()
    if norm:
        o = o.view(T, H, Dv)
        o = (o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * post_scale).reshape(T, H * Dv)
    if gate_logits is not None:
        g = gate_logits.float()
        o = o * (torch.sigmoid(g) if gate_act == "sigmoid" else torch.nn.functional.silu(g))
    return o.to(out_dtype)


def act_rows(x, act):
    """Elementwise activation of an ungated feed-forward: "relu2" (the square
    of relu), "silu", "gelu_tanh"; evaluated in float32."""
    z = x.float()
    if act == "relu2":
        z = torch.relu(z).square()
    elif act == "silu":
        z = torch.nn.functional.silu(z)
    else:
        z = gelu_tanh(z)
    return z.to(x.dtype)


def moe_pairs_plain(x, w1, w2, idx, wts, act):
    """out[t] = sum_j wts[t, j] * W2[e] act(W1[e] x_t), e = idx[t, j]; w1
    [E, I, K], w2 [E, C, I]."""
    T, top = idx.shape
    out = torch.zeros(T, w2.shape[1], dtype=torch.float32, device=x.device)
    for t in range(T):
        for j in range(top):
            e = int(idx[t, j])
            a = act_rows(torch.nn.functional.linear(x[t : t + 1], w1[e]), act)
            out[t] += wts[t, j] * torch.nn.functional.linear(a, w2[e])[0].float()
    return out.to(x.dtype)
