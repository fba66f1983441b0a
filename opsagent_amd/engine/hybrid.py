"""Hybrid decoders: a per-layer choice of token mixer and feed-forward
around a float32 residual stream, in four layer styles.

"post_canon" (the Povazen design): softmax attention with a linear distance
penalty, or a gated delta rule with per-channel decay.
Layer:  x <- x + norm1(mixer(h)),  h = x + canon(x);  x <- x + norm2(ff(x)).
The norms sit on the sublayer OUTPUTS (grouped RMS norm); the sublayers read
the raw stream. canon is a causal per-channel convolution over time whose
last inputs are carried per sequence, like the recurrent state.

"sandwich" (the Vazilorn design): rotary sliding-window attention with a
sink term, dense gelu or routed-expert feed-forwards.
Layer:  x <- x + post1(mixer(pre1(x)));  x <- x + post2(ff(pre2(x))),
every norm elementwise: tanh(a x) w + b with one scalar a, no statistics
over channels.

"pre_norm" (the Rafodra design): latent attention (a cached low-rank latent
and one rotated key part shared by the heads, optionally read from another
layer's cache), lightning attention (fixed per-head decay) or gated linear
attention (learned per-channel decay); dense silu or routed clamped-swish
feed-forwards.
Layer:  x <- x + mixer(ln1(x));  x <- x + ff(ln2(x)),
ln a layer norm with a weight and no bias.

"hyper" (the Suzulix design): latent attention whose queries also pass a
normed latent, differential attention (two rotary softmax maps per head over
the same values, soft-capped scores, combined as a difference and normed) or
retention (rotary linear attention with a fixed per-head decay); routed
ungated squared-relu experts with a biased router and a gated shared expert.
Layer: the same pre-norm sublayers (layer norm with weight and bias) on S
residual streams: a sublayer reads u = sum_s in_s x_s and writes
x_t <- sum_s mix[s, t] x_s + out_t y; the model's output is the streams' sum.
A run of layers may loop with the same weights; every pass has its own cache
and state. The head is the embedding table.

The mixers are modules of their own (BiasedAttentionMixer,
ChannelDeltaMixer, ...) with every constant a constructor argument, built on the
flat multi-sequence ops of opsagent_amd.ops.mixer_ops; the model keeps no
cache and no loop of its own — keys/values live in the engine's paged cache,
recurrent and convolution state in its StateSlotPool, and one forward serves
prompt portions and decoded tokens of several sequences at once.

Projections that read the same input are fused into one GEMM (library GEMM
for prompt-sized batches, the framework's GEMV kernels for decode).
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch
from torch import nn

from opsagent_amd import ops
from opsagent_amd.engine.config import HybridLayerSpec, HybridSpec, MixerSpec
from opsagent_amd.engine.model import ForwardBatch
from opsagent_amd.ops import mixer_ops as mx
from opsagent_amd.parallel import get_tp_size


def _rand(gen, *shape, std=1.0, dtype=torch.float32):
    dev = gen.device
    return (torch.randn(*shape, generator=gen, device=dev) * std).to(dtype)


def _param(t: torch.Tensor) -> nn.Parameter:
    return nn.Parameter(t, requires_grad=False)


def distance_slopes(heads: int, base_exp: float = 8.0) -> torch.Tensor:
    """slope_h = 2^(-base_exp * (h+1) / heads), float32 [heads]."""
    h = torch.arange(1, heads + 1, dtype=torch.float64)
    return torch.pow(2.0, -base_exp * h / heads).to(torch.float32)


def half_to_interleaved(rows: torch.Tensor, dims: int) -> torch.Tensor:
    """Reorder the first `dims` rows of a block from the "half" rotation
    layout (row i pairs with row i + dims/2) to the interleaved one (row 2i
    pairs with row 2i+1). Applied alike to the query and key projections it
    leaves every dot product unchanged."""
    idx = torch.arange(dims).view(2, dims // 2).t().reshape(-1)
    return torch.cat([rows[idx], rows[dims:]], 0)


def _relayout_heads(w: torch.Tensor, heads: int, dim: int, offset: int, dims: int,
                    layout: str) -> torch.Tensor:
    """w [heads * dim, K]: within every head, rows offset .. offset + dims go
    from `layout` to the interleaved rotation layout."""
    if layout != "half" or dims == 0:
        return w
    w = w.reshape(heads, dim, -1)
    parts = [torch.cat([w[h, :offset], half_to_interleaved(w[h, offset:], dims)], 0)
             for h in range(heads)]
    return torch.stack(parts).reshape(heads * dim, -1)


class BiasedAttentionMixer(nn.Module):
    """Causal softmax attention without rotation: position enters only as a
    per-head linear penalty slope_h * (i - j) on the score. Query and key
    are RMS-normed over their WHOLE projections (weighted), values per head
    (unweighted, cached normed); key and value sizes may differ; each head's
    output is scaled by a sigmoid gate read from the mixer input.

    Fused projection rows: q | k | v | gate."""

    def __init__(self, hidden: int, m: MixerSpec, eps: float, dtype, gen,
                 slope_base_exp: float = 8.0):
        super().__init__()
        self.H, self.G, self.D, self.Dv = m.heads, m.kv_heads, m.dim, m.vdim
        self.eps = eps
        self.scale = float(m.scale) if m.scale is not None else m.dim ** -0.5
        nq, nk, nv = self.H * self.D, self.G * self.D, self.G * self.Dv
        self.n_qkv = nq + nk + nv
        std = 1.0 / math.sqrt(hidden)
        self.proj_w = _param(_rand(gen, self.n_qkv + self.H, hidden, std=std, dtype=dtype))
        self.proj_b = _param(_rand(gen, self.n_qkv, std=0.02, dtype=dtype))
        self.q_norm_w = _param(torch.ones(nq, dtype=dtype, device=gen.device))
        self.k_norm_w = _param(torch.ones(nk, dtype=dtype, device=gen.device))
        self.o_w = _param(_rand(gen, hidden, self.H * self.Dv,
                                std=1.0 / math.sqrt(self.H * self.Dv), dtype=dtype))
        self.register_buffer("slopes", distance_slopes(self.H, slope_base_exp).to(gen.device),
                             persistent=False)

    def kv_shape(self):
        return (self.G, self.D, self.Dv)

    def state_shapes(self) -> Dict[str, tuple]:
        return {}

    def forward(self, h, sb: mx.SeqBatch, kv, state) -> torch.Tensor:
        k_cache, v_cache = kv
        proj = ops.linear(h, self.proj_w)                     # [T, q|k|v|gate]
        q = mx.attn_qkv_prepare(proj, self.proj_b, self.q_norm_w, self.k_norm_w,
                                self.H, self.G, self.D, self.Dv, self.eps,
                                k_cache, v_cache, sb)
        ctx = mx.attention_biased_paged(q, proj[:, self.n_qkv:], k_cache, v_cache, sb,
                                        self.scale, self.slopes)
        return ops.linear(ctx, self.o_w)


class RotaryWindowAttentionMixer(nn.Module):
    """Causal softmax attention with rotary positions. Order of operations
    on a query or key head: RMS norm over the head's `dim` channels (weight
    [dim], one per projection, the same for every head), then rotation of
    channels (2i, 2i+1), i < rot_dims/2, by position * f_i with
    f_i = rot_base^(-2i/rot_dims), optionally rescaled by wavelength.
    Visible keys: the last `window` positions up to the query (None: the
    whole past). With sink=True head h's normaliser is
    sum_j exp(score_j) + exp(sink_h), sink_h learned. Norm weights, sinks,
    angles, scores and softmax weights are float32.

    Fused projection rows: q | k | v."""

    def __init__(self, hidden: int, m: MixerSpec, eps: float, dtype, gen):
        super().__init__()
        self.H, self.G, self.D, self.Dv = m.heads, m.kv_heads, m.dim, m.vdim
        self.eps = eps
        self.scale = float(m.scale) if m.scale is not None else m.dim ** -0.5
        self.window = int(m.window) if m.window else None
        dev = gen.device
        n = self.H * self.D + self.G * (self.D + self.Dv)
        self.proj_w = _param(_rand(gen, n, hidden, std=1.0 / math.sqrt(hidden), dtype=dtype))
        self.q_norm_w = _param(1.0 + 0.1 * _rand(gen, self.D))
        self.k_norm_w = _param(1.0 + 0.1 * _rand(gen, self.D))
        self.sinks = _param(_rand(gen, self.H)) if m.sink else None
        self.o_w = _param(_rand(gen, hidden, self.H * self.Dv,
                                std=1.0 / math.sqrt(self.H * self.Dv), dtype=dtype))
        self.register_buffer(
            "inv_freq", mx.rotary_inv_freq(m.rot_dims, m.rot_base, m.rot_scaling).to(dev),
            persistent=False)

    def kv_shape(self):
        return (self.G, self.D, self.Dv)

    def state_shapes(self) -> Dict[str, tuple]:
        return {}

    def forward(self, h, sb: mx.SeqBatch, kv, state) -> torch.Tensor:
        k_cache, v_cache = kv
        proj = ops.linear(h, self.proj_w)                     # [T, q|k|v]
        q = mx.attn_rope_prepare(proj, self.q_norm_w, self.k_norm_w, self.inv_freq,
                                 self.H, self.G, self.D, self.Dv, self.eps,
                                 k_cache, v_cache, sb)
        ctx = mx.attention_paged(q, k_cache, v_cache, sb, self.scale,
                                 window=self.window, sinks=self.sinks)
        return ops.linear(ctx, self.o_w)

    def load(self, get, put, p: str) -> None:
        put(self.proj_w, [get(p + "q"), get(p + "k"), get(p + "v")])
        put(self.q_norm_w, [get(p + "q.norm")])
        put(self.k_norm_w, [get(p + "k.norm")])
        if self.sinks is not None:
            put(self.sinks, [get(p + "sink")])
        put(self.o_w, [get(p + "o")])


class ChannelDeltaMixer(nn.Module):
    """Gated delta rule with one decay per head and key channel.

    q, k (kv_heads x dim) and v (heads x vdim) pass a short causal
    convolution and silu; q and k become unit vectors per head (q also times
    dim^-1/2). Per head and token:
        S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
    with g = exp(-exp(A_log) softplus(W_a2 W_a1 h + dt_bias)) per key channel
    and beta = sigmoid(W_b h). o is RMS-normed per head (weight shared by
    heads) and gated by sigmoid(W_g2 W_g1 h). S and the convolution's last
    inputs are per-sequence state (float32).

    Fused projection rows: q | k | v | beta | a1 | g1."""

    def __init__(self, hidden: int, m: MixerSpec, eps: float, dtype, gen):
        super().__init__()
        self.H, self.G, self.D, self.Dv = m.heads, m.kv_heads, m.dim, m.vdim
        self.taps = m.conv
        self.eps = eps
        self.ra = m.decay_rank or max(4, hidden // 16)
        self.rg = m.gate_rank or max(4, hidden // 16)
        H, G, D, Dv = self.H, self.G, self.D, self.Dv
        self.n_conv = 2 * G * D + H * Dv
        std = 1.0 / math.sqrt(hidden)
        dev = gen.device
        self.proj_w = _param(_rand(gen, self.n_conv + H + self.ra + self.rg, hidden,
                                   std=std, dtype=dtype))
        self.conv_w = _param(_rand(gen, self.n_conv, self.taps, std=0.5, dtype=dtype))
        self.a2_w = _param(_rand(gen, H * D, self.ra, std=1.0 / math.sqrt(self.ra), dtype=dtype))
        self.g2_w = _param(_rand(gen, H * Dv, self.rg, std=1.0 / math.sqrt(self.rg), dtype=dtype))
        self.dt_bias = _param((_rand(gen, H * D) - 2.0).to(dtype))
        self.a_log = _param((_rand(gen, H, std=0.5) - 1.0).to(dtype))
        self.norm_w = _param(torch.ones(Dv, dtype=dtype, device=dev))
        self.o_w = _param(_rand(gen, hidden, H * Dv, std=1.0 / math.sqrt(H * Dv), dtype=dtype))

    def kv_shape(self):
        return None

    def state_shapes(self) -> Dict[str, tuple]:
        # S is kept column-major: [head, value column, key row]
        return {"conv": (self.taps - 1, self.n_conv), "S": (self.H, self.Dv, self.D)}

    def forward(self, h, sb: mx.SeqBatch, kv, state) -> torch.Tensor:
        H, G, D, Dv = self.H, self.G, self.D, self.Dv
        proj = ops.linear(h, self.proj_w)
        o0 = self.n_conv
        qkv = mx.causal_conv_seq(proj[:, :o0], self.conv_w, state["conv"], sb,
                                 add_input=False, act_silu=True)
        b_logits = proj[:, o0 : o0 + H]
        a1 = proj[:, o0 + H : o0 + H + self.ra]
        g1 = proj[:, o0 + H + self.ra :]
        a = ops.linear(a1, self.a2_w)                         # [T, H*D]
        gate = ops.linear(g1, self.g2_w)                      # [T, H*Dv]
        y = mx.channel_delta_rule(
            qkv[:, : G * D], qkv[:, G * D : 2 * G * D], qkv[:, 2 * G * D :],
            b_logits, a, self.dt_bias, self.a_log, self.norm_w, gate, state["S"], sb,
            H, G, D, Dv, self.eps)
        return ops.linear(y, self.o_w)


class LatentAttentionMixer(nn.Module):
    """Causal softmax attention whose keys and values are up-projections of
    one cached latent per token. With h the input, per token the cache row
    is [c | r]: c = rms_norm(first kv_rank rows of W_dkv h) (weighted), r =
    the last rot_dim rows rotated by position (one key part for all heads).
    Head h's score is (qu_h . W_uk,h c + qr_h . r) * scale with qu_h the
    `dim` unrotated and qr_h the rot_dim rotated channels of its query; its
    value is W_uv,h c. Because both up-projections are linear they are taken
    to the query side: qu_h^T W_uk,h is a query against c itself, the
    softmax weights average c, and W_uv,h is applied to that average. The
    attention kernel therefore sees ONE key/value head of size kv_rank +
    rot_dim whose values are the first kv_rank key channels, and the cache
    holds nothing else. The softmax normaliser also holds exp(sink_h); each
    head's output is scaled by sigmoid(W_g h)_h.

    A layer with kv_from = j projects no latent: it reads layer j's cache
    rows with its own queries, up-projections, sinks and gates.

    Options, each a MixerSpec field: q_rank > 0 sends the queries through a
    latent of their own, q = W_uq rms_norm(W_dq h) (weighted); sink=False
    leaves the sink term out; gate "channel" multiplies the concatenated head
    outputs elementwise by sigmoid(W_g h) ([heads * vdim] logits) instead of
    one logit per head; rot_layout "half" names the checkpoint's pairing of
    rotated channels (rows are reordered once at load).

    Fused projection rows: q (or dq) | dkv (own latent only) | gate."""

    def __init__(self, hidden: int, m: MixerSpec, eps: float, dtype, gen):
        super().__init__()
        self.H, self.D, self.Dv = m.heads, m.dim, m.vdim
        self.R, self.rot = m.kv_rank, m.rot_dim
        self.kv_source = m.kv_from
        self.own = m.kv_from is None
        self.eps = eps
        self.scale = float(m.scale) if m.scale is not None else (m.dim + m.rot_dim) ** -0.5
        H, D, Dv, R, rot = self.H, self.D, self.Dv, self.R, self.rot
        dev = gen.device
        self.n_q = H * (D + rot)
        self.q_rank = m.q_rank
        self.n_in = m.q_rank or self.n_q          # leading projection rows: dq or q
        self.n_kv = R + rot if self.own else 0
        self.gate = m.gate
        self.layout, self.rot_dims, self.dtype = m.rot_layout, m.rot_dims, dtype
        n_gate = {"head": H, "channel": H * Dv, "none": 0}[m.gate]
        std = 1.0 / math.sqrt(hidden)
        self.proj_w = _param(_rand(gen, self.n_in + self.n_kv + n_gate, hidden, std=std,
                                   dtype=dtype))
        if m.q_rank:
            self.dq_norm_w = _param((1.0 + 0.1 * _rand(gen, m.q_rank)).to(dtype))
            self.uq_w = _param(_rand(gen, self.n_q, m.q_rank, std=m.q_rank ** -0.5, dtype=dtype))
        if self.own:
            self.dkv_norm_w = _param(1.0 + 0.1 * _rand(gen, R))
        # up-projections per head: uk [H, D, R] (W_uk,h as stored), uv [H, Dv, R]
        self.uk_w = _param(_rand(gen, H, D, R, std=1.0 / math.sqrt(R), dtype=dtype))
        self.uv_w = _param(_rand(gen, H, Dv, R, std=1.0 / math.sqrt(R), dtype=dtype))
        self.sinks = _param(_rand(gen, H)) if m.sink else None
        self.o_w = _param(_rand(gen, hidden, H * Dv, std=1.0 / math.sqrt(H * Dv), dtype=dtype))
        self.register_buffer("inv_freq", mx.rotary_inv_freq(m.rot_dims, m.rot_base).to(dev),
                             persistent=False)

    def kv_shape(self):
        # one key head of kv_rank + rot_dim channels; the values are its
        # first kv_rank channels and take no storage of their own
        return (1, self.R + self.rot, self.R, "prefix") if self.own else None

    def state_shapes(self) -> Dict[str, tuple]:
        return {}

    def forward(self, h, sb: mx.SeqBatch, kv, state) -> torch.Tensor:
        k_cache, v_view = kv
        T = h.shape[0]
        H, D, Dv, R, rot = self.H, self.D, self.Dv, self.R, self.rot
        proj = ops.linear(h, self.proj_w)                     # [T, q or dq | dkv | gate]
        n_in = self.n_in
        if self.own:
            mx.latent_kv_prepare(proj[:, n_in : n_in + self.n_kv], self.dkv_norm_w,
                                 self.inv_freq, R, rot, self.eps, k_cache, sb)
        if self.q_rank:
            _, cq = mx.group_rms_norm(proj[:, :n_in], self.dq_norm_w, 1, self.eps)
            q = ops.linear(cq, self.uq_w)
        else:
            q = proj[:, :n_in]
        gate = proj[:, n_in + self.n_kv :]
        # the batched GEMMs over heads read and write token-major rows through
        # strided views: no head-major copies on either side of the attention
        q_un = q.view(T, H, D + rot)[..., :D].transpose(0, 1)  # [H, T, D]
        qf = torch.empty(T, H, R + rot, dtype=proj.dtype, device=proj.device)
        torch.bmm(q_un, self.uk_w, out=qf[..., :R].transpose(0, 1))
        mx.latent_q_assemble(q, None, self.inv_freq, H, D, rot, sb, out=qf)
        ctx = mx.attention_paged(qf, k_cache, v_view, sb, self.scale, sinks=self.sinks,
                                 gate_logits=gate if self.gate == "head" else None)
        val = torch.empty(T, H * Dv, dtype=proj.dtype, device=proj.device)
        torch.bmm(ctx.view(T, H, R).transpose(0, 1), self.uv_w.transpose(1, 2),
                  out=val.view(T, H, Dv).transpose(0, 1))
        if self.gate == "channel":
            val = mx.combine_norm_gate(val, H, Dv, self.dtype, gate_logits=gate)
        return ops.linear(val, self.o_w)

    def load(self, get, put, p: str) -> None:
        D, rot = self.D, self.rot
        relay_q = lambda w: _relayout_heads(w, self.H, D + rot, D, self.rot_dims,  # noqa: E731
                                            self.layout)
        if self.q_rank:
            parts = [get(p + "dq")]
            put(self.dq_norm_w, [get(p + "dq.norm")])
            put(self.uq_w, [relay_q(get(p + "uq"))])
        else:
            parts = [relay_q(get(p + "q"))]
        if self.own:
            parts.append(_relayout_heads(get(p + "dkv"), 1, self.R + rot, self.R,
                                         self.rot_dims, self.layout))
        if self.gate != "none":
            parts.append(get(p + "g"))
        put(self.proj_w, parts)
        if self.own:
            put(self.dkv_norm_w, [get(p + "dkv.norm")])
        self.uk_w.data.copy_(get(p + "uk").reshape(self.H, self.D, self.R)
                             .to(self.uk_w.device, self.uk_w.dtype))
        self.uv_w.data.copy_(get(p + "uv").reshape(self.H, self.Dv, self.R)
                             .to(self.uv_w.device, self.uv_w.dtype))
        if self.sinks is not None:
            put(self.sinks, [get(p + "sink")])
        put(self.o_w, [get(p + "o")])


class DiffAttentionMixer(nn.Module):
    """Differential attention: every head has two query/key maps over the
    same values. q = W_q h (heads x 2 x dim), k = W_k h (kv_heads x 2 x dim),
    v = W_v h (kv_heads x vdim); both maps are rotated by position on their
    first rot_dims channels; score = q . k * scale, optionally soft-capped
    (cap * tanh(score / cap)); each map is a causal softmax attention a_m.
    With lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff (one number for the
    layer), o = a_1 - lambda a_2, divided per head by its root mean square
    over vdim (eps inside the root, no weight), times (1 - diff), times
    sigmoid(W_g h) elementwise.

    The two maps are run as 2 * heads ordinary heads against 2 * kv_heads
    key heads: projection rows are kept map-major ([map, head, dim]) so that
    the grouped-query rule head // (heads / kv_heads) pairs map m of a query
    head with map m of its key head, and the cache holds kv_heads value heads
    which key head g reads as g mod kv_heads.

    Fused projection rows: q | k | v | gate."""

    def __init__(self, hidden: int, m: MixerSpec, eps: float, dtype, gen):
        super().__init__()
        self.H, self.G, self.D, self.Dv = m.heads, m.kv_heads, m.dim, m.vdim
        self.eps, self.dtype = eps, dtype
        self.scale = float(m.scale) if m.scale is not None else m.dim ** -0.5
        self.softcap = m.softcap
        self.diff = float(m.diff if m.diff is not None else 0.0)
        self.layout, self.rot_dims = m.rot_layout, m.rot_dims
        H, G, D, Dv = self.H, self.G, self.D, self.Dv
        dev = gen.device
        self.n_q, self.n_k, self.n_v = 2 * H * D, 2 * G * D, G * Dv
        self.proj_w = _param(_rand(gen, self.n_q + self.n_k + self.n_v + H * Dv, hidden,
                                   std=1.0 / math.sqrt(hidden), dtype=dtype))
        # lq1 | lk1 | lq2 | lk2
        self.lam_w = _param(0.3 * _rand(gen, 4, D))
        self.o_w = _param(_rand(gen, hidden, H * Dv, std=1.0 / math.sqrt(H * Dv), dtype=dtype))
        self.register_buffer("inv_freq", mx.rotary_inv_freq(m.rot_dims, m.rot_base).to(dev),
                             persistent=False)
        self._lam: Optional[float] = None

    def kv_shape(self):
        return (2 * self.G, self.D, self.Dv, "vheads", self.G)

    def state_shapes(self) -> Dict[str, tuple]:
        return {}

    def lam(self) -> float:
        """lambda, from the float32 parameters (a constant of the layer)."""
        if self._lam is None:
            w = self.lam_w.detach().float().cpu()
            self._lam = float(torch.exp((w[0] * w[1]).sum()) - torch.exp((w[2] * w[3]).sum())
                              + self.diff)
        return self._lam

    def forward(self, h, sb: mx.SeqBatch, kv, state) -> torch.Tensor:
        k_cache, v_cache = kv
        H, G, D, Dv = self.H, self.G, self.D, self.Dv
        proj = ops.linear(h, self.proj_w)                     # [T, q | k | v | gate]
        q = mx.attn_rope_prepare(proj, None, None, self.inv_freq, 2 * H, 2 * G, D, Dv, self.eps,
                                 k_cache, v_cache, sb, v_heads=G)
        ctx = mx.attention_paged(q, k_cache, v_cache, sb, self.scale, softcap=self.softcap)
        n = H * Dv                                            # map 1 | map 2
        y = mx.combine_norm_gate(ctx[:, :n], H, Dv, self.dtype, a2=ctx[:, n:], lam=self.lam(),
                                 norm=True, eps=self.eps, post_scale=1.0 - self.diff,
                                 gate_logits=proj[:, self.n_q + self.n_k + self.n_v :])
        return ops.linear(y, self.o_w)

    def load(self, get, put, p: str) -> None:
        def map_major(w, heads):      # [head, map, dim] rows -> [map, head, dim]
            w = _relayout_heads(w, heads * 2, self.D, 0, self.rot_dims, self.layout)
            return w.reshape(heads, 2, self.D, -1).transpose(0, 1).reshape(2 * heads * self.D, -1)

        put(self.proj_w, [map_major(get(p + "q"), self.H), map_major(get(p + "k"), self.G),
                          get(p + "v"), get(p + "g")])
        put(self.lam_w, [get(p + "lq1").reshape(1, -1), get(p + "lk1").reshape(1, -1),
                         get(p + "lq2").reshape(1, -1), get(p + "lk2").reshape(1, -1)])
        self._lam = None
        put(self.o_w, [get(p + "o")])


class RetentionMixer(nn.Module):
    """Retention: linear attention with one fixed decay per head and no
    softmax or denominator. q = W_q h, k = W_k h (heads x dim) are rotated by
    position on their first rot_dims channels, k is scaled by dim^-1/2;
    per head S <- decay_h S + k v^T, o = S^T q with S float32 per-sequence
    state. Each head's o is divided by its root mean square (no weight) and
    the concatenated heads are multiplied by silu(W_g h). Rotation and
    recurrence run on float32 copies of the projections.

    The scale dim^-1/2 is applied to q instead of k: the read-out is linear
    in both, only the stored state differs by that factor.

    Fused projection rows: q | k | v | gate."""

    def __init__(self, hidden: int, m: MixerSpec, eps: float, dtype, gen):
        super().__init__()
        self.H, self.D, self.Dv = m.heads, m.dim, m.vdim
        self.eps, self.dtype = eps, dtype
        self.layout, self.rot_dims = m.rot_layout, m.rot_dims
        H, D, Dv = self.H, self.D, self.Dv
        self.proj_w = _param(_rand(gen, 2 * H * D + 2 * H * Dv, hidden,
                                   std=1.0 / math.sqrt(hidden), dtype=dtype))
        self.o_w = _param(_rand(gen, hidden, H * Dv, std=1.0 / math.sqrt(H * Dv), dtype=dtype))
        self.register_buffer(
            "decay", torch.tensor([float(d) for d in m.decay], dtype=torch.float64)
            .to(torch.float32).to(gen.device), persistent=False)
        self.register_buffer("inv_freq",
                             mx.rotary_inv_freq(m.rot_dims, m.rot_base).to(gen.device),
                             persistent=False)

    def kv_shape(self):
        return None

    def state_shapes(self) -> Dict[str, tuple]:
        return {"S": (self.H, self.Dv, self.D)}      # S transposed: [head, value, key]

    def forward(self, h, sb: mx.SeqBatch, kv, state) -> torch.Tensor:
        H, D, Dv = self.H, self.D, self.Dv
        n, nv = H * D, H * Dv
        proj = ops.linear(h, self.proj_w)
        qkv = mx.rope_rows(proj[:, : 2 * n + nv], 2 * H, D, self.inv_freq, sb)   # float32
        o = mx.decay_linear_attention(qkv[:, :n], qkv[:, n : 2 * n], qkv[:, 2 * n :],
                                      state["S"], sb, H, D, Dv, head_decay=self.decay,
                                      q_scale=D ** -0.5)
        y = mx.combine_norm_gate(o, H, Dv, self.dtype, norm=True, eps=self.eps,
                                 gate_logits=proj[:, 2 * n + nv :], gate_act="silu")
        return ops.linear(y, self.o_w)

    def load(self, get, put, p: str) -> None:
        relay = lambda w: _relayout_heads(w, self.H, self.D, 0, self.rot_dims,  # noqa: E731
                                          self.layout)
        put(self.proj_w, [relay(get(p + "q")), relay(get(p + "k")), get(p + "v"), get(p + "g")])
        put(self.o_w, [get(p + "o")])


class LightningMixer(nn.Module):
    """Linear attention with one fixed decay per head: q, k (heads x dim) and
    v (heads x vdim) pass silu; per head S <- decay_h S + k v^T, o = S^T q
    with S float32 per-sequence state. The concatenated heads are RMS-normed
    as one vector (weight [heads * vdim]) and gated by sigmoid(W_g h).

    Fused projection rows: q | k | v | gate."""

    def __init__(self, hidden: int, m: MixerSpec, eps: float, dtype, gen):
        super().__init__()
        self.H, self.D, self.Dv = m.heads, m.dim, m.vdim
        self.eps, self.dtype = eps, dtype
        H, D, Dv = self.H, self.D, self.Dv
        self.proj_w = _param(_rand(gen, 2 * H * D + 2 * H * Dv, hidden,
                                   std=1.0 / math.sqrt(hidden), dtype=dtype))
        self.norm_w = _param(1.0 + 0.1 * _rand(gen, H * Dv))
        self.o_w = _param(_rand(gen, hidden, H * Dv, std=1.0 / math.sqrt(H * Dv), dtype=dtype))
        self.register_buffer(
            "decay", torch.tensor([float(d) for d in m.decay], dtype=torch.float64)
            .to(torch.float32).to(gen.device), persistent=False)

    def kv_shape(self):
        return None

    def state_shapes(self) -> Dict[str, tuple]:
        return {"S": (self.H, self.Dv, self.D)}      # S transposed: [head, value, key]

    def forward(self, h, sb: mx.SeqBatch, kv, state) -> torch.Tensor:
        n, nv = self.H * self.D, self.H * self.Dv
        proj = ops.linear(h, self.proj_w)
        o = mx.decay_linear_attention(proj[:, :n], proj[:, n : 2 * n], proj[:, 2 * n : 2 * n + nv],
                                      state["S"], sb, self.H, self.D, self.Dv,
                                      head_decay=self.decay, act="silu")
        y = mx.gated_rms_norm(o, self.norm_w, 1, proj[:, 2 * n + nv :], "sigmoid", self.eps,
                              self.dtype)
        return ops.linear(y, self.o_w)

    def load(self, get, put, p: str) -> None:
        put(self.proj_w, [get(p + "q"), get(p + "k"), get(p + "v"), get(p + "g")])
        put(self.norm_w, [get(p + "norm")])
        put(self.o_w, [get(p + "o")])


class GatedLinearAttentionMixer(nn.Module):
    """Linear attention with a learned decay per head and key channel:
    q = W_q h * dim^-1/2, k = W_k h, v = W_v h; a = sigmoid(W_a2 W_a1 h +
    b)^(1/tau) (float32); per head S <- diag(a) S + k v^T, o = S^T q with S
    float32 per-sequence state. Each head's o is RMS-normed over vdim (weight
    [vdim], the same for every head) and gated by silu(W_g h).

    Fused projection rows: q | k | v | gate | a1."""

    def __init__(self, hidden: int, m: MixerSpec, eps: float, dtype, gen):
        super().__init__()
        self.H, self.D, self.Dv = m.heads, m.dim, m.vdim
        self.eps, self.dtype = eps, dtype
        self.inv_tau = 1.0 / float(m.tau)
        self.ra = m.decay_rank or max(4, hidden // 16)
        H, D, Dv = self.H, self.D, self.Dv
        self.proj_w = _param(_rand(gen, 2 * H * D + 2 * H * Dv + self.ra, hidden,
                                   std=1.0 / math.sqrt(hidden), dtype=dtype))
        self.a2_w = _param(_rand(gen, H * D, self.ra, std=1.0 / math.sqrt(self.ra), dtype=dtype))
        self.a2_b = _param(_rand(gen, H * D) + 2.0)
        self.norm_w = _param(1.0 + 0.1 * _rand(gen, Dv))
        self.o_w = _param(_rand(gen, hidden, H * Dv, std=1.0 / math.sqrt(H * Dv), dtype=dtype))

    def kv_shape(self):
        return None

    def state_shapes(self) -> Dict[str, tuple]:
        return {"S": (self.H, self.Dv, self.D)}

    def forward(self, h, sb: mx.SeqBatch, kv, state) -> torch.Tensor:
        n, nv = self.H * self.D, self.H * self.Dv
        proj = ops.linear(h, self.proj_w)
        z = ops.linear(proj[:, 2 * n + 2 * nv :], self.a2_w)  # [T, H*D]
        o = mx.decay_linear_attention(proj[:, :n], proj[:, n : 2 * n], proj[:, 2 * n : 2 * n + nv],
                                      state["S"], sb, self.H, self.D, self.Dv, z=z,
                                      z_bias=self.a2_b, inv_tau=self.inv_tau,
                                      q_scale=self.D ** -0.5)
        y = mx.gated_rms_norm(o, self.norm_w, self.H, proj[:, 2 * n + nv : 2 * n + 2 * nv],
                              "silu", self.eps, self.dtype)
        return ops.linear(y, self.o_w)

    def load(self, get, put, p: str) -> None:
        put(self.proj_w, [get(p + "q"), get(p + "k"), get(p + "v"), get(p + "g"), get(p + "a1")])
        put(self.a2_w, [get(p + "a2")])
        put(self.a2_b, [get(p + "a2.b")])
        put(self.norm_w, [get(p + "norm")])
        put(self.o_w, [get(p + "o")])


MIXERS = {"attention": BiasedAttentionMixer, "channel_delta": ChannelDeltaMixer,
          "rotary_window": RotaryWindowAttentionMixer,
          "latent_attention": LatentAttentionMixer, "lightning": LightningMixer,
          "gla": GatedLinearAttentionMixer, "diff_attention": DiffAttentionMixer,
          "retention": RetentionMixer}


class GatedMLP(nn.Module):
    """down(act(gate x) * (up x)); gate|up fused; act "silu" | "gelu_tanh" |
    ("clamp_swish", limit, alpha)."""

    def __init__(self, hidden: int, ff: int, dtype, gen, act: str = "silu"):
        super().__init__()
        self.ff = ff
        self.act = act
        self.gate_up_w = _param(_rand(gen, 2 * ff, hidden, std=1.0 / math.sqrt(hidden), dtype=dtype))
        self.down_w = _param(_rand(gen, hidden, ff, std=1.0 / math.sqrt(ff), dtype=dtype))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        M, K = x.shape
        if (
            x.is_cuda and x.dtype == torch.bfloat16 and K % 8 == 0 and self.ff % 8 == 0
            and isinstance(self.act, str)
            and (ops._gemv_m_ok(M) or ops._bf16_mfma_ok(M, K, gateup=True))
        ):
            act = ops.gateup_act(x, self.gate_up_w, self.ff, self.act)   # fused decode GEMV
        else:
            act = mx.act_mul_rows(ops.linear(x, self.gate_up_w), self.ff, self.act)
        return ops.linear(act, self.down_w)

    def load(self, get, put, p: str) -> None:
        put(self.gate_up_w, [get(p + "gate"), get(p + "up")])
        put(self.down_w, [get(p + "down")])


class PlainMLP(nn.Module):
    """down(act(up x)) without a gate branch; act "relu2" (the square of
    relu) | "silu" | "gelu_tanh"."""

    def __init__(self, hidden: int, ff: int, dtype, gen, act: str = "relu2"):
        super().__init__()
        self.ff, self.act = ff, act
        self.up_w = _param(_rand(gen, ff, hidden, std=1.0 / math.sqrt(hidden), dtype=dtype))
        self.down_w = _param(_rand(gen, hidden, ff, std=1.0 / math.sqrt(ff), dtype=dtype))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.linear(mx.act_rows(ops.linear(x, self.up_w), self.act), self.down_w)

    def load(self, get, put, p: str) -> None:
        put(self.up_w, [get(p + "up")])
        put(self.down_w, [get(p + "down")])


class HybridLayer(nn.Module):
    def __init__(self, spec: HybridSpec, ls: HybridLayerSpec, dtype, gen):
        super().__init__()
        C = spec.hidden_size
        self.groups, self.eps = spec.norm_groups, spec.norm_eps
        self.canon_w = _param(_rand(gen, C, spec.canon_taps, std=0.2, dtype=dtype))
        self.mixer = MIXERS[ls.mixer.kind](C, ls.mixer, spec.norm_eps, dtype, gen)
        self.norm1_w = _param(torch.ones(C, dtype=dtype, device=gen.device))
        self.mlp: Optional[GatedMLP] = None
        if ls.mlp_kind is not None:
            self.mlp = GatedMLP(C, ls.mlp_ff, dtype, gen)
            self.norm2_w = _param(torch.ones(C, dtype=dtype, device=gen.device))

    def state_shapes(self) -> Dict[str, tuple]:
        shapes = dict(self.mixer.state_shapes())
        shapes["canon"] = (self.canon_w.shape[1] - 1, self.canon_w.shape[0])
        return shapes

    def forward(self, x: torch.Tensor, sb: mx.SeqBatch, kv, state) -> torch.Tensor:
        """x: float32 residual [T, C], updated in place and returned."""
        h = mx.causal_conv_seq(x, self.canon_w, state["canon"], sb,
                               add_input=True, act_silu=False)
        y = self.mixer(h, sb, kv, state)
        narrow = self.mlp is not None and self.norm1_w.dtype != torch.float32
        x, copy = mx.group_rms_norm(y, self.norm1_w, self.groups, self.eps,
                                    residual=x, want_copy=narrow)
        if self.mlp is not None:
            m = self.mlp(copy if narrow else x)
            x, _ = mx.group_rms_norm(m, self.norm2_w, self.groups, self.eps,
                                     residual=x, want_copy=False)
        return x


class DyTNorm(nn.Module):
    """Dynamic-tanh norm tanh(a x) w + b: weight and bias per channel, one
    scalar a; float32 parameters whatever the model's type."""

    def __init__(self, width: int, gen, alpha: float = 0.5):
        super().__init__()
        dev = gen.device
        self.w = _param(torch.ones(width, device=dev) + 0.05 * _rand(gen, width))
        self.b = _param(0.02 * _rand(gen, width))
        self.alpha = _param(torch.full((1,), float(alpha), device=dev))

    def params(self):
        return (self.w, self.b, self.alpha)

    def load(self, get, put, name: str) -> None:
        put(self.w, [get(name)])
        put(self.b, [get(name + ".b")])
        put(self.alpha, [get(name + ".alpha").reshape(1)])


class SandwichLayer(nn.Module):
    """x <- x + post1(mixer(pre1(x)));  x <- x + post2(ff(pre2(x))) with
    dynamic-tanh norms. The add after a sublayer and the norm before the
    next one (also the next layer's) are one launch: forward takes the
    already-normed mixer input and returns the next layer's."""

    def __init__(self, spec: HybridSpec, ls: HybridLayerSpec, dtype, gen):
        super().__init__()
        C = spec.hidden_size
        self.dtype = dtype
        self.pre1, self.post1 = DyTNorm(C, gen), DyTNorm(C, gen)
        self.mixer = MIXERS[ls.mixer.kind](C, ls.mixer, spec.norm_eps, dtype, gen)
        self.mlp = None
        if ls.mlp_kind == "dense":
            self.mlp = GatedMLP(C, ls.mlp_ff, dtype, gen, act=ls.mlp_act)
        elif ls.mlp_kind == "moe":
            from opsagent_amd.engine.moe import RoutedExperts

            self.mlp = RoutedExperts(C, ls.router, dtype, gen)
        self.routed = ls.mlp_kind == "moe"
        if self.mlp is not None:
            self.pre2, self.post2 = DyTNorm(C, gen), DyTNorm(C, gen)

    def state_shapes(self) -> Dict[str, tuple]:
        return dict(self.mixer.state_shapes())

    def first_norm(self):
        return self.pre1.params()

    def forward(self, x, h, sb: mx.SeqBatch, kv, state, next_norm):
        """x: float32 residual [T, C] (updated in place); h = pre1(x).
        next_norm: the following layer's first norm (None after the last
        layer). Returns (x, next layer's h or None)."""
        y = self.mixer(h, sb, kv, state)
        if self.mlp is None:
            return x, mx.dyt_norm(x, next_norm, self.dtype, y=y, post=self.post1.params())
        h2 = mx.dyt_norm(x, self.pre2.params(), self.dtype, y=y, post=self.post1.params())
        m = self.mlp(h2, decode=sb.max_chunk == 1) if self.routed else self.mlp(h2)
        return x, mx.dyt_norm(x, next_norm, self.dtype, y=m, post=self.post2.params())

    def load(self, get, put, p: str) -> None:
        self.pre1.load(get, put, p + "norm1")
        self.post1.load(get, put, p + "norm1b")
        self.mixer.load(get, put, p + "mix.")
        if self.mlp is not None:
            self.pre2.load(get, put, p + "norm2")
            self.post2.load(get, put, p + "norm2b")
            self.mlp.load(get, put, p + "mlp.")


class PreNormLayer(nn.Module):
    """x <- x + mixer(ln1(x));  x <- x + ff(ln2(x)) with weighted layer norms
    (no bias; float32 weights and statistics). The add after a sublayer and
    the norm before the next one (also the next layer's) are one launch:
    forward takes the already-normed mixer input and returns the next
    layer's. A routed feed-forward hands its routed sum, its shared expert's
    output and that expert's gate logits to the same launch."""

    def __init__(self, spec: HybridSpec, ls: HybridLayerSpec, dtype, gen):
        super().__init__()
        C = spec.hidden_size
        self.dtype, self.eps = dtype, spec.norm_eps
        self.norm1_w = _param(1.0 + 0.05 * _rand(gen, C))
        self.mixer = MIXERS[ls.mixer.kind](C, ls.mixer, spec.norm_eps, dtype, gen)
        self.mlp = None
        if ls.mlp_kind == "dense":
            self.mlp = GatedMLP(C, ls.mlp_ff, dtype, gen, act=ls.mlp_act)
        elif ls.mlp_kind == "moe":
            from opsagent_amd.engine.moe import RoutedExperts

            self.mlp = RoutedExperts(C, ls.router, dtype, gen)
        self.routed = ls.mlp_kind == "moe"
        if self.mlp is not None:
            self.norm2_w = _param(1.0 + 0.05 * _rand(gen, C))

    def state_shapes(self) -> Dict[str, tuple]:
        return dict(self.mixer.state_shapes())

    def first_norm(self):
        return self.norm1_w

    def forward(self, x, h, sb: mx.SeqBatch, kv, state, next_norm):
        """x: float32 residual [T, C] (updated in place); h = ln1(x).
        next_norm: the following layer's first norm weight (None after the
        last layer). Returns (x, next layer's h or None)."""
        y = self.mixer(h, sb, kv, state)
        if self.mlp is None:
            return x, mx.add_layer_norm(x, next_norm, self.eps, self.dtype, y=y)
        h2 = mx.add_layer_norm(x, self.norm2_w, self.eps, self.dtype, y=y)
        if self.routed:
            m, shared, gate = self.mlp.forward_parts(h2, decode=sb.max_chunk == 1)
            return x, mx.add_layer_norm(x, next_norm, self.eps, self.dtype, y=m, y2=shared,
                                        y2_gate=gate)
        return x, mx.add_layer_norm(x, next_norm, self.eps, self.dtype, y=self.mlp(h2))

    def load(self, get, put, p: str) -> None:
        put(self.norm1_w, [get(p + "norm1")])
        self.mixer.load(get, put, p + "mix.")
        if self.mlp is not None:
            put(self.norm2_w, [get(p + "norm2")])
            self.mlp.load(get, put, p + "mlp.")


class HyperLayer(nn.Module):
    """Pre-norm sublayers on S hyper-connected residual streams. Sublayer q
    (1: mixer, 2: feed-forward) reads u = sum_s in_q[s] x_s, computes
    y = sublayer(layer_norm(u)) (weight and bias), and writes every stream
    from the old ones: x_t <- sum_s mix_q[s, t] x_s + out_q[t] y. The write
    of one sublayer and the read and norm of the next (also the next
    layer's) are one launch: forward takes the already-normed mixer input
    and returns the next layer's. Without learned coefficients (hyper=False)
    all of them are 1 on a single stream: the plain residual sum."""

    def __init__(self, spec: HybridSpec, ls: HybridLayerSpec, dtype, gen):
        super().__init__()
        C, S = spec.hidden_size, spec.streams
        dev = gen.device
        self.dtype, self.eps, self.hyper = dtype, spec.norm_eps, spec.hyper
        self.norm1_w = _param(1.0 + 0.05 * _rand(gen, C))
        self.norm1_b = _param(0.02 * _rand(gen, C))
        self.mixer = MIXERS[ls.mixer.kind](C, ls.mixer, spec.norm_eps, dtype, gen)
        self.mlp = None
        if ls.mlp_kind == "moe":
            from opsagent_amd.engine.moe import RoutedExperts

            self.mlp = RoutedExperts(C, ls.router, dtype, gen)
        elif ls.mlp_kind is not None:
            raise ValueError(f"hyper layers take routed feed-forwards, not {ls.mlp_kind!r}")

        def coeffs(q):
            if spec.hyper:
                rd = _param(1.0 / S + 0.1 * _rand(gen, S))
                wr = _param(1.0 + 0.1 * _rand(gen, S))
                mix = _param(torch.eye(S, device=dev) + 0.1 * _rand(gen, S, S))
            else:
                rd, wr = _param(torch.ones(S, device=dev)), _param(torch.ones(S, device=dev))
                mix = _param(torch.eye(S, device=dev))
            setattr(self, f"hc{q}_in", rd)
            setattr(self, f"hc{q}_out", wr)
            setattr(self, f"hc{q}_mix", mix)

        coeffs(1)
        if self.mlp is not None:
            self.norm2_w = _param(1.0 + 0.05 * _rand(gen, C))
            self.norm2_b = _param(0.02 * _rand(gen, C))
            coeffs(2)

    def state_shapes(self) -> Dict[str, tuple]:
        return dict(self.mixer.state_shapes())

    def first_read(self):
        return self.hc1_in, self.norm1_w, self.norm1_b

    def forward(self, xs, h, sb: mx.SeqBatch, kv, state, nxt):
        """xs: float32 streams [T, S, C] (updated in place); h: the normed
        read of this layer's mixer. nxt: (read, w, b) of what follows (None
        after the last layer). Returns the next normed read or None."""
        rd, w, b = nxt if nxt is not None else (None, None, None)
        y = self.mixer(h, sb, kv, state)
        if self.mlp is None:
            return mx.hyper_norm(xs, rd, w, b, self.eps, self.dtype, y=y, mix=self.hc1_mix,
                                 write=self.hc1_out)
        h2 = mx.hyper_norm(xs, self.hc2_in, self.norm2_w, self.norm2_b, self.eps, self.dtype,
                           y=y, mix=self.hc1_mix, write=self.hc1_out)
        m, shared, gate = self.mlp.forward_parts(h2, decode=sb.max_chunk == 1)
        return mx.hyper_norm(xs, rd, w, b, self.eps, self.dtype, y=m, mix=self.hc2_mix,
                             write=self.hc2_out, y2=shared, y2_gate=gate)

    def load(self, get, put, p: str) -> None:
        put(self.norm1_w, [get(p + "norm1")])
        put(self.norm1_b, [get(p + "norm1.b")])
        self.mixer.load(get, put, p + "mix.")
        subs = [1]
        if self.mlp is not None:
            put(self.norm2_w, [get(p + "norm2")])
            put(self.norm2_b, [get(p + "norm2.b")])
            self.mlp.load(get, put, p + "mlp.")
            subs.append(2)
        if self.hyper:
            for q in subs:
                put(getattr(self, f"hc{q}_in"), [get(f"{p}hc{q}.in")])
                put(getattr(self, f"hc{q}_out"), [get(f"{p}hc{q}.out")])
                put(getattr(self, f"hc{q}_mix"), [get(f"{p}hc{q}.mix")])


LAYER_STYLES = {"post_canon": HybridLayer, "sandwich": SandwichLayer, "pre_norm": PreNormLayer,
                "hyper": HyperLayer}


class HybridForCausalLM(nn.Module):
    """Embedding -> hybrid layers -> final norm -> head (-> soft cap)."""

    def __init__(self, spec: HybridSpec, dtype: torch.dtype = torch.bfloat16,
                 device: str = "cpu", seed: int = 1234):
        super().__init__()
        if get_tp_size() != 1:
            raise NotImplementedError("hybrid decoders run at tensor-parallel size 1")
        self.spec = spec
        self.dtype = dtype
        gen = torch.Generator(device=device).manual_seed(seed)
        C = spec.hidden_size
        self.embed = _param(_rand(gen, spec.vocab_size, C, dtype=dtype))
        self.sandwich = spec.layer_style == "sandwich"
        self.pre_norm = spec.layer_style == "pre_norm"
        self.hyper = spec.layer_style == "hyper"
        # the order the layers run in (a looped layer once per pass); caches
        # and state are kept per RUN, weights per layer
        self.runs = spec.layer_runs()
        self.layers = nn.ModuleList(
            [LAYER_STYLES[spec.layer_style](spec, ls, dtype, gen) for ls in spec.layers]
        )
        if self.sandwich:
            self.final_norm = DyTNorm(C, gen)
        elif self.hyper:
            self.final_norm_w = _param(torch.ones(C, device=device))
            self.final_norm_b = _param(torch.zeros(C, device=device))
            self.register_buffer("sum_read", torch.ones(spec.streams, device=device),
                                 persistent=False)
            self.register_buffer("one_read", torch.ones(1, device=device), persistent=False)
        elif self.pre_norm:
            self.final_norm_w = _param(torch.ones(C, device=device))
        else:
            self.final_norm_w = _param(torch.ones(C, dtype=dtype, device=device))
        # layer i reads the cache of layer kv_source[i] (its own unless its
        # mixer names another layer)
        self.kv_source = [getattr(layer.mixer, "kv_source", None) for layer in self.layers]
        if spec.tied_head:
            self.lm_head = self.embed           # the head IS the embedding table
        else:
            self.lm_head = _param(_rand(gen, spec.vocab_size, C, std=1.0 / math.sqrt(C),
                                        dtype=dtype))
        self.vocab_local = spec.vocab_size
        self.to(device)
        # residual stream after every layer of the last forward (debug aid)
        self.trace_layers: Optional[List[torch.Tensor]] = None

    # -- cache geometry the engine sizes its pools from ---------------------
    def kv_layer_shapes(self):
        return [self.layers[i].mixer.kv_shape() for i in self.runs]

    def state_layer_shapes(self) -> List[Dict[str, tuple]]:
        return [self.layers[i].state_shapes() for i in self.runs]

    def forward(self, fb: ForwardBatch, kv_caches, state=None) -> torch.Tensor:
        sb = fb.seq_batch
        assert sb is not None and state is not None, "hybrid models run flat multi-sequence steps"
        x = mx.embed_rows(self.embed, fb.input_ids, self.spec.embed_scale)
        if self.hyper:
            S, eps = self.spec.streams, self.spec.norm_eps
            # every stream starts as the embedding output
            xs = x.unsqueeze(1).expand(-1, S, -1).contiguous() if S > 1 else x.unsqueeze(1)
            rd, w, b = self.layers[self.runs[0]].first_read()
            h = mx.hyper_norm(xs, rd, w, b, eps, self.dtype)
            for r, i in enumerate(self.runs):
                nxt = self.layers[self.runs[r + 1]].first_read() if r + 1 < len(self.runs) else None
                h = self.layers[i](xs, h, sb, kv_caches[r], state[r], nxt)
                if self.trace_layers is not None:
                    self.trace_layers.append(xs.sum(1))
            return xs.sum(1) if S > 1 else xs.squeeze(1)
        if self.sandwich or self.pre_norm:
            n = len(self.layers)
            if self.sandwich:
                h = mx.dyt_norm(x, self.layers[0].first_norm(), self.dtype)
            else:
                h = mx.add_layer_norm(x, self.layers[0].first_norm(), self.spec.norm_eps,
                                      self.dtype)
            for i, layer in enumerate(self.layers):
                nxt = self.layers[i + 1].first_norm() if i + 1 < n else None
                src = self.kv_source[i]
                x, h = layer(x, h, sb, kv_caches[i if src is None else src], state[i], nxt)
                if self.trace_layers is not None:
                    self.trace_layers.append(x.clone())
            return x
        for i, layer in enumerate(self.layers):
            x = layer(x, sb, kv_caches[i], state[i])
            if self.trace_layers is not None:
                self.trace_layers.append(x.clone())
        return x  # float32 residual [T, C]; compute_logits norms the rows it needs

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """hidden: float32 residual rows. Returns float32 logits (soft-capped
        if the design caps them)."""
        if self.sandwich:
            normed = mx.dyt_norm(hidden.contiguous(), self.final_norm.params(), self.dtype)
        elif self.hyper:
            normed = mx.hyper_norm(hidden.contiguous().unsqueeze(1), self.one_read,
                                   self.final_norm_w, self.final_norm_b, self.spec.norm_eps,
                                   self.dtype)
        elif self.pre_norm:
            normed = mx.add_layer_norm(hidden.contiguous(), self.final_norm_w,
                                       self.spec.norm_eps, self.dtype)
        else:
            _, normed = mx.group_rms_norm(hidden, self.final_norm_w, self.spec.norm_groups,
                                          self.spec.norm_eps, residual=None)
        logits = ops.linear(normed, self.lm_head)
        if self.spec.logit_scale != 1.0:
            return logits.float() * self.spec.logit_scale
        if self.spec.logit_softcap is None:
            return logits.float()
        return mx.softcap(logits, self.spec.logit_softcap)

    # -- checkpoint names ----------------------------------------------------
    @torch.no_grad()
    def load_named_tensors(self, tensors: Dict[str, torch.Tensor]) -> int:
        """Fill the parameters from a checkpoint under the design's tensor
        names (embed, l<i>.norm1, l<i>.mix.q, ..., final.norm, head)."""
        n = 0
        dev, dtype = self.embed.device, self.dtype

        def put(param, parts):
            nonlocal n
            t = torch.cat([p.reshape(p.shape[0], -1) if param.dim() == 2 else p.reshape(-1)
                           for p in parts], 0)
            assert tuple(t.shape) == tuple(param.shape), (tuple(t.shape), tuple(param.shape))
            # float32 parameters (norms, sinks, routers) stay float32
            param.data.copy_(t.to(device=dev, dtype=param.dtype))
            n += len(parts)

        def get(name):
            if name not in tensors:
                raise KeyError(f"checkpoint has no tensor {name!r}")
            return tensors[name]

        put(self.embed, [get("embed")])
        if not self.spec.tied_head:
            put(self.lm_head, [get("head")])
        if self.hyper:
            put(self.final_norm_w, [get("final.norm")])
            put(self.final_norm_b, [get("final.norm.b")])
            for i, layer in enumerate(self.layers):
                layer.load(get, put, f"l{i}.")
            return n
        if self.sandwich or self.pre_norm:
            if self.sandwich:
                self.final_norm.load(get, put, "final.norm")
            else:
                put(self.final_norm_w, [get("final.norm")])
            for i, layer in enumerate(self.layers):
                layer.load(get, put, f"l{i}.")
            return n
        put(self.final_norm_w, [get("final.norm")])
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            put(layer.norm1_w, [get(p + "norm1")])
            put(layer.canon_w, [get(p + "canon1")])
            mixer = layer.mixer
            if isinstance(mixer, BiasedAttentionMixer):
                put(mixer.proj_w, [get(p + "mix.q"), get(p + "mix.k"), get(p + "mix.v"),
                                   get(p + "mix.g")])
                put(mixer.proj_b, [get(p + "mix.q.b"), get(p + "mix.k.b"), get(p + "mix.v.b")])
                put(mixer.q_norm_w, [get(p + "mix.q.norm")])
                put(mixer.k_norm_w, [get(p + "mix.k.norm")])
                put(mixer.o_w, [get(p + "mix.o")])
            else:
                put(mixer.proj_w, [get(p + "mix.q"), get(p + "mix.k"), get(p + "mix.v"),
                                   get(p + "mix.b"), get(p + "mix.a1"), get(p + "mix.g1")])
                put(mixer.conv_w, [get(p + "mix.q.conv"), get(p + "mix.k.conv"),
                                   get(p + "mix.v.conv")])
                put(mixer.a2_w, [get(p + "mix.a2")])
                put(mixer.g2_w, [get(p + "mix.g2")])
                put(mixer.dt_bias, [get(p + "mix.dt_bias")])
                put(mixer.a_log, [get(p + "mix.A_log")])
                put(mixer.norm_w, [get(p + "mix.norm")])
                put(mixer.o_w, [get(p + "mix.o")])
            if layer.mlp is not None:
                put(layer.norm2_w, [get(p + "norm2")])
                put(layer.mlp.gate_up_w, [get(p + "mlp.gate"), get(p + "mlp.up")])
                put(layer.mlp.down_w, [get(p + "mlp.down")])
        return n
