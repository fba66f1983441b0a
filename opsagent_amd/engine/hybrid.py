"""Hybrid decoders: a per-layer choice of token mixer and feed-forward
around a float32 residual stream, in two layer styles.

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

    Fused projection rows: q | dkv (own latent only) | gate."""

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
        self.n_kv = R + rot if self.own else 0
        std = 1.0 / math.sqrt(hidden)
        self.proj_w = _param(_rand(gen, self.n_q + self.n_kv + H, hidden, std=std, dtype=dtype))
        if self.own:
            self.dkv_norm_w = _param(1.0 + 0.1 * _rand(gen, R))
        # up-projections per head: uk [H, D, R] (W_uk,h as stored), uv [H, Dv, R]
        self.uk_w = _param(_rand(gen, H, D, R, std=1.0 / math.sqrt(R), dtype=dtype))
        self.uv_w = _param(_rand(gen, H, Dv, R, std=1.0 / math.sqrt(R), dtype=dtype))
        self.sinks = _param(_rand(gen, H))
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
        proj = ops.linear(h, self.proj_w)                     # [T, q | dkv | gate]
        if self.own:
            mx.latent_kv_prepare(proj[:, self.n_q : self.n_q + self.n_kv], self.dkv_norm_w,
                                 self.inv_freq, R, rot, self.eps, k_cache, sb)
        q = proj[:, : self.n_q]
        # the batched GEMMs over heads read and write token-major rows through
        # strided views: no head-major copies on either side of the attention
        q_un = q.view(T, H, D + rot)[..., :D].transpose(0, 1)  # [H, T, D]
        qf = torch.empty(T, H, R + rot, dtype=proj.dtype, device=proj.device)
        torch.bmm(q_un, self.uk_w, out=qf[..., :R].transpose(0, 1))
        mx.latent_q_assemble(q, None, self.inv_freq, H, D, rot, sb, out=qf)
        ctx = mx.attention_paged(qf, k_cache, v_view, sb, self.scale, sinks=self.sinks,
                                 gate_logits=proj[:, self.n_q + self.n_kv :])
        val = torch.empty(T, H * Dv, dtype=proj.dtype, device=proj.device)
        torch.bmm(ctx.view(T, H, R).transpose(0, 1), self.uv_w.transpose(1, 2),
                  out=val.view(T, H, Dv).transpose(0, 1))
        return ops.linear(val, self.o_w)

    def load(self, get, put, p: str) -> None:
        parts = [get(p + "q")] + ([get(p + "dkv")] if self.own else []) + [get(p + "g")]
        put(self.proj_w, parts)
        if self.own:
            put(self.dkv_norm_w, [get(p + "dkv.norm")])
        self.uk_w.data.copy_(get(p + "uk").reshape(self.H, self.D, self.R)
                             .to(self.uk_w.device, self.uk_w.dtype))
        self.uv_w.data.copy_(get(p + "uv").reshape(self.H, self.Dv, self.R)
                             .to(self.uv_w.device, self.uv_w.dtype))
        put(self.sinks, [get(p + "sink")])
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
          "gla": GatedLinearAttentionMixer}


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


LAYER_STYLES = {"post_canon": HybridLayer, "sandwich": SandwichLayer, "pre_norm": PreNormLayer}


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
        self.layers = nn.ModuleList(
            [LAYER_STYLES[spec.layer_style](spec, ls, dtype, gen) for ls in spec.layers]
        )
        if self.sandwich:
            self.final_norm = DyTNorm(C, gen)
        elif self.pre_norm:
            self.final_norm_w = _param(torch.ones(C, device=device))
        else:
            self.final_norm_w = _param(torch.ones(C, dtype=dtype, device=device))
        # layer i reads the cache of layer kv_source[i] (its own unless its
        # mixer names another layer)
        self.kv_source = [getattr(layer.mixer, "kv_source", None) for layer in self.layers]
        self.lm_head = _param(_rand(gen, spec.vocab_size, C, std=1.0 / math.sqrt(C), dtype=dtype))
        self.vocab_local = spec.vocab_size
        self.to(device)
        # residual stream after every layer of the last forward (debug aid)
        self.trace_layers: Optional[List[torch.Tensor]] = None

    # -- cache geometry the engine sizes its pools from ---------------------
    def kv_layer_shapes(self):
        return [layer.mixer.kv_shape() for layer in self.layers]

    def state_layer_shapes(self) -> List[Dict[str, tuple]]:
        return [layer.state_shapes() for layer in self.layers]

    def forward(self, fb: ForwardBatch, kv_caches, state=None) -> torch.Tensor:
        sb = fb.seq_batch
        assert sb is not None and state is not None, "hybrid models run flat multi-sequence steps"
        x = mx.embed_rows(self.embed, fb.input_ids, self.spec.embed_scale)
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
        elif self.pre_norm:
            normed = mx.add_layer_norm(hidden.contiguous(), self.final_norm_w,
                                       self.spec.norm_eps, self.dtype)
        else:
            _, normed = mx.group_rms_norm(hidden, self.final_norm_w, self.spec.norm_groups,
                                          self.spec.norm_eps, residual=None)
        logits = ops.linear(normed, self.lm_head)
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
        put(self.lm_head, [get("head")])
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
