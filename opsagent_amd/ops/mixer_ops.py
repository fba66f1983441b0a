"""Dispatch of the sequence-mixer ops of hybrid decoders: GPU -> the HIP
kernels of mixers.hip (loud failure if the library is missing), CPU ->
torch_ref. All ops take a SeqBatch: T new tokens of B sequences laid end to
end, each continuing its sequence from its own past length, so a prompt
portion and a decoded token are one case.

Activations and weights are bfloat16 or float32 (`dt`); norms, scores,
softmax weights, decays, gates, recurrent state and the residual are float32
in both.
"""

from __future__ import annotations

import ctypes
import dataclasses
import os
from typing import List, Optional, Tuple

import torch

from opsagent_amd.ops import torch_ref


@dataclasses.dataclass
class SeqBatch:
    """Geometry of one flat multi-sequence step. Host lists mirror the
    device tensors (launch geometry and the CPU path read the lists)."""

    cu: List[int]                 # [B+1] token offsets
    past: List[int]               # [B] tokens already in cache/state
    slots: List[int]              # [B] state-slot rows
    cu_t: torch.Tensor            # int32 [B+1]
    past_t: torch.Tensor          # int32 [B]
    slots_t: torch.Tensor         # int32 [B]
    seq_of_t: torch.Tensor        # int32 [T]
    slot_mapping: torch.Tensor    # int32 [T] flat kv-cache slot per token
    block_table: torch.Tensor     # int32 [B, max_blocks]
    # upper bounds used for launch geometry; a captured graph keeps them
    max_chunk: int = 0
    max_total: int = 0

    @property
    def num_seqs(self) -> int:
        return len(self.cu) - 1

    @property
    def num_tokens(self) -> int:
        return self.cu[-1]

    @staticmethod
    def build(chunks: List[Tuple[int, int, int, List[int]]], block_size: int,
              device, max_blocks: Optional[int] = None) -> "SeqBatch":
        """chunks: per sequence (past_len, count, state_slot, block ids)."""
        cu, past, slots, seq_of, slot_map, bt = [0], [], [], [], [], []
        nb = max((len(c[3]) for c in chunks), default=1)
        max_blocks = max(max_blocks or 0, nb, 1)
        for b, (p, n, slot, blocks) in enumerate(chunks):
            cu.append(cu[-1] + n)
            past.append(p)
            slots.append(slot if slot is not None else 0)
            seq_of.extend([b] * n)
            for pos in range(p, p + n):
                slot_map.append(blocks[pos // block_size] * block_size + pos % block_size)
            bt.extend(blocks)
            bt.extend([0] * (max_blocks - len(blocks)))
        # one host->device copy; the tensors are views of it
        B, T = len(chunks), cu[-1]
        flat = torch.tensor(cu + past + slots + seq_of + slot_map + bt,
                            dtype=torch.int32).to(device)
        o1, o2, o3, o4, o5 = B + 1, 2 * B + 1, 3 * B + 1, 3 * B + 1 + T, 3 * B + 1 + 2 * T
        return SeqBatch(
            cu=cu, past=past, slots=slots, cu_t=flat[:o1], past_t=flat[o1:o2],
            slots_t=flat[o2:o3], seq_of_t=flat[o3:o4], slot_mapping=flat[o4:o5],
            block_table=flat[o5:].view(B, max_blocks),
            max_chunk=max((c[1] for c in chunks), default=0),
            max_total=max((c[0] + c[1] for c in chunks), default=0),
        )


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return 0
    if t.dtype == torch.float32:
        return 1
    raise TypeError(f"unsupported activation type {t.dtype}")


def _lib():
    from opsagent_amd.ops import hip_lib

    return hip_lib.get_mixers_lib(), hip_lib


def _rows(t: torch.Tensor) -> int:
    """Row stride of a 2-D view whose rows are contiguous."""
    assert t.dim() == 2 and (t.shape[1] == 1 or t.stride(1) == 1), "rows must be contiguous"
    return t.stride(0)


def embed_rows(table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """table[ids] * scale as a float32 residual stream [T, C]."""
    if not table.is_cuda:
        return table[ids].float() * scale if scale != 1.0 else table[ids].float()
    lib, hip = _lib()
    T, C = ids.shape[0], table.shape[1]
    out = torch.empty(T, C, dtype=torch.float32, device=table.device)
    assert ids.dtype == torch.int64 and table.is_contiguous()
    hip.check(lib.oa_embed_rows(hip.current_stream_ptr(), table.data_ptr(), ids.data_ptr(),
                                out.data_ptr(), T, C, _dt(table), float(scale)), "oa_embed_rows")
    return out


def causal_conv_seq(x: torch.Tensor, w: torch.Tensor, state: torch.Tensor, sb: SeqBatch,
                    add_input: bool, act_silu: bool) -> torch.Tensor:
    """(x +) causal per-channel convolution over time (-> silu), continued
    from and carried into state [slots, taps-1, C] float32. x [T, C] may be a
    column slice of a wider buffer; out has w's type."""
    T, C = x.shape
    taps = w.shape[1]
    assert w.shape[0] == C and state.shape[1:] == (taps - 1, C)
    if not x.is_cuda:
        return torch_ref.causal_conv_seq(x, w, state, sb.cu, sb.past, sb.slots,
                                         add_input, act_silu, w.dtype)
    lib, hip = _lib()
    out = torch.empty(T, C, dtype=w.dtype, device=x.device)
    assert w.is_contiguous() and state.is_contiguous() and state.dtype == torch.float32
    rc = lib.oa_causal_conv_seq(
        hip.current_stream_ptr(), x.data_ptr(), _rows(x), _dt(x), w.data_ptr(),
        state.data_ptr(), out.data_ptr(), C, sb.seq_of_t.data_ptr(), sb.cu_t.data_ptr(),
        sb.past_t.data_ptr(), sb.slots_t.data_ptr(), T, sb.num_seqs, C, taps,
        int(add_input), int(act_silu), _dt(w), sb.max_chunk)
    hip.check(rc, "oa_causal_conv_seq")
    return out


def group_rms_norm(y: torch.Tensor, w: torch.Tensor, groups: int, eps: float,
                   residual: Optional[torch.Tensor] = None,
                   want_copy: bool = True) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
    """RMS norm over `groups` consecutive parts, times w. With `residual`
    (float32 [T, C], updated in place): residual += norm. Returns (residual,
    copy) where copy is the result in w's type (None unless want_copy)."""
    T, C = y.shape
    if not y.is_cuda:
        if residual is not None:
            r = torch_ref.group_rms_norm(y, w, groups, eps, residual, w.dtype)
            return r, (r.to(w.dtype) if want_copy else None)
        return None, torch_ref.group_rms_norm(y, w, groups, eps, None, w.dtype)
    lib, hip = _lib()
    copy = torch.empty(T, C, dtype=w.dtype, device=y.device) if (want_copy or residual is None) else None
    if residual is not None:
        assert residual.dtype == torch.float32 and residual.is_contiguous()
    rc = lib.oa_group_rmsnorm(
        hip.current_stream_ptr(), y.data_ptr(), _rows(y), _dt(y), w.data_ptr(),
        residual.data_ptr() if residual is not None else None,
        copy.data_ptr() if copy is not None else None, T, C, groups, eps, _dt(w))
    hip.check(rc, "oa_group_rmsnorm")
    return residual, copy


def attn_qkv_prepare(qkv: torch.Tensor, bias: Optional[torch.Tensor], q_norm_w: torch.Tensor, k_norm_w: torch.Tensor,
                     H: int, G: int, D: int, Dv: int, eps: float, k_cache: torch.Tensor,
                     v_cache: torch.Tensor, sb: SeqBatch) -> torch.Tensor:
    """qkv [T, >= H*D + G*D + G*Dv] (q | k | v columns first; bias over these
    columns is added first, if given). Norms q and k over their whole
    projections, v per head; writes k, v to the paged cache; returns q
    [T, H, D]."""
    T = qkv.shape[0]
    if not qkv.is_cuda:
        return torch_ref.attn_qkv_prepare(qkv, bias, q_norm_w, k_norm_w, H, G, D, Dv, eps,
                                          k_cache, v_cache, sb.slot_mapping)
    lib, hip = _lib()
    assert k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype
    assert k_cache.shape[2:] == (G, D) and v_cache.shape[2:] == (G, Dv)
    q = torch.empty(T, H, D, dtype=qkv.dtype, device=qkv.device)
    rc = lib.oa_attn_prepare(
        hip.current_stream_ptr(), qkv.data_ptr(), _rows(qkv),
        bias.data_ptr() if bias is not None else None, q_norm_w.data_ptr(),
        k_norm_w.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
        sb.slot_mapping.data_ptr(), sb.cu_t.data_ptr(), sb.num_seqs, T, H, G, D, Dv, eps,
        _dt(qkv))
    hip.check(rc, "oa_attn_prepare")
    return q


_GEOM = {}


# value channels per head that one launch of the paged attention kernels takes
ATTN_MAX_VALUES = 256


def attn_geometry(H: int, G: int, D: int, Dv: int, dt: int, max_chunk: int) -> Tuple[int, int]:
    """(query tokens per tile, keys per staged tile) of the attention kernel
    for steps whose longest portion is max_chunk tokens."""
    key = (H, G, D, Dv, dt, max_chunk >= 32)
    if key not in _GEOM:
        lib, hip = _lib()
        vals = [ctypes.c_int() for _ in range(4)]
        rc = lib.oa_attn_bias_geometry(H, G, D, Dv, dt, max_chunk,
                                       *[ctypes.byref(v) for v in vals])
        hip.check(rc, "oa_attn_bias_geometry")
        _GEOM[key] = (vals[0].value, vals[1].value)
    return _GEOM[key]


def attention_paged(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    sb: SeqBatch, scale: float, slopes: Optional[torch.Tensor] = None,
                    gate_logits: Optional[torch.Tensor] = None,
                    window: Optional[int] = None,
                    sinks: Optional[torch.Tensor] = None,
                    softcap: Optional[float] = None) -> torch.Tensor:
    """Causal softmax attention over each sequence's cached keys, score
    q.k*scale. Options, each a parameter: `slopes` [H] float32 subtracts
    slope_h*(i-j); `window` hides keys with i - j >= window; `sinks` [H]
    float32 enlarges head h's softmax normaliser by exp(sink_h) and leaves
    the numerator alone; `softcap` replaces the scaled score by
    softcap * tanh(score / softcap);
    `gate_logits` [T,H] (may be a column slice) scales each head's output by
    its sigmoid. q [T,H,D]. The cache may hold fewer value heads than key
    heads (Gv divides G): key head g reads value head g mod Gv.
    Returns [T, H*Dv]."""
    T, H, D = q.shape
    nb, bs, Gv, Dv = v_cache.shape
    G = k_cache.shape[2]
    window = int(window) if window else 0
    softcap = float(softcap) if softcap else 0.0
    assert G % Gv == 0 and H % G == 0
    # v_cache may be a view of the leading channels of wider rows (values
    # that are a prefix of the cached keys): its token stride is passed on
    assert v_cache.stride(3) == 1 and (Gv == 1 or v_cache.stride(2) == Dv)
    assert v_cache.stride(0) == bs * v_cache.stride(1)
    if not q.is_cuda:
        return torch_ref.attention_paged(q, k_cache, v_cache, sb.cu, sb.past, sb.block_table,
                                         scale, slopes, gate_logits, window or None, sinks,
                                         softcap or None)
    if Dv > ATTN_MAX_VALUES:
        # a lane of the kernels holds at most 4 value channels: wider value
        # heads run as slices of the value channels with the same scores
        if Gv != 1:
            raise ValueError(f"value heads wider than {ATTN_MAX_VALUES} need a single value head")
        out = torch.empty(T, H, Dv, dtype=q.dtype, device=q.device)
        for lo in range(0, Dv, ATTN_MAX_VALUES):
            hi = min(Dv, lo + ATTN_MAX_VALUES)
            part = attention_paged(q, k_cache, v_cache[..., lo:hi], sb, scale, slopes, gate_logits,
                                   window, sinks, softcap)
            out[..., lo:hi] = part.view(T, H, hi - lo)
        return out.view(T, H * Dv)
    lib, hip = _lib()
    dt = _dt(q)
    TQ, KT = attn_geometry(H, G, D, Dv, dt, sb.max_chunk)
    ntiles = sum((sb.cu[b + 1] - sb.cu[b] + TQ - 1) // TQ for b in range(sb.num_seqs))
    # few tiles and long contexts: split the keys over blocks to fill the chip
    reach = sb.max_total
    if window:
        reach = min(reach, window + min(sb.max_chunk, TQ) + KT)
    nkt = max(1, (reach + KT - 1) // KT)
    nsplit = 1
    if ntiles * G < 256 and nkt >= 8:
        nsplit = int(min(nkt // 4, max(1, 512 // max(1, ntiles * G)), 64))
    # decode steps of many query heads per kv head run one block per 64 heads
    # (the heads share each staged tile): fewer blocks, so finer key splits
    if (sb.max_chunk == 1 and H // G >= 16 and dt == 0 and D % 16 == 0 and Dv % 16 == 0
            and D <= 256 and Dv <= 256 and (D <= 128 or D % 32 == 0) and nkt >= 4):
        blocks = ntiles * G * ((H // G + 63) // 64)
        if blocks < 128:
            # at most 16: a captured step sizes nkt for the longest context
            # the pool allows, and merging many (mostly empty) partials costs
            # more than the splits save
            nsplit = int(min(nkt // 2, max(1, 256 // blocks), 16))
            if os.environ.get("OPSAGENT_ATTN_DECODE_SPLITS"):
                nsplit = max(1, min(nkt, int(os.environ["OPSAGENT_ATTN_DECODE_SPLITS"])))
    out = torch.empty(T, H * Dv, dtype=q.dtype, device=q.device)
    part_o = part_ml = None
    if nsplit > 1:
        part_o = torch.empty(T * H * nsplit, Dv, dtype=torch.float32, device=q.device)
        part_ml = torch.empty(T * H * nsplit, 2, dtype=torch.float32, device=q.device)
    assert q.is_contiguous()
    assert slopes is None or (slopes.dtype == torch.float32 and slopes.numel() == H)
    assert sinks is None or (sinks.dtype == torch.float32 and sinks.numel() == H
                             and sinks.is_contiguous())
    rc = lib.oa_attn_bias_paged(
        hip.current_stream_ptr(), q.data_ptr(),
        gate_logits.data_ptr() if gate_logits is not None else None,
        _rows(gate_logits) if gate_logits is not None else 0,
        k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(),
        part_o.data_ptr() if part_o is not None else None,
        part_ml.data_ptr() if part_ml is not None else None,
        sb.cu_t.data_ptr(), sb.past_t.data_ptr(), sb.block_table.data_ptr(),
        sb.block_table.shape[1], bs, slopes.data_ptr() if slopes is not None else None,
        sinks.data_ptr() if sinks is not None else None,
        T, sb.num_seqs, ntiles, H, G, D, Dv,
        float(scale), nsplit, dt, sb.max_chunk, window, v_cache.stride(1), Gv, softcap)
    hip.check(rc, "oa_attn_bias_paged")
    return out


def attention_biased_paged(q: torch.Tensor, gate_logits: torch.Tensor, k_cache: torch.Tensor,
                           v_cache: torch.Tensor, sb: SeqBatch, scale: float,
                           slopes: torch.Tensor) -> torch.Tensor:
    """attention_paged with a distance penalty and an output gate."""
    return attention_paged(q, k_cache, v_cache, sb, scale, slopes=slopes,
                           gate_logits=gate_logits)


def dyt_norm(residual: torch.Tensor, nxt: Optional[Tuple[torch.Tensor, ...]], out_dtype,
             y: Optional[torch.Tensor] = None,
             post: Optional[Tuple[torch.Tensor, ...]] = None) -> Optional[torch.Tensor]:
    """Dynamic-tanh norm dyt(x; w, b, a) = tanh(a x) * w + b, computed in
    float32; a norm is the tuple (w [C], b [C], a [1]) of float32 tensors.
    With y [T, C] and post: residual (float32 [T, C]) += dyt(y; post) in
    place. With nxt: returns dyt(residual; nxt) in out_dtype — one launch
    for the add after a sublayer and the norm before the next one."""
    T, C = residual.shape
    assert residual.dtype == torch.float32 and residual.is_contiguous()
    assert (y is None) == (post is None) and (y is not None or nxt is not None)
    if not residual.is_cuda:
        return torch_ref.dyt_norm(y, post, residual, nxt, out_dtype)
    lib, hip = _lib()
    for t in (post or ()) + (nxt or ()):
        assert t.dtype == torch.float32 and t.is_contiguous()
    out = torch.empty(T, C, dtype=out_dtype, device=residual.device) if nxt is not None else None
    pw, pb, pa = (t.data_ptr() for t in post) if post is not None else (None, None, None)
    nw, nb, na = (t.data_ptr() for t in nxt) if nxt is not None else (None, None, None)
    rc = lib.oa_dyt_norm(
        hip.current_stream_ptr(), y.data_ptr() if y is not None else None,
        _rows(y) if y is not None else 0, _dt(y) if y is not None else 1, pw, pb, pa,
        residual.data_ptr(), nw, nb, na, out.data_ptr() if out is not None else None,
        _dt(out) if out is not None else 1, T, C)
    hip.check(rc, "oa_dyt_norm")
    return out


def rotary_inv_freq(dims: int, base: float, scaling: Optional[dict] = None) -> torch.Tensor:
    """float32 [dims/2] rotation frequencies base^(-2i/dims). `scaling`
    {factor, low, high, original} slows long waves: a wavelength below
    original/high keeps its frequency, one above original/low gets
    frequency/factor, between them the two are blended linearly in
    original/wavelength."""
    import math

    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, orig = (float(scaling[k])
                                       for k in ("factor", "low", "high", "original"))
            wavelen = 2.0 * math.pi / f
            if wavelen > orig / low:
                f = f / factor
            elif wavelen >= orig / high:
                smooth = (orig / wavelen - low) / (high - low)
                f = (1.0 - smooth) * f / factor + smooth * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float32)


def attn_rope_prepare(qkv: torch.Tensor, q_norm_w: Optional[torch.Tensor],
                      k_norm_w: Optional[torch.Tensor],
                      inv_freq: torch.Tensor, H: int, G: int, D: int, Dv: int, eps: float,
                      k_cache: torch.Tensor, v_cache: torch.Tensor, sb: SeqBatch,
                      v_heads: Optional[int] = None) -> torch.Tensor:
    """qkv [T, >= H*D + G*D + Gv*Dv] (q | k | v columns; Gv = v_heads or G).
    RMS norm of every query and key head over its D channels with the float32
    weights [D] (shared by heads; both None: no norm), then rotation of the
    channel pairs (2i, 2i+1), i < len(inv_freq), by position * inv_freq[i] —
    all in float32; k and v are written to their pages; returns q [T, H, D]."""
    T = qkv.shape[0]
    Gv = v_heads or G
    assert 2 * inv_freq.numel() <= D and (q_norm_w is None) == (k_norm_w is None)
    if not qkv.is_cuda:
        return torch_ref.attn_rope_prepare(qkv, q_norm_w, k_norm_w, inv_freq, H, G, D, Dv, eps,
                                           k_cache, v_cache, _positions(sb), sb.slot_mapping,
                                           Gv)
    lib, hip = _lib()
    assert k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype
    assert k_cache.shape[2:] == (G, D) and v_cache.shape[2:] == (Gv, Dv)
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    for t in (q_norm_w, k_norm_w, inv_freq):
        assert t is None or (t.dtype == torch.float32 and t.is_contiguous())
    assert q_norm_w is None or (q_norm_w.numel() == D and k_norm_w.numel() == D)
    q = torch.empty(T, H, D, dtype=qkv.dtype, device=qkv.device)
    rc = lib.oa_attn_rope_prepare(
        hip.current_stream_ptr(), qkv.data_ptr(), _rows(qkv),
        q_norm_w.data_ptr() if q_norm_w is not None else None,
        k_norm_w.data_ptr() if k_norm_w is not None else None,
        inv_freq.data_ptr(), inv_freq.numel(), q.data_ptr(),
        k_cache.data_ptr(), v_cache.data_ptr(), sb.slot_mapping.data_ptr(),
        sb.seq_of_t.data_ptr(), sb.cu_t.data_ptr(), sb.past_t.data_ptr(), sb.num_seqs, T,
        H, G, Gv, D, Dv, eps, _dt(qkv))
    hip.check(rc, "oa_attn_rope_prepare")
    return q


ACTS = {"silu": 0, "gelu_tanh": 1, "clamp_swish": 2, "relu2": 3}


def act_args(act) -> Tuple[int, float, float]:
    """(code, limit, alpha) of a gate activation given as a name or as
    ("clamp_swish", limit, alpha)."""
    if isinstance(act, tuple):
        return ACTS[act[0]], float(act[1]), float(act[2])
    return ACTS[act], 0.0, 0.0


def act_mul_rows(gu: torch.Tensor, inter: int, act="silu") -> torch.Tensor:
    """act(gu[:, :I]) * gu[:, I:] for a contiguous [M, 2I] buffer; act is
    "silu", "gelu_tanh" (the tanh form of gelu) or ("clamp_swish", limit,
    alpha): g = min(gate, limit), u = clamp(up, -limit, limit),
    g sigmoid(alpha g) (u + 1); evaluated in float32."""
    if not gu.is_cuda:
        g, u = gu.split([inter, inter], dim=-1)
        return torch_ref.act_mul(g, u, act)
    lib, hip = _lib()
    assert gu.is_contiguous() and gu.shape[-1] == 2 * inter
    M = gu.numel() // (2 * inter)
    out = torch.empty(*gu.shape[:-1], inter, dtype=gu.dtype, device=gu.device)
    code, limit, alpha = act_args(act)
    hip.check(lib.oa_act_mul_rows(hip.current_stream_ptr(), gu.data_ptr(), out.data_ptr(),
                                  M, inter, _dt(gu), code, limit, alpha), "oa_act_mul_rows")
    return out


def route_topk(logits: torch.Tensor, correction: Optional[torch.Tensor], top: int,
               groups: int = 1, keep: int = 1, scale: float = 1.0,
               score: str = "sigmoid", rating: str = "top2",
               renorm: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """Expert choice from float32 router logits [T, E]: returns (experts
    int32 [T, top], weights float32 [T, top]). score "sigmoid" | "softmax";
    c = score + correction (float32 [E], optional) ranks the experts; with
    groups > 1 the experts are cut into `groups` runs of E/groups neighbours,
    each run is rated max1(c) + max2(c) (rating "top2") or max(c) ("max"),
    and only the `keep` top-rated runs may be picked from. Weights:
    w_j = scale * s_j / (sum_k s_k + 1e-20) over the picked experts'
    uncorrected scores s; renorm=False leaves out the division. logits may
    be the leading columns of wider rows."""
    T, E = logits.shape
    assert logits.dtype == torch.float32 and E % max(groups, 1) == 0 and top <= E
    if groups > 1:
        assert keep * (E // groups) >= top, "too few eligible experts"
    if not logits.is_cuda:
        return torch_ref.route_topk(logits, correction, top, groups, keep, scale, score,
                                    rating, renorm)
    lib, hip = _lib()
    idx = torch.empty(T, top, dtype=torch.int32, device=logits.device)
    w = torch.empty(T, top, dtype=torch.float32, device=logits.device)
    assert correction is None or (correction.dtype == torch.float32 and correction.is_contiguous())
    rc = lib.oa_route_topk(
        hip.current_stream_ptr(), logits.data_ptr(), _rows(logits),
        correction.data_ptr() if correction is not None else None, idx.data_ptr(),
        w.data_ptr(), T, E, top, max(groups, 1), keep, float(scale),
        0 if score == "sigmoid" else 1, 1 if rating == "max" else 0, int(bool(renorm)))
    hip.check(rc, "oa_route_topk")
    return idx, w


def moe_pairs_mlp(x: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor, idx: torch.Tensor,
                  wts: torch.Tensor, act="silu") -> torch.Tensor:
    """Routed experts for few tokens, two launches, no host sync and no
    atomics: out[t] = sum_j wts[t,j] * W2[e_tj] (act(Wg[e_tj] x_t) * (Wu[e_tj] x_t)).
    x [T, K]; w13 [E, 2I, K] (gate rows, then up rows); w2 [E, C, I]; idx
    int32 [T, top]; wts float32 [T, top]. Any sizes, bf16 or float32. A
    token's result does not depend on the other tokens of the batch."""
    T, K = x.shape
    E, I2, _ = w13.shape
    I, C, top = I2 // 2, w2.shape[1], idx.shape[1]
    if not x.is_cuda:
        return torch_ref.moe_pairs_mlp(x, w13, w2, idx, wts, act)
    lib, hip = _lib()
    assert x.is_contiguous() and w13.is_contiguous() and w2.is_contiguous()
    assert idx.is_contiguous() and idx.dtype == torch.int32
    assert wts.is_contiguous() and wts.dtype == torch.float32
    assert w13.dtype == x.dtype and w2.dtype == x.dtype and w2.shape == (E, C, I)
    mid = torch.empty(T * top, I, dtype=x.dtype, device=x.device)
    out = torch.empty(T, C, dtype=x.dtype, device=x.device)
    code, limit, alpha = act_args(act)
    hip.check(lib.oa_moe_pairs_gateup(
        hip.current_stream_ptr(), x.data_ptr(), w13.data_ptr(), idx.data_ptr(), mid.data_ptr(),
        T, top, E, I, K, _dt(x), code, limit, alpha), "oa_moe_pairs_gateup")
    hip.check(lib.oa_moe_pairs_down(
        hip.current_stream_ptr(), mid.data_ptr(), w2.data_ptr(), idx.data_ptr(), wts.data_ptr(),
        out.data_ptr(), T, top, E, C, I, _dt(x)), "oa_moe_pairs_down")
    return out


def channel_delta_rule(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                       b_logits: torch.Tensor, a: torch.Tensor, dt_bias: torch.Tensor,
                       a_log: torch.Tensor, norm_w: torch.Tensor, gate_logits: torch.Tensor,
                       state: torch.Tensor, sb: SeqBatch, H: int, G: int, D: int, Dv: int,
                       eps: float) -> torch.Tensor:
    """Gated delta rule with one decay per head and key channel, through to
    the gated read-out norm. q,k [T, G*D], v [T, H*Dv] (after convolution and
    silu), b_logits [T,H], a [T,H*D], gate_logits [T,H*Dv] — all may be
    column slices. state [slots,H,Dv,D] float32 (S transposed: a value
    column's key rows contiguous) is continued and updated.
    Returns rms_norm_per_head(S^T q) * norm_w * sigmoid(gate) as [T, H*Dv]
    in norm_w's type."""
    T = q.shape[0]
    if not q.is_cuda:
        o = torch_ref.channel_delta_rule(
            q.reshape(T, G, D), k.reshape(T, G, D), v.reshape(T, H, Dv), b_logits, a,
            dt_bias, a_log, state, sb.cu, sb.past, sb.slots)
        return torch_ref.gated_head_rms_norm(o, norm_w, gate_logits, eps, norm_w.dtype)
    lib, hip = _lib()
    out = torch.empty(T, H * Dv, dtype=norm_w.dtype, device=q.device)
    assert state.dtype == torch.float32 and state.is_contiguous()
    assert state.shape[1:] == (H, Dv, D)
    # one block per (sequence, head) runs the recurrence of ALL value columns
    # on one CU; long portions of few sequences split the columns over blocks
    # instead (the head norm then runs as its own launch on a float32 buffer)
    csplit, o_raw = 1, None
    pairs = sb.num_seqs * H
    if sb.max_chunk >= 64 and pairs < 192:
        for c in (8, 4, 2):
            if Dv % (4 * c) == 0 and Dv // c >= 16 and pairs * c <= 512:
                csplit = c
                break
    if D > 128 and Dv // csplit > 64:
        # 256-row columns: more than 64 columns per block would hold two or
        # four columns per lane pass and spill registers; split instead
        for c in (2, 4):
            if c >= csplit and Dv % (4 * c) == 0 and Dv // c <= 64:
                csplit = c
                break
    if csplit > 1:
        o_raw = torch.empty(T, H * Dv, dtype=torch.float32, device=q.device)
    rc = lib.oa_delta_rule_fused(
        hip.current_stream_ptr(), q.data_ptr(), _rows(q), k.data_ptr(), _rows(k),
        v.data_ptr(), _rows(v), b_logits.data_ptr(), _rows(b_logits), a.data_ptr(), _rows(a),
        dt_bias.data_ptr(), a_log.data_ptr(), norm_w.data_ptr(), gate_logits.data_ptr(),
        _rows(gate_logits), state.data_ptr(), out.data_ptr(),
        o_raw.data_ptr() if o_raw is not None else None, sb.cu_t.data_ptr(),
        sb.past_t.data_ptr(), sb.slots_t.data_ptr(), T, sb.num_seqs, H, G, D, Dv, eps, _dt(q),
        csplit)
    hip.check(rc, "oa_delta_rule_fused")
    return out


def add_layer_norm(residual: torch.Tensor, w: Optional[torch.Tensor], eps: float, out_dtype,
                   y: Optional[torch.Tensor] = None, y2: Optional[torch.Tensor] = None,
                   y2_gate: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """One launch for the add after a sublayer and the layer norm before the
    next: residual (float32 [T, C], in place) += y + sigmoid(y2_gate) * y2
    (each optional; y2_gate float32 [T], may be a column of a wider buffer,
    scales y2's rows; without it y2 is added as it is). With w (float32 [C]):
    returns (x - mean) / sqrt(mean((x - mean)^2) + eps) * w of the new
    residual in out_dtype; statistics in float32, two passes."""
    T, C = residual.shape
    assert residual.dtype == torch.float32 and residual.is_contiguous()
    assert y2_gate is None or (y2 is not None and y2_gate.dtype == torch.float32
                               and y2_gate.dim() == 1)
    if not residual.is_cuda:
        return torch_ref.add_layer_norm(residual, y, w, eps, out_dtype, y2, y2_gate)
    lib, hip = _lib()
    assert w is None or (w.dtype == torch.float32 and w.is_contiguous() and w.numel() == C)
    out = torch.empty(T, C, dtype=out_dtype, device=residual.device) if w is not None else None
    rc = lib.oa_add_layer_norm(
        hip.current_stream_ptr(), residual.data_ptr(),
        y.data_ptr() if y is not None else None, _rows(y) if y is not None else 0,
        _dt(y) if y is not None else 1,
        y2.data_ptr() if y2 is not None else None, _rows(y2) if y2 is not None else 0,
        _dt(y2) if y2 is not None else 1,
        y2_gate.data_ptr() if y2_gate is not None else None,
        y2_gate.stride(0) if y2_gate is not None else 0,
        w.data_ptr() if w is not None else None,
        out.data_ptr() if out is not None else None, _dt(out) if out is not None else 1,
        T, C, float(eps))
    hip.check(rc, "oa_add_layer_norm")
    return out


def _positions(sb: SeqBatch) -> torch.Tensor:
    return torch.tensor([sb.past[b] + i for b in range(sb.num_seqs)
                         for i in range(sb.cu[b + 1] - sb.cu[b])], dtype=torch.float32)


def latent_kv_prepare(dkv: torch.Tensor, norm_w: torch.Tensor, inv_freq: torch.Tensor,
                      rank: int, rot: int, eps: float, k_cache: torch.Tensor,
                      sb: SeqBatch) -> None:
    """What latent attention caches per token, from dkv [T, rank + rot] (may
    be a column slice): the first `rank` columns RMS-normed with the float32
    weight norm_w (the latent), the last `rot` with channel pairs (2i, 2i+1),
    i < len(inv_freq), rotated by position * inv_freq[i] (one key part for
    all heads). Both go to the token's row of k_cache [blocks, page, 1,
    rank + rot]; everything between load and store is float32."""
    T = dkv.shape[0]
    assert dkv.shape[1] == rank + rot and 2 * inv_freq.numel() <= rot
    assert k_cache.shape[2:] == (1, rank + rot) and k_cache.is_contiguous()
    if not dkv.is_cuda:
        torch_ref.latent_kv_prepare(dkv, norm_w, inv_freq, rank, rot, eps, k_cache,
                                    _positions(sb), sb.slot_mapping)
        return
    lib, hip = _lib()
    assert k_cache.dtype == dkv.dtype
    for t in (norm_w, inv_freq):
        assert t.dtype == torch.float32 and t.is_contiguous()
    rc = lib.oa_latent_kv_prepare(
        hip.current_stream_ptr(), dkv.data_ptr(), _rows(dkv), norm_w.data_ptr(),
        inv_freq.data_ptr(), inv_freq.numel(), k_cache.data_ptr(), sb.slot_mapping.data_ptr(),
        sb.seq_of_t.data_ptr(), sb.cu_t.data_ptr(), sb.past_t.data_ptr(), sb.num_seqs, T,
        rank, rot, float(eps), _dt(dkv))
    hip.check(rc, "oa_latent_kv_prepare")


def latent_q_assemble(q: torch.Tensor, q_lat: Optional[torch.Tensor], inv_freq: torch.Tensor,
                      H: int, D: int, rot: int, sb: SeqBatch,
                      out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Queries against the cached latent rows: q [T, H*(D+rot)] (per head D
    unrotated, then rot rotated channels; may be a column slice) and q_lat
    [H, T, rank], the unrotated parts already taken through the key
    up-projection. Returns [T, H, rank + rot]: q_lat beside the part rotated
    by position (float32 angles). With `out` given and q_lat None the latent
    part is already in out[..., :rank] (a batched GEMM can write it there
    directly) and only the rotated part is filled in."""
    T = q.shape[0]
    assert (q_lat is None) == (out is not None)
    if out is not None:
        rank = out.shape[2] - rot
        assert out.shape[:2] == (T, H) and out.is_contiguous() and out.dtype == q.dtype
    else:
        rank = q_lat.shape[2]
        assert q_lat.shape[:2] == (H, T) and q_lat.is_contiguous() and q_lat.dtype == q.dtype
    if not q.is_cuda:
        if out is not None:
            out[..., rank:] = torch_ref.latent_q_assemble(
                q, out[..., :rank].transpose(0, 1), inv_freq, H, D, rot, _positions(sb))[..., rank:]
            return out
        return torch_ref.latent_q_assemble(q, q_lat, inv_freq, H, D, rot, _positions(sb))
    lib, hip = _lib()
    if out is None:
        out = torch.empty(T, H, rank + rot, dtype=q.dtype, device=q.device)
    rc = lib.oa_latent_q_assemble(
        hip.current_stream_ptr(), q.data_ptr(), _rows(q),
        q_lat.data_ptr() if q_lat is not None else None,
        inv_freq.data_ptr(), inv_freq.numel(), out.data_ptr(), sb.seq_of_t.data_ptr(),
        sb.cu_t.data_ptr(), sb.past_t.data_ptr(), sb.num_seqs, T, H, D, rot, rank, _dt(q))
    hip.check(rc, "oa_latent_q_assemble")
    return out


def decay_linear_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                           state: torch.Tensor, sb: SeqBatch, H: int, D: int, Dv: int,
                           head_decay: Optional[torch.Tensor] = None,
                           z: Optional[torch.Tensor] = None,
                           z_bias: Optional[torch.Tensor] = None, inv_tau: float = 1.0,
                           act: str = "none", q_scale: float = 1.0) -> torch.Tensor:
    """Linear attention with decay: per head S_t = diag(a_t) S_{t-1} + k_t v_t^T,
    o_t = S_t^T q_t. a_t is head_decay[h] (float32 [H]) for every key channel,
    or, with z [T, H*D], sigmoid(z_t + z_bias)^(inv_tau) per key channel
    (z_bias float32 [H*D]; computed as exp(inv_tau * log sigmoid) in
    float32). act "silu" is applied to q, k, v first; q is then scaled by
    q_scale. q, k [T, H*D], v [T, H*Dv] may be column slices. state [slots,
    H, Dv, D] float32 (S transposed) is continued and updated; a sequence at
    position 0 starts from zero whatever its slot holds. Returns the
    read-out [T, H*Dv] float32."""
    T = q.shape[0]
    assert (head_decay is None) != (z is None)
    assert state.dtype == torch.float32 and state.is_contiguous()
    assert state.shape[1:] == (H, Dv, D)
    if not q.is_cuda:
        return torch_ref.decay_linear_attention(q, k, v, z, z_bias, inv_tau, head_decay, state,
                                                sb.cu, sb.past, sb.slots, H, D, Dv, act, q_scale)
    lib, hip = _lib()
    for t in (head_decay, z_bias):
        assert t is None or (t.dtype == torch.float32 and t.is_contiguous())
    assert z is None or (z_bias is not None and z_bias.numel() == H * D)
    assert head_decay is None or head_decay.numel() == H
    out = torch.empty(T, H * Dv, dtype=torch.float32, device=q.device)
    # one block per (sequence, head) holds all value columns; long portions
    # of few sequences split the columns over blocks to fill the chip
    csplit, pairs = 1, sb.num_seqs * H
    if sb.max_chunk >= 64 and pairs < 192:
        for c in (8, 4, 2):
            if Dv % (4 * c) == 0 and Dv // c >= 16 and pairs * c <= 512:
                csplit = c
                break
    if Dv // csplit > 256 or (D > 128 and Dv // csplit > 64):
        # at most 256 columns per block; 256-row columns: more than 64 per
        # block would hold two or four per lane pass and spill registers
        cap = 64 if D > 128 else 256
        for c in range(csplit, Dv + 1):
            if Dv % c == 0 and Dv // c <= cap:
                csplit = c
                break
    rc = lib.oa_decay_scan(
        hip.current_stream_ptr(), q.data_ptr(), _rows(q), k.data_ptr(), _rows(k),
        v.data_ptr(), _rows(v), z.data_ptr() if z is not None else None,
        _rows(z) if z is not None else 0,
        z_bias.data_ptr() if z_bias is not None else None, float(inv_tau),
        head_decay.data_ptr() if head_decay is not None else None, state.data_ptr(),
        out.data_ptr(), sb.cu_t.data_ptr(), sb.past_t.data_ptr(), sb.slots_t.data_ptr(),
        T, sb.num_seqs, H, D, Dv, 1 if act == "silu" else 0, float(q_scale), _dt(q), csplit)
    hip.check(rc, "oa_decay_scan")
    return out


def gated_rms_norm(o: torch.Tensor, w: torch.Tensor, groups: int, gate_logits: torch.Tensor,
                   gate_act: str, eps: float, out_dtype) -> torch.Tensor:
    """o float32 [T, N]: RMS norm over each of `groups` equal parts, times the
    float32 weight w ([N/groups], shared by the parts, or [N]), times sigmoid
    or silu (gate_act) of gate_logits [T, N] (may be a column slice). Returns
    [T, N] in out_dtype."""
    T, N = o.shape
    assert o.dtype == torch.float32 and o.is_contiguous() and N % groups == 0
    assert w.numel() in (N, N // groups) and gate_act in ("sigmoid", "silu")
    if not o.is_cuda:
        return torch_ref.gated_rms_norm(o, w, groups, gate_logits, gate_act, eps, out_dtype)
    lib, hip = _lib()
    assert w.dtype == torch.float32 and w.is_contiguous()
    out = torch.empty(T, N, dtype=out_dtype, device=o.device)
    rc = lib.oa_gated_rms_norm(
        hip.current_stream_ptr(), o.data_ptr(), w.data_ptr(), w.numel(), gate_logits.data_ptr(),
        _rows(gate_logits), _dt(gate_logits), 0 if gate_act == "sigmoid" else 1, out.data_ptr(),
        _dt(out), T, N, groups, float(eps))
    hip.check(rc, "oa_gated_rms_norm")
    return out


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """cap * tanh(logits / cap) in float32."""
    if not logits.is_cuda:
        return torch_ref.softcap(logits, cap)
    lib, hip = _lib()
    x = logits.contiguous()
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    hip.check(lib.oa_softcap(hip.current_stream_ptr(), x.data_ptr(), out.data_ptr(),
                             x.numel(), float(cap), _dt(x)), "oa_softcap")
    return out


def silu_mul_rows(gu: torch.Tensor, inter: int) -> torch.Tensor:
    """silu(gu[:, :I]) * gu[:, I:] for a contiguous [M, 2I] buffer of any
    supported float type."""
    if not gu.is_cuda:
        g, u = gu.split([inter, inter], dim=-1)
        return torch_ref.silu_mul(g, u)
    lib, hip = _lib()
    assert gu.is_contiguous() and gu.shape[-1] == 2 * inter
    M = gu.numel() // (2 * inter)
    out = torch.empty(*gu.shape[:-1], inter, dtype=gu.dtype, device=gu.device)
    hip.check(lib.oa_silu_mul_rows(hip.current_stream_ptr(), gu.data_ptr(), out.data_ptr(),
                                   M, inter, _dt(gu)), "oa_silu_mul_rows")
    return out


def hyper_norm(streams: torch.Tensor, read: Optional[torch.Tensor], w: Optional[torch.Tensor],
               b: Optional[torch.Tensor], eps: float, out_dtype,
               y: Optional[torch.Tensor] = None, mix: Optional[torch.Tensor] = None,
               write: Optional[torch.Tensor] = None, y2: Optional[torch.Tensor] = None,
               y2_gate: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """One launch for a sublayer's write into hyper-connected residual streams
    and the read and layer norm before the next sublayer. streams float32
    [T, S, C], in place. With y [T, C] (plus sigmoid(y2_gate) * y2, as in
    add_layer_norm), mix float32 [S, S] indexed [from, to] and write float32
    [S]:  new_t = sum_s mix[s, t] old_s + write[t] * y, every stream from the
    old ones. With read float32 [S], w and (optionally) b float32 [C]: returns
    the layer norm of u = sum_s read[s] new_s, (u - mean) / sqrt(var + eps) *
    w + b, in out_dtype. One stream with mix = write = read = 1 is the plain
    residual sum."""
    T, S, C = streams.shape
    assert streams.dtype == torch.float32 and streams.is_contiguous()
    assert (y is None) == (mix is None) == (write is None)
    assert y2 is None or y is not None
    assert y2_gate is None or (y2 is not None and y2_gate.dtype == torch.float32
                               and y2_gate.dim() == 1)
    assert (read is None) == (w is None) and (y is not None or read is not None)
    if not streams.is_cuda:
        return torch_ref.hyper_norm(streams, y, y2, y2_gate, mix, write, read, w, b, eps,
                                    out_dtype)
    lib, hip = _lib()
    for t, n in ((mix, S * S), (write, S), (read, S), (w, C), (b, C)):
        assert t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.numel() == n)
    out = torch.empty(T, C, dtype=out_dtype, device=streams.device) if read is not None else None
    ptr = lambda t: t.data_ptr() if t is not None else None  # noqa: E731
    rc = lib.oa_hyper_norm(
        hip.current_stream_ptr(), streams.data_ptr(), S, ptr(y), _rows(y) if y is not None else 0,
        _dt(y) if y is not None else 1, ptr(y2), _rows(y2) if y2 is not None else 0,
        _dt(y2) if y2 is not None else 1, ptr(y2_gate),
        y2_gate.stride(0) if y2_gate is not None else 0, ptr(mix), ptr(write), ptr(read),
        ptr(w), ptr(b), ptr(out), _dt(out) if out is not None else 1, T, C, float(eps))
    hip.check(rc, "oa_hyper_norm")
    return out


def rope_rows(x: torch.Tensor, n_rot: int, D: int, inv_freq: torch.Tensor,
              sb: SeqBatch) -> torch.Tensor:
    """x [T, n] (may be a column slice): the first n_rot * D columns are heads
    of D channels whose pairs (2i, 2i+1), i < len(inv_freq), are rotated by
    position * inv_freq[i] in float32; the other columns are copied. Returns
    float32 [T, n]: what enters a recurrence stays unrounded."""
    T, n = x.shape
    assert n_rot * D <= n and 2 * inv_freq.numel() <= D
    if not x.is_cuda:
        return torch_ref.rope_rows(x, n_rot, D, inv_freq, _positions(sb))
    lib, hip = _lib()
    assert inv_freq.dtype == torch.float32 and inv_freq.is_contiguous()
    out = torch.empty(T, n, dtype=torch.float32, device=x.device)
    rc = lib.oa_rope_rows(
        hip.current_stream_ptr(), x.data_ptr(), _rows(x), _dt(x), out.data_ptr(), n, n_rot, D,
        inv_freq.data_ptr(), inv_freq.numel(), sb.seq_of_t.data_ptr(), sb.cu_t.data_ptr(),
        sb.past_t.data_ptr(), sb.num_seqs, T)
    hip.check(rc, "oa_rope_rows")
    return out


def combine_norm_gate(a: torch.Tensor, H: int, Dv: int, out_dtype,
                      a2: Optional[torch.Tensor] = None, lam: float = 0.0, norm: bool = False,
                      eps: float = 0.0, post_scale: float = 1.0,
                      gate_logits: Optional[torch.Tensor] = None,
                      gate_act: str = "sigmoid") -> torch.Tensor:
    """What follows a mixer's read-out, one launch: o = a - lam * a2 (a2
    optional; both [T, H*Dv], may be column slices, float32 or bf16); with
    `norm` each head's Dv values are divided by sqrt(mean(o^2) + eps) and
    multiplied by post_scale; then o * sigmoid|silu(gate_logits) ([T, H*Dv],
    may be a column slice; None: no gate). Computed in float32; returns
    [T, H*Dv] in out_dtype."""
    T = a.shape[0]
    assert a.shape[1] == H * Dv and gate_act in ("sigmoid", "silu")
    assert a2 is None or (a2.shape == a.shape and a2.dtype == a.dtype)
    if not a.is_cuda:
        return torch_ref.combine_norm_gate(a, a2, lam, H, Dv, norm, eps, post_scale,
                                           gate_logits, gate_act, out_dtype)
    lib, hip = _lib()
    out = torch.empty(T, H * Dv, dtype=out_dtype, device=a.device)
    assert gate_logits is None or gate_logits.dtype == out_dtype
    rc = lib.oa_combine_norm_gate(
        hip.current_stream_ptr(), a.data_ptr(), _rows(a), _dt(a),
        a2.data_ptr() if a2 is not None else None, _rows(a2) if a2 is not None else 0,
        float(lam), gate_logits.data_ptr() if gate_logits is not None else None,
        _rows(gate_logits) if gate_logits is not None else 0,
        0 if gate_act == "sigmoid" else 1, out.data_ptr(), _dt(out), T, H, Dv,
        int(bool(norm)), float(eps), float(post_scale))
    hip.check(rc, "oa_combine_norm_gate")
    return out


def act_rows(x: torch.Tensor, act: str = "relu2") -> torch.Tensor:
    """Elementwise activation of an ungated feed-forward on a contiguous
    buffer: "relu2" (the square of relu), "silu" or "gelu_tanh"; float32
    inside."""
    if not x.is_cuda:
        return torch_ref.act_rows(x, act)
    lib, hip = _lib()
    assert x.is_contiguous()
    out = torch.empty_like(x)
    hip.check(lib.oa_act_rows(hip.current_stream_ptr(), x.data_ptr(), out.data_ptr(),
                              x.numel(), _dt(x), ACTS[act]), "oa_act_rows")
    return out


def moe_pairs_plain(x: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, idx: torch.Tensor,
                    wts: torch.Tensor, act: str = "relu2") -> torch.Tensor:
    """Routed ungated experts for few tokens, two launches, no host sync:
    out[t] = sum_j wts[t,j] * W2[e_tj] act(W1[e_tj] x_t). x [T, K]; w1
    [E, I, K]; w2 [E, C, I]; idx int32 [T, top]; wts float32 [T, top]. Any
    sizes, bf16 or float32. A token's result does not depend on the other
    tokens of the batch."""
    T, K = x.shape
    E, I, _ = w1.shape
    C, top = w2.shape[1], idx.shape[1]
    if not x.is_cuda:
        return torch_ref.moe_pairs_plain(x, w1, w2, idx, wts, act)
    lib, hip = _lib()
    assert x.is_contiguous() and w1.is_contiguous() and w2.is_contiguous()
    assert idx.is_contiguous() and idx.dtype == torch.int32
    assert wts.is_contiguous() and wts.dtype == torch.float32
    assert w1.dtype == x.dtype and w2.dtype == x.dtype and w2.shape == (E, C, I)
    mid = torch.empty(T * top, I, dtype=x.dtype, device=x.device)
    out = torch.empty(T, C, dtype=x.dtype, device=x.device)
    hip.check(lib.oa_moe_pairs_up(
        hip.current_stream_ptr(), x.data_ptr(), w1.data_ptr(), idx.data_ptr(), mid.data_ptr(),
        T, top, E, I, K, _dt(x), ACTS[act]), "oa_moe_pairs_up")
    hip.check(lib.oa_moe_pairs_down(
        hip.current_stream_ptr(), mid.data_ptr(), w2.data_ptr(), idx.data_ptr(), wts.data_ptr(),
        out.data_ptr(), T, top, E, C, I, _dt(x)), "oa_moe_pairs_down")
    return out
