"""Op dispatch layer.

GPU (ROCm) path → hand-written HIP/CDNA4 kernels from the in-tree library
(fails LOUDLY if the library is missing — no silent eager fallback on a GPU
box, per the build contract). CPU path → opsagent_amd.ops.torch_ref (also the
numerics oracle for the GPU parity tests).

GEMM-shaped work that is a plain library GEMM (QKV/O/MLP projections,
lm_head) goes through torch.nn.functional.linear → hipBLASLt/rocBLAS, which
is the sanctioned path for non-fused GEMMs; the fused hot ops (norms, RoPE,
attention, activation, sampling) are the HIP kernels here.
"""

from __future__ import annotations

import os
from typing import Optional, Tuple

import torch

from opsagent_amd.ops import torch_ref

__all__ = [
    "rms_norm",
    "fused_add_rms_norm",
    "rope_apply_",
    "silu_mul",
    "kv_cache_write",
    "attention_prefill",
    "attention_decode_paged",
    "greedy_sample_masked",
    "rope_cos_sin",
]

rope_cos_sin = torch_ref.rope_cos_sin

# VALU-gemv M instantiations (the dot-per-lane form; measured crossover
# notes below). Batched decode M 3..8 rides the MFMA gemv instead
# (_bf16_mfma_ok); M > 8 bf16 stays on hipBLASLt.
_GEMV_MS = frozenset(range(1, 9))

# Measured crossover vs hipBLASLt (concurrent bench, within-box A/B):
#   M=1: custom ~2.5x faster        M=2: custom +19% (c=2 3.42 vs 2.88 t/s)
#   M=4: tie (5.20 vs 5.28)         M=8: custom ~2x SLOWER (c=8 4.6 vs 9.2)
# The per-lane-dot form goes VALU-bound as M grows; hipBLASLt's MFMA kernels
# take over. Default cap 2; OPSAGENT_GEMV_MAX_M overrides for experiments.


def _bf16_mfma_ok(M: int, K: int, gateup: bool = False) -> bool:
    """Mirror of gemv.hip's gemv_bf16_use_mfma: the MFMA batched-decode
    kernel (M 3..16) — concurrent decode's hipBLASLt fallback measured
    ~2.5x off the stream roofline."""
    e = os.environ.get("OPSAGENT_BF16_GEMV_MFMA", "")
    if e == "0":
        return False
    min_m = int(e[1:]) if e.startswith("m") else 3
    if M < min_m or M > 16:
        return False
    if K % (512 if gateup else 1024) != 0:
        return False
    if not e.startswith("m"):
        # measured win region only (see gemv.hip's gemv_bf16_use_mfma)
        if K > 6144 or M > 8:
            return False
    return M * (K * 2 + 16) <= 147456


def _gemv_m_ok(M: int) -> bool:
    import os

    cap = int(os.environ.get("OPSAGENT_GEMV_MAX_M", "2"))
    return M in _GEMV_MS and M <= cap


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """F.linear with custom HIP fast paths for decode shapes: the VALU
    skinny GEMV at M <= 2 (hipBLASLt's M=1 kernels run ~2.5x off the HBM
    roofline on gfx950) and the MFMA batched GEMV at M 3..8 / K <= 6144
    (_bf16_mfma_ok); everything else goes to hipBLASLt."""
    M = x.numel() // x.shape[-1]
    if (
        x.is_cuda
        and x.dtype == torch.bfloat16
        and (_gemv_m_ok(M) or _bf16_mfma_ok(M, x.shape[-1]))
        and x.shape[-1] % 8 == 0
        and w.stride(1) == 1
        and x.is_contiguous()
        # the kernels read 16 bytes at a time: a column slice of a wider
        # buffer may start anywhere
        and x.data_ptr() % 16 == 0
        and w.data_ptr() % 16 == 0
        and w.stride(0) % 8 == 0
    ):
        from opsagent_amd.ops import hip_lib

        lib = hip_lib.get_lib()
        N, K = w.shape
        out = torch.empty(*x.shape[:-1], N, dtype=x.dtype, device=x.device)
        rc = lib.oa_gemv(
            hip_lib.current_stream_ptr(), x.data_ptr(), w.data_ptr(), out.data_ptr(),
            M, N, K,
        )
        hip_lib.check(rc, "oa_gemv")
        return out
    return torch.nn.functional.linear(x, w)


def _is_gpu(t: torch.Tensor) -> bool:
    return t.is_cuda


def _lib():
    from opsagent_amd.ops import hip_lib

    return hip_lib.get_lib(), hip_lib


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    if not _is_gpu(x):
        return torch_ref.rms_norm(x, weight, eps)
    assert x.dtype == torch.bfloat16 and x.is_contiguous()
    lib, hip = _lib()
    rows = x.numel() // x.shape[-1]
    out = torch.empty_like(x)
    rc = lib.oa_rmsnorm(
        hip.current_stream_ptr(), x.data_ptr(), weight.data_ptr(), out.data_ptr(),
        rows, x.shape[-1], eps,
    )
    hip.check(rc, "oa_rmsnorm")
    return out


def fused_add_rms_norm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns (rmsnorm(x+residual), x+residual). GPU path updates `residual`
    in place as the new residual stream and returns it."""
    if not _is_gpu(x):
        return torch_ref.fused_add_rms_norm(x, residual, weight, eps)
    assert x.dtype == torch.bfloat16 and x.is_contiguous() and residual.is_contiguous()
    lib, hip = _lib()
    rows = x.numel() // x.shape[-1]
    out = torch.empty_like(x)
    rc = lib.oa_fused_add_rmsnorm(
        hip.current_stream_ptr(), x.data_ptr(), residual.data_ptr(), weight.data_ptr(),
        out.data_ptr(), rows, x.shape[-1], eps,
    )
    hip.check(rc, "oa_fused_add_rmsnorm")
    return out, residual


def rope_apply_(
    q: torch.Tensor,
    k: torch.Tensor,
    cos: torch.Tensor,
    sin: torch.Tensor,
    positions: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """In-place on GPU; q [T, Hq, D], k [T, Hk, D], positions int32 [T]."""
    if not _is_gpu(q):
        return torch_ref.rope_apply(q, k, cos, sin, positions)
    assert q.dtype == torch.bfloat16 and q.is_contiguous() and k.is_contiguous()
    assert cos.dtype == torch.float32 and positions.dtype == torch.int32
    lib, hip = _lib()
    T, Hq, D = q.shape
    Hk = k.shape[1]
    rc = lib.oa_rope(
        hip.current_stream_ptr(), q.data_ptr(), k.data_ptr(), cos.data_ptr(),
        sin.data_ptr(), positions.data_ptr(), T, Hq, Hk, D,
    )
    hip.check(rc, "oa_rope")
    return q, k


def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    if not _is_gpu(gate):
        return torch_ref.silu_mul(gate, up)
    assert gate.dtype == torch.bfloat16 and gate.is_contiguous() and up.is_contiguous()
    lib, hip = _lib()
    out = torch.empty_like(gate)
    rc = lib.oa_silu_mul(
        hip.current_stream_ptr(), gate.data_ptr(), up.data_ptr(), out.data_ptr(),
        gate.numel(),
    )
    hip.check(rc, "oa_silu_mul")
    return out


def quant_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-row OCP e4m3 quantization: bf16 [T, K] -> (uint8 [T, K], f32 [T])."""
    T = x.numel() // x.shape[-1]
    K = x.shape[-1]
    if not _is_gpu(x):
        return torch_ref.quant_fp8(x)
    assert x.dtype == torch.bfloat16 and x.is_contiguous() and K % 8 == 0
    lib, hip = _lib()
    q = torch.empty(*x.shape, dtype=torch.uint8, device=x.device)
    scales = torch.empty(T, dtype=torch.float32, device=x.device)
    rc = lib.oa_quant_fp8(
        hip.current_stream_ptr(), x.data_ptr(), q.data_ptr(), scales.data_ptr(), T, K
    )
    hip.check(rc, "oa_quant_fp8")
    return q, scales


def linear_fp8(
    x: torch.Tensor, w8: torch.Tensor, w_scale: torch.Tensor
) -> torch.Tensor:
    """out = (x @ dequant(w8)^T) with per-row weight scales.

    GPU: M <= 8 -> fp8 weight-streaming GEMV (half the bytes of bf16);
    M <= 16 -> the same GEMV padded to the next instantiation (catch-up /
    speculative verify passes); larger M (real prefill) -> quantize x per
    token and run the fp8 MFMA tile GEMM. (A dequant-to-bf16 + hipBLASLt
    variant was measured and REVERTED: 70B fp8 turn 723 ms vs 573 with the
    tile GEMM — the per-call dequant round-trip costs more than the GEMM's
    tile-pipeline inefficiency.)
    CPU: dequantized torch reference."""
    M = x.numel() // x.shape[-1]
    K = x.shape[-1]
    N = w8.shape[0]
    if not _is_gpu(x):
        return torch_ref.linear_fp8(x, w8, w_scale)
    assert x.dtype == torch.bfloat16 and x.is_contiguous() and K % 64 == 0
    lib, hip = _lib()
    # NOTE: the bf16 _gemv_m_ok cap (M<=2) encodes the crossover vs
    # hipBLASLt, which does not apply here — for fp8 weights the alternative
    # pays a dequant round-trip. Keep bf16-activation GEMV for skinny M.
    # M>8 goes to the MX tile GEMM: the padded M=12/16 gemv instantiations
    # are VALU-bound (16 dots/lane) and measured 276 us/call on the 70B
    # jump-ahead catch-up passes vs ~80-150 us through the tile GEMM.
    if (M <= 8 or _fp8_mfma_ok(M, K)) and K % 16 == 0:
        out = torch.empty(M, N, dtype=x.dtype, device=x.device)
        rc = lib.oa_gemv_fp8(
            hip.current_stream_ptr(), x.reshape(M, K).data_ptr(), w8.data_ptr(),
            w_scale.data_ptr(), out.data_ptr(), M, N, K,
        )
        hip.check(rc, "oa_gemv_fp8")
        return out.reshape(*x.shape[:-1], N)
    if K % 128 != 0:
        # the pipelined tile GEMM unrolls K in 128-byte steps; shapes below
        # that (tiny test experts) chunk through the skinny-M gemv instead
        xm = x.reshape(M, K).contiguous()
        parts = [
            linear_fp8(xm[m0 : m0 + 8].contiguous(), w8, w_scale)
            for m0 in range(0, M, 8)
        ]
        return torch.cat(parts, dim=0).reshape(*x.shape[:-1], N)
    out = torch.empty(*x.shape[:-1], N, dtype=x.dtype, device=x.device)
    a8, a_scale = quant_fp8(x.reshape(M, K))
    rc = lib.oa_gemm_fp8(
        hip.current_stream_ptr(), a8.data_ptr(), w8.data_ptr(),
        a_scale.data_ptr(), w_scale.data_ptr(), out.data_ptr(), M, N, K,
    )
    hip.check(rc, "oa_gemm_fp8")
    return out


def linear_norm(
    x: torch.Tensor, norm_w: torch.Tensor, eps: float, w: torch.Tensor
) -> torch.Tensor:
    """rmsnorm(x) @ W^T with the norm fused into the GEMV prologue (decode
    fast path: the standalone norm kernel + its output round-trip disappear).
    Fused form normalizes in fp32 without the intermediate bf16 rounding of
    the two-kernel form (slightly MORE precise)."""
    M = x.numel() // x.shape[-1]
    if M == 1 and _bf16_prenorm():
        return linear(rms_norm(x, norm_w, eps), w)
    if (
        x.is_cuda and x.dtype == torch.bfloat16
        and (_gemv_m_ok(M) or _bf16_mfma_ok(M, x.shape[-1]))
        and x.shape[-1] % 8 == 0 and x.is_contiguous()
    ):
        from opsagent_amd.ops import hip_lib

        lib = hip_lib.get_lib()
        N, K = w.shape
        out = torch.empty(*x.shape[:-1], N, dtype=x.dtype, device=x.device)
        rc = lib.oa_gemv_ex(
            hip_lib.current_stream_ptr(), x.data_ptr(), w.data_ptr(), out.data_ptr(),
            norm_w.data_ptr(), None, M, N, K, eps, 1,
        )
        hip_lib.check(rc, "oa_gemv_ex(norm)")
        return out
    return linear(rms_norm(x, norm_w, eps), w)


def linear_addres(x: torch.Tensor, w: torch.Tensor, res: torch.Tensor) -> torch.Tensor:
    """x @ W^T + res — the projection emits the new residual stream directly."""
    M = x.numel() // x.shape[-1]
    if (
        x.is_cuda and x.dtype == torch.bfloat16
        and (_gemv_m_ok(M) or _bf16_mfma_ok(M, x.shape[-1]))
        and x.shape[-1] % 8 == 0 and x.is_contiguous() and res.is_contiguous()
    ):
        from opsagent_amd.ops import hip_lib

        lib = hip_lib.get_lib()
        N, K = w.shape
        out = torch.empty(*x.shape[:-1], N, dtype=x.dtype, device=x.device)
        rc = lib.oa_gemv_ex(
            hip_lib.current_stream_ptr(), x.data_ptr(), w.data_ptr(), out.data_ptr(),
            None, res.data_ptr(), M, N, K, 0.0, 2,
        )
        hip_lib.check(rc, "oa_gemv_ex(addres)")
        return out
    return linear(x, w) + res


def gateup_silu_norm(
    x: torch.Tensor, norm_w: torch.Tensor, eps: float, gate_up_w: torch.Tensor,
    i_local: int
) -> torch.Tensor:
    """silu(norm(x) @ gate^T) * (norm(x) @ up^T), norm fused in the prologue."""
    M = x.numel() // x.shape[-1]
    if M == 1 and _bf16_prenorm():
        return gateup_silu(rms_norm(x, norm_w, eps), gate_up_w, i_local)
    if (
        x.is_cuda and x.dtype == torch.bfloat16
        and (_gemv_m_ok(M) or _bf16_mfma_ok(M, x.shape[-1]))
        and x.shape[-1] % 8 == 0 and x.is_contiguous()
    ):
        from opsagent_amd.ops import hip_lib

        lib = hip_lib.get_lib()
        out = torch.empty(*x.shape[:-1], i_local, dtype=x.dtype, device=x.device)
        rc = lib.oa_gemv_gateup_ex(
            hip_lib.current_stream_ptr(), x.data_ptr(), gate_up_w.data_ptr(),
            out.data_ptr(), norm_w.data_ptr(), M, i_local, x.shape[-1], eps, 1,
        )
        hip_lib.check(rc, "oa_gemv_gateup_ex(norm)")
        return out
    return gateup_silu(rms_norm(x, norm_w, eps), gate_up_w, i_local)


def moe_grouped_mlp(
    x: torch.Tensor,
    w13: torch.Tensor,
    w13_scale: Optional[torch.Tensor],
    w2: torch.Tensor,
    w2_scale: Optional[torch.Tensor],
    expert_ids: torch.Tensor,
    token_ids: torch.Tensor,
    pair_weights: torch.Tensor,
    i_local: int,
    fp8: bool,
    num_experts: int = 0,
    act=None,
) -> torch.Tensor:
    """Grouped MoE expert MLP (GPU decode path): one gateup launch + one down
    launch for ALL (token, expert) pairs of a layer — no per-expert loop, no
    host sync, shape-static (graph-capturable). Returns y [P, H] to be
    index_add-ed into the output by token.

    Two kernel families, both static-shaped:
      * pair-major (default): one block column per PAIR; the expert's weight
        rows stream once per pair — lowest latency at tiny P
      * expert-major (P > OPSAGENT_MOE_EMAJ_MIN_P, needs num_experts): one
        block column per EXPERT; weights stream once per GROUP of 8 matched
        pairs, cutting the weight traffic up to 8x at big decode batches
    act: None / "silu", or ("clamp_swish", limit, alpha) for the clamped gate
    g' = min(g, limit), u' = clamp(u, -limit, limit), g' sigmoid(alpha g') (u' + 1),
    or "relu2" for UNGATED experts: w13 is [E, I, K] (up rows alone) and the
    middle activation is relu(up x)^2.
    """
    if isinstance(act, tuple):
        assert act[0] == "clamp_swish"
        actk, limit, alpha = 2, float(act[1]), float(act[2])
    elif act == "relu2":
        assert w13.shape[1] == i_local
        actk, limit, alpha = 3, 0.0, 0.0
    else:
        assert act in (None, "silu")
        actk, limit, alpha = 0, 0.0, 0.0
    assert x.is_cuda and x.dtype == torch.bfloat16 and x.is_contiguous()
    # stride-0 expand views have a data_ptr that covers ONE element — the
    # kernels index these linearly, so contiguity is load-bearing
    assert expert_ids.is_contiguous() and expert_ids.dtype == torch.int32
    assert token_ids.is_contiguous() and token_ids.dtype == torch.int32
    assert pair_weights.is_contiguous() and pair_weights.dtype == torch.float32
    lib, hip = _lib()
    P = expert_ids.shape[0]
    K = x.shape[-1]
    H = w2.shape[1]
    emaj_min = int(os.environ.get("OPSAGENT_MOE_EMAJ_MIN_P", "64"))
    use_emaj = num_experts > 0 and P >= emaj_min and P <= 2048
    mid = torch.empty(P, i_local, dtype=x.dtype, device=x.device)
    if use_emaj:
        rc = lib.oa_moe_gateup_emaj_act(
            hip.current_stream_ptr(), x.data_ptr(), w13.data_ptr(),
            w13_scale.data_ptr() if fp8 else None,
            expert_ids.data_ptr(), token_ids.data_ptr(), mid.data_ptr(),
            P, num_experts, i_local, K, 1 if fp8 else 0, actk, limit, alpha,
        )
        hip.check(rc, "oa_moe_gateup_emaj")
    else:
        rc = lib.oa_moe_gateup_act(
            hip.current_stream_ptr(), x.data_ptr(), w13.data_ptr(),
            w13_scale.data_ptr() if fp8 else None,
            expert_ids.data_ptr(), token_ids.data_ptr(), mid.data_ptr(),
            P, i_local, K, 1 if fp8 else 0, actk, limit, alpha,
        )
        hip.check(rc, "oa_moe_gateup")
    y = torch.empty(P, H, dtype=x.dtype, device=x.device)
    if use_emaj:
        rc = lib.oa_moe_down_emaj(
            hip.current_stream_ptr(), mid.data_ptr(), w2.data_ptr(),
            w2_scale.data_ptr() if fp8 else None,
            expert_ids.data_ptr(), pair_weights.data_ptr(), y.data_ptr(),
            P, num_experts, H, i_local, 1 if fp8 else 0,
        )
        hip.check(rc, "oa_moe_down_emaj")
    else:
        rc = lib.oa_moe_down(
            hip.current_stream_ptr(), mid.data_ptr(), w2.data_ptr(),
            w2_scale.data_ptr() if fp8 else None,
            expert_ids.data_ptr(), pair_weights.data_ptr(), y.data_ptr(),
            P, H, i_local, 1 if fp8 else 0,
        )
        hip.check(rc, "oa_moe_down")
    return y


def rope_kv_fused(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    cos: torch.Tensor,
    sin: torch.Tensor,
    positions: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Fused RoPE(q,k in place) + paged KV write of k,v. Returns (q, k, v).

    q/k/v may be head-slices of ONE fused [T, (Hq+2Hk)*D] qkv buffer sharing
    a token stride — no .contiguous() copies (those cost ~5.8 ms per 736-token
    prefill). Requires contiguous (head, dim) inner layout and equal token
    strides across q/k/v."""
    if not _is_gpu(q):
        q2, k2 = torch_ref.rope_apply(q, k, cos, sin, positions)
        torch_ref.kv_cache_write(k_cache, v_cache, k2, v, slot_mapping.long())
        return q2, k2, v
    T, Hq, D = q.shape
    Hk = k.shape[1]
    assert q.dtype == torch.bfloat16
    assert q.stride(2) == 1 and q.stride(1) == D, "q heads must be inner-contiguous"
    assert k.stride(2) == 1 and k.stride(1) == D and v.stride(2) == 1 and v.stride(1) == D
    assert cos.dtype == torch.float32
    assert positions.dtype == torch.int32 and slot_mapping.dtype == torch.int32
    lib, hip = _lib()
    rc = lib.oa_rope_kv(
        hip.current_stream_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
        k_cache.data_ptr(), v_cache.data_ptr(), cos.data_ptr(), sin.data_ptr(),
        positions.data_ptr(), slot_mapping.data_ptr(), T, Hq, Hk, D,
        q.stride(0), k.stride(0), v.stride(0),
    )
    hip.check(rc, "oa_rope_kv")
    return q, k, v


def gateup_silu(x: torch.Tensor, gate_up_w: torch.Tensor, i_local: int) -> torch.Tensor:
    """silu(x @ gate^T) * (x @ up^T) with gate_up_w = [gate; up] rows.

    GPU decode (M <= 8): one fused HIP kernel, no [*, 2I] intermediate.
    Otherwise: library GEMM + the silu_mul kernel."""
    M = x.numel() // x.shape[-1]
    if (
        x.is_cuda
        and x.dtype == torch.bfloat16
        and (_gemv_m_ok(M) or _bf16_mfma_ok(M, x.shape[-1], gateup=True))
        and x.shape[-1] % 8 == 0
        and x.is_contiguous()
    ):
        from opsagent_amd.ops import hip_lib

        lib = hip_lib.get_lib()
        out = torch.empty(*x.shape[:-1], i_local, dtype=x.dtype, device=x.device)
        rc = lib.oa_gemv_gateup(
            hip_lib.current_stream_ptr(), x.data_ptr(), gate_up_w.data_ptr(),
            out.data_ptr(), M, i_local, x.shape[-1],
        )
        hip_lib.check(rc, "oa_gemv_gateup")
        return out
    gu = linear(x, gate_up_w)
    gate, up = gu.split([i_local, i_local], dim=-1)
    return silu_mul(gate.contiguous(), up.contiguous())


def gateup_act(x: torch.Tensor, gate_up_w: torch.Tensor, i_local: int,
               act: str = "silu") -> torch.Tensor:
    """act(x @ gate^T) * (x @ up^T), act "silu" | "gelu_tanh", for decode-sized
    bf16 batches: one fused GEMV launch."""
    if act == "silu":
        return gateup_silu(x, gate_up_w, i_local)
    from opsagent_amd.ops import hip_lib

    M = x.numel() // x.shape[-1]
    assert x.is_cuda and x.dtype == torch.bfloat16 and x.is_contiguous() and act == "gelu_tanh"
    lib = hip_lib.get_lib()
    out = torch.empty(*x.shape[:-1], i_local, dtype=x.dtype, device=x.device)
    rc = lib.oa_gemv_gateup_act(
        hip_lib.current_stream_ptr(), x.data_ptr(), gate_up_w.data_ptr(),
        out.data_ptr(), M, i_local, x.shape[-1], 1,
    )
    hip_lib.check(rc, "oa_gemv_gateup_act")
    return out


def kv_cache_write(
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    """k/v: [T, Hk, D]; caches [num_blocks, block_size, Hk, D]; slots int32 [T]."""
    if not _is_gpu(k):
        torch_ref.kv_cache_write(k_cache, v_cache, k, v, slot_mapping.long())
        return
    assert k.dtype == torch.bfloat16 and k.is_contiguous() and v.is_contiguous()
    assert slot_mapping.dtype == torch.int32
    lib, hip = _lib()
    T, Hk, D = k.shape
    rc = lib.oa_kv_write(
        hip.current_stream_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
        k.data_ptr(), v.data_ptr(), slot_mapping.data_ptr(), T, Hk, D,
    )
    hip.check(rc, "oa_kv_write")


def attention_prefill(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: Optional[float] = None,
    causal: bool = True,
) -> torch.Tensor:
    """q [B, Sq, Hq, D]; k, v [B, Skv, Hk, D] (token-major layouts; the CPU
    reference uses [B, H, S, D], so the dispatch transposes for it)."""
    if not _is_gpu(q):
        out = torch_ref.attention_prefill(
            q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), scale, causal
        )
        return out.transpose(1, 2).contiguous()
    assert causal, "GPU prefill kernel is causal-only"
    assert q.dtype == torch.bfloat16
    B, Sq, Hq, D = q.shape
    Skv, Hk = k.shape[1], k.shape[2]
    for t, name in ((q, "q"), (k, "k"), (v, "v")):
        assert t.stride(3) == 1 and t.stride(2) == D, f"{name} heads must be inner-contiguous"
        assert t.shape[0] == 1 or t.stride(0) == t.shape[1] * t.stride(1), f"{name} batch stride"
    scale = scale if scale is not None else D ** -0.5
    lib, hip = _lib()
    out = torch.empty(B, Sq, Hq, D, dtype=q.dtype, device=q.device)
    rc = lib.oa_attention_prefill(
        hip.current_stream_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
        out.data_ptr(), B, Hq, Hk, Sq, Skv, D, scale,
        q.stride(1), k.stride(1), v.stride(1),
    )
    hip.check(rc, "oa_attention_prefill")
    return out


def decode_nsplit(batch: int, n_kv_heads: int, max_len: int) -> int:
    """Split the key range so the grid covers 256 CUs with a couple of
    blocks each (≫256 workgroups rule). Minimum split granule is 64 keys
    (16 per wave). Target 512 blocks, not more: each extra split adds a
    partial the combine must re-read, and the 4-deep load pipeline wants
    ≥8 key-quads per wave to hide HBM latency (A/B at B=1 len 8192:
    nsplit 128 -> 64 cut the step's attention+combine time)."""
    tgt_blocks = int(os.environ.get("OPSAGENT_DECODE_NSPLIT_TARGET", "512"))
    target = max(1, tgt_blocks // max(1, batch * n_kv_heads))
    return int(max(1, min(target, (max_len + 63) // 64)))


def attention_decode_paged(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_lens: torch.Tensor,
    scale: Optional[float] = None,
    workspace: Optional[Tuple[torch.Tensor, ...]] = None,
    nsplit: Optional[int] = None,
    fused_combine: bool = False,
) -> torch.Tensor:
    """q [B, Hq, D]; caches [num_blocks, block_size, Hk, D]; out [B, Hq, D].

    fused_combine folds the split reduction into the attention launch via the
    in-launch G16 release/acquire hand-off (one kernel + a memset node
    instead of two kernels per layer). Measured on MI355X it is ~0.4 ms/step
    SLOWER than the two-kernel form at 8B decode (the single last-arriving
    block serializes a reduction the combine kernel spreads over B*Hq blocks)
    — kept as a correct, tested option; default off."""
    if not _is_gpu(q):
        return torch_ref.attention_decode_paged(q, k_cache, v_cache, block_table, seq_lens, scale)
    assert q.dtype == torch.bfloat16
    assert q.stride(2) == 1 and q.stride(1) == q.shape[2], "q heads must be inner-contiguous"
    assert block_table.dtype == torch.int32 and seq_lens.dtype == torch.int32
    B, Hq, D = q.shape
    nb, block_size, Hk, _ = k_cache.shape
    G = Hq // Hk
    scale = scale if scale is not None else D ** -0.5
    if nsplit is None:
        nsplit = decode_nsplit(B, Hk, int(block_table.shape[1] * block_size))
    if workspace is None:
        o_part = torch.empty(B * Hk * nsplit, G, D, dtype=torch.float32, device=q.device)
        ml_part = torch.empty(B * Hk * nsplit, G, 2, dtype=torch.float32, device=q.device)
        cnt_ws = torch.empty(B * Hk, dtype=torch.int32, device=q.device)
    else:
        o_part, ml_part, cnt_ws = workspace
    lib, hip = _lib()
    out = torch.empty(B, Hq, D, dtype=q.dtype, device=q.device)
    rc = lib.oa_attention_decode(
        hip.current_stream_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
        block_table.data_ptr(), seq_lens.data_ptr(), o_part.data_ptr(),
        ml_part.data_ptr(), cnt_ws.data_ptr(), out.data_ptr(), B, Hq, Hk, D,
        block_table.shape[1], block_size, nsplit, scale, q.stride(0),
        1 if fused_combine else 0,
    )
    hip.check(rc, "oa_attention_decode")
    return out


def _bf16_prenorm() -> bool:
    """OPSAGENT_BF16_PRENORM=1: at M=1 run rmsnorm as its own pass and the
    PLAIN bf16 gemv (A/B knob mirroring the fp8 M=1 prenorm win)."""
    return os.environ.get("OPSAGENT_BF16_PRENORM", "0") == "1"


def _fp8_mfma_ok(M: int, K: int, gateup: bool = False) -> bool:
    """Mirror of fp8_moe.hip's gemv_fp8_use_mfma for the M 9..16 range
    (the VALU kernels have no 9-11/13-15 instantiations — those batch
    sizes are only reachable through the MFMA stream)."""
    if os.environ.get("OPSAGENT_FP8_GEMV_MFMA", "") == "0":
        return False
    # unlike bf16 (whose M>8 alternative is a decent hipBLASLt skinny
    # kernel), fp8's M 9..16 alternative is the 128-row tile GEMM on an
    # underfilled grid — in-engine c16 fp8: MFMA gemv 8.93 t/s vs 7.40
    # through the GEMM. Keep the full M 2..16 range here.
    if K % 512 != 0 or (K // 512) % (4 if gateup else 8) != 0:
        return False
    return 2 <= M <= 16 and M * K <= 131072


def _fp8_gemv_ok(x: torch.Tensor) -> bool:
    M = x.numel() // x.shape[-1]
    K = x.shape[-1]
    return (
        x.is_cuda and x.dtype == torch.bfloat16
        and (M <= 8 or _fp8_mfma_ok(M, K))
        and K % 16 == 0 and x.is_contiguous()
    )


def linear_norm_fp8(
    x: torch.Tensor, norm_w: torch.Tensor, eps: float,
    w8: torch.Tensor, w_scale: torch.Tensor,
) -> torch.Tensor:
    """rmsnorm(x) @ dequant(W8)^T with the norm fused into the fp8 GEMV
    prologue (fp8 decode fast path). At M=1 the VALU stream kernel runs the
    norm per ELEMENT inside the weight loop (measured 2.7 vs 5.1 TB/s on the
    70B qkv shape), so a single rmsnorm pass + the plain kernel wins; the
    M>=2 MFMA path fuses the norm into its one-shot x-quant instead."""
    if not _fp8_gemv_ok(x):
        return linear_fp8(rms_norm(x, norm_w, eps), w8, w_scale)
    lib, hip = _lib()
    M = x.numel() // x.shape[-1]
    if M == 1:
        return linear_fp8(rms_norm(x, norm_w, eps), w8, w_scale)
    N, K4 = w8.shape[0], x.shape[-1]
    out = torch.empty(*x.shape[:-1], N, dtype=x.dtype, device=x.device)
    rc = lib.oa_gemv_fp8_ex(
        hip.current_stream_ptr(), x.data_ptr(), w8.data_ptr(),
        w_scale.data_ptr(), out.data_ptr(), norm_w.data_ptr(), None,
        M, N, K4, eps, 1,
    )
    hip.check(rc, "oa_gemv_fp8_ex(norm)")
    return out


def linear_addres_fp8(
    x: torch.Tensor, w8: torch.Tensor, w_scale: torch.Tensor,
    res: torch.Tensor,
) -> torch.Tensor:
    """x @ dequant(W8)^T + res (fp8 residual-producing projection)."""
    if not (_fp8_gemv_ok(x) and res.is_contiguous()):
        return linear_fp8(x, w8, w_scale) + res
    lib, hip = _lib()
    M = x.numel() // x.shape[-1]
    N = w8.shape[0]
    out = torch.empty(*x.shape[:-1], N, dtype=x.dtype, device=x.device)
    rc = lib.oa_gemv_fp8_ex(
        hip.current_stream_ptr(), x.data_ptr(), w8.data_ptr(),
        w_scale.data_ptr(), out.data_ptr(), None, res.data_ptr(),
        M, N, x.shape[-1], 0.0, 2,
    )
    hip.check(rc, "oa_gemv_fp8_ex(addres)")
    return out


def gateup_silu_fp8(
    x: torch.Tensor, w8: torch.Tensor, w_scale: torch.Tensor, i_local: int,
    norm_w: Optional[torch.Tensor] = None, eps: float = 0.0,
) -> torch.Tensor:
    """silu(x @ gate8^T) * (x @ up8^T) with fp8 [gate; up] weights; optional
    fused rmsnorm prologue. Falls back to linear_fp8 + silu_mul."""
    use_norm = norm_w is not None
    _Mgu = x.numel() // x.shape[-1]
    if not _fp8_gemv_ok(x) or (
        _Mgu in (5, 7) and not _fp8_mfma_ok(_Mgu, x.shape[-1], gateup=True)
    ):
        xin = rms_norm(x, norm_w, eps) if use_norm else x
        gu = linear_fp8(xin, w8, w_scale)
        g, u = gu.split([i_local, i_local], dim=-1)
        return silu_mul(g.contiguous(), u.contiguous())
    lib, hip = _lib()
    M = x.numel() // x.shape[-1]
    if use_norm and M == 1:  # see linear_norm_fp8: prenorm beats in-loop norm
        x = rms_norm(x, norm_w, eps)
        norm_w = None
        use_norm = False
    out = torch.empty(*x.shape[:-1], i_local, dtype=x.dtype, device=x.device)
    rc = lib.oa_gemv_gateup_fp8(
        hip.current_stream_ptr(), x.data_ptr(), w8.data_ptr(),
        w_scale.data_ptr(), out.data_ptr(),
        norm_w.data_ptr() if use_norm else None,
        M, i_local, x.shape[-1], eps, 1 if use_norm else 0,
    )
    hip.check(rc, "oa_gemv_gateup_fp8")
    return out


def attention_decode_rope(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_lens: torch.Tensor,
    cos: torch.Tensor,
    sin: torch.Tensor,
    slots: torch.Tensor,
    scale: Optional[float] = None,
    workspace: Optional[Tuple[torch.Tensor, ...]] = None,
    nsplit: Optional[int] = None,
) -> torch.Tensor:
    """Fully-fused decode attention: RoPE(q, k) + paged-KV scatter + split-K
    attention + combine in two launches, replacing the separate rope_kv
    launch per layer. q [B, Hq, D], k/v [B, Hk, D] are the RAW (un-roped)
    GEMV outputs (head-slice views of the fused qkv buffer are fine —
    per-tensor token strides); slots [B] int32 gives the new token's cache
    slot. CPU path: rope_kv then the torch reference attention."""
    if not _is_gpu(q):
        positions = (seq_lens.to(torch.int64) - 1).to(torch.int32)
        q2, k2 = torch_ref.rope_apply(q, k, cos, sin, positions)
        torch_ref.kv_cache_write(k_cache, v_cache, k2, v, slots.long())
        return torch_ref.attention_decode_paged(
            q2, k_cache, v_cache, block_table, seq_lens, scale
        )
    assert q.dtype == torch.bfloat16
    assert q.stride(2) == 1 and q.stride(1) == q.shape[2]
    assert k.stride(2) == 1 and k.stride(1) == k.shape[2]
    assert v.stride(2) == 1 and v.stride(1) == v.shape[2]
    assert block_table.dtype == torch.int32 and seq_lens.dtype == torch.int32
    assert slots.dtype == torch.int32
    B, Hq, D = q.shape
    nb, block_size, Hk, _ = k_cache.shape
    G = Hq // Hk
    scale = scale if scale is not None else D ** -0.5
    if nsplit is None:
        nsplit = decode_nsplit(B, Hk, int(block_table.shape[1] * block_size))
    if workspace is None:
        o_part = torch.empty(B * Hk * nsplit, G, D, dtype=torch.float32, device=q.device)
        ml_part = torch.empty(B * Hk * nsplit, G, 2, dtype=torch.float32, device=q.device)
    else:
        o_part, ml_part = workspace[0], workspace[1]
    lib, hip = _lib()
    out = torch.empty(B, Hq, D, dtype=q.dtype, device=q.device)
    rc = lib.oa_attention_decode_rope(
        hip.current_stream_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
        k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(),
        seq_lens.data_ptr(), cos.data_ptr(), sin.data_ptr(), slots.data_ptr(),
        o_part.data_ptr(), ml_part.data_ptr(), out.data_ptr(), B, Hq, Hk, D,
        block_table.shape[1], block_size, nsplit, scale, q.stride(0),
        k.stride(0), v.stride(0),
    )
    hip.check(rc, "oa_attention_decode_rope")
    return out


def greedy_sample_masked(
    logits: torch.Tensor, mask_bits: Optional[torch.Tensor]
) -> torch.Tensor:
    """logits [B, V] bf16 (GPU) / any float (CPU); mask_bits uint32-packed
    [B, ceil(V/32)] on GPU, bool [B, V] on CPU. Returns int32/int64 [B]."""
    if not _is_gpu(logits):
        return torch_ref.greedy_sample_masked(logits, mask_bits)
    lib, hip = _lib()
    B, V = logits.shape
    out = torch.empty(B, dtype=torch.int32, device=logits.device)
    if logits.dtype == torch.float32:
        # float32 rows of any width (hybrid models' soft-capped logits)
        assert logits.is_contiguous()
        if mask_bits is not None:
            assert mask_bits.dtype == torch.int32 and mask_bits.is_contiguous()
        ws32 = torch.empty(B * 16 * 2, dtype=torch.int32, device=logits.device)
        rc = lib.oa_masked_argmax_f32(
            hip.current_stream_ptr(), logits.data_ptr(),
            mask_bits.data_ptr() if mask_bits is not None else None,
            ws32.data_ptr(), out.data_ptr(), B, V,
        )
        hip.check(rc, "oa_masked_argmax_f32")
        return out
    assert logits.dtype == torch.bfloat16 and logits.is_contiguous()
    ws = torch.empty(B, dtype=torch.int64, device=logits.device)
    mask_ptr = mask_bits.data_ptr() if mask_bits is not None else None
    if mask_bits is not None:
        assert mask_bits.dtype == torch.int32 and mask_bits.is_contiguous()
    rc = lib.oa_masked_argmax(
        hip.current_stream_ptr(), logits.data_ptr(), mask_ptr, ws.data_ptr(),
        out.data_ptr(), B, V,
    )
    hip.check(rc, "oa_masked_argmax")
    return out
