"""DeepSeek-V3-style Mixture-of-Experts MLP (BASELINE config #5).

Routing: softmax top-k over a router linear, normalized weights, plus
`moe_shared_experts` always-on shared experts (DeepSeek style). Experts are
TP-sharded on the intermediate dim (column-parallel w1/w3, row-parallel w2,
one all-reduce with the shared-expert output folded in).

Compute path v1: dense grouped GEMMs via torch (hipBLASLt batched) with
token gather/scatter. The CDNA4 fp8-MFMA expert GEMM kernel (spec.moe_dtype
== "fp8") is the planned upgrade — see ops/csrc/ notes.
"""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F
from torch import nn

from opsagent_amd import ops
from opsagent_amd.engine.config import ModelSpec
from opsagent_amd.engine.model import _init_linear, _shard  # noqa: F401
from opsagent_amd.parallel import get_tp_rank, get_tp_size, tp_all_reduce


class MoEMLP(nn.Module):
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, gen: torch.Generator):
        super().__init__()
        tp, rank = get_tp_size(), get_tp_rank()
        h = spec.hidden_size
        e = spec.moe_num_experts
        i_moe = spec.moe_intermediate_size
        assert i_moe % tp == 0
        self.top_k = spec.moe_top_k
        self.num_experts = e
        self.i_local = i_moe // tp

        self.router_w = nn.Parameter(_init_linear(gen, e, h, torch.float32), requires_grad=False)
        w13 = torch.stack(
            [
                torch.cat([_init_linear(gen, i_moe, h, dtype), _init_linear(gen, i_moe, h, dtype)], 0)
                for _ in range(e)
            ]
        )  # [E, 2*I, H]
        w2 = torch.stack([_init_linear(gen, h, i_moe, dtype) for _ in range(e)])  # [E, H, I]
        # shard: w13 rows (both gate and up halves), w2 cols
        if tp > 1:
            gate = w13[:, :i_moe, :]
            up = w13[:, i_moe:, :]
            w13 = torch.cat(
                [_shard(gate, 1, rank, tp), _shard(up, 1, rank, tp)], dim=1
            )
            w2 = _shard(w2, 2, rank, tp)
        self.fp8 = spec.moe_dtype == "fp8"
        if self.fp8:
            # CDNA4 OCP-e4m3 expert weights (per-row scales): halves the
            # expert weight stream at decode and enables the fp8 MFMA GEMM
            # at prefill (ops/csrc/fp8_moe.hip)
            from opsagent_amd.ops import torch_ref as _tr

            q13 = torch.empty(*w13.shape, dtype=torch.uint8)
            s13 = torch.empty(e, w13.shape[1], dtype=torch.float32)
            q2 = torch.empty(*w2.shape, dtype=torch.uint8)
            s2 = torch.empty(e, w2.shape[1], dtype=torch.float32)
            for ei in range(e):
                q13[ei], s13[ei] = _tr.quant_fp8(w13[ei])
                q2[ei], s2[ei] = _tr.quant_fp8(w2[ei])
            self.w13_q = nn.Parameter(q13, requires_grad=False)
            self.w13_s = nn.Parameter(s13, requires_grad=False)
            self.w2_q = nn.Parameter(q2, requires_grad=False)
            self.w2_s = nn.Parameter(s2, requires_grad=False)
            self.w13 = self.w2 = None
        else:
            self.w13 = nn.Parameter(w13.contiguous(), requires_grad=False)
            self.w2 = nn.Parameter(w2.contiguous(), requires_grad=False)

        self._force_loop = False  # tests compare grouped vs loop paths
        self.n_shared = spec.moe_shared_experts
        if self.n_shared > 0:
            from opsagent_amd.engine.model import DenseMLP
            import copy

            shared_spec = copy.copy(spec)
            shared_spec.intermediate_size = i_moe * self.n_shared
            shared_spec.moe_num_experts = None
            self.shared = DenseMLP(shared_spec, dtype, gen)
        else:
            self.shared = None

    def forward(self, x: torch.Tensor, decode: bool = False) -> torch.Tensor:
        T, H = x.shape
        router_logits = F.linear(x.float(), self.router_w)  # [T, E]
        probs = torch.softmax(router_logits, dim=-1)
        topw, topi = probs.topk(self.top_k, dim=-1)           # [T, K]
        topw = (topw / topw.sum(dim=-1, keepdim=True)).to(x.dtype)

        # grouped path: pair-major kernels for tiny T; for DECODE batches
        # past 64 the expert-major kernels keep the stage in one
        # static-shaped launch pair (graph-capturable to batch 256).
        # Prefill-sized T stays on the sorted per-expert hipBLASLt loop —
        # extending the GEMV-style grouped path to 65..341-token prefill
        # chunks measured -18% on the moe-small c=4 turn.
        grouped_ok = T <= 64 or (decode and T * self.top_k <= 2048)
        if x.is_cuda and grouped_ok and not self._force_loop:
            # grouped-kernel path: one launch per stage for all pairs, no
            # host sync, shape-static -> hipGraph-capturable decode
            flat_e = topi.reshape(-1).to(torch.int32).contiguous()
            # NOTE: for T=1 expand().reshape(-1) is a stride-0 VIEW whose
            # data_ptr covers one element — must materialize contiguously
            flat_t = (
                torch.arange(T, device=x.device, dtype=torch.int32)
                .repeat_interleave(self.top_k)
                .contiguous()
            )
            flat_w = topw.reshape(-1).float().contiguous()
            y = ops.moe_grouped_mlp(
                x.contiguous(),
                self.w13_q if self.fp8 else self.w13,
                self.w13_s if self.fp8 else None,
                self.w2_q if self.fp8 else self.w2,
                self.w2_s if self.fp8 else None,
                flat_e, flat_t, flat_w, self.i_local, self.fp8,
                num_experts=self.num_experts,
            )
            out = torch.zeros_like(x)
            out.index_add_(0, flat_t.long(), y)
            if self.shared is not None:
                return tp_all_reduce(out) + self.shared(x)
            return tp_all_reduce(out)

        out = torch.zeros_like(x)
        # token gather per expert (sorted dispatch)
        flat_e = topi.reshape(-1)                              # [T*K]
        flat_t = (
            torch.arange(T, device=x.device).unsqueeze(1).expand(T, self.top_k).reshape(-1)
        )
        flat_w = topw.reshape(-1)
        order = torch.argsort(flat_e)
        flat_e, flat_t, flat_w = flat_e[order], flat_t[order], flat_w[order]
        # ONE host sync for the whole dispatch (a per-expert .item() would be
        # num_experts GPU->CPU round trips per layer per token)
        counts = torch.bincount(flat_e, minlength=self.num_experts).cpu().tolist()
        start = 0
        for e in range(self.num_experts):
            c = counts[e]
            if c == 0:
                continue
            toks = flat_t[start : start + c]
            wts = flat_w[start : start + c].unsqueeze(1)
            start += c
            xe = x[toks].contiguous()
            if self.fp8:
                gu = ops.linear_fp8(xe, self.w13_q[e], self.w13_s[e])
                gate, up = gu.split([self.i_local, self.i_local], dim=-1)
                act = ops.silu_mul(gate.contiguous(), up.contiguous())
                ye = ops.linear_fp8(act.contiguous(), self.w2_q[e], self.w2_s[e])
            else:
                gu = ops.linear(xe, self.w13[e])
                gate, up = gu.split([self.i_local, self.i_local], dim=-1)
                act = ops.silu_mul(gate.contiguous(), up.contiguous())
                ye = ops.linear(act, self.w2[e])
            out.index_add_(0, toks, ye * wts)
        if self.shared is not None:
            # shared expert runs its own all-reduce; fold by adding after
            out = tp_all_reduce(out) + self.shared(x)
            return out
        return tp_all_reduce(out)

    def forward_loop(self, x: torch.Tensor) -> torch.Tensor:
        """Force the per-expert loop path (test oracle for the grouped kernels)."""
        self._force_loop = True
        try:
            return self.forward(x)
        finally:
            self._force_loop = False


class RoutedExperts(nn.Module):
    """Mixture of gated feed-forwards with a score-and-choose router whose
    every constant is a RouterSpec field: sigmoid (or softmax) scores, a
    learned correction that enters the CHOICE only, group-limited choice
    (groups rated by their two best scores or their best one), weights
    normalised over the chosen experts (or not) and scaled, the experts'
    gate activation with its constants, an optional always-on shared expert
    with an optional per-token sigmoid gate whose projection is one more row
    of the float32 router matrix. Router logits, scores and weights are
    float32. With r.bias the router adds a learned vector to its logits;
    with r.gated False an expert (and the shared one) is down(act(up x)).

    Expert weights are stacked: w13 [E, 2I, C] (gate rows, then up rows; up
    rows alone, [E, I, C], for ungated experts) and w2 [E, C, I]. Few (token, expert) pairs run through two static-shaped
    launches without host sync (hipGraph-capturable); prompt-sized batches
    are sorted by expert and run one library GEMM pair per used expert.
    """

    def __init__(self, hidden: int, r, dtype: torch.dtype, gen: torch.Generator,
                 act: Optional[str] = None):
        super().__init__()
        if get_tp_size() != 1:
            raise NotImplementedError("routed experts run at tensor-parallel size 1")
        from opsagent_amd.engine.hybrid import GatedMLP, PlainMLP, _param, _rand

        act = act or r.act
        shared_act = act
        if act == "clamp_swish":
            act = ("clamp_swish", float(r.limit), float(r.alpha))
            shared_act = ("clamp_swish", float(r.shared_limit or r.limit), float(r.alpha))
        self.r, self.act, self.hidden = r, act, hidden
        E, I = r.experts, r.ff
        self.shared_gate = bool(r.shared_gate and r.shared_ff)
        # router rows, then (optionally) the shared expert's gate row
        self.router_w = _param(_rand(gen, E + int(self.shared_gate), hidden, std=hidden ** -0.5))
        self.correction = _param(0.1 * _rand(gen, E)) if r.correction else None
        # the shared expert's gate row carries no bias
        self.router_b = (_param(torch.cat([0.5 * _rand(gen, E),
                                           torch.zeros(int(self.shared_gate), device=gen.device)]))
                         if r.bias else None)
        self.gated = bool(r.gated)
        self.w13 = _param(_rand(gen, E, (2 if self.gated else 1) * I, hidden,
                                std=hidden ** -0.5, dtype=dtype))
        self.w2 = _param(_rand(gen, E, hidden, I, std=I ** -0.5, dtype=dtype))
        self.shared = None
        if r.shared_ff:
            self.shared = (GatedMLP(hidden, r.shared_ff, dtype, gen, act=shared_act)
                           if self.gated else PlainMLP(hidden, r.shared_ff, dtype, gen, act=act))
        # weight bytes one launch pair may stream through the pair kernels
        self.pair_budget = 64 << 20
        self.force_path = None     # "pairs" | "sorted" (tests)

    def route(self, x: torch.Tensor, with_gate: bool = False):
        from opsagent_amd.ops import mixer_ops as mx

        logits = F.linear(x.float(), self.router_w, self.router_b)
        E = self.r.experts
        idx, wts = mx.route_topk(logits[:, :E], self.correction, self.r.top, self.r.groups,
                                 self.r.keep, self.r.scale, self.r.score, self.r.rating,
                                 self.r.renorm)
        if with_gate:
            return idx, wts, (logits[:, E] if self.shared_gate else None)
        return idx, wts

    def forward(self, x: torch.Tensor, decode: bool = False) -> torch.Tensor:
        """decode: the step holds one token per sequence; such batches stay on
        the static-shaped pair kernels up to 2048 pairs, so the step can be
        captured in a hipGraph."""
        out, shared, gate = self.forward_parts(x, decode)
        if shared is not None:
            if gate is not None:
                shared = (torch.sigmoid(gate).unsqueeze(1) * shared.float()).to(out.dtype)
            out = out + shared
        return out

    def forward_parts(self, x: torch.Tensor, decode: bool = False):
        """(routed sum, shared expert's output or None, float32 gate logits
        [T] of the shared expert or None): a caller that adds them to a
        residual can do so in one launch."""
        T, C = x.shape
        idx, wts, gate = self.route(x, with_gate=True)
        P, I = T * self.r.top, self.r.ff
        esz = 4 if x.dtype == torch.float32 else 2
        pairs = (P <= 64 or P * (3 if self.gated else 2) * I * C * esz <= self.pair_budget
                 or (decode and P <= 2048))
        if self.force_path is not None:
            pairs = self.force_path == "pairs"
        if pairs:
            out = self._pairs(x, idx, wts)
        else:
            out = self._sorted(x, idx, wts)
        return out, (self.shared(x) if self.shared is not None else None), gate

    def _pairs(self, x, idx, wts):
        from opsagent_amd.ops import mixer_ops as mx

        T, C = x.shape
        I, top = self.r.ff, self.r.top
        fast_act = (self.act == "silu" or (isinstance(self.act, tuple)
                                           and self.act[0] == "clamp_swish")
                    or (not self.gated and self.act == "relu2"))
        if (x.is_cuda and x.dtype == torch.bfloat16 and fast_act
                and C % 16 == 0 and I % 16 == 0 and self.force_path is None):
            # the framework's grouped expert GEMV kernels (pair- or expert-major)
            flat_t = torch.arange(T, device=x.device, dtype=torch.int32).repeat_interleave(top)
            y = ops.moe_grouped_mlp(x.contiguous(), self.w13, None, self.w2, None,
                                    idx.reshape(-1), flat_t.contiguous(),
                                    wts.reshape(-1).contiguous(), I, False,
                                    num_experts=self.r.experts, act=self.act)
            return y.view(T, top, C).float().sum(1).to(x.dtype)
        if not self.gated:
            return mx.moe_pairs_plain(x.contiguous(), self.w13, self.w2, idx, wts, self.act)
        return mx.moe_pairs_mlp(x.contiguous(), self.w13, self.w2, idx, wts, self.act)

    def _sorted(self, x, idx, wts):
        from opsagent_amd.ops import mixer_ops as mx

        T, C = x.shape
        top, I = self.r.top, self.r.ff
        flat_e = idx.reshape(-1).long()
        order = torch.argsort(flat_e, stable=True)
        tok = torch.div(order, top, rounding_mode="floor")
        w_sorted = wts.reshape(-1)[order]
        # ONE host sync for the whole dispatch
        counts = torch.bincount(flat_e, minlength=self.r.experts).cpu().tolist()
        xs = x.index_select(0, tok)
        ys = torch.empty(T * top, C, dtype=torch.float32, device=x.device)
        start = 0
        for e, c in enumerate(counts):
            if c == 0:
                continue
            gu = ops.linear(xs[start : start + c], self.w13[e])
            a = mx.act_mul_rows(gu, I, self.act) if self.gated else mx.act_rows(gu, self.act)
            ys[start : start + c] = ops.linear(a, self.w2[e]).float()
            start += c
        ys *= w_sorted.unsqueeze(1)
        # back to (token, choice) order: a token's experts are summed in its
        # own order whatever else the batch holds
        inv = torch.empty_like(order)
        inv[order] = torch.arange(order.numel(), device=order.device)
        return ys.index_select(0, inv).view(T, top, C).sum(1).to(x.dtype)

    def load(self, get, put, p: str) -> None:
        E = self.r.experts
        put(self.router_w, [get(p + "router")]
            + ([get(p + "shared.sg")] if self.shared_gate else []))
        if self.correction is not None:
            put(self.correction, [get(p + "correction")])
        if self.router_b is not None:
            put(self.router_b, [get(p + "router.b")]
                + ([torch.zeros(1)] if self.shared_gate else []))
        if self.gated:
            w13 = torch.stack([torch.cat([get(f"{p}e{k}.gate"), get(f"{p}e{k}.up")], 0)
                               for k in range(E)])
        else:
            w13 = torch.stack([get(f"{p}e{k}.up") for k in range(E)])
        w2 = torch.stack([get(f"{p}e{k}.down") for k in range(E)])
        self.w13.data.copy_(w13.to(self.w13.device, self.w13.dtype))
        self.w2.data.copy_(w2.to(self.w2.device, self.w2.dtype))
        if self.shared is not None:
            self.shared.load(get, put, p + "shared.")
