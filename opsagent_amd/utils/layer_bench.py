"""Prefill and decode throughput of a hybrid decoder beside the llama model
of equal width, depth, head geometry and feed-forward size (random weights,
random token ids). Used by `bench.py --mode layers`.

For each size both engines get the same workload through the same public
path (add_request + step): B prompts of P tokens are read, then D tokens are
decoded greedily per request. Prefill tokens/s = B*P / time until every
prompt is read; decode tokens/s = B*D / time of the decode steps.
"""

from __future__ import annotations

import dataclasses
import time
from typing import Dict, List

import torch

from opsagent_amd.engine.config import (
    ModelSpec,
    povazen_config_dict,
    povazen_spec_from_dict,
    rafodra_config_dict,
    rafodra_spec_from_dict,
    suzulix_config_dict,
    suzulix_spec_from_dict,
    vazilorn_config_dict,
    vazilorn_spec_from_dict,
)

# (name, width, heads, kv_heads, head dim, ff, layers)
SIZES = [
    ("1b-class", 2048, 16, 4, 128, 8192, 4),
    ("8b-class", 4096, 32, 8, 128, 14336, 4),
]


def specs_for(size) -> Dict[str, object]:
    name, width, heads, kv, dim, ff, layers = size
    llama = ModelSpec(
        name=f"llama-{name}", vocab_size=32000, hidden_size=width, intermediate_size=ff,
        num_layers=layers, num_heads=heads, num_kv_heads=kv, head_dim=dim, max_seq_len=8192,
    )
    pattern = ("da" * layers)[:layers]           # delta and attention layers alternate
    hybrid = povazen_spec_from_dict(
        povazen_config_dict(vocab=32000, width=width, pattern=pattern, heads=heads,
                            kv_heads=kv, dim=dim, vdim=dim, ff=ff, delta_heads=heads),
        name=f"povazen-{name}",
    )
    # routed feed-forwards of equal shape in both families: 16 experts of
    # ff/8, 4 per token, one shared expert of the same size
    experts, top, eff = 16, 4, ff // 8
    llama_moe = dataclasses.replace(
        llama, name=f"llama-moe-{name}", moe_num_experts=experts, moe_top_k=top,
        moe_intermediate_size=eff, moe_shared_experts=1,
    )

    def vz(pattern, window, tag):
        return vazilorn_spec_from_dict(
            vazilorn_config_dict(vocab=32000, width=width, pattern=pattern * layers, heads=heads,
                                 kv_heads=kv, dim=dim, vdim=dim, ff=ff, window=window,
                                 experts=experts, top=top, expert_ff=eff, groups=4, keep=2,
                                 router_scale=2.0, shared_ff=eff, rot_base=500000.0),
            name=f"vazilorn-{tag}-{name}",
        )

    def rf(pattern, tag):
        # every mixer kind once per four layers: lightning, gated linear
        # attention, latent attention, latent attention on the same latent.
        # Linear-attention heads have llama's head size; the cached latent is
        # 192 + 64 wide (one row per token for all heads)
        return rafodra_spec_from_dict(
            rafodra_config_dict(vocab=32000, width=width, pattern=(pattern * layers)[:2 * layers],
                                heads=heads, dim=dim, vdim=dim, ff=ff, kv_rank=192, rot_dim=64,
                                rot_base=500000.0, lin_heads=heads, lin_dim=dim, lin_vdim=dim,
                                experts=experts, top=top, expert_ff=eff, groups=4, keep=2,
                                router_scale=2.0, limit=7.0, shared_ff=eff, shared_limit=7.0,
                                embed_scale=1.0),
            name=f"rafodra-{tag}-{name}",
        )

    def sz(pattern, streams, tag):
        # latent attention, differential attention (two maps of half a head
        # each: llama's query/key width), retention twice; the cached latent
        # and the routed feed-forwards have Rafodra's shapes (experts ungated)
        return suzulix_spec_from_dict(
            suzulix_config_dict(vocab=32000, width=width, pattern=(pattern * layers)[:2 * layers],
                                heads=heads, kv_heads=kv, dim=dim // 2, vdim=dim, kv_rank=192,
                                q_rank=width // 4, rot_dim=64, lat_dim=dim, lat_vdim=dim,
                                rot_base=500000.0, ret_heads=heads, ret_dim=dim, ret_vdim=dim,
                                experts=experts, top=top, expert_ff=eff, shared_ff=eff,
                                streams=streams),
            name=f"suzulix-{tag}-{name}",
        )

    return {
        "suzulix": sz("LmAmRmRm", 2, "moe"),
        # mixers alone (no feed-forward) beside Rafodra's: what the streams,
        # the two maps and the rotation cost without the experts
        "suzulix-mix": sz("L-A-R-R-", 2, "mix"), "rafodra-mix": rf("L-G-A-S-", "mix"),
        "llama": llama, "povazen": hybrid, "llama-moe": llama_moe,
        "rafodra": rf("LdGdAdSd", "dense"), "rafodra-moe": rf("LmGmAmSm", "moe"),
        # a window wider than the prompt: the attention kernels do llama's work
        "vazilorn": vz("d", 8192, "dense"),
        # a window that pays: keys beyond it are never read
        "vazilorn-w512": vz("d", 512, "w512"),
        "vazilorn-moe": vz("m", 8192, "moe"),
    }


# which model each one is measured against
BASELINE_OF = {"povazen": "llama", "vazilorn": "llama", "vazilorn-w512": "llama",
               "vazilorn-moe": "llama-moe", "rafodra": "povazen", "rafodra-moe": "vazilorn-moe",
               "suzulix": "rafodra-moe", "suzulix-mix": "rafodra-mix"}


def _run(spec, batch: int, prompt: int, decode: int, reps: int) -> Dict[str, float]:
    from opsagent_amd.engine.engine import LLMEngine, SamplingParams

    eng = LLMEngine({
        "model": spec, "dtype": "bf16", "kv_block_size": 32,
        "kv_num_blocks": max(64, 2 * batch * ((prompt + decode) // 32 + 2)),
        "max_batch_size": max(batch, 1), "max_seq_len": 8192, "max_prefill_chunk": 8192,
        "tokenizer_check": False, "spec_decode": False, "seed": 7,
    })
    gen = torch.Generator().manual_seed(0)
    params = SamplingParams(max_new_tokens=decode, stop_on_eos=False)
    pre_s: List[float] = []
    dec_s: List[float] = []
    for rep in range(reps + 1):                  # first repetition warms up
        prompts = [torch.randint(300, 30000, (prompt,), generator=gen).tolist()
                   for _ in range(batch)]
        rids = [eng.add_request(p, params) for p in prompts]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while any(len(eng.requests[r].output_ids) == 0 for r in rids):
            eng.step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        while not all(eng.requests[r].finished for r in rids):
            eng.step()
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        for r in rids:
            eng.requests.pop(r)
        if rep:
            pre_s.append(t1 - t0)
            dec_s.append(t2 - t1)
    pre, dec = min(pre_s), min(dec_s)
    del eng
    torch.cuda.empty_cache()
    return {"prefill_tok_s": batch * prompt / pre, "decode_tok_s": batch * (decode - 1) / dec,
            "prefill_ms": pre * 1e3, "decode_ms_per_step": dec * 1e3 / (decode - 1)}


def run(sizes=None, prompt: int = 2048, decode: int = 64, batches=(1, 8), reps: int = 2,
        models=("llama", "povazen")) -> List[dict]:
    rows = []
    for size in (sizes or SIZES):
        specs = specs_for(size)
        for b in batches:
            row = {"size": size[0], "batch": b, "prompt": prompt, "decode": decode}
            for m in models:
                r = _run(specs[m], b, prompt, decode, reps)
                row[m] = {k: round(v, 2) for k, v in r.items()}
            for m, base in BASELINE_OF.items():
                if m in row and base in row:
                    row[f"{m}_vs_{base}".replace("-", "_")] = {
                        "prefill": round(row[m]["prefill_tok_s"] / row[base]["prefill_tok_s"], 3),
                        "decode": round(row[m]["decode_tok_s"] / row[base]["decode_tok_s"], 3),
                    }
            rows.append(row)
    return rows
