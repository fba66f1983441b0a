"""Model architecture registry.

Llama-3 family dims (8B / 70B per BASELINE.json configs #2-#4), a tiny config
for CPU tests, and DeepSeek-V3-style MoE configs (BASELINE config #5). Random
initialization is the benchmark mode (no network for checkpoints); safetensors
loading is supported for real weights.
"""

from __future__ import annotations

import dataclasses
from typing import List, Optional


@dataclasses.dataclass
class ModelSpec:
    name: str
    vocab_size: int = 128256
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    rope_theta: float = 500000.0
    rms_eps: float = 1e-5
    max_seq_len: int = 8192
    tie_embeddings: bool = False
    # MoE (None => dense MLP)
    moe_num_experts: Optional[int] = None
    moe_top_k: int = 2
    moe_intermediate_size: Optional[int] = None
    moe_shared_experts: int = 0
    moe_dtype: str = "bf16"  # "fp8" enables the CDNA4 fp8 expert GEMM path

    is_hybrid = False

    @property
    def is_moe(self) -> bool:
        return self.moe_num_experts is not None


MODEL_REGISTRY = {
    # Llama-3 8B (BASELINE configs #2/#3)
    "llama3-8b": ModelSpec(
        name="llama3-8b",
        hidden_size=4096,
        intermediate_size=14336,
        num_layers=32,
        num_heads=32,
        num_kv_heads=8,
    ),
    # Llama-3 70B (BASELINE config #4, TP=8)
    "llama3-70b": ModelSpec(
        name="llama3-70b",
        hidden_size=8192,
        intermediate_size=28672,
        num_layers=80,
        num_heads=64,
        num_kv_heads=8,
    ),
    # tiny model for CPU tests (vocab covers the byte tokenizer's ~260 ids)
    "llama3-tiny": ModelSpec(
        name="llama3-tiny",
        vocab_size=512,
        hidden_size=128,
        intermediate_size=256,
        num_layers=2,
        num_heads=4,
        num_kv_heads=2,
        head_dim=32,
        max_seq_len=512,
    ),
    # tiny model whose head/vocab geometry divides by 4 (CPU world=4 TP tests)
    "llama3-tiny-w4": ModelSpec(
        name="llama3-tiny-w4",
        vocab_size=512,
        hidden_size=128,
        intermediate_size=256,
        num_layers=2,
        num_heads=8,
        num_kv_heads=4,
        head_dim=16,
        max_seq_len=512,
    ),
    # GPU-smoke-sized model (real head_dim for the HIP kernels)
    "llama3-micro": ModelSpec(
        name="llama3-micro",
        vocab_size=2048,
        hidden_size=1024,
        intermediate_size=2816,
        num_layers=4,
        num_heads=8,
        num_kv_heads=2,
        head_dim=128,
        max_seq_len=4096,
    ),
    # 8B-class projection shapes at 2 layers: exercises the K=4096 MFMA
    # GEMV paths (fp8 and bf16) end-to-end without an 8B weight build
    "llama3-2l4k": ModelSpec(
        name="llama3-2l4k",
        vocab_size=2048,
        hidden_size=4096,
        intermediate_size=14336,
        num_layers=2,
        num_heads=32,
        num_kv_heads=8,
        head_dim=128,
        max_seq_len=4096,
    ),
    # tiny MoE for CPU tests
    "moe-tiny": ModelSpec(
        name="moe-tiny",
        vocab_size=512,
        hidden_size=128,
        intermediate_size=256,
        num_layers=2,
        num_heads=4,
        num_kv_heads=2,
        head_dim=32,
        max_seq_len=512,
        moe_num_experts=8,
        moe_top_k=2,
        moe_intermediate_size=64,
        moe_shared_experts=1,
    ),
    # GPU-smoke-sized MoE (real head_dim, fp8-capable expert shapes)
    "moe-micro": ModelSpec(
        name="moe-micro",
        vocab_size=2048,
        hidden_size=1024,
        intermediate_size=2816,
        num_layers=4,
        num_heads=8,
        num_kv_heads=2,
        head_dim=128,
        max_seq_len=4096,
        moe_num_experts=16,
        moe_top_k=4,
        moe_intermediate_size=512,
        moe_shared_experts=1,
    ),
    # DeepSeek-V3-style MoE, scaled down to fit one MI355X comfortably
    # (BASELINE config #5: fp8 experts on CDNA4 MFMA)
    "deepseek-moe-small": ModelSpec(
        name="deepseek-moe-small",
        vocab_size=128256,
        hidden_size=2048,
        intermediate_size=8192,       # dense MLP for the first layer(s)
        num_layers=12,
        num_heads=16,
        num_kv_heads=4,
        moe_num_experts=64,
        moe_top_k=6,
        moe_intermediate_size=1408,
        moe_shared_experts=2,
    ),
    "deepseek-moe": ModelSpec(
        name="deepseek-moe",
        vocab_size=128256,
        hidden_size=4096,
        intermediate_size=14336,
        num_layers=28,
        num_heads=32,
        num_kv_heads=8,
        moe_num_experts=128,
        moe_top_k=8,
        moe_intermediate_size=2048,
        moe_shared_experts=1,
    ),
}


def get_model_spec(name):
    """A registry name, a checkpoint folder, or an already-built spec."""
    import os

    if not isinstance(name, str):
        return name
    if name in HYBRID_REGISTRY:
        cfg = HYBRID_REGISTRY[name]()
        return ARCHITECTURE_PARSERS[cfg["architecture"]](cfg, name=name)
    if os.path.isdir(name) and os.path.exists(os.path.join(name, "config.json")):
        return load_spec_from_dir(name)
    if name not in MODEL_REGISTRY:
        raise KeyError(f"unknown model {name!r}; known: {sorted(MODEL_REGISTRY)}")
    return MODEL_REGISTRY[name]


# ---------------------------------------------------------------------------
# Hybrid designs: a per-layer list of mixers (softmax attention, recurrent
# delta rule, ...) read from a checkpoint folder's config.json. Every size
# and every constant that can differ between checkpoints lives in the spec;
# nothing is taken from a particular checkpoint.


@dataclasses.dataclass
class MixerSpec:
    """One layer's token mixer. kind: "attention" (distance-penalty softmax
    attention) | "channel_delta" (gated delta rule) | "rotary_window"
    (rotary softmax attention with per-head query/key norm, an optional
    sliding window and an optional sink term) | "latent_attention" (softmax
    attention over a cached low-rank latent and one rotated key part shared
    by the heads) | "lightning" (linear attention with one fixed decay per
    head) | "gla" (linear attention with a learned decay per key channel) |
    "diff_attention" (rotary softmax attention in two maps per head over the
    same values, combined as a difference) | "retention" (rotary linear
    attention with one fixed decay per head)."""

    kind: str
    heads: int
    kv_heads: int
    dim: int                      # per-head query/key size
    vdim: int                     # per-head value size
    scale: Optional[float] = None  # attention score scale
    conv: int = 0                 # short-convolution taps (recurrent mixers)
    # inner sizes of the low-rank decay / output-gate projections; only the
    # checkpoint's tensor shapes give them (None => the mixer's default)
    decay_rank: Optional[int] = None
    gate_rank: Optional[int] = None
    # rotary attention: rotated channels per head (0 = none), frequency base,
    # wavelength-dependent rescaling {factor, low, high, original} or None
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_scaling: Optional[dict] = None
    # keys a query sees, itself included (None = all earlier keys)
    window: Optional[int] = None
    # a learned per-head term in the softmax denominator
    sink: bool = False
    # latent attention: size of the cached latent, rotated channels per head
    # (query) and of the shared key part, and the layer whose cached latent
    # this layer reads instead of projecting its own (None = its own)
    kv_rank: int = 0
    rot_dim: int = 0
    kv_from: Optional[int] = None
    # linear attention: fixed per-head decays ("lightning"), temperature of
    # the learned per-channel decay sigmoid(z)^(1/tau) ("gla")
    decay: Optional[List[float]] = None
    tau: float = 1.0
    # which channels a rotation pairs: "interleaved" (2i, 2i+1) or "half"
    # (i, i + rot_dims/2); the pairs' order does not change a dot product, so
    # a checkpoint in the "half" layout has its rows permuted once at load
    rot_layout: str = "interleaved"
    # score <- softcap * tanh(score / softcap) before the softmax (None = off)
    softcap: Optional[float] = None
    # differential attention: the constant of lambda and of the output scale
    diff: Optional[float] = None
    # latent attention: size of the normed latent the queries are projected
    # through (0 = queries come straight from the input)
    q_rank: int = 0
    # output gate read from the mixer input: "head" (one logit per head),
    # "channel" (one per output channel), "none"
    gate: str = "head"

    @property
    def has_kv(self) -> bool:
        return self.kind in ("attention", "rotary_window", "diff_attention") or (
            self.kind == "latent_attention" and self.kv_from is None)

    @property
    def has_state(self) -> bool:
        return self.kind in ("channel_delta", "lightning", "gla", "retention")


@dataclasses.dataclass
class RouterSpec:
    """Expert choice of a mixture-of-experts feed-forward. score: how router
    logits become scores s ("sigmoid" | "softmax"); with `correction` the
    ranking uses c = s + a learned vector while the mixing weights keep s;
    `groups` > 1 cuts the experts into runs of neighbours rated
    max1(c) + max2(c) (`rating` "top2") or max(c) ("max"), of which the
    `keep` top-rated may be picked from; w_j = scale * s_j / sum_k s_k over
    the `top` picked experts, or scale * s_j with renorm=False.
    act: the experts' gate activation ("silu" | "gelu_tanh" | "clamp_swish":
    g = min(gate, limit), u = clamp(up, -limit, limit),
    y = g sigmoid(alpha g) (u + 1)); the shared expert has its own limit and,
    with shared_gate, is scaled per token by the sigmoid of a learned
    projection. gated=False: an expert is down(act(up x)) with no gate
    branch (act "relu2": the square of relu). bias: the router adds a learned
    vector to its logits (it enters scores and choice alike)."""

    experts: int
    top: int
    ff: int                          # an expert's inner size
    score: str = "sigmoid"
    correction: bool = True
    groups: int = 1
    keep: int = 1
    scale: float = 1.0
    shared_ff: int = 0               # inner size of the always-on expert (0 = none)
    rating: str = "top2"
    renorm: bool = True
    act: str = "silu"
    limit: float = 0.0
    alpha: float = 1.702
    shared_limit: float = 0.0
    shared_gate: bool = False
    gated: bool = True
    bias: bool = False


@dataclasses.dataclass
class HybridLayerSpec:
    mixer: MixerSpec
    mlp_kind: Optional[str] = None   # None => no feed-forward; "dense" | "moe"
    mlp_ff: int = 0
    mlp_act: str = "silu"            # dense feed-forward gate activation
    router: Optional[RouterSpec] = None


@dataclasses.dataclass
class HybridSpec:
    """Architecture of a hybrid decoder (the Povazen design)."""

    name: str
    architecture: str
    vocab_size: int
    hidden_size: int
    layers: List[HybridLayerSpec]
    norm_eps: float
    norm_groups: int = 1
    canon_taps: int = 0
    logit_softcap: Optional[float] = None
    # "post_canon": grouped RMS norm on sublayer outputs, sublayers read
    # x + canon(x). "sandwich": a dynamic-tanh norm before and after every
    # sublayer. "pre_norm": a weighted layer norm before every sublayer.
    # "hyper": pre-norm sublayers (layer norm with weight and bias) around
    # `streams` residual streams joined by learned hyper-connections.
    layer_style: str = "post_canon"
    embed_scale: float = 1.0
    streams: int = 1
    # learned read/mix/write coefficients between the streams (False: the
    # plain residual sum, which is one stream with all coefficients 1)
    hyper: bool = False
    # layers [start, stop) run `times` times in a row with the same weights;
    # every pass keeps its own keys, values and state
    loop: Optional[tuple] = None
    # logits = head(norm(x)) * logit_scale; tied_head: the head is the
    # embedding table itself (without its scale)
    logit_scale: float = 1.0
    tied_head: bool = False
    max_seq_len: int = 1 << 20
    weights_path: Optional[str] = None

    is_moe = False
    is_hybrid = True

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def layer_runs(self) -> List[int]:
        """The layers in the order they run (a looped layer once per pass)."""
        n = len(self.layers)
        if not self.loop:
            return list(range(n))
        start, stop, times = self.loop
        return (list(range(start)) + list(range(start, stop)) * times
                + list(range(stop, n)))


def povazen_spec_from_dict(cfg: dict, name: str = "povazen") -> HybridSpec:
    """Parse a Povazen config.json dict."""
    layers = []
    for entry in cfg["layers"]:
        m = entry["mixer"]
        kind = entry["type"]
        if kind not in ("attention", "channel_delta"):
            raise ValueError(f"unknown Povazen layer type {kind!r}")
        mixer = MixerSpec(
            kind=kind,
            heads=int(m["heads"]),
            kv_heads=int(m["kv_heads"]),
            dim=int(m["dim"]),
            vdim=int(m["vdim"]),
            scale=float(m["scale"]) if "scale" in m else None,
            conv=int(m.get("conv", 0)),
        )
        if mixer.heads % mixer.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        mlp = entry.get("mlp")
        if mlp is not None and mlp.get("kind") != "dense":
            raise ValueError(f"unknown Povazen feed-forward kind {mlp.get('kind')!r}")
        layers.append(
            HybridLayerSpec(
                mixer=mixer,
                mlp_kind=None if mlp is None else "dense",
                mlp_ff=0 if mlp is None else int(mlp["ff"]),
            )
        )
    width = int(cfg["width"])
    groups = int(cfg["norm"]["groups"])
    if width % groups:
        raise ValueError("width must be a multiple of norm.groups")
    return HybridSpec(
        name=name,
        architecture="Povazen",
        vocab_size=int(cfg["vocab"]),
        hidden_size=width,
        layers=layers,
        norm_eps=float(cfg["norm"]["eps"]),
        norm_groups=groups,
        canon_taps=int(cfg["canon"]["taps"]),
        logit_softcap=float(cfg["logit_softcap"]),
    )


def povazen_config_dict(
    vocab: int, width: int, pattern: str, heads: int, kv_heads: int, dim: int,
    vdim: int, ff: int, delta_heads: Optional[int] = None, conv: int = 4,
    taps: int = 3, groups: int = 4, eps: float = 1e-6, softcap: float = 30.0,
) -> dict:
    """A Povazen config.json dict from a layer pattern: 'D' = channel_delta
    layer without feed-forward, 'd' = with one, 'A'/'a' likewise attention."""
    layers = []
    for ch in pattern:
        mlp = {"kind": "dense", "ff": ff} if ch.islower() else None
        if ch in "Aa":
            mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                     "vdim": vdim, "scale": dim ** -0.5}
            layers.append({"type": "attention", "mixer": mixer, "mlp": mlp})
        else:
            dh = delta_heads or heads
            mixer = {"heads": dh, "kv_heads": dh, "dim": dim, "vdim": vdim, "conv": conv}
            layers.append({"type": "channel_delta", "mixer": mixer, "mlp": mlp})
    return {"architecture": "Povazen", "canon": {"taps": taps}, "layers": layers,
            "logit_softcap": softcap, "norm": {"eps": eps, "groups": groups},
            "vocab": vocab, "width": width}


def vazilorn_spec_from_dict(cfg: dict, name: str = "vazilorn") -> HybridSpec:
    """Parse a Vazilorn config.json dict: rotary sliding-window attention with
    sinks between dynamic-tanh norms, dense or routed feed-forwards."""
    layers = []
    for entry in cfg["layers"]:
        if entry["type"] != "attention":
            raise ValueError(f"unknown Vazilorn layer type {entry['type']!r}")
        m = entry["mixer"]
        rot = m.get("rot") or {}
        mask = m.get("mask") or {}
        mixer = MixerSpec(
            kind="rotary_window",
            heads=int(m["heads"]),
            kv_heads=int(m["kv_heads"]),
            dim=int(m["dim"]),
            vdim=int(m["vdim"]),
            scale=float(m["scale"]) if "scale" in m else None,
            rot_dims=int(rot.get("dims", 0)),
            rot_base=float(rot.get("base", 10000.0)),
            rot_scaling=dict(rot["scaling"]) if rot.get("scaling") else None,
            window=int(mask["size"]) if mask.get("size") else None,
            sink=True,
        )
        if mixer.heads % mixer.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        if mixer.rot_dims % 2 or mixer.rot_dims > mixer.dim:
            raise ValueError("rot.dims must be even and at most dim")
        mlp = entry.get("mlp")
        ls = HybridLayerSpec(mixer=mixer)
        if mlp is not None:
            kind = mlp.get("kind")
            if kind == "dense":
                ls.mlp_kind, ls.mlp_ff, ls.mlp_act = "dense", int(mlp["ff"]), "gelu_tanh"
            elif kind == "moe":
                r = mlp["router"]
                grp = r.get("groups") or {}
                shared = mlp.get("shared") or {}
                ls.mlp_kind = "moe"
                ls.router = RouterSpec(
                    experts=int(r["experts"]), top=int(r["top"]), ff=int(mlp["expert"]["ff"]),
                    score="sigmoid", correction=True,
                    groups=int(grp.get("count", 1)), keep=int(grp.get("keep", grp.get("count", 1))),
                    scale=float(r.get("scale", 1.0)), shared_ff=int(shared.get("ff", 0)),
                )
                if ls.router.experts % ls.router.groups:
                    raise ValueError("experts must be a multiple of groups.count")
            else:
                raise ValueError(f"unknown Vazilorn feed-forward kind {kind!r}")
        layers.append(ls)
    return HybridSpec(
        name=name,
        architecture="Vazilorn",
        vocab_size=int(cfg["vocab"]),
        hidden_size=int(cfg["width"]),
        layers=layers,
        norm_eps=float(cfg["norm"]["eps"]),
        layer_style="sandwich",
    )


def vazilorn_config_dict(
    vocab: int, width: int, pattern: str, heads: int, kv_heads: int, dim: int,
    vdim: int, ff: int, window: Optional[int] = 64, rot_dims: Optional[int] = None,
    rot_base: float = 10000.0, rot_scaling: Optional[dict] = None, experts: int = 8,
    top: int = 2, expert_ff: int = 64, groups: int = 2, keep: int = 1,
    router_scale: float = 1.0, shared_ff: int = 0, eps: float = 1e-6,
    scale: Optional[float] = None,
) -> dict:
    """A Vazilorn config.json dict from a layer pattern: 'd' = attention +
    dense feed-forward, 'm' = attention + routed experts, 'a' = attention
    alone."""
    layers = []
    for ch in pattern:
        mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                 "scale": scale if scale is not None else dim ** -0.5,
                 "rot": {"base": rot_base, "dims": dim if rot_dims is None else rot_dims}}
        if rot_scaling:
            mixer["rot"]["scaling"] = dict(rot_scaling)
        if window:
            mixer["mask"] = {"size": window}
        if ch == "d":
            mlp = {"kind": "dense", "ff": ff}
        elif ch == "m":
            mlp = {"kind": "moe", "expert": {"ff": expert_ff},
                   "router": {"experts": experts, "top": top, "scale": router_scale,
                              "groups": {"count": groups, "keep": keep}}}
            if shared_ff:
                mlp["shared"] = {"ff": shared_ff}
        elif ch == "a":
            mlp = None
        else:
            raise ValueError(f"unknown layer letter {ch!r}")
        layers.append({"type": "attention", "mixer": mixer, "mlp": mlp})
    return {"architecture": "Vazilorn", "layers": layers, "norm": {"eps": eps},
            "vocab": vocab, "width": width}


def rafodra_spec_from_dict(cfg: dict, name: str = "rafodra") -> HybridSpec:
    """Parse a Rafodra config.json dict: pre-norm layers whose mixer is
    latent attention (optionally reading another layer's cached latent),
    lightning attention or gated linear attention, with dense silu or routed
    clamped-swish feed-forwards."""
    layers = []
    for i, entry in enumerate(cfg["layers"]):
        kind, m = entry["type"], entry["mixer"]
        if kind == "latent_attention":
            rot = m.get("rot") or {}
            src = m.get("kv_from")
            mixer = MixerSpec(
                kind=kind, heads=int(m["heads"]), kv_heads=1, dim=int(m["dim"]),
                vdim=int(m["vdim"]), scale=float(m["scale"]) if "scale" in m else None,
                rot_dims=int(rot.get("dims", m["rot_dim"])),
                rot_base=float(rot.get("base", 10000.0)),
                kv_rank=int(m["kv_rank"]), rot_dim=int(m["rot_dim"]),
                kv_from=None if src is None else int(src), sink=True,
            )
            if mixer.rot_dims % 2 or mixer.rot_dims > mixer.rot_dim:
                raise ValueError("rot.dims must be even and at most rot_dim")
            if mixer.kv_from is not None:
                j = mixer.kv_from
                if not 0 <= j < i or layers[j].mixer.kind != kind or layers[j].mixer.kv_from is not None:
                    raise ValueError(f"layer {i}: kv_from must name an earlier latent-attention "
                                     "layer that projects its own latent")
                o = layers[j].mixer
                if (o.kv_rank, o.rot_dim, o.rot_dims, o.rot_base) != (
                        mixer.kv_rank, mixer.rot_dim, mixer.rot_dims, mixer.rot_base):
                    raise ValueError(f"layer {i}: latent sizes differ from layer {j}'s")
        elif kind == "lightning":
            mixer = MixerSpec(kind=kind, heads=int(m["heads"]), kv_heads=int(m["heads"]),
                              dim=int(m["dim"]), vdim=int(m["vdim"]),
                              decay=[float(d) for d in m["decay"]])
            if len(mixer.decay) != mixer.heads:
                raise ValueError("lightning: one decay per head")
        elif kind == "gla":
            mixer = MixerSpec(kind=kind, heads=int(m["heads"]), kv_heads=int(m["heads"]),
                              dim=int(m["dim"]), vdim=int(m["vdim"]), tau=float(m["tau"]))
        else:
            raise ValueError(f"unknown Rafodra layer type {kind!r}")
        mlp = entry.get("mlp")
        ls = HybridLayerSpec(mixer=mixer)
        if mlp is not None:
            mk = mlp.get("kind")
            if mk == "dense":
                ls.mlp_kind, ls.mlp_ff, ls.mlp_act = "dense", int(mlp["ff"]), "silu"
            elif mk == "moe":
                r = mlp["router"]
                grp = r.get("groups") or {}
                shared = mlp.get("shared") or {}
                ls.mlp_kind = "moe"
                ls.router = RouterSpec(
                    experts=int(r["experts"]), top=int(r["top"]), ff=int(mlp["expert"]["ff"]),
                    score="softmax", correction=False, groups=int(grp.get("count", 1)),
                    keep=int(grp.get("keep", grp.get("count", 1))),
                    scale=float(r.get("scale", 1.0)), shared_ff=int(shared.get("ff", 0)),
                    rating="max", renorm=False, act="clamp_swish",
                    limit=float(mlp["expert"]["limit"]),
                    shared_limit=float(shared.get("limit", 0.0)), shared_gate=bool(shared),
                )
                if ls.router.experts % ls.router.groups:
                    raise ValueError("experts must be a multiple of groups.count")
            else:
                raise ValueError(f"unknown Rafodra feed-forward kind {mk!r}")
        layers.append(ls)
    return HybridSpec(
        name=name, architecture="Rafodra", vocab_size=int(cfg["vocab"]),
        hidden_size=int(cfg["width"]), layers=layers, norm_eps=float(cfg["norm"]["eps"]),
        layer_style="pre_norm", embed_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
    )


def rafodra_config_dict(
    vocab: int, width: int, pattern: str, heads: int = 4, dim: int = 16, vdim: int = 16,
    ff: int = 128, kv_rank: int = 24, rot_dim: int = 8, rot_base: float = 10000.0,
    scale: Optional[float] = None, lin_heads: Optional[int] = None, lin_dim: Optional[int] = None,
    lin_vdim: Optional[int] = None, decay: Optional[List[float]] = None, tau: float = 16.0,
    experts: int = 8, top: int = 2, expert_ff: int = 32, groups: int = 2, keep: int = 1,
    router_scale: float = 1.0, limit: float = 1.5, shared_ff: int = 0, shared_limit: float = 2.0,
    embed_scale: float = 1.0, eps: float = 1e-6,
) -> dict:
    """A Rafodra config.json dict from a layer pattern, one or two characters
    per layer: the mixer 'A' (latent attention), 'S' (latent attention
    reading the latest 'A' layer's latent), 'L' (lightning), 'G' (gla),
    followed by the feed-forward 'd' (dense), 'm' (routed experts) or '-'
    (none)."""
    if len(pattern) % 2:
        raise ValueError("pattern: two characters per layer")
    lh, ld, lv = lin_heads or heads, lin_dim or dim, lin_vdim or vdim
    if decay is None:
        decay = [1.0 - 2.0 ** (-(2 + 2 * h)) for h in range(lh)]
    layers, last_a = [], None
    for i in range(0, len(pattern), 2):
        mk, fk = pattern[i], pattern[i + 1]
        if mk in "AS":
            mixer = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank,
                     "rot_dim": rot_dim, "rot": {"base": rot_base, "dims": rot_dim},
                     "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
            if mk == "S":
                if last_a is None:
                    raise ValueError("'S' needs an earlier 'A' layer")
                mixer["kv_from"] = last_a
            else:
                last_a = len(layers)
            kind = "latent_attention"
        elif mk == "L":
            mixer, kind = {"heads": lh, "dim": ld, "vdim": lv, "decay": list(decay)}, "lightning"
        elif mk == "G":
            mixer, kind = {"heads": lh, "dim": ld, "vdim": lv, "tau": tau}, "gla"
        else:
            raise ValueError(f"unknown mixer letter {mk!r}")
        if fk == "d":
            mlp = {"kind": "dense", "ff": ff}
        elif fk == "m":
            mlp = {"kind": "moe", "expert": {"ff": expert_ff, "limit": limit},
                   "router": {"experts": experts, "top": top, "scale": router_scale,
                              "groups": {"count": groups, "keep": keep}}}
            if shared_ff:
                mlp["shared"] = {"ff": shared_ff, "limit": shared_limit}
        elif fk == "-":
            mlp = None
        else:
            raise ValueError(f"unknown feed-forward letter {fk!r}")
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    return {"architecture": "Rafodra", "embedding": {"scale": embed_scale}, "layers": layers,
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


def suzulix_spec_from_dict(cfg: dict, name: str = "suzulix") -> HybridSpec:
    """Parse a Suzulix config.json dict: pre-norm sublayers (layer norm with
    weight and bias) on `streams` hyper-connected residual streams; mixers
    latent attention with a query latent, differential rotary attention with
    a score soft cap, or retention; routed feed-forwards of ungated
    squared-relu experts with a biased router and a gated shared expert; a
    run of layers may loop; the head is the embedding table."""
    layers = []
    for i, entry in enumerate(cfg["layers"]):
        kind, m = entry["type"], entry["mixer"]
        rot = m.get("rot") or {}
        if kind == "latent_attention":
            mixer = MixerSpec(
                kind=kind, heads=int(m["heads"]), kv_heads=1, dim=int(m["dim"]),
                vdim=int(m["vdim"]), scale=float(m["scale"]) if "scale" in m else None,
                rot_dims=int(rot.get("dims", m["rot_dim"])),
                rot_base=float(rot.get("base", 10000.0)), rot_layout="half",
                kv_rank=int(m["kv_rank"]), rot_dim=int(m["rot_dim"]),
                q_rank=int(m.get("q_rank", 0)), sink=False, gate="channel",
            )
            if mixer.rot_dims % 2 or mixer.rot_dims > mixer.rot_dim:
                raise ValueError("rot.dims must be even and at most rot_dim")
        elif kind == "attention":
            mixer = MixerSpec(
                kind="diff_attention", heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
                dim=int(m["dim"]), vdim=int(m["vdim"]),
                scale=float(m["scale"]) if "scale" in m else None,
                rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                rot_layout="interleaved",
                softcap=float(m["softcap"]) if m.get("softcap") else None,
                diff=float(m["diff"]), gate="channel",
            )
            if mixer.heads % mixer.kv_heads:
                raise ValueError("heads must be a multiple of kv_heads")
            if mixer.rot_dims % 2 or mixer.rot_dims > mixer.dim:
                raise ValueError("rot.dims must be even and at most dim")
        elif kind == "retention":
            mixer = MixerSpec(
                kind=kind, heads=int(m["heads"]), kv_heads=int(m["heads"]), dim=int(m["dim"]),
                vdim=int(m["vdim"]), decay=[float(d) for d in m["decay"]],
                rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                rot_layout="half", gate="channel",
            )
            if len(mixer.decay) != mixer.heads:
                raise ValueError("retention: one decay per head")
            if mixer.rot_dims % 2 or mixer.rot_dims > mixer.dim:
                raise ValueError("rot.dims must be even and at most dim")
        else:
            raise ValueError(f"unknown Suzulix layer type {kind!r}")
        mlp = entry.get("mlp")
        ls = HybridLayerSpec(mixer=mixer)
        if mlp is not None:
            mk = mlp.get("kind", "moe")
            if mk != "moe":
                raise ValueError(f"unknown Suzulix feed-forward kind {mk!r}")
            r = mlp["router"]
            shared = mlp.get("shared") or {}
            ls.mlp_kind = "moe"
            ls.router = RouterSpec(
                experts=int(r["experts"]), top=int(r["top"]), ff=int(mlp["expert"]["ff"]),
                score="softmax", correction=False, groups=1, keep=1, scale=1.0,
                shared_ff=int(shared.get("ff", 0)), rating="max", renorm=True, act="relu2",
                shared_gate=bool(shared), gated=False, bias=True,
            )
            if ls.router.top > ls.router.experts:
                raise ValueError("router.top exceeds router.experts")
        layers.append(ls)
    loop = cfg.get("loop")
    if loop:
        start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
        if not (0 <= start <= stop <= len(layers)) or times < 1:
            raise ValueError("loop: need 0 <= start <= stop <= layers and times >= 1")
        loop = (start, stop, times) if stop > start and times != 1 else None
    streams = int(cfg.get("streams", 1))
    if streams < 1:
        raise ValueError("streams must be at least 1")
    return HybridSpec(
        name=name, architecture="Suzulix", vocab_size=int(cfg["vocab"]),
        hidden_size=int(cfg["width"]), layers=layers, norm_eps=float(cfg["norm"]["eps"]),
        layer_style="hyper", embed_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
        streams=streams, hyper="streams" in cfg, loop=loop or None,
        logit_scale=float(cfg.get("logit_scale", 1.0)), tied_head=True,
    )


def suzulix_config_dict(
    vocab: int, width: int, pattern: str, heads: int = 4, kv_heads: int = 2, dim: int = 16,
    vdim: int = 16, kv_rank: int = 24, q_rank: int = 24, rot_dim: int = 8,
    lat_heads: Optional[int] = None, lat_dim: Optional[int] = None,
    lat_vdim: Optional[int] = None, rot_dims: Optional[int] = None, rot_base: float = 10000.0,
    scale: Optional[float] = None, softcap: Optional[float] = 50.0, diff: float = 0.5,
    ret_heads: Optional[int] = None, ret_dim: Optional[int] = None,
    ret_vdim: Optional[int] = None, ret_rot_dims: Optional[int] = None,
    decay: Optional[List[float]] = None, experts: int = 8, top: int = 2, expert_ff: int = 32,
    shared_ff: int = 0, streams: Optional[int] = 2, loop: Optional[tuple] = None,
    embed_scale: float = 1.0, logit_scale: float = 1.0, eps: float = 1e-5,
) -> dict:
    """A Suzulix config.json dict from a layer pattern, two characters per
    layer: the mixer 'L' (latent attention), 'A' (differential attention) or
    'R' (retention), then the feed-forward 'm' (routed experts) or '-'
    (none). loop = (start, stop, times); streams=None leaves the key out (one
    plain residual stream)."""
    if len(pattern) % 2:
        raise ValueError("pattern: two characters per layer")
    lh, ld, lv = lat_heads or heads, lat_dim or dim, lat_vdim or vdim
    rh, rd, rv = ret_heads or heads, ret_dim or dim, ret_vdim or vdim
    if decay is None:
        decay = [1.0 - 2.0 ** (-(3 + 2 * h)) for h in range(rh)]
    layers = []
    for i in range(0, len(pattern), 2):
        mk, fk = pattern[i], pattern[i + 1]
        if mk == "L":
            mixer = {"heads": lh, "dim": ld, "vdim": lv, "kv_rank": kv_rank, "q_rank": q_rank,
                     "rot_dim": rot_dim, "rot": {"base": rot_base, "dims": rot_dim},
                     "scale": scale if scale is not None else (ld + rot_dim) ** -0.5}
            kind = "latent_attention"
        elif mk == "A":
            mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff,
                     "rot": {"base": rot_base, "dims": dim if rot_dims is None else rot_dims},
                     "scale": scale if scale is not None else dim ** -0.5}
            if softcap:
                mixer["softcap"] = softcap
            kind = "attention"
        elif mk == "R":
            mixer = {"heads": rh, "dim": rd, "vdim": rv, "decay": list(decay),
                     "rot": {"base": rot_base,
                             "dims": rd if ret_rot_dims is None else ret_rot_dims}}
            kind = "retention"
        else:
            raise ValueError(f"unknown mixer letter {mk!r}")
        if fk == "m":
            mlp = {"kind": "moe", "expert": {"ff": expert_ff},
                   "router": {"experts": experts, "top": top}}
            if shared_ff:
                mlp["shared"] = {"ff": shared_ff}
        elif fk == "-":
            mlp = None
        else:
            raise ValueError(f"unknown feed-forward letter {fk!r}")
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    cfg = {"architecture": "Suzulix", "embedding": {"scale": embed_scale}, "layers": layers,
           "logit_scale": logit_scale, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if streams is not None:
        cfg["streams"] = streams
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


# config.json "architecture" -> parser
ARCHITECTURE_PARSERS = {"Povazen": povazen_spec_from_dict,
                        "Vazilorn": vazilorn_spec_from_dict,
                        "Rafodra": rafodra_spec_from_dict,
                        "Suzulix": suzulix_spec_from_dict}

# named hybrid configurations (random-weight benchmarking and tests)
HYBRID_REGISTRY = {
    # CPU-test size
    "povazen-tiny": lambda: povazen_config_dict(
        vocab=512, width=64, pattern="Dad", heads=4, kv_heads=2, dim=16, vdim=8,
        ff=128, delta_heads=2),
    # GPU-smoke size
    "povazen-micro": lambda: povazen_config_dict(
        vocab=2048, width=1024, pattern="DdaD", heads=8, kv_heads=2, dim=128,
        vdim=128, ff=2816, delta_heads=8),
    # layer shapes of an ~8B-class model at 4 layers (speed measurements
    # beside llama3 layers of equal width)
    "povazen-4l4k": lambda: povazen_config_dict(
        vocab=2048, width=4096, pattern="dada", heads=32, kv_heads=8, dim=128,
        vdim=128, ff=14336, delta_heads=32),
    # CPU-test size
    "vazilorn-tiny": lambda: vazilorn_config_dict(
        vocab=512, width=64, pattern="dma", heads=4, kv_heads=2, dim=16, vdim=8,
        ff=128, window=24, rot_dims=8, experts=8, top=2, expert_ff=32, groups=2,
        keep=1, router_scale=1.5, shared_ff=48),
    # GPU-smoke size
    "vazilorn-micro": lambda: vazilorn_config_dict(
        vocab=2048, width=1024, pattern="dmdm", heads=8, kv_heads=2, dim=128,
        vdim=128, ff=2816, window=512, experts=16, top=4, expert_ff=512, groups=4,
        keep=2, router_scale=2.0, shared_ff=512,
        rot_scaling={"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}),
    # dense layer shapes of an ~8B-class model at 4 layers (speed beside
    # llama3 layers of equal width)
    "vazilorn-4l4k": lambda: vazilorn_config_dict(
        vocab=2048, width=4096, pattern="dddd", heads=32, kv_heads=8, dim=128,
        vdim=128, ff=14336, window=1024),
    "vazilorn-4l2k": lambda: vazilorn_config_dict(
        vocab=2048, width=2048, pattern="dddd", heads=16, kv_heads=4, dim=128,
        vdim=128, ff=8192, window=1024),
    # CPU-test size: every mixer and feed-forward kind once
    "rafodra-tiny": lambda: rafodra_config_dict(
        vocab=512, width=64, pattern="LdGmAdSmL-", heads=4, dim=16, vdim=8, ff=128,
        kv_rank=24, rot_dim=8, lin_heads=2, lin_dim=16, lin_vdim=24, experts=8, top=2,
        expert_ff=32, groups=2, keep=1, router_scale=1.5, shared_ff=48, embed_scale=4.0),
    # GPU-smoke size
    "rafodra-micro": lambda: rafodra_config_dict(
        vocab=2048, width=1024, pattern="LdGmAdLmSd", heads=8, dim=64, vdim=64, ff=2816,
        kv_rank=128, rot_dim=32, lin_heads=8, lin_dim=128, lin_vdim=128, experts=16, top=4,
        expert_ff=512, groups=4, keep=2, router_scale=2.0, shared_ff=512, embed_scale=8.0),
    # layer shapes of ~1B- and ~8B-class models at 4 layers (speed beside
    # Povazen and llama layers of equal width)
    "rafodra-4l2k": lambda: rafodra_config_dict(
        vocab=2048, width=2048, pattern="LdGdAdSd", heads=16, dim=128, vdim=128, ff=8192,
        kv_rank=192, rot_dim=64, lin_heads=16, lin_dim=128, lin_vdim=128),
    "rafodra-4l4k": lambda: rafodra_config_dict(
        vocab=2048, width=4096, pattern="LdGdAdSd", heads=32, dim=128, vdim=128, ff=14336,
        kv_rank=192, rot_dim=64, lin_heads=32, lin_dim=128, lin_vdim=128),
    # CPU-test size: every mixer once, a looped pair of layers, three streams
    "suzulix-tiny": lambda: suzulix_config_dict(
        vocab=512, width=64, pattern="LmAmRmR-Am", heads=4, kv_heads=2, dim=16, vdim=24,
        kv_rank=24, q_rank=40, rot_dim=8, lat_dim=16, lat_vdim=8, rot_dims=12, ret_heads=2,
        ret_dim=32, ret_vdim=16, experts=8, top=3, expert_ff=32, shared_ff=48, streams=3,
        loop=(1, 3, 2), embed_scale=4.0, logit_scale=0.5),
    # GPU-smoke size
    "suzulix-micro": lambda: suzulix_config_dict(
        vocab=2048, width=1024, pattern="LmAmRmRmLm", heads=8, kv_heads=2, dim=64, vdim=128,
        kv_rank=128, q_rank=256, rot_dim=32, lat_dim=64, lat_vdim=64, ret_heads=8,
        ret_dim=128, ret_vdim=128, experts=16, top=4, expert_ff=512, shared_ff=512,
        streams=2, loop=(0, 2, 2), embed_scale=8.0, logit_scale=0.25),
    # layer shapes of ~1B- and ~8B-class models at 4 layers (speed beside
    # Rafodra layers of equal width): two maps of half a head each, a 192 + 64
    # wide cached latent, 16 experts of ff/8 with 4 per token
    "suzulix-4l2k": lambda: suzulix_config_dict(
        vocab=2048, width=2048, pattern="LmAmRmRm", heads=16, kv_heads=4, dim=64, vdim=128,
        kv_rank=192, q_rank=512, rot_dim=64, lat_dim=128, lat_vdim=128, rot_base=500000.0,
        ret_heads=16, ret_dim=128, ret_vdim=128, experts=16, top=4, expert_ff=1024,
        shared_ff=1024, streams=2),
    "suzulix-4l4k": lambda: suzulix_config_dict(
        vocab=2048, width=4096, pattern="LmAmRmRm", heads=32, kv_heads=8, dim=64, vdim=128,
        kv_rank=192, q_rank=1024, rot_dim=64, lat_dim=128, lat_vdim=128, rot_base=500000.0,
        ret_heads=32, ret_dim=128, ret_vdim=128, experts=16, top=4, expert_ff=1792,
        shared_ff=1792, streams=2),
}


def load_spec_from_dir(path: str):
    """Model spec from a checkpoint folder (config.json + model.safetensors);
    the model class follows config.json's "architecture"."""
    import json
    import os

    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    arch = cfg.get("architecture")
    if arch not in ARCHITECTURE_PARSERS:
        raise KeyError(
            f"unknown architecture {arch!r} in {path}/config.json; "
            f"known: {sorted(ARCHITECTURE_PARSERS)}"
        )
    spec = ARCHITECTURE_PARSERS[arch](cfg, name=os.path.basename(os.path.normpath(path)))
    spec.weights_path = os.path.join(path, "model.safetensors")
    if os.path.exists(spec.weights_path):
        apply_tensor_shapes(spec, safetensors_shapes(spec.weights_path))
    return spec


def apply_tensor_shapes(spec: HybridSpec, shapes: dict) -> HybridSpec:
    """Fill the sizes that only tensor shapes give (name -> shape): the inner
    ranks of the low-rank decay and output-gate projections, whether an
    attention mixer carries a sink and a router a correction."""
    for i, layer in enumerate(spec.layers):
        if layer.mixer.kind == "rotary_window":
            layer.mixer.sink = f"l{i}.mix.sink" in shapes
        if layer.router is not None:
            layer.router.correction = f"l{i}.mlp.correction" in shapes
        a1, g1 = shapes.get(f"l{i}.mix.a1"), shapes.get(f"l{i}.mix.g1")
        if a1 is not None:
            layer.mixer.decay_rank = int(a1[0])
        if g1 is not None:
            layer.mixer.gate_rank = int(g1[0])
    return spec


def safetensors_shapes(path: str) -> dict:
    """name -> shape from a safetensors header (8-byte little-endian length,
    then that many bytes of JSON); reads no tensor data."""
    import json
    import struct

    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
    return {k: tuple(v["shape"]) for k, v in header.items() if k != "__metadata__"}
