"""Plain float64 oracle of the Suzulix design: one slow function per
mechanism, written from the equations, sharing no code with the product
path. Weights come in as a dict name -> tensor under the design's
checkpoint names; the config is the config.json dict.

Notation: h is a sublayer's input [T, C]; matrices are stored [out, in];
positions count from 0.
"""

import math

import torch

F64 = torch.float64


# Where the product path may hold bfloat16 (projection outputs, normed sublayer
# inputs, mixer outputs before the output projection) the oracle can round too:
# the difference to the unrounded run shows how far rounding alone moves a
# position. Off by default.
_ROUND = [None]


class rounding:
    """with rounding(fn): every low-precision point applies fn."""

    def __init__(self, fn):
        self.fn = fn

    def __enter__(self):
        _ROUND[0] = self.fn

    def __exit__(self, *a):
        _ROUND[0] = None


def lowp(x):
    return x if _ROUND[0] is None else _ROUND[0](x)


def proj(x, w):
    return lowp(x @ w.T)


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def turn(x, pos, dims, base, layout):
    """x [T, n]: `dims` leading channels are rotated by pos * base^(-2i/dims);
    layout "half" pairs channel i with i + dims/2, "interleaved" 2i with 2i+1."""
    out = x.clone()
    for i in range(dims // 2):
        a, b = (i, i + dims // 2) if layout == "half" else (2 * i, 2 * i + 1)
        ang = pos.to(F64) * base ** (-2.0 * i / dims)
        c, s = torch.cos(ang), torch.sin(ang)
        out[:, a] = x[:, a] * c - x[:, b] * s
        out[:, b] = x[:, b] * c + x[:, a] * s
    return out


def softmax_rows(scores):
    """Causal softmax of scores [T, T] (row i sees columns j <= i)."""
    T = scores.shape[0]
    p = torch.zeros_like(scores)
    for i in range(T):
        s = scores[i, : i + 1]
        e = torch.exp(s - s.max())
        p[i, : i + 1] = e / e.sum()
    return p


def latent_attention(h, W, p, m, eps):
    T = h.shape[0]
    H, D, rot, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rd, rb = m["rot"]["dims"], m["rot"]["base"]
    pos = torch.arange(T)
    cq = lowp(unit_rms(proj(h, W[p + "dq"]), eps) * W[p + "dq.norm"])
    q = proj(cq, W[p + "uq"]).reshape(T, H, D + rot)
    d = proj(h, W[p + "dkv"])
    c = unit_rms(d[:, :R], eps) * W[p + "dkv.norm"]
    kr = turn(d[:, R:R + rot], pos, rd, rb, "half")
    ku = proj(c, W[p + "uk"]).reshape(T, H, D)
    v = proj(c, W[p + "uv"]).reshape(T, H, Dv)
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        qr = turn(q[:, hh, D:], pos, rd, rb, "half")
        s = (q[:, hh, :D] @ ku[:, hh].T + qr @ kr.T) * m["scale"]
        out[:, hh] = softmax_rows(s) @ v[:, hh]
    out = lowp(out.reshape(T, H * Dv) * sigmoid(proj(h, W[p + "g"])))
    return proj(out, W[p + "o"])


def diff_lambda(W, p, m):
    return (math.exp(float((W[p + "lq1"] * W[p + "lk1"]).sum()))
            - math.exp(float((W[p + "lq2"] * W[p + "lk2"]).sum())) + m["diff"])


def diff_attention(h, W, p, m, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    pos = torch.arange(T)
    q = proj(h, W[p + "q"]).reshape(T, H, 2, D)
    k = proj(h, W[p + "k"]).reshape(T, G, 2, D)
    v = proj(h, W[p + "v"]).reshape(T, G, Dv)
    lam = diff_lambda(W, p, m)
    cap = m.get("softcap")
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        maps = []
        for mm in range(2):
            qq = turn(q[:, hh, mm], pos, rot["dims"], rot["base"], "interleaved")
            kk = turn(k[:, g, mm], pos, rot["dims"], rot["base"], "interleaved")
            s = qq @ kk.T * m["scale"]
            if cap:
                s = cap * torch.tanh(s / cap)
            maps.append(softmax_rows(s) @ v[:, g])
        o = maps[0] - lam * maps[1]
        out[:, hh] = unit_rms(o, eps) * (1.0 - m["diff"])
    out = lowp(out.reshape(T, H * Dv) * sigmoid(proj(h, W[p + "g"])))
    return proj(out, W[p + "o"])


def retention(h, W, p, m, eps):
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    pos = torch.arange(T)
    q = proj(h, W[p + "q"]).reshape(T, H, D)
    k = proj(h, W[p + "k"]).reshape(T, H, D)
    v = proj(h, W[p + "v"]).reshape(T, H, Dv)
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        qq = turn(q[:, hh], pos, rot["dims"], rot["base"], "half")
        kk = turn(k[:, hh], pos, rot["dims"], rot["base"], "half") * D ** -0.5
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            S = float(m["decay"][hh]) * S + torch.outer(kk[t], v[t, hh])
            out[t, hh] = S.T @ qq[t]
    z = proj(h, W[p + "g"])
    y = lowp(unit_rms(out, eps).reshape(T, H * Dv) * (z * sigmoid(z)))
    return proj(y, W[p + "o"])


def expert(h, W, p):
    return proj(lowp(torch.clamp(proj(h, W[p + "up"]), min=0.0) ** 2), W[p + "down"])


def moe_ff(h, W, p, mlp):
    top = mlp["router"]["top"]
    z = h @ W[p + "router"].T + W[p + "router.b"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = sorted(range(z.shape[1]), key=lambda e: (-float(z[t, e]), e))[:top]
        zs = torch.stack([z[t, e] for e in chosen])
        w = torch.exp(zs - zs.max())
        w = w / w.sum()
        for j, e in enumerate(chosen):
            out[t] += w[j] * expert(h[t:t + 1], W, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + sigmoid(h @ W[p + "shared.sg"].T) * expert(h, W, p + "shared.")
    return out


MIXERS = {"latent_attention": latent_attention, "attention": diff_attention,
          "retention": retention}


def run_order(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    return (list(range(lp["start"])) + list(range(lp["start"], lp["stop"])) * lp["times"]
            + list(range(lp["stop"], n)))


def forward(cfg, W, tokens, layers_out=None):
    """Logits [T, vocab] of one whole sequence; layers_out collects the sum of
    the residual streams after every layer run."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x0 = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    hyper = "streams" in cfg
    S = cfg.get("streams", 1)
    xs = [x0.clone() for _ in range(S)]
    for i in run_order(cfg):
        L = cfg["layers"][i]
        p = f"l{i}."
        subs = [(1, lambda h: MIXERS[L["type"]](h, W, p + "mix.", L["mixer"], eps))]
        if L.get("mlp") is not None:
            subs.append((2, lambda h: moe_ff(h, W, p + "mlp.", L["mlp"])))
        for q, fn in subs:
            if hyper:
                rd, wr, mix = W[f"{p}hc{q}.in"], W[f"{p}hc{q}.out"], W[f"{p}hc{q}.mix"]
            else:
                rd, wr, mix = torch.ones(1, dtype=F64), torch.ones(1, dtype=F64), torch.ones(1, 1, dtype=F64)
            u = sum(rd[s] * xs[s] for s in range(S))
            y = fn(lowp(layer_norm(u, W[f"{p}norm{q}"], W[f"{p}norm{q}.b"], eps)))
            xs = [sum(mix[s, t] * xs[s] for s in range(S)) + wr[t] * y for t in range(S)]
        if layers_out is not None:
            layers_out.append(sum(xs))
    x = sum(xs)
    return (proj(lowp(layer_norm(x, W["final.norm"], W["final.norm.b"], eps)), W["embed"])
            * cfg.get("logit_scale", 1.0))


def greedy(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, W, toks)[-1].argmax()))
    return toks[len(prompt):]


def random_weights(cfg, seed=0):
    """Random tensors under the checkpoint's names for a config dictionary."""
    g = torch.Generator().manual_seed(seed)
    C, V = cfg["width"], cfg["vocab"]
    rn = lambda *s, std=1.0: torch.randn(*s, generator=g) * std   # noqa: E731
    W = {"embed": rn(V, C, std=0.5), "final.norm": 1.0 + 0.2 * rn(C), "final.norm.b": 0.1 * rn(C)}
    S = cfg.get("streams", 1)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        subs = [1] + ([2] if layer.get("mlp") is not None else [])
        for q in subs:
            W[f"{p}norm{q}"] = 1.0 + 0.2 * rn(C)
            W[f"{p}norm{q}.b"] = 0.1 * rn(C)
            if "streams" in cfg:
                W[f"{p}hc{q}.in"] = 1.0 / S + 0.3 * rn(S)
                W[f"{p}hc{q}.out"] = 1.0 + 0.3 * rn(S)
                W[f"{p}hc{q}.mix"] = torch.eye(S) * 0.9 + 0.2 * rn(S, S)
        if layer["type"] == "latent_attention":
            R, rot, Q = m["kv_rank"], m["rot_dim"], m["q_rank"]
            W[p + "mix.dq"] = rn(Q, C, std=C ** -0.5)
            W[p + "mix.dq.norm"] = 1.0 + 0.2 * rn(Q)
            W[p + "mix.uq"] = rn(H * (D + rot), Q, std=1.5 * Q ** -0.5)
            W[p + "mix.dkv"] = rn(R + rot, C, std=C ** -0.5)
            W[p + "mix.dkv.norm"] = 1.0 + 0.2 * rn(R)
            W[p + "mix.uk"] = rn(H * D, R, std=1.5 * R ** -0.5)
            W[p + "mix.uv"] = rn(H * Dv, R, std=R ** -0.5)
        elif layer["type"] == "attention":
            G = m["kv_heads"]
            W[p + "mix.q"] = rn(H * 2 * D, C, std=1.5 * C ** -0.5)
            W[p + "mix.k"] = rn(G * 2 * D, C, std=1.5 * C ** -0.5)
            W[p + "mix.v"] = rn(G * Dv, C, std=C ** -0.5)
            for nm in ("lq1", "lk1", "lq2", "lk2"):
                W[p + "mix." + nm] = rn(D, std=0.6 * D ** -0.5)
        else:
            W[p + "mix.q"] = rn(H * D, C, std=C ** -0.5)
            W[p + "mix.k"] = rn(H * D, C, std=C ** -0.5)
            W[p + "mix.v"] = rn(H * Dv, C, std=C ** -0.5)
        W[p + "mix.g"] = rn(H * Dv, C, std=C ** -0.5)
        W[p + "mix.o"] = rn(C, H * Dv, std=(H * Dv) ** -0.5)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        n, inner = mlp["router"]["experts"], mlp["expert"]["ff"]
        W[p + "mlp.router"] = rn(n, C, std=2.0 * C ** -0.5)
        W[p + "mlp.router.b"] = 0.5 * rn(n)
        for e in range(n):
            W[f"{p}mlp.e{e}.up"] = rn(inner, C, std=1.5 * C ** -0.5)
            W[f"{p}mlp.e{e}.down"] = rn(C, inner, std=inner ** -0.5)
        if mlp.get("shared"):
            sf = mlp["shared"]["ff"]
            W[p + "mlp.shared.up"] = rn(sf, C, std=1.5 * C ** -0.5)
            W[p + "mlp.shared.down"] = rn(C, sf, std=sf ** -0.5)
            W[p + "mlp.shared.sg"] = rn(1, C, std=C ** -0.5)
    return W
