"""Plain float64 oracle of the Rafodra design: one slow function per
mechanism, written from the equations, sharing no code with the product
path. Weights come in as a dict name -> tensor under the design's
checkpoint names; the config is the config.json dict.

Notation: h is a mixer's input [T, C]; matrices are stored [out, in].
"""

import math

import torch

F64 = torch.float64


def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def rotate_pairs(x, pos, dims, base):
    """x [T, n]: channels (2i, 2i+1), i < dims/2, turn by pos * base^(-2i/dims)."""
    out = x.clone()
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        ang = pos.to(F64) * f
        c, s = torch.cos(ang), torch.sin(ang)
        u, v = x[:, 2 * i], x[:, 2 * i + 1]
        out[:, 2 * i] = u * c - v * s
        out[:, 2 * i + 1] = v * c + u * s
    return out


def latent_kv(h, W, p, m, eps, pos):
    """What a latent-attention layer caches: (c [T, rank], rotated shared key [T, rot])."""
    rank, rot = m["kv_rank"], m["rot_dim"]
    d = h @ W[p + "dkv"].T
    c = rms_norm(d[:, :rank], W[p + "dkv.norm"], eps)
    kr = rotate_pairs(d[:, rank:rank + rot], pos, m["rot"]["dims"], m["rot"]["base"])
    return c, kr


def latent_attention(h, W, p, m, eps, shared=None):
    """Whole-sequence latent attention. shared: (c, kr) of another layer."""
    T = h.shape[0]
    H, D, rot, Dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    pos = torch.arange(T)
    c, kr = shared if shared is not None else latent_kv(h, W, p, m, eps, pos)
    q = (h @ W[p + "q"].T).reshape(T, H, D + rot)
    k_un = (c @ W[p + "uk"].T).reshape(T, H, D)
    v = (c @ W[p + "uv"].T).reshape(T, H, Dv)
    gate = sigmoid(h @ W[p + "g"].T)                       # [T, H]
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        q_un = q[:, hh, :D]
        q_ro = rotate_pairs(q[:, hh, D:], pos, m["rot"]["dims"], m["rot"]["base"])
        for i in range(T):
            s = (k_un[: i + 1, hh] @ q_un[i] + kr[: i + 1] @ q_ro[i]) * m["scale"]
            mx = max(float(s.max()), float(W[p + "sink"][hh]))
            e = torch.exp(s - mx)
            z = e.sum() + math.exp(float(W[p + "sink"][hh]) - mx)
            out[i, hh] = (e / z) @ v[: i + 1, hh] * gate[i, hh]
    return out.reshape(T, H * Dv) @ W[p + "o"].T


def decay_recurrence(q, k, v, decay):
    """S_t = diag(decay_t) S_{t-1} + k_t v_t^T, o_t = S_t^T q_t for one head.
    q, k [T, D]; v [T, Dv]; decay [T, D]."""
    T, D = k.shape
    S = torch.zeros(D, v.shape[1], dtype=F64)
    o = torch.zeros(T, v.shape[1], dtype=F64)
    for t in range(T):
        S = decay[t].unsqueeze(1) * S + torch.outer(k[t], v[t])
        o[t] = S.T @ q[t]
    return o


def lightning(h, W, p, m, eps):
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ W[p + "q"].T).reshape(T, H, D)
    k = silu(h @ W[p + "k"].T).reshape(T, H, D)
    v = silu(h @ W[p + "v"].T).reshape(T, H, Dv)
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        dec = torch.full((T, D), float(m["decay"][hh]), dtype=F64)
        o[:, hh] = decay_recurrence(q[:, hh], k[:, hh], v[:, hh], dec)
    y = rms_norm(o.reshape(T, H * Dv), W[p + "norm"], eps) * sigmoid(h @ W[p + "g"].T)
    return y @ W[p + "o"].T


def gla(h, W, p, m, eps):
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T * D ** -0.5).reshape(T, H, D)
    k = (h @ W[p + "k"].T).reshape(T, H, D)
    v = (h @ W[p + "v"].T).reshape(T, H, Dv)
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    alpha = (sigmoid(z) ** (1.0 / m["tau"])).reshape(T, H, D)
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hh in range(H):
        o[:, hh] = decay_recurrence(q[:, hh], k[:, hh], v[:, hh], alpha[:, hh])
    o = rms_norm(o, W[p + "norm"], eps).reshape(T, H * Dv)
    return (o * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def dense_ff(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def clamped_expert(h, W, p, limit):
    g = torch.clamp(h @ W[p + "gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


def choose_experts(scores, top, groups, keep):
    """scores [E] -> chosen expert ids, best first. Groups of neighbours are
    rated by their best score; only the `keep` best groups stay eligible."""
    E = scores.shape[0]
    per = E // groups
    rating = [float(scores[g * per:(g + 1) * per].max()) for g in range(groups)]
    kept = sorted(range(groups), key=lambda g: (-rating[g], g))[:keep]
    ok = [e for e in range(E) if e // per in kept]
    return sorted(ok, key=lambda e: (-float(scores[e]), e))[:top]


def moe_ff(h, W, p, mlp):
    r = mlp["router"]
    E, top = r["experts"], r["top"]
    grp = r.get("groups") or {"count": 1, "keep": 1}
    s = torch.softmax(h @ W[p + "router"].T, -1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in choose_experts(s[t], top, grp["count"], grp["keep"]):
            out[t] += s[t, e] * r["scale"] * clamped_expert(
                h[t:t + 1], W, f"{p}e{e}.", mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        sg = sigmoid(h @ W[p + "shared.sg"].T)              # [T, 1]
        out = out + sg * clamped_expert(h, W, p + "shared.", mlp["shared"]["limit"])
    return out


def forward(cfg, W, tokens, layers_out=None):
    """Logits [T, vocab] of one whole sequence; layers_out collects the
    residual stream after every layer."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    T = x.shape[0]
    kept = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        h = layer_norm(x, W[p + "norm1"], eps)
        if L["type"] == "latent_attention":
            if "kv_from" in m and m["kv_from"] is not None:
                y = latent_attention(h, W, p + "mix.", m, eps, shared=kept[m["kv_from"]])
            else:
                kept[i] = latent_kv(h, W, p + "mix.", m, eps, torch.arange(T))
                y = latent_attention(h, W, p + "mix.", m, eps, shared=kept[i])
        elif L["type"] == "lightning":
            y = lightning(h, W, p + "mix.", m, eps)
        elif L["type"] == "gla":
            y = gla(h, W, p + "mix.", m, eps)
        else:
            raise ValueError(L["type"])
        x = x + y
        mlp = L.get("mlp")
        if mlp is not None:
            h = layer_norm(x, W[p + "norm2"], eps)
            x = x + (dense_ff(h, W, p + "mlp.") if mlp["kind"] == "dense"
                     else moe_ff(h, W, p + "mlp.", mlp))
        if layers_out is not None:
            layers_out.append(x.clone())
    return layer_norm(x, W["final.norm"], eps) @ W["head"].T


def greedy(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, W, toks)[-1].argmax()))
    return toks[len(prompt):]


def random_weights(cfg, seed=0, decay_rank=5):
    """Random tensors under the checkpoint's names for a config dictionary."""
    g = torch.Generator().manual_seed(seed)
    C, V = cfg["width"], cfg["vocab"]
    rn = lambda *s, std=1.0: torch.randn(*s, generator=g) * std
    W = {"embed": rn(V, C, std=0.5), "head": rn(V, C, std=C ** -0.5),
         "final.norm": 1.0 + 0.2 * rn(C)}

    def ff(prefix, inner):
        W[prefix + "gate"] = rn(inner, C, std=1.5 * C ** -0.5)
        W[prefix + "up"] = rn(inner, C, std=1.5 * C ** -0.5)
        W[prefix + "down"] = rn(C, inner, std=inner ** -0.5)

    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        W[p + "norm1"] = 1.0 + 0.2 * rn(C)
        if layer["type"] == "latent_attention":
            R, rot = m["kv_rank"], m["rot_dim"]
            W[p + "mix.q"] = rn(H * (D + rot), C, std=C ** -0.5)
            if m.get("kv_from") is None:
                W[p + "mix.dkv"] = rn(R + rot, C, std=C ** -0.5)
                W[p + "mix.dkv.norm"] = 1.0 + 0.2 * rn(R)
            W[p + "mix.uk"] = rn(H * D, R, std=R ** -0.5)
            W[p + "mix.uv"] = rn(H * Dv, R, std=R ** -0.5)
            W[p + "mix.sink"] = rn(H)
            W[p + "mix.g"] = rn(H, C, std=C ** -0.5)
        else:
            W[p + "mix.q"] = rn(H * D, C, std=C ** -0.5)
            W[p + "mix.k"] = rn(H * D, C, std=C ** -0.5)
            W[p + "mix.v"] = rn(H * Dv, C, std=C ** -0.5)
            W[p + "mix.g"] = rn(H * Dv, C, std=C ** -0.5)
            if layer["type"] == "gla":
                W[p + "mix.a1"] = rn(decay_rank, C, std=C ** -0.5)
                W[p + "mix.a2"] = rn(H * D, decay_rank, std=2.0 * decay_rank ** -0.5)
                W[p + "mix.a2.b"] = 1.0 + rn(H * D)
                W[p + "mix.norm"] = 1.0 + 0.2 * rn(Dv)
            else:
                W[p + "mix.norm"] = 1.0 + 0.2 * rn(H * Dv)
        W[p + "mix.o"] = rn(C, H * Dv, std=(H * Dv) ** -0.5)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        W[p + "norm2"] = 1.0 + 0.2 * rn(C)
        if mlp["kind"] == "dense":
            ff(p + "mlp.", mlp["ff"])
        else:
            n = mlp["router"]["experts"]
            W[p + "mlp.router"] = rn(n, C, std=2.0 * C ** -0.5)
            for e in range(n):
                ff(f"{p}mlp.e{e}.", mlp["expert"]["ff"])
            if mlp.get("shared"):
                ff(p + "mlp.shared.", mlp["shared"]["ff"])
                W[p + "mlp.shared.sg"] = rn(1, C, std=C ** -0.5)
    return W
