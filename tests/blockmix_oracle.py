"""Plain float64 forms of the mechanisms of the parallel-residual decoders
(Masezen layout), one function per mechanism, written from their equations.
Slow and simple on purpose; shares no code with the package.

A model is (cfg, W): ``cfg`` in the checkpoint's config.json layout, ``W`` a
dict name -> tensor (as stored: bf16 values, [out, in]).
"""
import math

import torch

F64 = torch.float64


# ------------------------------------------------------------------ configurations
def attn_layer(heads=4, kv_heads=2, dim=16, dims=None, base=10000.0, scale=None, scaling=None, mlp=None):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
                      "rot": {"dims": dims if dims is not None else dim, "base": base, "scaling": scaling},
                      "scale": scale if scale is not None else dim ** -0.5},
            "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, limit=2.0, shared_ff=0, shared_limit=1.0):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared_ff:
        m["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return m


def config(layers, width=48, vocab=97, taps=3, side=6, eps=1e-5):
    cfg = {"architecture": "Masezen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if taps:
        cfg["canon"] = {"taps": taps}
    if side:
        cfg["token_side"] = {"dim": side}
    return cfg


def random_weights(cfg, seed=0):
    """name -> bf16 tensor of every tensor of ``cfg``"""
    g = torch.Generator().manual_seed(seed)
    Wd, V = cfg["width"], cfg["vocab"]
    taps = (cfg.get("canon") or {}).get("taps", 0)
    sd = (cfg.get("token_side") or {}).get("dim", 0)
    n = len(cfg["layers"])

    def mat(o, i, s=None):
        return torch.randn(o, i, generator=g) * (s if s is not None else i ** -0.5)

    W = {"embed": torch.randn(V, Wd, generator=g), "head": mat(V, Wd), "final.norm": 1 + 0.2 * torch.randn((), generator=g)}
    if sd:
        W["side.embed"] = torch.randn(V, sd * n, generator=g)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, d = m["heads"], m["kv_heads"], m["dim"]
        W[p + "norm1"] = 1 + 0.2 * torch.randn((), generator=g)
        W[p + "mix.q"], W[p + "mix.k"] = mat(H * d, Wd), mat(G * d, Wd)
        W[p + "mix.q.norm"] = 1 + 0.3 * torch.randn(d, generator=g)
        W[p + "mix.k.norm"] = 1 + 0.3 * torch.randn(d, generator=g)
        W[p + "mix.talk"] = torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)
        W[p + "mix.g"], W[p + "mix.o"] = mat(H * d, Wd), mat(Wd, H * d)
        W[p + "ls1"] = 0.7 + 0.2 * torch.randn(Wd, generator=g)
        mlp = L["mlp"]
        if mlp is not None:
            W[p + "ls2"] = 0.7 + 0.2 * torch.randn(Wd, generator=g)
            if mlp["kind"] == "dense":
                W[p + "mlp.up"], W[p + "mlp.down"] = mat(mlp["ff"], Wd), mat(Wd, mlp["ff"])
            else:
                ff = mlp["expert"]["ff"]
                for e in range(mlp["router"]["experts"]):
                    q = f"{p}mlp.e{e}."
                    W[q + "gate"], W[q + "up"], W[q + "down"] = mat(ff, Wd, 2 * Wd ** -0.5), mat(ff, Wd, 2 * Wd ** -0.5), mat(Wd, ff)
                W[p + "mlp.router"] = mat(mlp["router"]["experts"], Wd)
                if mlp.get("shared"):
                    sf = mlp["shared"]["ff"]
                    q = p + "mlp.shared."
                    W[q + "gate"], W[q + "up"], W[q + "down"] = mat(sf, Wd, 2 * Wd ** -0.5), mat(sf, Wd, 2 * Wd ** -0.5), mat(Wd, sf)
        if taps:
            W[p + "canon1"] = 0.4 * torch.randn(Wd, taps, generator=g)
        if sd:
            W[p + "side.gate"], W[p + "side.proj"] = mat(sd, Wd), mat(Wd, sd)
            W[p + "side.norm"] = 0.5 + 0.2 * torch.randn(Wd, generator=g)
    return {k: v.to(torch.bfloat16) for k, v in W.items()}


def random_tokens(cfg, n, seed=0):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


# ------------------------------------------------------------------ mechanisms
def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def rotary_angles(rot, positions):
    """cos, sin [n, dims / 2] (f64) with YaRN when rot['scaling'] is set"""
    dims, base = rot["dims"], float(rot["base"])
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2 * i / dims)
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        def where(turns):
            return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
        lo, hi = max(math.floor(where(sc["fast"])), 0), min(math.ceil(where(sc["slow"])), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        f = f / sc["factor"] * ramp + f * (1 - ramp)
        mag = 0.1 * math.log(sc["factor"]) + 1
    a = torch.tensor(list(positions), dtype=F64)[:, None] * f[None]
    return a.cos() * mag, a.sin() * mag


def rotate_half(x, rot, positions):
    """x [n, heads, dim]: value i < dims / 2 pairs with value i + dims / 2; the rest passes"""
    dims = rot["dims"]
    c, s = rotary_angles(rot, positions)
    c, s = c[:, None], s[:, None]
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def canon(h, w):
    """h [n, W] -> h + causal convolution of h with w [W, taps] over time"""
    n, taps = h.shape[0], w.shape[1]
    out = h.clone()
    for t in range(n):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def attention(W, p, m, h, eps):
    n = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ W[p + "q"].T).view(n, H, d)
    k = (h @ W[p + "k"].T).view(n, G, d)
    v = k
    qn = rotate_half(unit_rms(q, eps) * W[p + "q.norm"], m["rot"], range(n))
    kn = rotate_half(unit_rms(k, eps) * W[p + "k.norm"], m["rot"], range(n))
    out = torch.zeros(n, H, d, dtype=F64)
    for t in range(n):
        s = torch.stack([(kn[:t + 1, hh // (H // G)] @ qn[t, hh]) * m["scale"] for hh in range(H)])    # [H, t + 1]
        s = W[p + "talk"] @ s
        pr = torch.softmax(s, -1)
        for hh in range(H):
            out[t, hh] = pr[hh] @ v[:t + 1, hh // (H // G)]
    o = out.reshape(n, H * d) * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def expert(W, p, x, limit):
    g = torch.clamp(x @ W[p + "gate"].T, max=limit)
    u = torch.clamp(x @ W[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ W[p + "down"].T


def feed_forward(W, p, mlp, h):
    if mlp["kind"] == "dense":
        return torch.relu(h @ W[p + "up"].T) ** 2 @ W[p + "down"].T
    s = torch.sigmoid(h @ W[p + "router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(s.shape[1]), key=lambda e: (-float(s[t, e]), e))[:mlp["router"]["top"]]
        for e in order:
            out[t] += expert(W, f"{p}e{e}.", s[t, e] * h[t], mlp["expert"]["limit"])
    if mlp.get("shared"):
        out = out + expert(W, p + "shared.", h, mlp["shared"]["limit"])
    return out


def router_margin(cfg, W, tokens):
    """smallest gap between the last chosen and the first rejected score over all layers and tokens
    (tests that compare 16-bit runs keep away from near ties)"""
    gaps = []
    forward(cfg, W, tokens, gaps=gaps)
    return min(gaps) if gaps else 1.0


def forward(cfg, W, tokens, layers_out=None, gaps=None):
    """logits [n, vocab] (f64) of one sequence run whole"""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    taps = (cfg.get("canon") or {}).get("taps", 0)
    sd = (cfg.get("token_side") or {}).get("dim", 0)
    tok = torch.tensor(tokens)
    x = W["embed"][tok]
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = unit_rms(x, eps) * W[p + "norm1"]
        hm = canon(h, W[p + "canon1"]) if taps else h
        y = attention(W, p + "mix.", L["mixer"], hm, eps) * W[p + "ls1"]
        if L["mlp"] is not None:
            if gaps is not None and L["mlp"]["kind"] == "moe":
                s = torch.sigmoid(h @ W[p + "mlp.router"].T).sort(-1, descending=True).values
                k = L["mlp"]["router"]["top"]
                if k < s.shape[1]:
                    gaps.append(float((s[:, k - 1] - s[:, k]).min()))
            y = y + feed_forward(W, p + "mlp.", L["mlp"], h) * W[p + "ls2"]
        x = x + y
        if sd:
            e = W["side.embed"][tok][:, i * sd:(i + 1) * sd]
            z = (gelu_tanh(x @ W[p + "side.gate"].T) * e) @ W[p + "side.proj"].T
            x = x + unit_rms(z, eps) * W[p + "side.norm"]
        if layers_out is not None:
            layers_out.append(x.clone())
    return (unit_rms(x, eps) * W["final.norm"]) @ W["head"].T
