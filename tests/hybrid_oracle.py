"""Plain, slow float64 forms of the hybrid decoder's mechanisms, written from
their equations; the tests compare the framework against them.  One function
per mechanism, whole sequences only (no cache, no state carried between
calls, no batching), and no code shared with ``ipex_llm_amd``.

A model is a configuration dict in the Zamelix checkpoint layout and a dict
name -> tensor (linear weights [out, in]).
"""
import math

import torch

F64 = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rotary_angles(rot, positions):
    """cos, sin [len(positions), dims / 2] (YaRN-scaled when rot has 'scaling')"""
    dims, base = rot["dims"], rot["base"]
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2 * i / dims)
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        def d_of(t):
            return dims * math.log(sc["original"] / (2 * math.pi * t)) / (2 * math.log(base))
        lo = max(math.floor(d_of(sc["fast"])), 0)
        hi = min(math.ceil(d_of(sc["slow"])), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        f = f / sc["factor"] * ramp + f * (1 - ramp)
        mag = 0.1 * math.log(sc["factor"]) + 1
    a = torch.as_tensor(positions, dtype=F64)[:, None] * f[None]
    return a.cos() * mag, a.sin() * mag


def rotate(x, cos, sin, dims):
    """x [T, ..., D]: the first dims values as interleaved pairs (2i, 2i + 1)"""
    out = x.clone()
    for i in range(dims // 2):
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        c = cos[:, i].reshape([-1] + [1] * (x.dim() - 2))
        s = sin[:, i].reshape([-1] + [1] * (x.dim() - 2))
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def latent_attention(h, W, p, mx, eps):
    """h [T, width] -> [T, width]; W[p + name]"""
    T = h.shape[0]
    H, dim, dr, dv, r = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    q = (h @ W[p + "q"].T).view(T, H, dim + dr)
    dkv = h @ W[p + "dkv"].T
    c = unit_rms(dkv[:, :r], eps) * W[p + "dkv.norm"]
    cos, sin = rotary_angles(mx["rot"], range(T))
    dims = mx["rot"]["dims"]
    q_rot = rotate(q[..., dim:], cos, sin, dims)
    k_rot = rotate(dkv[:, r:], cos, sin, dims)
    k = (c @ W[p + "uk"].T).view(T, H, dim)
    v = (c @ W[p + "uv"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        for hh in range(H):
            s = (k[:t + 1, hh] @ q[t, hh, :dim] + k_rot[:t + 1] @ q_rot[t, hh]) * mx["scale"]
            out[t, hh] = torch.softmax(s, 0) @ v[:t + 1, hh]
    gate = torch.sigmoid(h @ W[p + "g"].T)
    return (out * gate[..., None]).reshape(T, H * dv) @ W[p + "o"].T


def mlstm(h, W, p, mx, eps):
    T = h.shape[0]
    H, dim, dv, cap = mx["heads"], mx["dim"], mx["vdim"], mx["gate_cap"]
    q = (h @ W[p + "q"].T).view(T, H, dim) * dim ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, dim)
    v = (h @ W[p + "v"].T).view(T, H, dv)
    ig = cap * torch.tanh((h @ W[p + "i"].T + W[p + "i.b"]) / cap)
    fz = cap * torch.tanh((h @ W[p + "f"].T + W[p + "f.b"]) / cap)
    fg = -torch.log1p(torch.exp(-fz))
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        S = torch.zeros(dim, dv, dtype=F64)
        n = torch.zeros(dim, dtype=F64)
        m = 0.0
        for t in range(T):
            m_new = max(float(fg[t, hh]) + m, float(ig[t, hh]))
            a, b = math.exp(float(fg[t, hh]) + m - m_new), math.exp(float(ig[t, hh]) - m_new)
            S = a * S + b * torch.outer(k[t, hh], v[t, hh])
            n = a * n + b * k[t, hh]
            m = m_new
            out[t, hh] = (S.T @ q[t, hh]) / (max(abs(float(n @ q[t, hh])), math.exp(-m)) + 1e-6)
    o = unit_rms(out, eps).reshape(T, H * dv) * W[p + "norm"]
    return (o * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def dense_ff(h, W, p):
    return (gelu_tanh(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def embed(cfg, W, tokens):
    bg = cfg["embedding"]["bigram"]
    x = torch.zeros(len(tokens), cfg["width"], dtype=F64)
    for t, tok in enumerate(tokens):
        row = bg["buckets"] if t == 0 else (tokens[t - 1] * bg["mul_prev"] + tok * bg["mul_cur"]) % bg["buckets"]
        x[t] = W["embed"][tok] + W["bigram"][row]
    return x


def forward(cfg, W, tokens, layers_out=None):
    """logits f64 [T, vocab] of one whole sequence"""
    W = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in W.items()}
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = embed(cfg, W, list(tokens))
    for li, L in enumerate(cfg["layers"]):
        fn = {"latent_attention": latent_attention, "mlstm": mlstm}[L["type"]]
        x = x + mult * layer_norm(fn(x, W, f"l{li}.mix.", L["mixer"], eps), W[f"l{li}.norm1"], eps)
        if L["mlp"] is not None:
            x = x + mult * layer_norm(dense_ff(x, W, f"l{li}.mlp."), W[f"l{li}.norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return layer_norm(x, W["final.norm"], eps) @ W["head"].T


def greedy(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, W, toks)[-1].argmax()))
    return toks[len(prompt):]


# ---------------------------------------------------------------- test models
def attn_layer(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, scale=0.21, base=10000.0, dims=None, scaling=None,
               ff=48):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
                      "rot": {"base": base, "dims": dims or rot_dim, "scaling": scaling}},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def mlstm_layer(heads=2, dim=12, vdim=20, gate_cap=3.0, ff=0):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": gate_cap},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, vocab=97, width=40, eps=1e-5, mult=0.45, buckets=53, mul_prev=31, mul_cur=5):
    return {"architecture": "Zamelix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
            "embedding": {"bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}, "layers": layers}


def random_weights(cfg, seed=0):
    """bf16-representable random weights, name -> f32 tensor"""
    g = torch.Generator().manual_seed(seed)
    Wd = cfg["width"]

    def lin(o, i, gain=1.0):
        return torch.randn(o, i, generator=g) * gain * i ** -0.5

    def near_one(n):
        return 1.0 + 0.2 * torch.randn(n, generator=g)

    W = {"embed": torch.randn(cfg["vocab"], Wd, generator=g),
         "bigram": 0.5 * torch.randn(cfg["embedding"]["bigram"]["buckets"] + 1, Wd, generator=g)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        W[p + "norm1"] = near_one(Wd)
        if L["type"] == "latent_attention":
            H, r = m["heads"], m["kv_rank"]
            W[p + "mix.q"] = lin(H * (m["dim"] + m["rot_dim"]), Wd, 2.0)
            W[p + "mix.dkv"] = lin(r + m["rot_dim"], Wd, 2.0)
            W[p + "mix.dkv.norm"] = near_one(r)
            W[p + "mix.uk"] = lin(H * m["dim"], r, 2.0)
            W[p + "mix.uv"] = lin(H * m["vdim"], r)
            W[p + "mix.g"] = lin(H, Wd)
            W[p + "mix.o"] = lin(Wd, H * m["vdim"])
        else:
            H = m["heads"]
            W[p + "mix.q"] = lin(H * m["dim"], Wd, 2.0)
            W[p + "mix.k"] = lin(H * m["dim"], Wd, 2.0)
            W[p + "mix.v"] = lin(H * m["vdim"], Wd)
            W[p + "mix.g"] = lin(H * m["vdim"], Wd)
            W[p + "mix.o"] = lin(Wd, H * m["vdim"])
            W[p + "mix.norm"] = near_one(H * m["vdim"])
            W[p + "mix.i"] = lin(H, Wd, 2.0)
            W[p + "mix.i.b"] = torch.randn(H, generator=g)
            W[p + "mix.f"] = lin(H, Wd, 2.0)
            W[p + "mix.f.b"] = 1.5 + torch.randn(H, generator=g)
        if L["mlp"] is not None:
            W[p + "norm2"] = near_one(Wd)
            W[p + "mlp.gate"] = lin(L["mlp"]["ff"], Wd)
            W[p + "mlp.up"] = lin(L["mlp"]["ff"], Wd)
            W[p + "mlp.down"] = lin(Wd, L["mlp"]["ff"])
    W["final.norm"] = near_one(Wd)
    W["head"] = lin(cfg["vocab"], Wd)
    return {k: v.to(torch.bfloat16).float() for k, v in W.items()}


def random_tokens(cfg, n, seed=0):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()
