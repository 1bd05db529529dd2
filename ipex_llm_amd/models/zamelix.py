"""Zamelix: a hybrid decoder of latent-attention and mLSTM layers with a
hashed-bigram embedding, read from its own checkpoint layout.

A checkpoint folder holds ``config.json`` (``"architecture": "Zamelix"``) and
``model.safetensors`` (bf16 weights, linear weights stored [out, in]).  The
configuration lists the layers in order; each entry names its mixer type, the
mixer's sizes and its feed-forward (or none).  Tensor names: ``embed``,
``bigram``, ``l<i>.norm1`` / ``norm2``, ``l<i>.mix.<name>``, ``l<i>.mlp.<name>``,
``final.norm``, ``head``.  Every size and constant comes from the
configuration; the building blocks are the generic ones of ``models/hybrid.py``.
"""
from __future__ import annotations

import json
import os
from typing import Dict, Optional

import torch

from .hybrid import (BigramSpec, DenseFF, DenseFFSpec, HybridCausalLM, HybridLayer, HybridSpec, LatentAttention,
                     LatentAttentionSpec, LayerSpec, MLSTM, MLSTMSpec, RotarySpec)

ARCHITECTURE = "Zamelix"


def spec_from_config(cfg: dict) -> HybridSpec:
    layers = []
    for i, L in enumerate(cfg["layers"]):
        m, kind = L["mixer"], L["type"]
        if kind == "latent_attention":
            rot = m["rot"]
            mixer = LatentAttentionSpec(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]),
                                        vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]), scale=float(m["scale"]),
                                        rot=RotarySpec(int(rot["dims"]), float(rot["base"]), rot.get("scaling") or None),
                                        out_gate=True)
            if mixer.rot.dims > mixer.rot_dim or mixer.rot.dims % 2:
                raise ValueError(f"layer {i}: rot.dims must be even and at most rot_dim")
        elif kind == "mlstm":
            mixer = MLSTMSpec(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                              gate_cap=float(m["gate_cap"]))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        mlp = L.get("mlp")
        if mlp is not None:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            mlp = DenseFFSpec(int(mlp["ff"]))
        layers.append(LayerSpec(kind, mixer, mlp))
    bg = (cfg.get("embedding") or {}).get("bigram")
    bigram = BigramSpec(int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"])) if bg else None
    return HybridSpec(model_type="zamelix", vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]), layers=layers,
                      norm_eps=float(cfg["norm"]["eps"]), residual_mult=float(cfg.get("residual_mult", 1.0)),
                      bigram=bigram)


def tensor_shapes(spec: HybridSpec) -> Dict[str, tuple]:
    """name -> shape of every tensor of a checkpoint of ``spec``"""
    W = spec.hidden_size
    out = {"embed": (spec.vocab_size, W)}
    if spec.bigram is not None:
        out["bigram"] = (spec.bigram.buckets + 1, W)
    for i, L in enumerate(spec.layers):
        p, m = f"l{i}.", L.mixer
        out[p + "norm1"] = (W,)
        if L.kind == "latent_attention":
            out.update({p + "mix.q": (m.heads * (m.dim + m.rot_dim), W), p + "mix.dkv": (m.kv_rank + m.rot_dim, W),
                        p + "mix.dkv.norm": (m.kv_rank,), p + "mix.uk": (m.heads * m.dim, m.kv_rank),
                        p + "mix.uv": (m.heads * m.vdim, m.kv_rank), p + "mix.g": (m.heads, W),
                        p + "mix.o": (W, m.heads * m.vdim)})
        else:
            out.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.k": (m.heads * m.dim, W),
                        p + "mix.v": (m.heads * m.vdim, W), p + "mix.g": (m.heads * m.vdim, W),
                        p + "mix.o": (W, m.heads * m.vdim), p + "mix.norm": (m.heads * m.vdim,),
                        p + "mix.i": (m.heads, W), p + "mix.i.b": (m.heads,), p + "mix.f": (m.heads, W),
                        p + "mix.f.b": (m.heads,)})
        if L.mlp is not None:
            out.update({p + "norm2": (W,), p + "mlp.gate": (L.mlp.ff, W), p + "mlp.up": (L.mlp.ff, W),
                        p + "mlp.down": (W, L.mlp.ff)})
    out["final.norm"] = (W,)
    out["head"] = (spec.vocab_size, W)
    return out


def build(spec: HybridSpec, tensors: Dict[str, torch.Tensor], dtype=torch.bfloat16, device="cuda") -> HybridCausalLM:
    """Assemble the model from name -> tensor (any float dtype; cast to ``dtype``)."""
    want = tensor_shapes(spec)
    for name, shape in want.items():
        if name not in tensors:
            raise KeyError(f"checkpoint lacks tensor {name!r}")
        if tuple(tensors[name].shape) != tuple(shape):
            raise ValueError(f"tensor {name!r}: shape {tuple(tensors[name].shape)}, configuration says {tuple(shape)}")

    def t(name):
        return tensors[name].to(device=device, dtype=dtype).contiguous()

    layers = []
    for i, L in enumerate(spec.layers):
        p = f"l{i}.mix."
        if L.kind == "latent_attention":
            mixer = LatentAttention(L.mixer, t(p + "q"), t(p + "dkv"), t(p + "dkv.norm"), t(p + "uk"), t(p + "uv"),
                                    t(p + "g"), t(p + "o"))
        else:
            mixer = MLSTM(L.mixer, t(p + "q"), t(p + "k"), t(p + "v"), t(p + "g"), t(p + "i"), t(p + "f"),
                          t(p + "i.b"), t(p + "f.b"), t(p + "norm"), t(p + "o"))
        mlp, n2 = None, None
        if L.mlp is not None:
            q = f"l{i}.mlp."
            mlp, n2 = DenseFF(t(q + "gate"), t(q + "up"), t(q + "down")), t(f"l{i}.norm2")
        layers.append(HybridLayer(mixer, t(f"l{i}.norm1"), mlp, n2))
    return HybridCausalLM(spec, t("embed"), t("bigram") if spec.bigram is not None else None, layers,
                          t("final.norm"), t("head"), dtype).eval()


def load(path: str, dtype=torch.bfloat16, device="cuda") -> HybridCausalLM:
    """Read ``config.json`` + ``model.safetensors`` of a checkpoint folder."""
    from safetensors import safe_open
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    spec = spec_from_config(cfg)
    tensors = {}
    with safe_open(os.path.join(path, "model.safetensors"), "pt") as f:
        names = set(f.keys())
        for name in tensor_shapes(spec):
            if name in names:
                tensors[name] = f.get_tensor(name)
    model = build(spec, tensors, dtype, device)
    model.config = cfg
    return model


@torch.no_grad()
def random_tensors(spec: HybridSpec, seed: int = 0, std: Optional[float] = None) -> Dict[str, torch.Tensor]:
    """Random bf16 weights of ``spec``'s shapes (benchmarks and tests)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(spec).items():
        if name.endswith(("norm1", "norm2", "final.norm", "mix.norm", "dkv.norm")):
            w = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif name.endswith(".b"):
            w = torch.randn(shape, generator=g) + (3.0 if name.endswith("f.b") else 0.0)
        elif len(shape) == 2 and name not in ("embed", "bigram"):
            w = torch.randn(shape, generator=g) * (std if std is not None else shape[1] ** -0.5)
        else:
            w = torch.randn(shape, generator=g) * (std if std is not None else 1.0)
        out[name] = w.to(torch.bfloat16)
    return out


def random_model(spec: HybridSpec, seed: int = 0, dtype=torch.bfloat16, device="cuda") -> HybridCausalLM:
    return build(spec, random_tensors(spec, seed), dtype, device)
