"""Masezen: a decoder of parallel-residual blocks -- grouped-query attention
with mixed head scores beside a squared-ReLU feed-forward or a sigmoid-routed
mixture of experts -- read from its own checkpoint layout.

A checkpoint folder holds ``config.json`` (``"architecture": "Masezen"``) and
``model.safetensors`` (bf16 weights, linear weights stored [out, in]).  The
configuration lists the layers in order; each entry names its mixer type
(``attention``), the mixer's sizes and its feed-forward (``dense``, ``moe`` or
none).  Tensor names: ``embed``, ``side.embed``, ``l<i>.norm1`` (one number),
``l<i>.mix.<name>``, ``l<i>.mlp.<name>`` (experts ``e<k>.``, ``shared.``,
``router``), ``l<i>.ls1`` / ``ls2``, ``l<i>.canon1``, ``l<i>.side.<name>``,
``final.norm``, ``head``.  Every size and constant comes from the
configuration; the building blocks are the generic ones of ``models/hybrid.py``.
"""
from __future__ import annotations

import json
import os
from typing import Dict, Optional

import torch

from .hybrid import (ExpertSpec, GroupedAttention, GroupedAttentionSpec, HybridCausalLM, HybridSpec, LayerSpec, MoESpec,
                     ParallelLayer, ReluSqFF, ReluSqFFSpec, RotarySpec, SigmoidMoE, TokenSide)

ARCHITECTURE = "Masezen"


def _expert(c: dict) -> ExpertSpec:
    return ExpertSpec(ff=int(c["ff"]), limit=float(c["limit"]))


def spec_from_config(cfg: dict) -> HybridSpec:
    layers = []
    for i, L in enumerate(cfg["layers"]):
        m, kind = L["mixer"], L["type"]
        if kind != "attention":
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        rot = m.get("rot") or {"dims": 0, "base": 10000.0}
        if int(m.get("vdim", m["dim"])) != int(m["dim"]):
            raise ValueError(f"layer {i}: the values are the keys, so vdim must equal dim")
        mixer = GroupedAttentionSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
                                     scale=float(m["scale"]),
                                     rot=RotarySpec(int(rot["dims"]), float(rot["base"]), rot.get("scaling") or None))
        if mixer.rot.dims > mixer.dim or mixer.rot.dims % 2:
            raise ValueError(f"layer {i}: rot.dims must be even and at most dim")
        if mixer.heads % mixer.kv_heads:
            raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
        mlp = L.get("mlp")
        if mlp is not None:
            k = mlp.get("kind", "dense")
            if k == "dense":
                mlp = ReluSqFFSpec(int(mlp["ff"]))
            elif k == "moe":
                r = mlp["router"]
                mlp = MoESpec(experts=int(r["experts"]), top=int(r["top"]), expert=_expert(mlp["expert"]),
                              shared=_expert(mlp["shared"]) if mlp.get("shared") else None)
                if not 1 <= mlp.top <= mlp.experts:
                    raise ValueError(f"layer {i}: router.top must be 1..experts")
            else:
                raise ValueError(f"layer {i}: unknown feed-forward kind {k!r}")
        layers.append(LayerSpec("grouped_attention", mixer, mlp))
    return HybridSpec(model_type="masezen", vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]), layers=layers,
                      norm_eps=float(cfg["norm"]["eps"]), block="parallel", norm="rms_scalar", layer_scale=True,
                      canon_taps=int((cfg.get("canon") or {}).get("taps", 0)),
                      side_dim=int((cfg.get("token_side") or {}).get("dim", 0)))


def tensor_shapes(spec: HybridSpec) -> Dict[str, tuple]:
    """name -> shape of every tensor of a checkpoint of ``spec``"""
    W = spec.hidden_size
    out = {"embed": (spec.vocab_size, W)}
    if spec.side_dim:
        out["side.embed"] = (spec.vocab_size, spec.side_dim * spec.num_layers)
    for i, L in enumerate(spec.layers):
        p, m = f"l{i}.", L.mixer
        out[p + "norm1"] = ()
        out.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.k": (m.kv_heads * m.dim, W),
                    p + "mix.q.norm": (m.dim,), p + "mix.k.norm": (m.dim,), p + "mix.talk": (m.heads, m.heads),
                    p + "mix.g": (m.heads * m.dim, W), p + "mix.o": (W, m.heads * m.dim)})
        if isinstance(L.mlp, ReluSqFFSpec):
            out.update({p + "mlp.up": (L.mlp.ff, W), p + "mlp.down": (W, L.mlp.ff)})
        elif isinstance(L.mlp, MoESpec):
            for e in range(L.mlp.experts):
                q = f"{p}mlp.e{e}."
                out.update({q + "gate": (L.mlp.expert.ff, W), q + "up": (L.mlp.expert.ff, W),
                            q + "down": (W, L.mlp.expert.ff)})
            out[p + "mlp.router"] = (L.mlp.experts, W)
            if L.mlp.shared is not None:
                q = p + "mlp.shared."
                out.update({q + "gate": (L.mlp.shared.ff, W), q + "up": (L.mlp.shared.ff, W),
                            q + "down": (W, L.mlp.shared.ff)})
        if spec.layer_scale:
            out[p + "ls1"] = (W,)
            if L.mlp is not None:
                out[p + "ls2"] = (W,)
        if spec.canon_taps:
            out[p + "canon1"] = (W, spec.canon_taps)
        if spec.side_dim:
            out.update({p + "side.gate": (spec.side_dim, W), p + "side.proj": (W, spec.side_dim), p + "side.norm": (W,)})
    out["final.norm"] = ()
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
        mixer = GroupedAttention(L.mixer, t(p + "q"), t(p + "k"), t(p + "q.norm"), t(p + "k.norm"), t(p + "talk"),
                                 t(p + "g"), t(p + "o"))
        mlp = None
        q = f"l{i}.mlp."
        if isinstance(L.mlp, ReluSqFFSpec):
            mlp = ReluSqFF(t(q + "up"), t(q + "down"))
        elif isinstance(L.mlp, MoESpec):
            E = L.mlp.experts
            w_gu = torch.stack([torch.cat([t(f"{q}e{e}.gate"), t(f"{q}e{e}.up")], 0) for e in range(E)])
            w_down = torch.stack([t(f"{q}e{e}.down") for e in range(E)])
            sh_gu = sh_down = None
            if L.mlp.shared is not None:
                sh_gu = torch.cat([t(q + "shared.gate"), t(q + "shared.up")], 0).contiguous()
                sh_down = t(q + "shared.down")
            mlp = SigmoidMoE(L.mlp, t(q + "router"), w_gu, w_down, sh_gu, sh_down)
        side = None
        if spec.side_dim:
            r = f"l{i}.side."
            side = TokenSide(t(r + "gate"), t(r + "proj"), t(r + "norm"), i * spec.side_dim)
        layers.append(ParallelLayer(mixer, t(f"l{i}.norm1").reshape(1), mlp,
                                    canon=t(f"l{i}.canon1") if spec.canon_taps else None,
                                    ls1=t(f"l{i}.ls1") if spec.layer_scale else None,
                                    ls2=t(f"l{i}.ls2") if spec.layer_scale and L.mlp is not None else None, side=side))
    return HybridCausalLM(spec, t("embed"), None, layers, t("final.norm").reshape(1), t("head"), dtype,
                          side_embed=t("side.embed") if spec.side_dim else None).eval()


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
        if name.endswith(("norm1", "final.norm", "q.norm", "k.norm", "side.norm")):
            w = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif name.endswith(("ls1", "ls2")):
            w = 0.5 + 0.1 * torch.randn(shape, generator=g)
        elif name.endswith("talk"):
            w = torch.eye(shape[0]) + 0.2 * torch.randn(shape, generator=g)
        elif name.endswith("canon1"):
            w = 0.3 * torch.randn(shape, generator=g)
        elif len(shape) == 2 and name not in ("embed", "side.embed"):
            w = torch.randn(shape, generator=g) * (std if std is not None else shape[1] ** -0.5)
        else:
            w = torch.randn(shape, generator=g) * (std if std is not None else 1.0)
        out[name] = w.to(torch.bfloat16)
    return out


def random_model(spec: HybridSpec, seed: int = 0, dtype=torch.bfloat16, device="cuda") -> HybridCausalLM:
    return build(spec, random_tensors(spec, seed), dtype, device)
