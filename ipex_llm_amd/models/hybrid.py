"""Hybrid decoders: a layer list that mixes attention over a paged cache with
recurrent layers over per-sequence state, driven by data (``HybridSpec``).

Building blocks (each usable by any design that lists it in its layer specs):

* ``LatentAttention``   low-rank latent attention: one cached row per token,
  ``[latent c (kv_rank) | shared rotated key (rot_dim)]``; per-head keys and
  values are ``W_uk c`` / ``W_uv c``, so scores and outputs are formed in the
  latent space with the up-projections absorbed (as models/mla.py does for
  the DeepSeek family):  q_lat[h] = W_uk[h]^T q_nope[h],
  s = (q_lat[h] . c + q_rot[h] . k_rot) scale,  o[h] = W_uv[h] (softmax(s) C).
  Interleaved-pair rotary positions with optional YaRN scaling, an optional
  per-head sigmoid output gate.
* ``MLSTM``             matrix-memory recurrence (xLSTM's mLSTM) with capped
  exponential gates, running-maximum stabiliser, per-head RMS norm and a
  sigmoid output gate; f32 state in the cache's slots.
* ``DenseFF``           gated feed-forward, tanh-GELU.
* ``GroupedAttention``  grouped-query attention over a paged cache of
  ``[keys | values]`` rows: per-head RMS norm of queries and keys, half-split
  rotary positions (optionally on part of the head, optional YaRN), the
  values are the key projection itself (before norm and rotation), the
  heads' scores are mixed by an [H, H] matrix before the softmax, an
  element-wise sigmoid output gate.
* ``ReluSqFF``          two-matrix feed-forward with a squared-ReLU activation.
* ``SigmoidMoE``        experts behind a sigmoid router: the chosen experts'
  scores weigh the experts' *inputs*; clamped GLU experts
  ``W_down (g sigmoid(alpha g) (u + 1))``; an optional shared expert.
* ``TokenSide``         a per-layer token input: a slice of a second
  embedding table, gated by the residual stream, projected, RMS-normed and
  added.

Block layouts.  ``post_norm`` (``HybridLayer``): the sublayers read the
residual stream ``x`` itself and their *output* is normalised:
x += mult * LN(mixer(x)), x += mult * LN(ff(x)).  ``parallel``
(``ParallelLayer``): one norm, both sublayers read it, their scaled results
are summed and added: h = norm(x), x += ls1 * mixer(h + conv(h)) + ls2 * ff(h),
with an optional short causal convolution in front of the mixer (its last
inputs are per-sequence state) and an optional token-side input afterwards.
The residual stream is f32 throughout; projections run in the model's
activation dtype through the vendor GEMM, everything else in the kernels of
``ops/seqmix.py`` and ``ops/blockmix.py``.

``forward_tokens`` takes a *ragged* step (``AttnMeta.cu_q`` ...): sequences
bring different numbers of new tokens, prompt portions beside single decoded
tokens, and is what ``serving.engine.LLMEngine`` drives for these models.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..ops import blockmix as BM
from ..ops import seqmix as SM
from .decoder import AttnMeta


# ---------------------------------------------------------------------- specs
@dataclass
class RotarySpec:
    dims: int
    base: float = 10000.0
    scaling: Optional[dict] = None          # YaRN: factor, original, fast, slow


@dataclass
class LatentAttentionSpec:
    heads: int
    dim: int                                # unrotated query / key size per head
    rot_dim: int                            # rotated part (one key shared by all heads)
    vdim: int
    kv_rank: int
    scale: float
    rot: RotarySpec = None
    out_gate: bool = True


@dataclass
class MLSTMSpec:
    heads: int
    dim: int
    vdim: int
    gate_cap: float = 15.0


@dataclass
class DenseFFSpec:
    ff: int


@dataclass
class GroupedAttentionSpec:
    heads: int
    kv_heads: int
    dim: int                                # query / key size per head; the values are the keys as projected
    scale: float
    rot: RotarySpec = None                  # half-split pairs on the first rot.dims values of a head
    qk_norm: bool = True
    talk: bool = True                       # [H, H] mixing of the heads' scores before the softmax
    out_gate: bool = True                   # element-wise sigmoid gate on the concatenated heads


@dataclass
class ReluSqFFSpec:
    ff: int


@dataclass
class ExpertSpec:
    ff: int
    limit: float
    alpha: float = 1.702


@dataclass
class MoESpec:
    experts: int
    top: int
    expert: ExpertSpec = None
    shared: Optional[ExpertSpec] = None


@dataclass
class LayerSpec:
    kind: str                               # key of MIXERS
    mixer: object
    mlp: Optional[object] = None            # DenseFFSpec | ReluSqFFSpec | MoESpec


@dataclass
class BigramSpec:
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass
class HybridSpec:
    model_type: str
    vocab_size: int
    hidden_size: int
    layers: List[LayerSpec]
    norm_eps: float = 1e-6
    residual_mult: float = 1.0
    bigram: Optional[BigramSpec] = None
    final_softcap: float = 0.0              # read by the engines' shared helpers
    block: str = "post_norm"                # "post_norm" | "parallel"
    norm: str = "layer_norm"                # "layer_norm" | "rms_scalar" (one number) | "rms" (a vector)
    layer_scale: bool = False               # parallel blocks: per-coordinate scales on both sublayers' results
    canon_taps: int = 0                     # parallel blocks: taps of the convolution in front of the mixer (0: none)
    side_dim: int = 0                       # per-layer slice of the token-side table (0: none)

    @property
    def num_layers(self) -> int:
        return len(self.layers)


# ---------------------------------------------------------------------- mixers
class LatentAttention(nn.Module):
    cache_kind = "rows"

    def __init__(self, s: LatentAttentionSpec, w_q, w_dkv, dkv_norm, w_uk, w_uv, w_g, w_o):
        super().__init__()
        self.s = s
        H, r = s.heads, s.kv_rank
        # one projection launch: [q | dkv | gate] rows
        parts = [w_q, w_dkv] + ([w_g] if w_g is not None else [])
        self.w_in = nn.Parameter(torch.cat(parts, 0).contiguous(), requires_grad=False)
        self.n_q, self.n_dkv = w_q.shape[0], w_dkv.shape[0]
        self.dkv_norm = nn.Parameter(dkv_norm, requires_grad=False)
        self.w_uk = nn.Parameter(w_uk.view(H, s.dim, r).contiguous(), requires_grad=False)               # [H, dim, r]
        self.w_uv_t = nn.Parameter(w_uv.view(H, s.vdim, r).transpose(1, 2).contiguous(), requires_grad=False)  # [H, r, dv]
        self.w_o = nn.Parameter(w_o, requires_grad=False)
        self.table: Optional[torch.Tensor] = None

    def cache_spec(self):
        return ("rows", self.s.kv_rank + self.s.rot_dim)

    def ensure_table(self, max_pos: int):
        if self.table is None or self.table.shape[0] < max_pos or self.table.device != self.w_o.device:
            n = max(256, 1 << (max_pos - 1).bit_length())
            self.table = SM.rope_table(n, self.s.rot.dims, self.s.rot.base, self.s.rot.scaling).to(self.w_o.device)
        return self.table

    def forward(self, xa, pos, slots, meta: AttnMeta, cache, li: int, eps: float):
        s = self.s
        T, H = xa.shape[0], s.heads
        y = F.linear(xa, self.w_in)
        q = y[:, :self.n_q].reshape(T, H, s.dim + s.rot_dim).contiguous()
        dkv = y[:, self.n_q:self.n_q + self.n_dkv]
        gate = y[:, self.n_q + self.n_dkv:] if s.out_gate else None
        table = self.table
        SM.latent_kv_store(dkv, self.dkv_norm, eps, s.kv_rank, table, pos, slots, cache.rows[li])
        SM.rope_rows_(q, s.dim, table, pos)
        # absorbed up-projection of the keys: per-head [T, dim] x [dim, r]
        q_lat = torch.bmm(q[..., :s.dim].transpose(0, 1), self.w_uk).transpose(0, 1)
        o_lat = SM.latent_attention(q_lat, q[..., s.dim:], cache.rows[li], meta.block_tables, meta.seq_of, pos,
                                    s.scale, gate, meta.q_lens_host, meta.seq_lens_host, xa.dtype)
        o = torch.bmm(o_lat.transpose(0, 1), self.w_uv_t).transpose(0, 1).reshape(T, H * s.vdim)
        return F.linear(o, self.w_o)


class MLSTM(nn.Module):
    cache_kind = "state"

    def __init__(self, s: MLSTMSpec, w_q, w_k, w_v, w_g, w_i, w_f, b_i, b_f, norm, w_o):
        super().__init__()
        self.s = s
        self.w_in = nn.Parameter(torch.cat([w_q, w_k, w_v, w_g, w_i, w_f], 0).contiguous(), requires_grad=False)
        self.b_i = nn.Parameter(b_i.float(), requires_grad=False)
        self.b_f = nn.Parameter(b_f.float(), requires_grad=False)
        self.norm = nn.Parameter(norm, requires_grad=False)
        self.w_o = nn.Parameter(w_o, requires_grad=False)

    def cache_spec(self):
        s = self.s
        return ("state", {"S": (s.heads, s.dim, s.vdim), "n": (s.heads, s.dim), "m": (s.heads,)})

    def ensure_table(self, max_pos: int):
        return None

    def forward(self, xa, pos, slots, meta: AttnMeta, cache, li: int, eps: float):
        s = self.s
        T, H = xa.shape[0], s.heads
        nqk, nv = H * s.dim, H * s.vdim
        y = F.linear(xa, self.w_in)
        q, k = y[:, :nqk].reshape(T, H, s.dim), y[:, nqk:2 * nqk].reshape(T, H, s.dim)
        v = y[:, 2 * nqk:2 * nqk + nv].reshape(T, H, s.vdim)
        g = y[:, 2 * nqk + nv:2 * nqk + 2 * nv]
        ip, fp = y[:, 2 * nqk + 2 * nv:2 * nqk + 2 * nv + H], y[:, 2 * nqk + 2 * nv + H:]
        h = SM.mlstm_scan(q, k, v, ip, fp, self.b_i, self.b_f, s.gate_cap, cache.state[li], meta.cu_q,
                          meta.state_slots, pos, meta.q_lens_host)
        o = SM.head_rms_gate(h, self.norm, g, eps, xa.dtype)
        return F.linear(o, self.w_o)


class DenseFF(nn.Module):
    def __init__(self, w_gate, w_up, w_down):
        super().__init__()
        self.w_gu = nn.Parameter(torch.cat([w_gate, w_up], 0).contiguous(), requires_grad=False)
        self.w_down = nn.Parameter(w_down, requires_grad=False)

    def forward(self, xa):
        return F.linear(SM.glu_gelu(F.linear(xa, self.w_gu)), self.w_down)


class GroupedAttention(nn.Module):
    cache_kind = "rows"

    def __init__(self, s: GroupedAttentionSpec, w_q, w_k, q_norm, k_norm, talk, w_g, w_o):
        super().__init__()
        if s.heads % s.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.s = s
        parts = [w_q, w_k] + ([w_g] if w_g is not None else [])
        self.w_in = nn.Parameter(torch.cat(parts, 0).contiguous(), requires_grad=False)      # [q | k | gate] rows
        self.q_norm = nn.Parameter(q_norm, requires_grad=False) if q_norm is not None else None
        self.k_norm = nn.Parameter(k_norm, requires_grad=False) if k_norm is not None else None
        self.talk = nn.Parameter(talk.float().contiguous(), requires_grad=False) if talk is not None else None
        self.w_o = nn.Parameter(w_o, requires_grad=False)
        self.table: Optional[torch.Tensor] = None

    def cache_spec(self):
        return ("rows", 2 * self.s.kv_heads * self.s.dim)

    def ensure_table(self, max_pos: int):
        if self.table is None or self.table.shape[0] < max_pos or self.table.device != self.w_o.device:
            n = max(256, 1 << (max_pos - 1).bit_length())
            if self.s.rot is None or self.s.rot.dims == 0:     # no rotation: one pair turned by the angle 0
                self.table = torch.tensor([1.0, 0.0]).repeat(n, 1, 1).contiguous().to(self.w_o.device)
            else:
                self.table = SM.rope_table(n, self.s.rot.dims, self.s.rot.base, self.s.rot.scaling).to(self.w_o.device)
        return self.table

    def forward(self, xa, pos, slots, meta: AttnMeta, cache, li: int, eps: float):
        s = self.s
        T, H, G, d = xa.shape[0], s.heads, s.kv_heads, s.dim
        y = BM.linear(xa, self.w_in)
        q = y[:, :H * d].view(T, H, d)
        k = y[:, H * d:(H + G) * d].view(T, G, d)
        gate = y[:, (H + G) * d:] if s.out_gate else None
        qf = BM.qk_norm_rope_store(q, k, self.q_norm, self.k_norm, eps, self.table, pos, slots, cache.rows[li])
        o = BM.talk_attention(qf, cache.rows[li], meta.block_tables, meta.seq_of, pos, s.scale, self.talk, gate, G,
                              meta.q_lens_host, meta.seq_lens_host, xa.dtype)
        return BM.linear(o, self.w_o)


class ReluSqFF(nn.Module):
    def __init__(self, w_up, w_down):
        super().__init__()
        self.w_up = nn.Parameter(w_up, requires_grad=False)
        self.w_down = nn.Parameter(w_down, requires_grad=False)

    def forward(self, xa, x32=None):
        return BM.linear(BM.relu_sq(BM.linear(xa, self.w_up)), self.w_down), None


class SigmoidMoE(nn.Module):
    """``w_gu`` [E, 2 ff, W] (every expert's gate rows, then its up rows),
    ``w_down`` [E, W, ff]; the router runs in f32 on the f32 input."""

    def __init__(self, s: MoESpec, router, w_gu, w_down, shared_gu=None, shared_down=None):
        super().__init__()
        self.s = s
        self.router = nn.Parameter(router.float().contiguous(), requires_grad=False)
        self.w_gu = nn.Parameter(w_gu.contiguous(), requires_grad=False)
        self.w_down = nn.Parameter(w_down.contiguous(), requires_grad=False)
        self.shared_gu = nn.Parameter(shared_gu, requires_grad=False) if shared_gu is not None else None
        self.shared_down = nn.Parameter(shared_down, requires_grad=False) if shared_down is not None else None

    def forward(self, xa, x32):
        s = self.s
        idx, wts = BM.moe_route(F.linear(x32, self.router), s.top)
        y = BM.moe_experts(xa, idx, wts, self.w_gu, self.w_down, s.expert.limit, s.expert.alpha)
        ys = None
        if self.shared_gu is not None:
            ys = BM.linear(BM.glu_clamp(BM.linear(xa, self.shared_gu), s.shared.limit, s.shared.alpha), self.shared_down)
        return y, ys


class TokenSide(nn.Module):
    """x += rms_norm(W_proj (gelu_tanh(W_gate x) * e)) * w, with e the layer's
    slice of the token-side table's row of the token."""

    def __init__(self, w_gate, w_proj, norm, offset: int):
        super().__init__()
        self.w_gate = nn.Parameter(w_gate, requires_grad=False)
        self.w_proj = nn.Parameter(w_proj, requires_grad=False)
        self.norm = nn.Parameter(norm, requires_grad=False)
        self.offset = offset

    def forward(self, x, xa, ids, table, eps: float, act):
        g = BM.side_gate(BM.linear(xa, self.w_gate), table, ids, self.offset)
        return BM.add_rms_norm_(x, BM.linear(g, self.w_proj), self.norm, eps, act)


class HybridLayer(nn.Module):
    def __init__(self, mixer: nn.Module, norm1: torch.Tensor, mlp: Optional[DenseFF], norm2: Optional[torch.Tensor]):
        super().__init__()
        self.mixer, self.mlp = mixer, mlp
        self.norm1 = nn.Parameter(norm1, requires_grad=False)
        self.norm2 = nn.Parameter(norm2, requires_grad=False) if norm2 is not None else None

    def cache_specs(self):
        return [self.mixer.cache_spec()]

    def forward(self, x, xa, ids, pos, slots, meta, cache, li: int, model):
        s, act = model.spec, model.dtype
        y = self.mixer(xa, pos, slots, meta, cache, li, s.norm_eps)
        xa = SM.add_scaled_layer_norm_(x, y, self.norm1, s.norm_eps, s.residual_mult, act)
        if self.mlp is not None:
            xa = SM.add_scaled_layer_norm_(x, self.mlp(xa), self.norm2, s.norm_eps, s.residual_mult, act)
        return xa


class ParallelLayer(nn.Module):
    """h = norm(x);  x += ls1 * mixer(h + conv(h)) + ls2 * ff(h);  then the
    token-side input.  ``canon`` [W, taps] or None, ``ls1`` / ``ls2`` [W] or
    None, ``mlp`` returns (result, second result or None) and may be None."""

    def __init__(self, mixer: nn.Module, norm1: torch.Tensor, mlp: Optional[nn.Module], canon=None, ls1=None, ls2=None,
                 side: Optional[TokenSide] = None):
        super().__init__()
        self.mixer, self.mlp, self.side = mixer, mlp, side
        self.norm1 = nn.Parameter(norm1, requires_grad=False)
        self.canon = nn.Parameter(canon.float().contiguous(), requires_grad=False) if canon is not None else None
        self.ls1 = nn.Parameter(ls1.float(), requires_grad=False) if ls1 is not None else None
        self.ls2 = nn.Parameter(ls2.float(), requires_grad=False) if ls2 is not None else None

    def cache_specs(self):
        out = [self.mixer.cache_spec()]
        if self.canon is not None and self.canon.shape[1] > 1:
            out.append(("state", {"canon": (self.canon.shape[1] - 1, self.canon.shape[0])}))
        return out

    def forward(self, x, xa, ids, pos, slots, meta, cache, li: int, model):
        s, act = model.spec, model.dtype
        if self.canon is not None and self.canon.shape[1] > 1:
            h32, ha, hm = BM.norm_canon(x, self.norm1, s.norm_eps, self.canon, cache.state[li]["canon"], meta.cu_q,
                                        meta.seq_of, meta.state_slots, pos, meta.q_lens_host, act)
        else:
            h32, ha = BM.rms_norm_rows(x, self.norm1, s.norm_eps, act)
            hm = ha if self.canon is None else (h32 * (1.0 + self.canon[:, 0])).to(act)
        ym = self.mixer(hm, pos, slots, meta, cache, li, s.norm_eps)
        y2, y3 = self.mlp(ha, h32) if self.mlp is not None else (None, None)
        xa = BM.residual_add_scaled_(x, ym, self.ls1, y2, y3, self.ls2, act)
        if self.side is not None:
            xa = self.side(x, xa, ids, model.side_embed, s.norm_eps, act)
        return xa


# name -> (spec class, module class): a design's config reader maps its layer
# types onto these
MIXERS: Dict[str, tuple] = {"latent_attention": (LatentAttentionSpec, LatentAttention), "mlstm": (MLSTMSpec, MLSTM),
                            "grouped_attention": (GroupedAttentionSpec, GroupedAttention)}


# ---------------------------------------------------------------------- model
class HybridCausalLM(nn.Module):
    ragged_step = True              # forward_tokens takes sequences of unequal new-token counts
    native_lib = "seqmix"           # the kernels it needs (ops.require_seqmix)

    def __init__(self, spec: HybridSpec, embed: torch.Tensor, bigram: Optional[torch.Tensor],
                 layers: List[nn.Module], final_norm: torch.Tensor, head: torch.Tensor, dtype=torch.bfloat16,
                 side_embed: Optional[torch.Tensor] = None):
        super().__init__()
        self.spec, self.dtype = spec, dtype
        self.embed_tokens = nn.Parameter(embed, requires_grad=False)
        self.bigram = nn.Parameter(bigram, requires_grad=False) if bigram is not None else None
        self.side_embed = nn.Parameter(side_embed, requires_grad=False) if side_embed is not None else None
        self.layers = nn.ModuleList(layers)
        self.norm = nn.Parameter(final_norm, requires_grad=False)
        self.lm_head = nn.Parameter(head, requires_grad=False)
        self.tp_group = None
        self.first_stage = self.last_stage = True
        self.capture_layers: Optional[list] = None      # debugging: residual stream after every layer

    @property
    def device(self):
        return self.norm.device

    @property
    def has_state(self) -> bool:
        return any(c[0] == "state" for L in self.layers for c in L.cache_specs())

    def graph_max_batch(self) -> int:
        return 0                    # ragged steps are launched eagerly

    def ensure_rope_cache(self, max_pos: int):
        for L in self.layers:
            L.mixer.ensure_table(max_pos)

    def cache_bytes_per_token(self) -> int:
        eb = torch.empty(0, dtype=self.dtype).element_size()
        return sum(c[1] * eb for L in self.layers for c in L.cache_specs() if c[0] == "rows")

    def make_cache(self, max_tokens: int, batch: int = 1, block_size: int = 64, kv_fp8: int = 0,
                   num_blocks: Optional[int] = None, num_slots: Optional[int] = None):
        from .cache import HybridCache
        if kv_fp8:
            raise ValueError("hybrid decoders keep their latent rows in the activation dtype (no fp8 cache)")
        nblk = num_blocks or batch * ((max_tokens + block_size - 1) // block_size)
        self.ensure_rope_cache(max_tokens + 1)
        return HybridCache([L.cache_specs() for L in self.layers], nblk, num_slots or batch, block_size,
                           self.dtype, self.device)

    @staticmethod
    def complete_meta(meta: AttnMeta, pos: torch.Tensor, T: int) -> AttnMeta:
        """fill the ragged fields of a uniform (B x Tq) step"""
        if meta.cu_q is None:
            dev = pos.device
            meta.cu_q = torch.arange(0, (meta.B + 1) * meta.Tq, meta.Tq, dtype=torch.int32, device=dev)
            meta.q_lens_host = [meta.Tq] * meta.B
            meta.seq_of = torch.arange(meta.B, dtype=torch.int32, device=dev).repeat_interleave(meta.Tq)
        if meta.seq_lens_host is None:
            meta.seq_lens_host = [int(v) for v in meta.seq_lens.tolist()]
        return meta

    def forward_tokens(self, ids: torch.Tensor, pos: torch.Tensor, slots: torch.Tensor, meta: AttnMeta, cache,
                       logits_idx: Optional[torch.Tensor] = None, return_hidden: bool = False,
                       hidden_in: Optional[torch.Tensor] = None):
        """ids / pos / slots [T] (sequence after sequence, ``meta.cu_q``);
        ``meta.prev_ids`` the token before each one (-1: none) when the model
        has a bigram table; ``meta.state_slots`` when it has recurrent layers.
        Returns f32 logits [len(logits_idx) or T, vocab]."""
        s = self.spec
        T = ids.shape[0]
        meta = self.complete_meta(meta, pos, T)
        if self.has_state and meta.state_slots is None:
            raise ValueError("a model with recurrent layers needs AttnMeta.state_slots")
        self.ensure_rope_cache(max(meta.seq_lens_host) + 1)
        act = self.dtype
        if hidden_in is not None:
            x = hidden_in.float().contiguous().clone()
        elif self.bigram is not None:
            if meta.prev_ids is None:
                raise ValueError("a model with a bigram table needs AttnMeta.prev_ids")
            b = s.bigram
            x = SM.embed_bigram(ids, meta.prev_ids, self.embed_tokens, self.bigram, b.mul_prev, b.mul_cur)
        else:
            x = F.embedding(ids, self.embed_tokens).float()
        xa = x if act == torch.float32 else x.to(act)
        for li, L in enumerate(self.layers):
            xa = L(x, xa, ids, pos, slots, meta, cache, li, self)
            if self.capture_layers is not None:
                self.capture_layers.append(x.clone())
        if not self.last_stage:
            return x
        if logits_idx is not None:
            x = x.index_select(0, logits_idx)
        if s.norm == "layer_norm":
            xn = SM.layer_norm_f32(x, self.norm, s.norm_eps, act)
        else:
            xn = BM.rms_norm_rows(x, self.norm, s.norm_eps, act)[1]
        if return_hidden:
            return xn
        return BM.linear(xn, self.lm_head).float()
