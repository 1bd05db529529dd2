"""Paged KV cache sized for MI355X's 288 GB HBM.

Reference: ``SRC/transformers/kv.py`` (DynamicNormalCache / DynamicFp8Cache:
contiguous caches grown 256 tokens at a time, fp8 as uint8) and the vLLM
block tables of ``VLLM_PATCH`` (reshape_and_cache / paged attention).

Here every layer owns two tensors ``[num_blocks, Hkv, block_size, D]``
(bf16/fp16, or fp8 bytes).  A sequence owns a list of blocks (its row of the
int32 block table).  Static single-request generation simply reserves
``ceil(max_len / bs)`` blocks per sequence up front -- there is no regrowth
(and so no re-allocation inside a captured hipGraph).
"""
from __future__ import annotations

from typing import List, Optional

import torch

KV_FP8_NONE, KV_FP8_E5M2, KV_FP8_E4M3 = 0, 1, 2


class BlockAllocator:
    def __init__(self, num_blocks: int):
        self.free: List[int] = list(range(num_blocks - 1, -1, -1))

    def alloc(self, n: int) -> List[int]:
        if n > len(self.free):
            raise RuntimeError(f"KV cache exhausted: need {n} blocks, {len(self.free)} free")
        return [self.free.pop() for _ in range(n)]

    def release(self, blocks: List[int]):
        self.free.extend(reversed(blocks))


class SlotAllocator:
    """Free list of recurrent-state slots (one per live sequence).  A slot's
    content is never cleared on release: a sequence whose first position is 0
    starts from the zero state inside the scan kernels, whatever the slot held."""

    def __init__(self, num_slots: int):
        self.free: List[int] = list(range(num_slots - 1, -1, -1))

    def alloc(self) -> int:
        if not self.free:
            raise RuntimeError("recurrent-state pool exhausted: no free slot")
        return self.free.pop()

    def release(self, slot: int):
        self.free.append(slot)


class HybridCache:
    """Cache of a model whose layers mix paged attention rows and recurrent
    state (models/hybrid.py).

    ``layer_specs[i]`` is ``("rows", width)`` for a layer that appends one
    ``width``-wide row per token to a paged pool (a latent-attention layer
    keeps ``[latent | rotated key]``, a grouped-attention layer ``[keys |
    values]``), ``("state", {name: shape})`` for a layer with per-sequence f32
    state tensors (``shape`` without the slot axis), ``None``, or a list of
    such entries for a layer that has both (paged rows and, say, the last
    inputs of a short convolution).  Row pools are ``[num_blocks + 1, block_size, width]`` and state
    pools ``[num_slots + 1, *shape]``: the last block / slot is a scratch
    target for padded batch rows.  ``k`` / ``v`` alias the row pools so the
    engines' device probes (``cache.k[0]``) keep working."""

    def __init__(self, layer_specs, num_blocks: int, num_slots: int, block_size: int = 64,
                 dtype=torch.bfloat16, device="cuda"):
        if block_size % 64:
            raise ValueError("block_size must be a multiple of 64")
        self.num_layers, self.num_blocks, self.num_slots = len(layer_specs), num_blocks, num_slots
        self.bs, self.dtype, self.kv_fp8 = block_size, dtype, 0
        self.k_scale = self.v_scale = 1.0
        self.device = torch.device(device)
        self.rows: List[Optional[torch.Tensor]] = []
        self.state: List[Optional[dict]] = []
        for entry in layer_specs:
            rows, st = None, None
            for spec in (entry if isinstance(entry, list) else [entry]):
                if spec is not None and spec[0] == "rows":
                    if rows is not None:
                        raise ValueError("one paged row pool per layer")
                    rows = torch.zeros(num_blocks + 1, block_size, int(spec[1]), dtype=dtype, device=device)
                elif spec is not None and spec[0] == "state":
                    st = dict(st or {})
                    st.update({n: torch.zeros(num_slots + 1, *shape, dtype=torch.float32, device=device)
                               for n, shape in spec[1].items()})
            self.rows.append(rows)
            self.state.append(st)
        probe = next((r for r in self.rows if r is not None), None)
        if probe is None:
            probe = torch.zeros(1, dtype=dtype, device=device)
        self.k = [r if r is not None else probe for r in self.rows]
        self.v = self.k
        self.allocator = BlockAllocator(num_blocks)
        self.slots = SlotAllocator(num_slots)

    def blocks_for(self, n_tokens: int) -> int:
        return (n_tokens + self.bs - 1) // self.bs

    def bytes(self) -> int:
        n = sum(r.numel() * r.element_size() for r in self.rows if r is not None)
        return n + sum(t.numel() * 4 for st in self.state if st for t in st.values())


class PagedKVCache:
    def __init__(self, num_layers: int, num_blocks: int, num_kv_heads: int, head_dim: int,
                 block_size: int = 64, dtype=torch.bfloat16, device="cuda", kv_fp8: int = 0,
                 k_scale: float = 1.0, v_scale: float = 1.0):
        if block_size % 64:
            raise ValueError("block_size must be a multiple of 64")
        self.num_layers, self.num_blocks = num_layers, num_blocks
        self.Hkv, self.D, self.bs = num_kv_heads, head_dim, block_size
        self.dtype, self.kv_fp8 = dtype, kv_fp8
        self.k_scale, self.v_scale = k_scale, v_scale
        store = torch.uint8 if kv_fp8 else dtype
        shape = (num_blocks, num_kv_heads, block_size, head_dim)
        self.k = [torch.zeros(shape, dtype=store, device=device) for _ in range(num_layers)]
        self.v = [torch.zeros(shape, dtype=store, device=device) for _ in range(num_layers)]
        self.allocator = BlockAllocator(num_blocks)
        self.device = torch.device(device)

    @staticmethod
    def bytes_per_token(num_layers, num_kv_heads, head_dim, dtype=torch.bfloat16, kv_fp8=0):
        eb = 1 if kv_fp8 else torch.empty(0, dtype=dtype).element_size()
        return 2 * num_layers * num_kv_heads * head_dim * eb

    def blocks_for(self, n_tokens: int) -> int:
        return (n_tokens + self.bs - 1) // self.bs


class SequenceState:
    """Host-side bookkeeping of one sequence in the cache."""

    def __init__(self, blocks: List[int], length: int = 0, slot: int = -1):
        self.blocks = blocks
        self.length = length
        self.slot = slot                 # recurrent-state slot (HybridCache), -1: none


def make_block_table(seqs: List[SequenceState], max_blocks: int, device) -> torch.Tensor:
    t = torch.zeros(len(seqs), max_blocks, dtype=torch.int32)
    for i, s in enumerate(seqs):
        t[i, :len(s.blocks)] = torch.tensor(s.blocks, dtype=torch.int32)
    return t.to(device)


def slots_for(seq: SequenceState, start: int, n: int, bs: int) -> torch.Tensor:
    pos = torch.arange(start, start + n)
    blk = torch.tensor(seq.blocks, dtype=torch.int64)[pos // bs]
    return blk * bs + pos % bs
