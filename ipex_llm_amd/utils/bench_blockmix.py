"""Prefill / decode throughput of a parallel-residual decoder (Masezen layout:
grouped attention with mixed head scores, canon convolution, token-side
input; dense or expert feed-forward) at layer sizes of a real model, beside
the framework's closest existing model -- the Qwen3-style grouped-query
decoder with per-head query / key norms (models/decoder.py) -- at equal
attention and feed-forward sizes.  Random bf16 weights, synthetic tokens.
Run through ``bench.py --blockmix``; one JSON line.

Both models go through their serving paths: the parallel-residual one through
``LLMEngine.feed`` (ragged steps), the reference through ``Engine.prefill``
and its decode step.  Prefill: one request of P tokens in one step, tokens / s.
Decode: B sequences at context P, one token each per step (hipGraph on both
sides), tokens / s.
"""
from __future__ import annotations

import json
import sys
import time
from typing import Dict, List

import torch

SIZES = {
    # width, vocab, heads, kv heads, head size, dense ff, experts (count, top, ff, shared ff), layers
    "small": dict(width=1024, vocab=32000, heads=8, kv=2, dim=128, ff=2816, moe=(8, 2, 1024, 1024), blocks=4),
    "base": dict(width=2048, vocab=32000, heads=16, kv=4, dim=128, ff=5632, moe=(16, 2, 1408, 1408), blocks=4),
}


def blockmix_config(sz: dict, experts: bool) -> dict:
    mixer = {"heads": sz["heads"], "kv_heads": sz["kv"], "dim": sz["dim"], "vdim": sz["dim"], "scale": sz["dim"] ** -0.5,
             "rot": {"base": 10000.0, "dims": sz["dim"] // 2,
                     "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}}}
    if experts:
        E, top, ff, sff = sz["moe"]
        mlp = {"kind": "moe", "router": {"experts": E, "top": top}, "expert": {"ff": ff, "limit": 7.0},
               "shared": {"ff": sff, "limit": 7.0}}
    else:
        mlp = {"kind": "dense", "ff": sz["ff"]}
    return {"architecture": "Masezen", "vocab": sz["vocab"], "width": sz["width"], "norm": {"eps": 1e-6},
            "canon": {"taps": 4}, "token_side": {"dim": 64},
            "layers": [{"type": "attention", "mixer": mixer, "mlp": mlp} for _ in range(sz["blocks"])]}


def _sync_time(fn, dev, reps: int) -> float:
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize(dev)
    return (time.perf_counter() - t0) / reps


def bench_blockmix(sz: dict, experts: bool, dev, prompt_len: int, batch: int, steps: int, warmup: int) -> Dict[str, float]:
    from ..models import masezen as Z
    from ..serving.engine import LLMEngine
    spec = Z.spec_from_config(blockmix_config(sz, experts))
    model = Z.random_model(spec, 0, torch.bfloat16, dev)
    total = prompt_len + warmup + steps + 8
    nblk = batch * (-(-total // 64))
    eng = LLMEngine(model, max_batch=batch, block_size=64, num_blocks=nblk, max_model_len=total,
                    max_prefill_tokens=1 << 30, use_graph=True, enable_prefix_caching=False)
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, spec.vocab_size, (prompt_len,), generator=g).tolist() for _ in range(batch)]
    times = []
    for rep in range(3):
        rid = eng.open_stream()
        torch.cuda.synchronize(dev)
        t0 = time.perf_counter()
        eng.feed([(rid, prompts[0], [prompt_len - 1])])
        torch.cuda.synchronize(dev)
        times.append(time.perf_counter() - t0)
        eng.close_stream(rid)
    prefill_s = min(times[1:])
    rids = [eng.open_stream() for _ in range(batch)]
    eng.feed([(r, p, [prompt_len - 1]) for r, p in zip(rids, prompts)])
    tok = [[1 + i] for i in range(batch)]

    def step():
        eng.feed([(r, t, [0]) for r, t in zip(rids, tok)])
    for _ in range(warmup):
        step()
    decode_s = _sync_time(step, dev, steps)
    for r in rids:
        eng.close_stream(r)
    return {"prefill_tok_s": prompt_len / prefill_s, "prefill_ms": prefill_s * 1e3,
            "decode_tok_s": batch / decode_s, "decode_ms_per_step": decode_s * 1e3}


def bench_gqa(sz: dict, dev, prompt_len: int, batch: int, steps: int, warmup: int) -> Dict[str, float]:
    """the closest existing model: Qwen3-style decoder (grouped-query attention, per-head query / key
    norms, gated feed-forward) with the same attention sizes, a feed-forward of the same number of
    weights (two matrices of ff there, three of 2/3 ff here), as many layers, bf16 weights"""
    import transformers as T
    from ..engine.runner import Engine
    from ..models.builder import random_native_model
    from ..models.cache import SequenceState
    ff = (sz["ff"] * 2 // 3 + 31) // 32 * 32
    total = prompt_len + warmup + steps + 8
    cfg = T.Qwen3Config(vocab_size=sz["vocab"], hidden_size=sz["width"], intermediate_size=ff,
                        num_hidden_layers=sz["blocks"], num_attention_heads=sz["heads"], num_key_value_heads=sz["kv"],
                        head_dim=sz["dim"], max_position_embeddings=total + 64, rms_norm_eps=1e-6,
                        tie_word_embeddings=False)
    model = random_native_model(cfg, "bf16", dev, torch.bfloat16, seed=0)
    eng = Engine(model)
    eng._ensure_cache(batch, total)
    nblk = -(-total // eng.block_size)
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, sz["vocab"], (batch, prompt_len), generator=g)
    times = []
    for rep in range(3):
        seq = SequenceState(eng.cache.allocator.alloc(nblk))
        torch.cuda.synchronize(dev)
        t0 = time.perf_counter()
        eng.prefill(seq, ids[0])
        torch.cuda.synchronize(dev)
        times.append(time.perf_counter() - t0)
        eng.cache.allocator.release(seq.blocks)
    prefill_s = min(times[1:])
    seqs = [SequenceState(eng.cache.allocator.alloc(nblk)) for _ in range(batch)]
    for b, s in enumerate(seqs):
        eng.prefill(s, ids[b])
    st = eng.decode_step_obj(seqs, total, greedy=True, use_graph=True)
    st.set_state(torch.ones(batch, dtype=torch.long, device=dev), torch.tensor([s.length for s in seqs], device=dev))
    for _ in range(warmup):
        st.step()
    decode_s = _sync_time(st.step, dev, steps)
    return {"prefill_tok_s": prompt_len / prefill_s, "prefill_ms": prefill_s * 1e3,
            "decode_tok_s": batch / decode_s, "decode_ms_per_step": decode_s * 1e3}


def main(args) -> dict:
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    out: List[dict] = []
    for name in args.blockmix_sizes.split(","):
        sz = SIZES[name]
        for P in [int(p) for p in args.blockmix_prompts.split(",")]:
            row = {"size": name, "prompt_len": P, "batch": args.batch}
            for key, experts in (("dense", False), ("experts", True)):
                row[key] = {k: round(v, 3) for k, v in
                            bench_blockmix(sz, experts, dev, P, args.batch, args.steps, args.warmup).items()}
            if not args.no_blockmix_ref:
                row["gqa_reference"] = {k: round(v, 3) for k, v in
                                        bench_gqa(sz, dev, P, args.batch, args.steps, args.warmup).items()}
            out.append(row)
            print(json.dumps(row), file=sys.stderr, flush=True)
    res = {"metric": "parallel-residual decoder prefill / decode throughput (random weights, synthetic tokens)",
           "unit": "tokens/s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "rows": out}
    print(json.dumps(res))
    return res
