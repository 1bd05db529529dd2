"""Prefill / decode throughput of a hybrid decoder (latent attention + mLSTM
layers, Zamelix layout) at layer sizes of a real model, beside the framework's
closest existing model -- the DeepSeek-style MLA decoder (models/mla.py) -- at
equal attention and feed-forward sizes.  Random bf16 weights, synthetic
tokens.  Run through ``bench.py --hybrid``; one JSON line.

Both models go through their serving paths: the hybrid one through
``LLMEngine.feed`` (ragged steps), the MLA one through ``Engine.prefill`` and
its decode step.  Prefill: one request of P tokens in one step, tokens / s.
Decode: B sequences at context P, one token each per step, tokens / s.
"""
from __future__ import annotations

import json
import time
from typing import Dict, List

import torch

SIZES = {
    # width, vocab, ff, attention (heads, dim, rot, vdim, rank), mLSTM (heads, dim, vdim), layers
    "small": dict(width=1024, vocab=32000, ff=2816, attn=(8, 64, 32, 64, 256), mlstm=(4, 64, 256), blocks=2),
    "base": dict(width=2048, vocab=32000, ff=5632, attn=(16, 128, 64, 128, 512), mlstm=(4, 256, 512), blocks=2),
}


def hybrid_config(sz: dict) -> dict:
    H, dim, rot, dv, r = sz["attn"]
    mh, md, mv = sz["mlstm"]
    attn = {"type": "latent_attention",
            "mixer": {"heads": H, "dim": dim, "rot_dim": rot, "vdim": dv, "kv_rank": r, "scale": (dim + rot) ** -0.5,
                      "rot": {"base": 10000.0, "dims": rot,
                              "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}}},
            "mlp": {"kind": "dense", "ff": sz["ff"]}}
    rec = {"type": "mlstm", "mixer": {"heads": mh, "dim": md, "vdim": mv, "gate_cap": 15.0}, "mlp": None}
    return {"architecture": "Zamelix", "vocab": sz["vocab"], "width": sz["width"], "norm": {"eps": 1e-6},
            "residual_mult": 0.5, "embedding": {"bigram": {"buckets": 65521, "mul_prev": 31, "mul_cur": 7}},
            "layers": [attn, rec] * sz["blocks"]}


def _sync_time(fn, dev, reps: int) -> float:
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize(dev)
    return (time.perf_counter() - t0) / reps


def bench_hybrid(sz: dict, dev, prompt_len: int, batch: int, steps: int, warmup: int) -> Dict[str, float]:
    from ..models import zamelix as Z
    from ..serving.engine import LLMEngine
    spec = Z.spec_from_config(hybrid_config(sz))
    model = Z.random_model(spec, 0, torch.bfloat16, dev)
    total = prompt_len + warmup + steps + 8
    nblk = batch * (-(-total // 64))
    eng = LLMEngine(model, max_batch=batch, block_size=64, num_blocks=nblk, max_model_len=total,
                    max_prefill_tokens=1 << 30, use_graph=True, enable_prefix_caching=False)
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, spec.vocab_size, (prompt_len,), generator=g).tolist() for _ in range(batch)]
    # prefill: one request, whole prompt, (warm-up run first)
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


def bench_mla(sz: dict, dev, prompt_len: int, batch: int, steps: int, warmup: int, tmpdir: str) -> Dict[str, float]:
    """the closest existing model: DeepSeek-style MLA decoder with the same
    attention sizes and as many (attention + dense feed-forward) layers"""
    import transformers as T
    from ..engine.runner import Engine
    from ..models.cache import SequenceState
    from ..transformers import AutoModelForCausalLM
    from ..transformers.hf_native import get_native
    H, dim, rot, dv, r = sz["attn"]
    cfg = T.AutoConfig.for_model("deepseek_v3", hidden_size=sz["width"], intermediate_size=sz["ff"],
                                 moe_intermediate_size=64, num_hidden_layers=sz["blocks"], num_attention_heads=H,
                                 num_key_value_heads=H, vocab_size=sz["vocab"],
                                 max_position_embeddings=prompt_len + warmup + steps + 64, n_routed_experts=2,
                                 num_experts_per_tok=1, n_group=1, topk_group=1, n_shared_experts=1,
                                 first_k_dense_replace=sz["blocks"], q_lora_rank=None, kv_lora_rank=r,
                                 qk_rope_head_dim=rot, qk_nope_head_dim=dim, v_head_dim=dv)
    torch.manual_seed(0)
    ref = T.AutoModelForCausalLM.from_config(cfg).to(torch.bfloat16).eval()
    ref.save_pretrained(tmpdir)
    del ref
    m = AutoModelForCausalLM.from_pretrained(tmpdir, load_in_low_bit="bf16", torch_dtype=torch.bfloat16).to(dev).eval()
    nm, eng = get_native(m)
    total = prompt_len + warmup + steps + 8
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
    st.set_state(torch.ones(batch, dtype=torch.long, device=dev),
                 torch.tensor([s.length for s in seqs], device=dev))
    for _ in range(warmup):
        st.step()
    decode_s = _sync_time(st.step, dev, steps)
    return {"prefill_tok_s": prompt_len / prefill_s, "prefill_ms": prefill_s * 1e3,
            "decode_tok_s": batch / decode_s, "decode_ms_per_step": decode_s * 1e3}


def main(args) -> dict:
    import tempfile
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    out: List[dict] = []
    for name in args.hybrid_sizes.split(","):
        sz = SIZES[name]
        for P in [int(p) for p in args.hybrid_prompts.split(",")]:
            row = {"size": name, "prompt_len": P, "batch": args.batch,
                   "hybrid": {k: round(v, 3) for k, v in
                              bench_hybrid(sz, dev, P, args.batch, args.steps, args.warmup).items()}}
            if not args.no_hybrid_ref:
                with tempfile.TemporaryDirectory() as td:
                    row["mla_reference"] = {k: round(v, 3) for k, v in
                                            bench_mla(sz, dev, P, args.batch, args.steps, args.warmup, td).items()}
            out.append(row)
            print(json.dumps(row), file=__import__("sys").stderr, flush=True)
    res = {"metric": "hybrid decoder prefill / decode throughput (random weights, synthetic tokens)", "unit": "tokens/s",
           "dtype": "bf16", "data": "synthetic", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "rows": out}
    print(json.dumps(res))
    return res
