"""Trace replay: feed given token ids through a model step by step and write
the logits at the asked places -- no sampling.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps arrive on standard input, one JSON object a line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries``: for each request its next tokens and the indices among them whose
logits are wanted; ``end``: requests that are finished after the step (their
cache blocks and state slot are given back).  A step's entries run as ONE
batch through ``serving.engine.LLMEngine`` -- the engine, scheduler / block
manager, cache and kernels that serve generation -- continuing from what
earlier steps left.  A step with wanted places writes ``<out>/<step>.f32``
(little-endian f32 ``[wanted, vocab]``, in entry order); after every step the
line ``done <step>`` is printed.  The engine is sized for ``--max-tokens``
live tokens (per request rounded up to whole cache blocks) and
``--max-requests`` live requests.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--max-requests", type=int, default=4)
    ap.add_argument("--device", default=os.environ.get("ILLM_TRACE_DEVICE", "cuda"))
    a = ap.parse_args(argv)
    import torch
    from ..models.registry import load_native, native_architecture
    if native_architecture(a.model) is None:
        print(f"trace_run: {a.model} is not a checkpoint of a registered native architecture", file=sys.stderr)
        return 2
    dtype = torch.bfloat16 if a.dtype == "bfloat16" else torch.float32
    if dtype == torch.float32:
        # true 32-bit products: no reduced-precision matrix mode
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    model = load_native(a.model, dtype=dtype, device=a.device)
    from ..serving.engine import LLMEngine
    bs = 64
    eng = LLMEngine(model, max_batch=a.max_requests, block_size=bs, num_blocks=max(1, -(-a.max_tokens // bs)),
                    max_model_len=max(bs, a.max_tokens), max_prefill_tokens=1 << 30, use_graph=False,
                    enable_prefix_caching=False)
    os.makedirs(a.out, exist_ok=True)
    live = {}
    out = sys.stdout
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries = []
        for e in step.get("entries", []):
            if not e["tokens"]:
                continue
            if e["id"] not in live:
                live[e["id"]] = eng.open_stream()
            entries.append((live[e["id"]], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]))
        if entries:
            logits = eng.feed(entries)
            if logits.shape[0]:
                data = logits.detach().to("cpu", torch.float32).contiguous().numpy().astype("<f4", copy=False)
                tmp = os.path.join(a.out, f".{step['step']}.part")
                with open(tmp, "wb") as f:
                    f.write(data.tobytes())
                os.replace(tmp, os.path.join(a.out, f"{step['step']}.f32"))
            elif a.device != "cpu":
                torch.cuda.synchronize()
        for rid in step.get("end", []):
            if rid in live:
                eng.close_stream(live.pop(rid))
        out.write(f"done {step['step']}\n")
        out.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
