"""Hybrid decoders (latent attention + mLSTM layers, Zamelix layout): the
framework -- checkpoint reader, cache / state slots, scheduler, ragged engine
steps, kernels -- against the plain float64 forms of tests/hybrid_oracle.py.

Every test runs on the CPU (torch forms of ops/seqmix.py) and, marked ``gpu``,
on the HIP kernels.  Models are small random ones made here; their sizes
differ from each other wherever the mechanisms allow it (heads, key / rotated
/ value sizes, latent rank, feed-forward or none, layer order).
"""
import json
import math
import os
import subprocess
import sys

import pytest
import torch

from . import hybrid_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEVS = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
YARN = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 2.0}


@pytest.fixture(params=DEVS)
def dev(request):
    if request.param == "cuda":
        if not torch.cuda.is_available():
            pytest.skip("no GPU")
        import ipex_llm_amd.ops as ops
        ops.require_seqmix()
    return torch.device(request.param)


def std_cfg():
    """mLSTM first, attention with and without feed-forward, YaRN on one layer,
    partial rotation on another"""
    return O.config([O.mlstm_layer(heads=2, dim=12, vdim=20, gate_cap=3.0, ff=0),
                     O.attn_layer(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, scaling=YARN, ff=48),
                     O.attn_layer(heads=5, dim=8, rot_dim=12, vdim=16, kv_rank=24, dims=8, scale=0.3, ff=0),
                     O.mlstm_layer(heads=3, dim=8, vdim=12, gate_cap=2.0, ff=56)])


def build(cfg, W, dev, dtype=torch.float32):
    from ipex_llm_amd.models import zamelix as Z
    return Z.build(Z.spec_from_config(cfg), W, dtype, dev)


def engine(cfg, W, dev, dtype=torch.float32, max_batch=4, num_blocks=16, prefill=1 << 30):
    from ipex_llm_amd.serving.engine import LLMEngine
    return LLMEngine(build(cfg, W, dev, dtype), max_batch=max_batch, block_size=64, num_blocks=num_blocks,
                     max_model_len=num_blocks * 64, max_prefill_tokens=prefill, use_graph=False,
                     enable_prefix_caching=False)


def replay(eng, prompts, schedule, keep_open=()):
    """schedule: steps of [(name, count)]; every token's logits are asked for.
    Returns name -> [T, V] (f64, on the CPU) of what was run."""
    at, rid, got = {}, {}, {}
    for step in schedule:
        entries, names = [], []
        for name, n in step:
            lo = at.get(name, 0)
            if name not in rid:
                rid[name] = eng.open_stream()
            entries.append((rid[name], prompts[name][lo:lo + n], list(range(n))))
            names.append((name, n))
            at[name] = lo + n
        lg = eng.feed(entries).double().cpu()
        o = 0
        for name, n in names:
            got.setdefault(name, []).append(lg[o:o + n])
            o += n
        for name, _ in names:
            if at[name] == len(prompts[name]) and name not in keep_open:
                eng.close_stream(rid.pop(name))
    return {k: torch.cat(v) for k, v in got.items()}


def rel_err(got, want):
    """largest row error: rms over the vocabulary of the centred difference, over the logits' spread"""
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / want.std()).max())


TOL = {torch.float32: 2e-4, torch.bfloat16: 0.12}


# ------------------------------------------------------------------ mechanisms alone
def test_rotary_table_plain_and_yarn():
    from ipex_llm_amd.ops.seqmix import rope_table
    for rot in ({"dims": 8, "base": 10000.0, "scaling": None}, {"dims": 12, "base": 500.0, "scaling": YARN},
                {"dims": 6, "base": 1e6, "scaling": {"factor": 2.0, "original": 16, "fast": 4.0, "slow": 1.0}}):
        cos, sin = O.rotary_angles(rot, range(300))
        tab = rope_table(300, rot["dims"], rot["base"], rot["scaling"]).double()
        assert tab.shape == (300, rot["dims"] // 2, 2)
        assert (tab[..., 0] - cos).abs().max() < 1e-6 and (tab[..., 1] - sin).abs().max() < 1e-6
    # YaRN really changes the slow pairs and the magnitude
    cos_p, _ = O.rotary_angles({"dims": 12, "base": 500.0}, range(300))
    cos_y, _ = O.rotary_angles({"dims": 12, "base": 500.0, "scaling": YARN}, range(300))
    assert (cos_p - cos_y).abs().max() > 0.1


@pytest.mark.parametrize("layer", [O.attn_layer(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, scaling=YARN, ff=0),
                                   O.attn_layer(heads=9, dim=4, rot_dim=6, vdim=8, kv_rank=72, dims=4, ff=0),
                                   O.attn_layer(heads=1, dim=8, rot_dim=2, vdim=4, kv_rank=8, ff=0)])
def test_latent_attention_alone(dev, layer):
    """one attention layer, residual multiplier 1: also > 8 heads, latent rank > 64, one head"""
    cfg = O.config([layer], mult=1.0)
    W = O.random_weights(cfg, 1)
    toks = O.random_tokens(cfg, 150, 1)
    got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", 150)]])["a"]
    assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.float32]


@pytest.mark.parametrize("layer", [O.mlstm_layer(heads=2, dim=12, vdim=20, gate_cap=3.0),
                                   O.mlstm_layer(heads=3, dim=70, vdim=72, gate_cap=50.0),
                                   O.mlstm_layer(heads=1, dim=4, vdim=130, gate_cap=1.0)])
def test_mlstm_alone(dev, layer):
    """one recurrent layer: also key size > 64, value size > 64 and > 128 (several column blocks)"""
    cfg = O.config([layer], mult=1.0)
    W = O.random_weights(cfg, 2)
    toks = O.random_tokens(cfg, 90, 2)
    got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", 90)]])["a"]
    assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.float32]


@pytest.mark.parametrize("C", [4, 32])
def test_mlstm_chunk_parallel_form(dev, C):
    """the chunk-parallel form of the recurrence against the token loop, continuing from a non-zero state"""
    from ipex_llm_amd.ops import seqmix as SM
    g = torch.Generator().manual_seed(C)
    n, H, d, dv = 96, 3, 10, 14
    q, k = torch.randn(n, H, d, generator=g) * d ** -0.5, torch.randn(n, H, d, generator=g)
    v = torch.randn(n, H, dv, generator=g)
    ig = 3.0 * torch.tanh(torch.randn(n, H, generator=g) * 2)
    fg = torch.nn.functional.logsigmoid(3.0 * torch.tanh(torch.randn(n, H, generator=g) * 2 + 1))
    S0, n0, m0 = torch.randn(H, d, dv, generator=g), torch.randn(H, d, generator=g), torch.rand(H, generator=g) * 2
    h, S1, n1, m1 = SM.mlstm_chunked(*(x.to(dev) for x in (q, k, v, ig, fg, S0, n0, m0)), C)
    S, nn, m = S0.double(), n0.double(), m0.double()
    want = torch.zeros(n, H, dv, dtype=torch.float64)
    for t in range(n):
        mn = torch.maximum(fg[t].double() + m, ig[t].double())
        a, b = torch.exp(fg[t].double() + m - mn), torch.exp(ig[t].double() - mn)
        S = a[:, None, None] * S + b[:, None, None] * k[t].double()[:, :, None] * v[t].double()[:, None, :]
        nn = a[:, None] * nn + b[:, None] * k[t].double()
        m = mn
        den = torch.maximum((nn * q[t].double()).sum(-1).abs(), torch.exp(-m)) + 1e-6
        want[t] = torch.einsum("hdv,hd->hv", S, q[t].double()) / den[:, None]
    assert (h.cpu().double() - want).abs().max() < 2e-4 * max(1.0, float(want.abs().max()))
    assert (S1.cpu().double() - S).abs().max() < 2e-4 * max(1.0, float(S.abs().max()))
    assert (n1.cpu().double() - nn).abs().max() < 2e-4 and (m1.cpu().double() - m).abs().max() < 1e-5


def test_mlstm_gates_saturate(dev):
    """large pre-activations: the cap bounds both gates, the running maximum keeps exp() finite"""
    cfg = O.config([O.mlstm_layer(heads=2, dim=8, vdim=8, gate_cap=6.0)], mult=1.0)
    W = O.random_weights(cfg, 3)
    for k in ("l0.mix.i", "l0.mix.f"):
        W[k] = (W[k] * 40).to(torch.bfloat16).float()
    toks = O.random_tokens(cfg, 70, 3)
    got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", 40)], [("a", 30)]])["a"]
    want = O.forward(cfg, W, toks)
    assert torch.isfinite(got).all() and rel_err(got, want) < TOL[torch.float32]


def test_elementwise_ops(dev):
    from ipex_llm_amd.ops import seqmix as SM
    g = torch.Generator().manual_seed(5)
    T, Wd = 7, 50
    for dt in (torch.float32, torch.bfloat16):
        tol = 1e-5 if dt == torch.float32 else 2e-2
        y = torch.randn(T, Wd, generator=g).to(dt)
        w = (1 + 0.3 * torch.randn(Wd, generator=g)).to(dt)
        x0 = torch.randn(T, Wd, generator=g)
        x = x0.clone().to(dev)
        xa = SM.add_scaled_layer_norm_(x, y.to(dev), w.to(dev), 1e-3, 0.37, dt)
        want = x0.double() + 0.37 * O.layer_norm(y.double(), w.double(), 1e-3)
        assert x.dtype == torch.float32 and (x.cpu().double() - want).abs().max() < 1e-5
        assert xa.dtype == dt and (xa.cpu().double() - want).abs().max() < tol * 5
        ln = SM.layer_norm_f32(x0.to(dev), w.to(dev), 1e-3, dt)
        assert (ln.cpu().double() - O.layer_norm(x0.double(), w.double(), 1e-3)).abs().max() < tol * 5
        gu = torch.randn(T, 2 * 36, generator=g).to(dt)
        a = SM.glu_gelu(gu.to(dev)).cpu().double()
        assert (a - O.gelu_tanh(gu[:, :36].double()) * gu[:, 36:].double()).abs().max() < tol * 4
        h = torch.randn(T, 3, 20, generator=g)
        nw, gate = (1 + 0.3 * torch.randn(60, generator=g)).to(dt), torch.randn(T, 60, generator=g).to(dt)
        o = SM.head_rms_gate(h.to(dev), nw.to(dev), gate.to(dev), 1e-3, dt).cpu().double()
        want = O.unit_rms(h.double(), 1e-3).reshape(T, 60) * nw.double() * torch.sigmoid(gate.double())
        assert (o - want).abs().max() < tol * 4


def test_bigram_embedding_rows(dev):
    """first token -> the table's last row; others -> the hashed row of (previous, current)"""
    from ipex_llm_amd.ops import seqmix as SM
    cfg = O.config([O.mlstm_layer()], buckets=11, mul_prev=7, mul_cur=3)
    W = O.random_weights(cfg, 4)
    toks = [5, 96, 0, 96, 96, 13]
    ids = torch.tensor(toks, device=dev)
    prev = torch.tensor([-1] + toks[:-1], device=dev)
    x = SM.embed_bigram(ids, prev, W["embed"].to(dev), W["bigram"].to(dev), 7, 3).cpu().double()
    assert (x - O.embed(cfg, {k: v.double() for k, v in W.items()}, toks)).abs().max() < 1e-6
    assert (x[0] - (W["embed"][5] + W["bigram"][11]).double()).abs().max() < 1e-6


# ------------------------------------------------------------------ far keys, page borders
@pytest.mark.parametrize("key_at", [0, 1, 63, 64, 127, 128, 191, 192, 300])
def test_far_key_stands_out(dev, key_at):
    """one key among hundreds matches the query (its score towers over the
    rest): the output must be that key's latent, wherever it lies relative to
    the 64-row pages -- for a query inside a long portion and for a single
    decoded token"""
    from ipex_llm_amd.ops import seqmix as SM
    g = torch.Generator().manual_seed(key_at)
    H, r, dr, bs, L = 3, 20, 6, 64, 333
    rows = 0.1 * torch.randn(8, bs, r + dr, generator=g)
    order = [5, 2, 7, 0, 3, 6]                           # pages in shuffled order
    flat = rows.view(-1, r + dr)
    mark = torch.randn(r + dr, generator=g)
    mark = mark / mark.norm()
    flat[order[key_at // bs] * bs + key_at % bs] = 3.0 * mark
    bt = torch.tensor([order], dtype=torch.int32)
    dense = torch.cat([rows[b] for b in order])[:L].double()
    for qpos in ([L - 1], list(range(L - 40, L))):
        T = len(qpos)
        q = 0.1 * torch.randn(T, H, r + dr, generator=g)
        q[:, 1] += 40.0 * mark                          # head 1 looks for the marked key
        pos = torch.tensor(qpos)
        out = SM.latent_attention(q[..., :r].contiguous().to(dev), q[..., r:].to(dev), rows.to(dev), bt.to(dev),
                                  torch.zeros(T, dtype=torch.int32, device=dev), pos.to(dev), 0.5, None, [T], [L],
                                  torch.float32).cpu().double()
        for i, p in enumerate(qpos):
            s = (dense[:p + 1] @ q[i].double().T) * 0.5                    # [keys, H]
            want = torch.softmax(s, 0).T @ dense[:p + 1, :r]
            assert (out[i] - want).abs().max() < 1e-4
            if key_at <= p:
                assert (out[i, 1] - 3.0 * mark[:r].double()).abs().max() < 1e-3


@pytest.mark.parametrize("H,r,dr", [(3, 20, 6), (16, 512, 64), (9, 72, 8), (16, 96, 32), (1, 4, 2)])
def test_latent_attention_op_bf16(dev, H, r, dr):
    """the 16-bit kernel variant (scores on the matrix cores, f32 softmax and
    weighted sum) on a ragged batch: a short portion of one sequence beside
    single tokens of two others, shuffled pages, gate on"""
    from ipex_llm_amd.ops import seqmix as SM
    g = torch.Generator().manual_seed(H * 1000 + r)
    bs = 64
    rows = (0.5 * torch.randn(12, bs, r + dr, generator=g)).to(torch.bfloat16)
    bt = torch.tensor([[7, 2, 9, 0], [4, 11, 1, 0], [5, 3, 0, 0]], dtype=torch.int32)
    ctx, qn = [200, 130, 70], [9, 1, 1]
    pos = torch.tensor(list(range(191, 200)) + [129, 69])
    seq = torch.tensor([0] * 9 + [1, 2], dtype=torch.int32)
    T = 11
    q = (torch.randn(T, H, r + dr, generator=g) * 0.7).to(torch.bfloat16)
    gate = torch.randn(T, H, generator=g).to(torch.bfloat16)
    out = SM.latent_attention(q[..., :r].contiguous().to(dev), q[..., r:].to(dev), rows.to(dev), bt.to(dev), seq.to(dev),
                              pos.to(dev), 0.11, gate.to(dev), qn, ctx, torch.bfloat16).float().cpu().double()
    for i in range(T):
        b = int(seq[i])
        dense = torch.cat([rows[int(x)] for x in bt[b]])[:int(pos[i]) + 1].double()
        sc = (dense @ q[i].double().T) * 0.11
        want = (torch.softmax(sc, 0).T @ dense[:, :r]) * torch.sigmoid(gate[i].double())[:, None]
        assert (out[i] - want).abs().max() < 6e-3 * max(1.0, float(want.abs().max())), i


@pytest.mark.parametrize("qpos", [62, 63, 64, 65, 127, 128, 129])
def test_causal_edge_at_page_borders(dev, qpos):
    """a towering key one position AFTER the query must not be seen; the same key AT the query must"""
    from ipex_llm_amd.ops import seqmix as SM
    g = torch.Generator().manual_seed(qpos)
    H, r, dr, bs = 2, 10, 4, 64
    rows = 0.1 * torch.randn(4, bs, r + dr, generator=g)
    flat = rows.view(-1, r + dr)
    mark = torch.randn(r + dr, generator=g)
    mark = mark / mark.norm()
    q = (30.0 * mark).repeat(1, H, 1)
    bt = torch.tensor([[0, 1, 2, 3]], dtype=torch.int32)
    for hot, seen in ((qpos + 1, False), (qpos, True)):
        rr = rows.clone()
        rr.view(-1, r + dr)[hot] = 3.0 * mark
        out = SM.latent_attention(q[..., :r].contiguous().to(dev), q[..., r:].to(dev), rr.to(dev), bt.to(dev),
                                  torch.zeros(1, dtype=torch.int32, device=dev), torch.tensor([qpos], device=dev), 1.0,
                                  None, [1], [qpos + 1], torch.float32).cpu()
        close = (out[0, 0] - 3.0 * mark[:r]).abs().max() < 1e-2
        assert bool(close) == seen


# ------------------------------------------------------------------ whole model, schedules
def test_whole_prompt_and_layers(dev):
    cfg = std_cfg()
    W = O.random_weights(cfg, 10)
    toks = O.random_tokens(cfg, 200, 10)
    eng = engine(cfg, W, dev)
    eng.model.capture_layers = []
    got = replay(eng, {"a": toks}, [[("a", 200)]])["a"]
    layers = []
    want = O.forward(cfg, W, toks, layers)
    for a, b in zip(eng.model.capture_layers, layers):
        assert (a.double().cpu() - b).abs().max() < 1e-3 * max(1.0, float(b.abs().max()))
    assert rel_err(got, want) < TOL[torch.float32]


def test_first_tokens(dev):
    """positions 0 and 1: the no-predecessor embedding row, state and running maximum starting at 0"""
    cfg = std_cfg()
    W = O.random_weights(cfg, 11)
    for toks in ([7], [7, 7], [0, 96, 3]):
        got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", 1)]] + [[("a", 1)] for _ in toks[1:]])["a"]
        assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.float32]


def test_prefill_equals_token_by_token(dev):
    cfg = std_cfg()
    W = O.random_weights(cfg, 12)
    toks = O.random_tokens(cfg, 140, 12)
    whole = replay(engine(cfg, W, dev), {"a": toks}, [[("a", 140)]])["a"]
    single = replay(engine(cfg, W, dev), {"a": toks}, [[("a", 1)] for _ in toks])["a"]
    assert rel_err(single, whole) < 1e-4
    assert rel_err(single, O.forward(cfg, W, toks)) < TOL[torch.float32]


@pytest.mark.parametrize("sizes", [[2] * 40, [63, 2, 64, 1, 3, 65], [5, 59, 1, 1, 62, 2, 70], [128, 2, 2, 66]])
def test_portions(dev, sizes):
    """portions cut inside pages, at their borders, down to two tokens"""
    cfg = std_cfg()
    W = O.random_weights(cfg, 13)
    n = sum(sizes)
    toks = O.random_tokens(cfg, n, 13)
    got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", s)] for s in sizes])["a"]
    assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.float32]


def test_unequal_batch_equals_each_alone(dev):
    cfg = std_cfg()
    W = O.random_weights(cfg, 14)
    prompts = {"a": O.random_tokens(cfg, 150, 1), "b": O.random_tokens(cfg, 9, 2), "c": O.random_tokens(cfg, 70, 3),
               "d": O.random_tokens(cfg, 3, 4)}
    schedule = [[("a", 100), ("b", 1), ("c", 2)], [("a", 1), ("b", 1), ("c", 64), ("d", 2)],
                [("b", 7), ("a", 30), ("d", 1)], [("c", 4), ("a", 19)]]
    got = replay(engine(cfg, W, dev), prompts, schedule)
    for name, toks in prompts.items():
        alone = replay(engine(cfg, W, dev), {name: toks}, [[(name, len(toks))]])[name]
        assert rel_err(got[name], alone) < 1e-4, name
        assert rel_err(got[name], O.forward(cfg, W, toks)) < TOL[torch.float32], name


def test_pages_and_slots_used_again(dev):
    """a pool of three pages and two slots serves five requests one after
    another and side by side: what an earlier request left in a page or a
    state slot must not reach a later one"""
    cfg = std_cfg()
    W = O.random_weights(cfg, 15)
    prompts = {k: O.random_tokens(cfg, n, i) for i, (k, n) in enumerate(
        [("a", 120), ("b", 60), ("c", 100), ("d", 64), ("e", 30)])}
    eng = engine(cfg, W, dev, max_batch=2, num_blocks=3)
    schedule = [[("a", 120)], [("b", 30)], [("b", 30), ("c", 50)], [("c", 50)], [("d", 60), ("e", 10)],
                [("d", 4), ("e", 20)]]
    got = replay(eng, prompts, schedule)
    assert int(eng.sched.num_free_blocks()) == 3 and int(eng.sched.num_free_slots()) == 2
    for name, toks in prompts.items():
        assert rel_err(got[name], O.forward(cfg, W, toks)) < TOL[torch.float32], name
    with pytest.raises(RuntimeError):                  # a third live request has no slot
        for _ in range(3):
            eng.open_stream()


def test_long_portions_chunk_parallel(dev, monkeypatch):
    """portions long enough for the chunk-parallel recurrence and the
    library-product attention (on the GPU), cut so that both leave remainders,
    beside a short request in the same steps"""
    from ipex_llm_amd.ops import seqmix as SM
    monkeypatch.setattr(SM, "MLSTM_CHUNK_MIN", 256)
    cfg = std_cfg()
    W = O.random_weights(cfg, 25)
    prompts = {"a": O.random_tokens(cfg, 700, 25), "b": O.random_tokens(cfg, 9, 26)}
    got = replay(engine(cfg, W, dev, num_blocks=16), prompts,
                 [[("a", 300), ("b", 3)], [("a", 390), ("b", 1)], [("a", 10), ("b", 5)]])
    for name, toks in prompts.items():
        assert rel_err(got[name], O.forward(cfg, W, toks)) < TOL[torch.float32], name


def test_long_decoding(dev):
    """a short prompt, then 200 tokens one by one across three page borders"""
    cfg = std_cfg()
    W = O.random_weights(cfg, 16)
    toks = O.random_tokens(cfg, 215, 16)
    got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", 15)]] + [[("a", 1)]] * 200)["a"]
    want = O.forward(cfg, W, toks)
    assert rel_err(got[-20:], want[-20:]) < TOL[torch.float32]
    assert rel_err(got, want) < TOL[torch.float32]


def test_bfloat16_serving_precision(dev):
    """16-bit projections, f32 residual / norms / scores / state: close to the
    exact forward, and chunking changes it only by rounding"""
    cfg = std_cfg()
    W = O.random_weights(cfg, 17)
    toks = O.random_tokens(cfg, 130, 17)
    want = O.forward(cfg, W, toks)
    whole = replay(engine(cfg, W, dev, torch.bfloat16), {"a": toks}, [[("a", 130)]])["a"]
    parts = replay(engine(cfg, W, dev, torch.bfloat16), {"a": toks}, [[("a", 66)], [("a", 2)]] + [[("a", 1)]] * 62)["a"]
    assert rel_err(whole, want) < TOL[torch.bfloat16]
    assert rel_err(parts, want) < TOL[torch.bfloat16]


def test_other_sizes_and_orders(dev):
    """attention only, recurrence only, sizes that are 1, equal sizes"""
    for layers in ([O.attn_layer(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=8, ff=16)] * 2,
                   [O.mlstm_layer(heads=1, dim=1, vdim=1, ff=8), O.mlstm_layer(heads=4, dim=2, vdim=3)],
                   [O.attn_layer(heads=1, dim=2, rot_dim=2, vdim=1, kv_rank=3, ff=0), O.mlstm_layer(ff=24),
                    O.attn_layer(ff=8)]):
        cfg = O.config(layers, vocab=31, width=24, eps=1e-6, mult=1.0, buckets=1, mul_prev=1, mul_cur=1)
        W = O.random_weights(cfg, 18)
        toks = O.random_tokens(cfg, 80, 18)
        got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", 70)]] + [[("a", 1)]] * 10)["a"]
        assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.float32]


ODD = [
    # sizes that are not multiples of 4 (no aligned chunks anywhere), partial rotation
    ([O.attn_layer(heads=5, dim=6, rot_dim=6, vdim=10, kv_rank=13, dims=4, ff=20), O.mlstm_layer(heads=3, dim=5, vdim=7)], 36),
    # > 16 heads, latent rank past 256, key size 256 in the recurrence
    ([O.attn_layer(heads=20, dim=16, rot_dim=16, vdim=16, kv_rank=300, ff=0, scaling=YARN),
      O.mlstm_layer(heads=2, dim=256, vdim=64, gate_cap=8.0, ff=32)], 64),
    # past what the flash kernel and the register-resident scan hold: the paths without size limits
    ([O.attn_layer(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=520, ff=0), O.mlstm_layer(heads=1, dim=260, vdim=8)], 32),
    # 16 heads with a small latent, key size that pads to the next wave slice
    ([O.mlstm_layer(heads=2, dim=100, vdim=36, ff=0), O.attn_layer(heads=16, dim=32, rot_dim=32, vdim=32, kv_rank=96, ff=40)], 48),
]


@pytest.mark.parametrize("case", range(len(ODD)))
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_odd_and_large_sizes(dev, case, dtype):
    """a long portion (the library-product path of the attention on the GPU),
    a short one, then single tokens -- in both number formats"""
    layers, width = ODD[case]
    cfg = O.config(layers, vocab=61, width=width, eps=1e-6, mult=0.7, buckets=17, mul_prev=3, mul_cur=11)
    W = O.random_weights(cfg, 30 + case)
    toks = O.random_tokens(cfg, 170, 30 + case)
    got = replay(engine(cfg, W, dev, dtype), {"a": toks}, [[("a", 140)], [("a", 20)]] + [[("a", 1)]] * 10)["a"]
    assert rel_err(got, O.forward(cfg, W, toks)) < TOL[dtype]


# ------------------------------------------------------------------ generation through the scheduler
def test_greedy_generation_scheduler(dev):
    """LLMEngine.generate: C++ scheduler, chunked prompts (7 tokens a step in
    all), requests of unequal length side by side, greedy sampling"""
    from ipex_llm_amd.serving.engine import SamplingParams
    cfg = std_cfg()
    W = O.random_weights(cfg, 19)
    prompts = [O.random_tokens(cfg, n, 20 + n) for n in (23, 3, 70, 11)]
    want = [O.greedy(cfg, W, p, 6) for p in prompts]
    for prefill, batch in ((7, 4), (1 << 30, 2)):
        eng = engine(cfg, W, dev, max_batch=batch, num_blocks=8, prefill=prefill)
        got = eng.generate(prompts, SamplingParams(max_new_tokens=6))
        assert got == want
        assert int(eng.sched.num_free_blocks()) == 8 and int(eng.sched.num_free_slots()) == batch


def test_generation_survives_preemption(dev):
    """a pool too small for all requests at once: the scheduler preempts and
    recomputes; the generated tokens do not change"""
    from ipex_llm_amd.serving.engine import SamplingParams
    cfg = std_cfg()
    W = O.random_weights(cfg, 21)
    prompts = [O.random_tokens(cfg, n, 30 + n) for n in (60, 62, 61)]
    want = [O.greedy(cfg, W, p, 8) for p in prompts]
    eng = engine(cfg, W, dev, max_batch=3, num_blocks=4, prefill=1 << 30)
    assert eng.generate(prompts, SamplingParams(max_new_tokens=8)) == want
    assert eng.stats["preemptions"] >= 1


@pytest.mark.gpu
def test_decode_graph_replays_equal_eager():
    """pure-decode steps replayed from a captured graph (padded batch bucket,
    scratch block and slot for the padding rows), with eager prefill steps and
    synchronisations between the replays: every replay equals the eager step"""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from ipex_llm_amd.serving.engine import LLMEngine
    dev = torch.device("cuda")
    cfg = std_cfg()
    W = O.random_weights(cfg, 24)
    prompts = {"a": O.random_tokens(cfg, 90, 1), "b": O.random_tokens(cfg, 40, 2), "c": O.random_tokens(cfg, 75, 3)}
    schedule = [[("a", 60), ("b", 20)], [("a", 1), ("b", 1)], [("a", 1), ("b", 1), ("c", 70)]] + \
        [[("a", 1), ("b", 1), ("c", 1)]] * 5 + [[("a", 23), ("b", 1)]] + [[("b", 1)]] * 12
    got = {}
    for graph in (False, True):
        eng = LLMEngine(build(cfg, W, dev, torch.float32), max_batch=4, block_size=64, num_blocks=12,
                        max_model_len=512, max_prefill_tokens=1 << 30, use_graph=graph, enable_prefix_caching=False)
        got[graph] = replay(eng, prompts, schedule)
        assert bool(eng._graphs) == graph
    for name, toks in prompts.items():
        n = got[True][name].shape[0]
        assert rel_err(got[True][name], got[False][name]) < 1e-4, name
        assert rel_err(got[True][name], O.forward(cfg, W, toks)[:n]) < TOL[torch.float32], name


# ------------------------------------------------------------------ checkpoint reader, registry, trace replay
def write_checkpoint(path, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))


def test_checkpoint_registry_and_generate(tmp_path):
    from ipex_llm_amd.models.registry import native_architecture
    from ipex_llm_amd.transformers import AutoModelForCausalLM
    cfg = std_cfg()
    W = O.random_weights(cfg, 22)
    write_checkpoint(str(tmp_path / "m"), cfg, W)
    assert native_architecture(str(tmp_path / "m")) == "Zamelix"
    assert native_architecture(str(tmp_path)) is None
    model = AutoModelForCausalLM.from_pretrained(str(tmp_path / "m"), torch_dtype=torch.float32)
    prompt = O.random_tokens(cfg, 12, 22)
    out = model.generate(torch.tensor([prompt]), max_new_tokens=5)
    assert out[0].tolist() == prompt + O.greedy(cfg, W, prompt, 5)
    bad = dict(cfg, width=cfg["width"] + 1)
    write_checkpoint(str(tmp_path / "bad"), bad, W)
    with pytest.raises(ValueError):
        AutoModelForCausalLM.from_pretrained(str(tmp_path / "bad"))


def test_trace_replay_program(tmp_path, dev):
    """bin/trace_run: steps on stdin, logits files, 'done' lines, requests ended and pages used again"""
    cfg = std_cfg()
    W = O.random_weights(cfg, 23)
    write_checkpoint(str(tmp_path / "m"), cfg, W)
    a, b = O.random_tokens(cfg, 100, 1), O.random_tokens(cfg, 66, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:70], "want": [0, 69]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[70:99], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[99:], "want": [0]}], "end": ["a"]},
             {"step": 3, "entries": [{"id": "b", "tokens": b[:2], "want": [1]}], "end": []},
             {"step": 4, "entries": [{"id": "b", "tokens": b[2:], "want": [63]}], "end": ["b"]}]
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(tmp_path / "m"), "--dtype",
                        "float32", "--out", str(out), "--max-tokens", "128", "--device", dev.type],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(5)]
    assert not (out / "1.f32").exists()
    wa, wb = O.forward(cfg, W, a), O.forward(cfg, W, b)
    import numpy as np
    V = cfg["vocab"]

    def rd(i):
        return torch.from_numpy(np.fromfile(str(out / f"{i}.f32"), dtype="<f4").reshape(-1, V).copy()).double()
    assert rel_err(rd(0), wa[[0, 69]]) < TOL[torch.float32]
    assert rel_err(rd(2), wa[[99]]) < TOL[torch.float32]
    assert rel_err(rd(3), wb[[1]]) < TOL[torch.float32]
    assert rel_err(rd(4), wb[[65]]) < TOL[torch.float32]
