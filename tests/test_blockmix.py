"""Parallel-residual decoders (Masezen layout): the framework -- checkpoint
reader, paged [keys | values] rows and convolution state slots, scheduler,
ragged engine steps, kernels -- against the plain float64 forms of
tests/blockmix_oracle.py.

Every test runs on the CPU (torch forms of ops/blockmix.py) and, marked
``gpu``, on the HIP kernels.  Models are small random ones made here.
"""
import json
import os
import subprocess
import sys

import pytest
import torch

from . import blockmix_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEVS = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
YARN = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 2.0}
F64 = torch.float64


@pytest.fixture(params=DEVS)
def dev(request):
    if request.param == "cuda":
        if not torch.cuda.is_available():
            pytest.skip("no GPU")
        import ipex_llm_amd.ops as ops
        ops.require_seqmix()
    return torch.device(request.param)


def std_cfg():
    """attention alone, beside a dense feed-forward, beside experts with a
    shared one (top 2), beside experts without (top 1); YaRN on one layer,
    partial rotation on another, one and several key / value heads"""
    return O.config([O.attn_layer(heads=4, kv_heads=2, dim=16, scaling=YARN, mlp=O.dense(40)),
                     O.attn_layer(heads=6, kv_heads=2, dim=8, dims=4, scale=0.4, mlp=O.moe(5, 2, 24, 1.5, 16, 0.8)),
                     O.attn_layer(heads=3, kv_heads=1, dim=24, dims=16, base=300.0, mlp=None),
                     O.attn_layer(heads=2, kv_heads=2, dim=32, mlp=O.moe(3, 1, 32, 2.5))], width=40, taps=3, side=6)


def build(cfg, W, dev, dtype=torch.float32):
    from ipex_llm_amd.models import masezen as Z
    return Z.build(Z.spec_from_config(cfg), W, dtype, dev)


def engine(cfg, W, dev, dtype=torch.float32, max_batch=4, num_blocks=16, prefill=1 << 30, graph=False):
    from ipex_llm_amd.serving.engine import LLMEngine
    return LLMEngine(build(cfg, W, dev, dtype), max_batch=max_batch, block_size=64, num_blocks=num_blocks,
                     max_model_len=num_blocks * 64, max_prefill_tokens=prefill, use_graph=graph,
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


def clear_tokens(cfg, W, n, seed):
    """random tokens whose router choices are not close calls (a tie decided in the last bits would
    compare rounding, not the mechanism)"""
    for s in range(seed, seed + 4000, 100):
        toks = O.random_tokens(cfg, n, s)
        if O.router_margin(cfg, W, toks) > 3e-5:
            return toks
    raise AssertionError("no prompt without a close router call")


def greedy(cfg, W, prompt, n):
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(O.forward(cfg, W, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out


TOL = {torch.float32: 2e-4, torch.bfloat16: 0.12}


# ------------------------------------------------------------------ mechanisms alone (ops)
def test_norms_and_elementwise(dev):
    from ipex_llm_amd.ops import blockmix as BM
    g = torch.Generator().manual_seed(0)
    T, Wd = 9, 70
    x = torch.randn(T, Wd, generator=g) * 3
    for w in (torch.tensor([1.3]), 1 + 0.2 * torch.randn(Wd, generator=g)):
        h, ha = BM.rms_norm_rows(x.to(dev), w.to(dev), 1e-5, torch.float32)
        assert (h.cpu().double() - O.unit_rms(x.double(), 1e-5) * w.double()).abs().max() < 1e-5 and ha is h
        _, hb = BM.rms_norm_rows(x.to(dev), w.to(dev).bfloat16(), 1e-5, torch.bfloat16)
        assert hb.dtype == torch.bfloat16
        assert (hb.cpu().double() - O.unit_rms(x.double(), 1e-5) * w.bfloat16().double()).abs().max() < 0.05
    y = torch.randn(T, Wd, generator=g)
    w = 0.5 + torch.rand(Wd, generator=g)
    xr = x.clone().to(dev)
    BM.add_rms_norm_(xr, y.to(dev), w.to(dev), 1e-5, torch.float32)
    assert (xr.cpu().double() - (x.double() + O.unit_rms(y.double(), 1e-5) * w.double())).abs().max() < 1e-5
    y2, y3 = torch.randn(T, Wd, generator=g), torch.randn(T, Wd, generator=g)
    s1, s2 = torch.rand(Wd, generator=g), torch.rand(Wd, generator=g)
    want = x.double() + y.double() * s1.double() + (y2.double() + y3.double()) * s2.double()
    xr = x.clone().to(dev)
    BM.residual_add_scaled_(xr, y.to(dev), s1.to(dev), y2.to(dev), y3.to(dev), s2.to(dev), torch.float32)
    assert (xr.cpu().double() - want).abs().max() < 1e-5
    xr = x.clone().to(dev)
    xa = BM.residual_add_scaled_(xr, y.to(dev).bfloat16(), None, y2.to(dev), None, s2.to(dev), torch.bfloat16)
    want = x.double() + y.bfloat16().double() + y2.double() * s2.double()
    assert (xr.cpu().double() - want).abs().max() < 1e-5 and xa.dtype == torch.bfloat16
    gu = torch.randn(T, 2 * 22, generator=g) * 3
    gg, uu = gu[:, :22].double().clamp(max=1.2), gu[:, 22:].double().clamp(-1.2, 1.2)
    assert (BM.glu_clamp(gu.to(dev), 1.2, 1.702).cpu().double() - gg * torch.sigmoid(1.702 * gg) * (uu + 1)).abs().max() < 1e-5
    assert (BM.relu_sq(gu.to(dev)).cpu().double() - torch.relu(gu.double()) ** 2).abs().max() < 1e-5
    table = torch.randn(31, 40, generator=g)
    ids = torch.randint(0, 31, (T,), generator=g)
    z = torch.randn(T, 7, generator=g)
    want = O.gelu_tanh(z.double()) * table.double()[ids][:, 14:21]
    assert (BM.side_gate(z.to(dev), table.to(dev), ids.to(dev), 14).cpu().double() - want).abs().max() < 1e-5


@pytest.mark.parametrize("taps", [2, 3, 5])
def test_canon_convolution_state(dev, taps):
    """two sequences fed in portions of unequal sizes (down to one token, shorter than the taps) through
    state slots that held something else before: equal to the convolution of each whole sequence"""
    from ipex_llm_amd.ops import blockmix as BM
    g = torch.Generator().manual_seed(taps)
    Wd, na, nb = 33, 23, 14
    ha, hb = torch.randn(na, Wd, generator=g), torch.randn(nb, Wd, generator=g)
    w = torch.randn(Wd, taps, generator=g)
    state = torch.randn(4, taps - 1, Wd, generator=g).to(dev) * 50            # garbage of earlier owners
    got_a, got_b = [], []
    plan = [(5, 1), (1, 1), (1, 3), (7, 2), (2, 1), (1, 1), (6, 5)]
    ia = ib = 0
    for ca, cb in plan:
        h = torch.cat([ha[ia:ia + ca], hb[ib:ib + cb]]).to(dev)
        cu = torch.tensor([0, ca, ca + cb], dtype=torch.int32, device=dev)
        seq_of = torch.tensor([0] * ca + [1] * cb, dtype=torch.int32, device=dev)
        pos = torch.tensor(list(range(ia, ia + ca)) + list(range(ib, ib + cb)), device=dev)
        out = BM.canon_conv(h, w.to(dev), state, cu, seq_of, torch.tensor([2, 0], dtype=torch.int32, device=dev), pos,
                            [ca, cb], torch.float32).cpu()
        got_a.append(out[:ca])
        got_b.append(out[ca:])
        ia, ib = ia + ca, ib + cb
    assert ia == na and ib == nb
    assert (torch.cat(got_a).double() - O.canon(ha.double(), w.double())).abs().max() < 1e-5
    assert (torch.cat(got_b).double() - O.canon(hb.double(), w.double())).abs().max() < 1e-5


@pytest.mark.parametrize("taps", [2, 4])
def test_norm_and_convolution_in_one(dev, taps):
    """the norm and the convolution as one op: mixed steps and steps in which both sequences bring one token
    (the state then advances inside the same launch), one number and a vector as norm weight"""
    from ipex_llm_amd.ops import blockmix as BM
    g = torch.Generator().manual_seed(10 + taps)
    Wd, na, nb = 21, 17, 12
    xa_, xb_ = torch.randn(na, Wd, generator=g) * 2, torch.randn(nb, Wd, generator=g) * 2
    w = torch.randn(Wd, taps, generator=g)
    for nw in (torch.tensor([0.8]), 1 + 0.2 * torch.randn(Wd, generator=g)):
        state = torch.randn(3, taps - 1, Wd, generator=g).to(dev) * 50
        outs_a, outs_b, hs = [], [], []
        plan = [(4, 1), (1, 1), (1, 1), (1, 3), (6, 2), (1, 1), (3, 3)]
        ia = ib = 0
        for ca, cb in plan:
            x = torch.cat([xa_[ia:ia + ca], xb_[ib:ib + cb]]).to(dev)
            cu = torch.tensor([0, ca, ca + cb], dtype=torch.int32, device=dev)
            seq_of = torch.tensor([0] * ca + [1] * cb, dtype=torch.int32, device=dev)
            pos = torch.tensor(list(range(ia, ia + ca)) + list(range(ib, ib + cb)), device=dev)
            h, ha, out = BM.norm_canon(x, nw.to(dev), 1e-5, w.to(dev), state, cu, seq_of,
                                       torch.tensor([1, 2], dtype=torch.int32, device=dev), pos, [ca, cb], torch.float32)
            assert ha is h
            outs_a.append(out[:ca].cpu())
            outs_b.append(out[ca:].cpu())
            hs.append(h[:ca].cpu())
            ia, ib = ia + ca, ib + cb
        assert ia == na and ib == nb
        ha64, hb64 = O.unit_rms(xa_.double(), 1e-5) * nw.double(), O.unit_rms(xb_.double(), 1e-5) * nw.double()
        assert (torch.cat(hs).double() - ha64).abs().max() < 1e-5
        assert (torch.cat(outs_a).double() - O.canon(ha64, w.double())).abs().max() < 2e-5
        assert (torch.cat(outs_b).double() - O.canon(hb64, w.double())).abs().max() < 2e-5


def plain_mixed_attention(q, k, v, talk, scale, positions):
    """q [n, H, d] at ``positions``; k, v [L, G, d] -> [n, H, d] (f64)"""
    n, H, d = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, d, dtype=F64)
    for t in range(n):
        L = positions[t] + 1
        s = torch.stack([(k[:L, h // (H // G)] @ q[t, h]) * scale for h in range(H)])
        pr = torch.softmax(talk @ s, -1)
        for h in range(H):
            out[t, h] = pr[h] @ v[:L, h // (H // G)]
    return out


def paged_rows(k, v, dev, dtype, bs=64, spare=3, seed=0):
    """[keys | values] rows of one sequence scattered over shuffled pages"""
    L, G, d = k.shape
    nb = (L + bs - 1) // bs
    perm = torch.randperm(nb + spare, generator=torch.Generator().manual_seed(seed))[:nb]
    rows = torch.randn(nb + spare + 1, bs, 2 * G * d, generator=torch.Generator().manual_seed(seed + 1)) * 30
    flat = torch.cat([k.reshape(L, G * d), v.reshape(L, G * d)], -1).float()
    for i in range(nb):
        part = flat[i * bs:(i + 1) * bs]
        rows[perm[i], :part.shape[0]] = part
    return rows.to(dev, dtype), perm.to(torch.int32)[None].to(dev)


@pytest.mark.parametrize("H,G,d", [(4, 2, 16), (8, 2, 64), (6, 6, 8), (5, 1, 24), (16, 4, 32), (3, 3, 128), (12, 1, 20),
                                   (2, 2, 12)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mixed_score_attention_op(dev, H, G, d, dtype):
    """decoded tokens and short portions over shuffled pages, keys past 200, with and without the mixing matrix"""
    from ipex_llm_amd.ops import blockmix as BM
    g = torch.Generator().manual_seed(H * 100 + d)
    L, n = 203, 5
    k = torch.randn(L, G, d, generator=g).to(dtype)
    v = torch.randn(L, G, d, generator=g).to(dtype)
    q = torch.randn(n, H, d, generator=g)
    talk = torch.eye(H) + 0.4 * torch.randn(H, H, generator=g)
    gate = torch.randn(n, H * d, generator=g).to(dtype)
    rows, bt = paged_rows(k, v, dev, dtype, seed=H)
    positions = list(range(L - n, L))
    for tk in (talk, None):
        got = BM.talk_attention(q.to(dev), rows, bt, torch.zeros(n, dtype=torch.int32, device=dev),
                                torch.tensor(positions, device=dev), 0.3, None if tk is None else tk.to(dev),
                                gate.to(dev), G, [n], [L], dtype).cpu().double()
        want = plain_mixed_attention(q.double(), k.double(), v.double(), (tk if tk is not None else torch.eye(H)).double(),
                                     0.3, positions).reshape(n, H * d) * torch.sigmoid(gate.double())
        assert (got - want).abs().max() < (2e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("key_at", [0, 1, 63, 64, 127, 128, 191, 192, 300, 511, 512])
def test_far_key_stands_out(dev, key_at):
    """one key among hundreds matches the query of one head strongly, at page borders and far back; the mixing
    matrix carries that score to the other heads; in a long portion and for a decoded token"""
    from ipex_llm_amd.ops import blockmix as BM
    g = torch.Generator().manual_seed(key_at)
    H, G, d, L = 4, 2, 16, 600
    k = torch.randn(L, G, d, generator=g) * 0.3
    v = torch.randn(L, G, d, generator=g)
    q = torch.randn(L, H, d, generator=g) * 0.3
    k[key_at, 1] = 0.0
    k[key_at, 1, 3] = 6.0
    q[:, 2] = 0.0
    q[:, 2, 3] = 5.0                                 # head 2 (kv head 1) finds it
    talk = torch.eye(H)
    talk[0, 2] = 0.8                                 # and head 0 hears of it
    rows, bt = paged_rows(k, v, dev, torch.float32, seed=key_at)
    want_all = plain_mixed_attention(q.double(), k.double(), v.double(), talk.double(), 1.0, list(range(L)))
    assert (want_all[L - 1, 2] - v[key_at, 1].double()).abs().max() < 1e-3       # the test's premise
    for positions in (list(range(L - 150, L)), [L - 1], list(range(max(key_at - 1, 0), min(key_at + 3, L)))):
        n = len(positions)
        got = BM.talk_attention(q[positions].to(dev), rows, bt, torch.zeros(n, dtype=torch.int32, device=dev),
                                torch.tensor(positions, device=dev), 1.0, talk.to(dev), None, G, [n], [positions[-1] + 1],
                                torch.float32).cpu().double()
        assert (got - want_all[positions].reshape(n, H * d)).abs().max() < 2e-5


@pytest.mark.parametrize("edge", [1, 62, 63, 64, 65, 127, 128, 129])
def test_causal_edge(dev, edge):
    """a towering key at position ``edge``: the query just before must not see it, the query at it must;
    inside a portion (the key is already in the cache when the earlier query runs) and token by token"""
    from ipex_llm_amd.ops import blockmix as BM
    g = torch.Generator().manual_seed(edge)
    H, G, d, L = 2, 1, 8, edge + 3
    k = torch.randn(L, G, d, generator=g) * 0.2
    v = torch.randn(L, G, d, generator=g)
    q = torch.randn(L, H, d, generator=g) * 0.2
    k[edge, 0, 0] = 8.0
    q[:, :, 0] = 4.0
    rows, bt = paged_rows(k, v, dev, torch.float32, seed=edge)
    want = plain_mixed_attention(q.double(), k.double(), v.double(), torch.eye(H, dtype=F64), 1.0, list(range(L)))
    assert (want[edge - 1] - want[edge]).abs().max() > 0.05
    for positions in (list(range(L)), [edge - 1], [edge], [edge + 1]):
        n = len(positions)
        got = BM.talk_attention(q[positions].to(dev), rows, bt, torch.zeros(n, dtype=torch.int32, device=dev),
                                torch.tensor(positions, device=dev), 1.0, None, None, G, [n], [L],
                                torch.float32).cpu().double()
        assert (got - want[positions].reshape(n, H * d)).abs().max() < 2e-5


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d", [(8, 2, 64), (16, 4, 128), (4, 4, 64), (8, 1, 128), (16, 2, 64), (4, 1, 128), (6, 3, 40),
                                   (5, 5, 16), (12, 1, 20), (3, 3, 12)])
@pytest.mark.parametrize("L,n", [(700, 633), (2300, 1101)])
def test_long_portion_paths_agree(H, G, d, dtype, L, n):
    """portions past the thresholds take the matrix-core kernel (16-bit, its sizes) or library products with the
    fused mixing softmax between them; the same rows through the one-pass kernel give the same result.  The
    portion starts inside a page, ends inside a 16-token tile and shares the step with a decoded token."""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from ipex_llm_amd.ops import blockmix as BM
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(d)
    if L > 1000 and (dtype == torch.float32 or d % 64):
        pytest.skip("the long case is for the matrix-core kernel's key splits")
    # the portion starts inside a page, 67 (1199) tokens into the sequence; past 2048 keys the kernel splits them
    k, v = torch.randn(L, G, d, generator=g).to(dtype), torch.randn(L, G, d, generator=g).to(dtype)
    q = torch.randn(n + 1, H, d, generator=g)
    talk = torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)
    gate = torch.randn(n + 1, H * d, generator=g).to(dtype)
    rows, bt = paged_rows(k, v, dev, dtype, seed=d)
    bt = torch.cat([bt, bt])                          # a second sequence over the same pages brings one token
    positions = list(range(L - n, L)) + [L - 5]
    seq_of = torch.tensor([0] * n + [1], dtype=torch.int32, device=dev)
    args = (q.to(dev), rows, bt, seq_of, torch.tensor(positions, device=dev), 0.25, talk.to(dev), gate.to(dev), G,
            [n, 1], [L, L - 4], dtype)
    want = plain_mixed_attention(q.double(), k.double(), v.double(), talk.double(), 0.25, positions).reshape(n + 1, H * d) * \
        torch.sigmoid(gate.double())
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    old = BM.GEMM_MIN_Q, BM.MFMA_MIN_Q
    try:
        for gemm_min, mfma_min in ((old,) if L > 1000 else (old, (128, 0), (1 << 30, 0))):
            BM.GEMM_MIN_Q, BM.MFMA_MIN_Q = gemm_min, mfma_min
            got = BM.talk_attention(*args).cpu().double()
            assert (got - want).abs().max() < tol, (gemm_min, mfma_min)
    finally:
        BM.GEMM_MIN_Q, BM.MFMA_MIN_Q = old


def test_qk_norm_rotation_and_rows(dev):
    """per-head norm, half-split rotation of part of the head with YaRN, and what lands in the cache rows"""
    from ipex_llm_amd.ops import blockmix as BM
    from ipex_llm_amd.ops.seqmix import rope_table
    g = torch.Generator().manual_seed(5)
    T, H, G, d = 7, 3, 2, 12
    rot = {"dims": 8, "base": 100.0, "scaling": YARN}
    y = torch.randn(T, (H + G) * d + 5, generator=g)
    q, k = y[:, :H * d].view(T, H, d), y[:, H * d:(H + G) * d].view(T, G, d)
    qn, kn = 1 + 0.3 * torch.randn(d, generator=g), 1 + 0.3 * torch.randn(d, generator=g)
    positions = [0, 1, 2, 70, 71, 130, 5]
    slots = torch.tensor([3, 64, 65, 130, 2, 190, 7])
    rows = torch.zeros(4, 64, 2 * G * d)
    table = rope_table(256, rot["dims"], rot["base"], rot["scaling"])
    yd = y.to(dev)
    qd, kd = yd[:, :H * d].view(T, H, d), yd[:, H * d:(H + G) * d].view(T, G, d)
    rows_d = rows.to(dev)
    qo = BM.qk_norm_rope_store(qd, kd, qn.to(dev), kn.to(dev), 1e-5, table.to(dev), torch.tensor(positions, device=dev),
                               slots.to(dev), rows_d).cpu().double()
    wq = O.rotate_half(O.unit_rms(q.double(), 1e-5) * qn.double(), rot, positions)
    wk = O.rotate_half(O.unit_rms(k.double(), 1e-5) * kn.double(), rot, positions)
    assert (qo - wq).abs().max() < 1e-5
    flat = rows_d.cpu().double().view(-1, 2 * G * d)
    assert (flat[slots][:, :G * d] - wk.reshape(T, G * d)).abs().max() < 1e-5
    assert (flat[slots][:, G * d:] - k.double().reshape(T, G * d)).abs().max() == 0
    # the part past rot.dims passes unrotated; YaRN changes the angles
    assert (qo[..., 8:] - (O.unit_rms(q.double(), 1e-5) * qn.double())[..., 8:]).abs().max() < 1e-5
    plain = O.rotate_half(O.unit_rms(q.double(), 1e-5) * qn.double(), {"dims": 8, "base": 100.0}, positions)
    assert (plain - wq).abs().max() > 0.05


def test_router_and_experts(dev):
    """the largest sigmoid scores win (lowest index among equals), their scores weigh the experts' inputs"""
    from ipex_llm_amd.ops import blockmix as BM
    g = torch.Generator().manual_seed(3)
    T, E, Wd, ff, top = 37, 7, 24, 20, 3
    z = torch.randn(T, E, generator=g) * 2
    z[0] = 0.5                                        # all equal: experts 0, 1, 2
    z[1, 4] = z[1, 2] = 3.0                           # two equal at the top: 2 before 4
    idx, w = BM.moe_route(z.to(dev), top)
    s = torch.sigmoid(z.double())
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-float(s[t, e]), e))[:top]
        assert idx[t].tolist() == order
        assert (w[t].cpu().double() - s[t, order]).abs().max() < 1e-6
    h = torch.randn(T, Wd, generator=g)
    Wt = {}
    for e in range(E):
        Wt[f"e{e}.gate"], Wt[f"e{e}.up"] = torch.randn(ff, Wd, generator=g) * 0.5, torch.randn(ff, Wd, generator=g) * 0.5
        Wt[f"e{e}.down"] = torch.randn(Wd, ff, generator=g) * 0.3
    w_gu = torch.stack([torch.cat([Wt[f"e{e}.gate"], Wt[f"e{e}.up"]]) for e in range(E)])
    w_down = torch.stack([Wt[f"e{e}.down"] for e in range(E)])
    got = BM.moe_experts(h.to(dev), idx, w, w_gu.to(dev), w_down.to(dev), 1.5, 1.702).cpu().double()
    W64 = {k: v.double() for k, v in Wt.items()}
    want = torch.zeros(T, Wd, dtype=F64)
    for t in range(T):
        for j in range(top):
            e = int(idx[t, j])
            want[t] += O.expert(W64, f"e{e}.", float(w[t, j]) * h[t].double(), 1.5)
    assert (got - want).abs().max() < 1e-4
    # the weight is inside the expert: scaling the output instead gives something else
    outside = sum(float(w[5, j]) * O.expert(W64, f"e{int(idx[5, j])}.", h[5].double(), 1.5) for j in range(top))
    assert (outside - want[5]).abs().max() > 1e-3


# ------------------------------------------------------------------ whole models through the engine
LAYER_CASES = [
    ([O.attn_layer(heads=4, kv_heads=2, dim=16, mlp=None)], dict(width=32, taps=0, side=0)),
    ([O.attn_layer(heads=4, kv_heads=4, dim=8, dims=6, scaling=YARN, mlp=O.dense(50))], dict(width=24, taps=2, side=0)),
    ([O.attn_layer(heads=6, kv_heads=1, dim=16, dims=8, mlp=O.moe(6, 2, 16, 1.0, 24, 3.0))], dict(width=40, taps=4, side=5)),
    ([O.attn_layer(heads=2, kv_heads=1, dim=40, mlp=O.moe(4, 4, 8, 2.0))], dict(width=16, taps=3, side=3)),
    ([O.attn_layer(heads=1, kv_heads=1, dim=8, mlp=O.moe(2, 1, 8, 0.5, 8, 0.5))], dict(width=8, taps=1, side=1)),
    # head sizes that are no multiple of 8 and more than 8 query heads per key / value head: no one-pass kernel
    ([O.attn_layer(heads=5, kv_heads=5, dim=12, dims=6, mlp=O.moe(3, 2, 12, 2.0, 20, 1.0))], dict(width=20, taps=3, side=2)),
    ([O.attn_layer(heads=12, kv_heads=1, dim=20, scaling=YARN, mlp=O.dense(36))], dict(width=36, taps=2, side=0)),
    # no rotated part at all
    ([O.attn_layer(heads=2, kv_heads=1, dim=16, dims=0, mlp=O.dense(24))], dict(width=24, taps=3, side=4)),
]


@pytest.mark.parametrize("case", [2, 5, 6])
def test_one_layer_models_bf16(dev, case):
    """16-bit serving of odd sizes: decoded tokens and portions through whatever path the sizes allow"""
    layers, kw = LAYER_CASES[case]
    cfg = O.config(layers, **kw)
    W = O.random_weights(cfg, case)
    seed = max(range(40), key=lambda s: O.router_margin(cfg, W, O.random_tokens(cfg, 80, s)))
    toks = O.random_tokens(cfg, 80, seed)
    got = replay(engine(cfg, W, dev, torch.bfloat16), {"a": toks}, [[("a", 70)], [("a", 3)]] + [[("a", 1)]] * 7)["a"]
    assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.bfloat16]


@pytest.mark.parametrize("case", range(len(LAYER_CASES)))
def test_one_layer_models(dev, case):
    layers, kw = LAYER_CASES[case]
    cfg = O.config(layers, **kw)
    W = O.random_weights(cfg, case)
    toks = clear_tokens(cfg, W, 150, case)
    got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", 150)]])["a"]
    assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.float32]


def test_whole_prompt_and_layers(dev):
    cfg = std_cfg()
    W = O.random_weights(cfg, 7)
    toks = clear_tokens(cfg, W, 131, 7)
    eng = engine(cfg, W, dev)
    eng.model.capture_layers = []
    got = replay(eng, {"a": toks}, [[("a", 131)]])["a"]
    layers = []
    want = O.forward(cfg, W, toks, layers_out=layers)
    assert rel_err(got, want) < TOL[torch.float32]
    assert len(eng.model.capture_layers) == len(layers)
    for a, b in zip(eng.model.capture_layers, layers):
        assert (a.double().cpu() - b).abs().max() < 1e-3 * float(b.abs().max())


def test_first_tokens(dev):
    """sequences of one, two and three tokens (shorter than the convolution), each alone and decoded one by one"""
    cfg = std_cfg()
    W = O.random_weights(cfg, 8)
    for n in (1, 2, 3):
        toks = clear_tokens(cfg, W, n, n)
        want = O.forward(cfg, W, toks)
        assert rel_err(replay(engine(cfg, W, dev), {"a": toks}, [[("a", n)]])["a"], want) < TOL[torch.float32]
        assert rel_err(replay(engine(cfg, W, dev), {"a": toks}, [[("a", 1)]] * n)["a"], want) < TOL[torch.float32]


def test_prefill_equals_token_by_token(dev):
    cfg = std_cfg()
    W = O.random_weights(cfg, 9)
    toks = clear_tokens(cfg, W, 70, 9)
    want = O.forward(cfg, W, toks)
    assert rel_err(replay(engine(cfg, W, dev), {"a": toks}, [[("a", 1)]] * 70)["a"], want) < TOL[torch.float32]


@pytest.mark.parametrize("sizes", [[2] * 40, [63, 2, 64, 1, 3, 65], [5, 59, 1, 1, 62, 2, 70], [130, 2, 2, 66]])
def test_portions(dev, sizes):
    cfg = std_cfg()
    W = O.random_weights(cfg, 10)
    toks = clear_tokens(cfg, W, sum(sizes), 10)
    got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", n)] for n in sizes])["a"]
    assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.float32]


def test_unequal_batch_equals_each_alone(dev):
    cfg = std_cfg()
    W = O.random_weights(cfg, 11)
    P = {"a": clear_tokens(cfg, W, 100, 1), "b": clear_tokens(cfg, W, 9, 2), "c": clear_tokens(cfg, W, 67, 3),
         "d": clear_tokens(cfg, W, 30, 4)}
    schedule = [[("a", 50), ("b", 1)], [("a", 14), ("b", 1), ("c", 64), ("d", 2)], [("a", 1), ("b", 2), ("c", 2), ("d", 27)],
                [("a", 35), ("b", 5), ("c", 1), ("d", 1)]]
    got = replay(engine(cfg, W, dev), P, schedule)
    for name, toks in P.items():
        assert rel_err(got[name], O.forward(cfg, W, toks)) < TOL[torch.float32], name


def test_pages_and_slots_used_again(dev):
    """a pool of three pages and two slots serves five requests one after another and side by side"""
    cfg = std_cfg()
    W = O.random_weights(cfg, 12)
    P = {n: clear_tokens(cfg, W, ln, i) for i, (n, ln) in enumerate([("a", 100), ("b", 60), ("c", 120), ("d", 3), ("e", 64)])}
    schedule = [[("a", 100)], [("b", 30)], [("b", 30)], [("c", 64), ("d", 1)], [("c", 56), ("d", 2)], [("e", 2)], [("e", 62)]]
    eng = engine(cfg, W, dev, max_batch=2, num_blocks=3)
    got = replay(eng, P, schedule)
    for name, toks in P.items():
        assert rel_err(got[name], O.forward(cfg, W, toks)) < TOL[torch.float32], name
    assert int(eng.sched.num_free_blocks()) == 3 and int(eng.sched.num_free_slots()) == 2


def test_long_decoding(dev):
    cfg = std_cfg()
    W = O.random_weights(cfg, 13)
    toks = clear_tokens(cfg, W, 200, 13)
    got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", 60)]] + [[("a", 1)]] * 140)["a"]
    assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.float32]


def test_bfloat16_serving_precision(dev):
    """16-bit serving against the f64 forms (a prompt whose router choices are far from close calls)"""
    cfg = std_cfg()
    W = O.random_weights(cfg, 14)
    seed = max(range(120), key=lambda s: O.router_margin(cfg, W, O.random_tokens(cfg, 48, s)))
    toks = O.random_tokens(cfg, 48, seed)
    want = O.forward(cfg, W, toks)
    got = replay(engine(cfg, W, dev, torch.bfloat16), {"a": toks}, [[("a", 33)], [("a", 2)]] + [[("a", 1)]] * 13)["a"]
    assert rel_err(got, want) < TOL[torch.bfloat16]


def test_greedy_generation_scheduler(dev):
    """LLMEngine.generate: C++ scheduler, chunked prompts (7 tokens a step in all), requests of unequal
    length side by side, greedy sampling"""
    from ipex_llm_amd.serving.engine import SamplingParams
    cfg = std_cfg()
    W = O.random_weights(cfg, 19)
    prompts = [clear_tokens(cfg, W, n, 20 + n) for n in (23, 3, 70, 11)]
    want = [greedy(cfg, W, p, 6) for p in prompts]
    for prefill, batch in ((7, 4), (1 << 30, 2)):
        eng = engine(cfg, W, dev, max_batch=batch, num_blocks=8, prefill=prefill)
        got = eng.generate(prompts, SamplingParams(max_new_tokens=6))
        assert got == want
        assert int(eng.sched.num_free_blocks()) == 8 and int(eng.sched.num_free_slots()) == batch


@pytest.mark.gpu
def test_decode_graph_replays_equal_eager():
    """pure-decode steps replayed from a captured graph (experts routed on the device, padded rows on the
    scratch page and slot), with eager prompt steps and synchronisations between the replays"""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    cfg = std_cfg()
    W = O.random_weights(cfg, 24)
    dev = torch.device("cuda")
    prompts = {"a": clear_tokens(cfg, W, 90, 1), "b": clear_tokens(cfg, W, 40, 2), "c": clear_tokens(cfg, W, 75, 3)}
    schedule = [[("a", 60), ("b", 20)], [("a", 1), ("b", 1)], [("a", 1), ("b", 1), ("c", 70)]] + \
        [[("a", 1), ("b", 1), ("c", 1)]] * 5 + [[("a", 23), ("b", 1)]] + [[("b", 1)]] * 12
    got = {}
    for graph in (False, True):
        eng = engine(cfg, W, dev, num_blocks=12, graph=graph)
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
    assert native_architecture(str(tmp_path / "m")) == "Masezen"
    model = AutoModelForCausalLM.from_pretrained(str(tmp_path / "m"), torch_dtype=torch.float32)
    prompt = clear_tokens(cfg, W, 12, 22)
    out = model.generate(torch.tensor([prompt]), max_new_tokens=5)
    assert out[0].tolist() == prompt + greedy(cfg, W, prompt, 5)
    bad = dict(cfg, width=cfg["width"] + 1)
    write_checkpoint(str(tmp_path / "bad"), bad, W)
    with pytest.raises(ValueError):
        AutoModelForCausalLM.from_pretrained(str(tmp_path / "bad"))


def test_trace_replay_program(tmp_path, dev):
    """bin/trace_run: steps on stdin, logits files, 'done' lines, requests ended and pages used again"""
    cfg = std_cfg()
    W = O.random_weights(cfg, 23)
    write_checkpoint(str(tmp_path / "m"), cfg, W)
    a, b = clear_tokens(cfg, W, 100, 1), clear_tokens(cfg, W, 66, 2)
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


@pytest.mark.parametrize("T,E,top,Wd,ff", [(300, 4, 2, 72, 40), (20, 6, 3, 64, 48), (5, 3, 1, 136, 24), (9, 3, 2, 20, 12)])
def test_experts_bf16(dev, T, E, top, Wd, ff):
    """16-bit experts (matrix cores on the GPU: row blocks of 128 and of 32, widths that are no multiple of the
    k step or of the column tile) against the f64 form on the same rounded weights"""
    from ipex_llm_amd.ops import blockmix as BM
    g = torch.Generator().manual_seed(T)
    h = torch.randn(T, Wd, generator=g).bfloat16()
    z = torch.randn(T, E, generator=g)
    idx, w = BM.moe_route(z.to(dev), top)
    Wt = {}
    for e in range(E):
        Wt[f"e{e}.gate"] = (torch.randn(ff, Wd, generator=g) * Wd ** -0.5).bfloat16()
        Wt[f"e{e}.up"] = (torch.randn(ff, Wd, generator=g) * Wd ** -0.5).bfloat16()
        Wt[f"e{e}.down"] = (torch.randn(Wd, ff, generator=g) * ff ** -0.5).bfloat16()
    w_gu = torch.stack([torch.cat([Wt[f"e{e}.gate"], Wt[f"e{e}.up"]]) for e in range(E)])
    w_down = torch.stack([Wt[f"e{e}.down"] for e in range(E)])
    got = BM.moe_experts(h.to(dev), idx, w, w_gu.to(dev), w_down.to(dev), 1.5, 1.702).cpu().double()
    W64 = {k: v.double() for k, v in Wt.items()}
    want = torch.zeros(T, Wd, dtype=F64)
    for t in range(T):
        for j in range(top):
            want[t] += O.expert(W64, f"e{int(idx[t, j])}.", float(w[t, j]) * h[t].double(), 1.5)
    assert (got - want).abs().max() < 0.03 * float(want.abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_matrix_core_sizes_model(dev, dtype):
    """a model whose head sizes and head counts fall into the matrix-core kernels' set (64-wide heads; 8, 4 and
    16 heads over 4, 1 and 2 key / value heads): portions past and below the kernels' thresholds beside decoded
    tokens of a second sequence, then decoding"""
    cfg = O.config([O.attn_layer(heads=8, kv_heads=4, dim=64, scaling=YARN, mlp=O.moe(4, 2, 32, 2.0, 32, 1.0)),
                    O.attn_layer(heads=4, kv_heads=1, dim=64, dims=32, mlp=O.dense(96)),
                    O.attn_layer(heads=16, kv_heads=2, dim=64, base=500.0, mlp=None)], width=64, taps=3, side=8)
    W = O.random_weights(cfg, 31)
    if dtype == torch.bfloat16:                      # 16-bit runs: prompts far from close router calls
        seeds = sorted(range(40), key=lambda s: -O.router_margin(cfg, W, O.random_tokens(cfg, 40, s)))
        P = {"a": O.random_tokens(cfg, 40, seeds[0]), "b": O.random_tokens(cfg, 40, seeds[1])}
        schedule = [[("a", 35), ("b", 1)], [("a", 2), ("b", 33)], [("a", 1), ("b", 1)], [("a", 1), ("b", 1)],
                    [("a", 1), ("b", 4)]]
    else:
        P = {"a": clear_tokens(cfg, W, 140, 1), "b": clear_tokens(cfg, W, 40, 2)}
        schedule = [[("a", 70), ("b", 1)], [("a", 3), ("b", 33)], [("a", 40), ("b", 1)]] + [[("a", 1), ("b", 1)]] * 5 + \
            [[("a", 22)]]
    got = replay(engine(cfg, W, dev, dtype), P, schedule)
    for name, toks in P.items():
        assert rel_err(got[name], O.forward(cfg, W, toks)) < TOL[dtype], name
