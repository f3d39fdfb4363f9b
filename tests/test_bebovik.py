"""Bebovik in the framework against the plain oracle (tests/bebovik_oracle.py): every mechanism
alone, then the model through the engine's scheduler, block pool and step — whole prompts,
token-by-token decoding, portions down to two tokens, unequal batches, reused pages, block
edges, first tokens, long decoding, greedy generation, the checkpoint layout and the trace
runner.  The same tests run the CPU reference ops here and the HIP kernels on a GPU box."""
import json
import math
import os
import subprocess
import sys

import pytest
import torch

import bebovik_oracle as orc
from dgi import ops
from dgi.engine import EngineConfig, LLMEngine
from dgi.models.config import AttentionSpec, BebovikConfig, GluSpec, LayerSpec, RotarySpec, get_config
from dgi.ops import mix
from dgi.ops.mix import DytNorm
from dgi.sched.request import SamplingParams

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F64 = torch.float64


def small_cfg() -> BebovikConfig:
    """Three layers that differ in everything: key size != value size, a key size that is no
    multiple of 8, heads == kv heads and one kv head, full and partial rotary with and without
    frequency scaling, three block sizes, a layer without feed-forward, logit scale 1."""
    sc = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}
    return BebovikConfig(name="t", vocab_size=61, hidden_size=48, layers=[
        LayerSpec("attention", AttentionSpec(4, 2, 16, 8, 0.3, RotarySpec(10000.0, 8, sc), "chunk", 8), GluSpec(40, 1.0)),
        LayerSpec("attention", AttentionSpec(2, 2, 12, 20, 0.25, RotarySpec(500.0, 12, None), "chunk", 5), None),
        LayerSpec("attention", AttentionSpec(3, 1, 8, 8, 0.5, RotarySpec(10000.0, 4, None), "chunk", 16), GluSpec(24, 0.7)),
    ], embedding_scale=3.0, logit_scale=1.0, logit_softcap=5.0, norm_eps=1e-5, max_position=512)


def engine(cfg, device, dtype=torch.float32, num_blocks=96, bs=4, seed=3, graphs=False, max_len=256):
    return LLMEngine(EngineConfig(model="bebovik-test", device=device, dtype=dtype, block_size=bs, num_blocks=num_blocks,
                                  max_num_seqs=4, max_model_len=max_len, max_num_batched_tokens=max_len,
                                  enable_prefix_caching=False, use_graphs=graphs, token_align=0, decode_lookahead=False,
                                  seed=seed), model_cfg=cfg)


def toks(n, seed=0, vocab=61):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def oracle_logits(eng, tokens):
    P, C = orc.from_model(eng.model)
    return orc.forward(tokens, P, C)


def feed_all(eng, rid, tokens, cuts):
    """Feed `tokens` in portions of the given sizes (the rest one by one); logits of every position."""
    out, at = [], 0
    sizes = list(cuts) + [1] * len(tokens)
    for n in sizes:
        if at >= len(tokens):
            break
        part = tokens[at:at + n]
        out.append(eng.feed([(rid, part, list(range(len(part))))])[0])
        at += len(part)
    return torch.cat(out, 0)


def close(a, b, tol):
    assert a.shape == b.shape
    err = (a.double() - b.double()).abs().max().item()
    assert err <= tol, f"max abs difference {err} > {tol}"


# ----------------------------------------------------------------------------------- mechanisms
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(5, 70), (37, 72), (16, 1032)])
def test_dyt_norms(device, dtype, shape):
    g = torch.Generator().manual_seed(1)
    T, W = shape             # scalar path, 16-byte path, and the row-tiled path with a ragged last tile
    mk = lambda: DytNorm(torch.rand(1, generator=g).add(0.3).to(device), torch.randn(W, generator=g).to(device),   # noqa: E731
                         torch.randn(W, generator=g).to(device))
    n1, n2 = mk(), mk()
    x = torch.randn(T, W, generator=g) * 3
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    close(mix.dyt(x.to(device), n1, dtype).cpu(), orc.dyt(x.double(), n1.alpha.cpu(), n1.w.cpu(), n1.b.cpu()), tol)
    h = (torch.randn(T, W, generator=g) * 2).to(dtype)
    ls = torch.randn(W, generator=g)
    res = x.clone().to(device)
    y = mix.dyt_add(res, h.to(device), n1, ls.to(device), n2)
    want = x.double() + orc.dyt(h.double(), n1.alpha.cpu(), n1.w.cpu(), n1.b.cpu()) * ls.double()
    close(res.cpu(), want, 1e-5)                                       # the stream stays fp32 in both dtypes
    close(y.cpu(), orc.dyt(want, n2.alpha.cpu(), n2.w.cpu(), n2.b.cpu()), tol)
    assert mix.dyt_add(res, h.to(device), n1, ls.to(device), None) is None
    table = torch.randn(9, W, generator=g).to(dtype)
    ids = torch.tensor([8, 0, 3, 3])
    e = mix.embed_dyt(ids.to(device), table.to(device), 2.5, n2)
    assert e.dtype == torch.float32
    close(e.cpu(), orc.dyt(table.double()[ids] * 2.5, n2.alpha.cpu(), n2.w.cpu(), n2.b.cpu()), 1e-5)


def test_rotary_table_scaling_regimes():
    sc = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}
    fr = orc.rotary_freqs(10000.0, 32, sc)
    plain = orc.rotary_freqs(10000.0, 32, None)
    kept, scaled = (fr == plain).sum().item(), torch.isclose(fr, plain / 4.0).sum().item()
    assert kept > 0 and scaled > 0 and kept + scaled < 16          # all three regimes occur
    t = ops.rope_cos_sin(32, 300, 10000.0, sc)
    pos = torch.tensor([0, 1, 17, 299], dtype=F64)
    a = pos[:, None] * fr[None]
    close(t[pos.long()], torch.cat([a.cos(), a.sin()], -1), 2e-6)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("geom", [(3, 1, 16, 8, 8), (2, 2, 12, 20, 12), (4, 2, 64, 64, 32), (1, 1, 10, 6, 0)])
def test_qknorm_rope_cache(device, dtype, geom):
    H, G, dk, dv, rd = geom
    g = torch.Generator().manual_seed(2)
    T, bs, NB = 6, 4, 40
    width = (H + G) * dk + G * dv + H * dv + 3
    qkv = (torch.randn(T, width, generator=g) * 2).to(dtype)
    pos = torch.tensor([0, 1, 7, 130, 131, 5], dtype=torch.int32)
    slots = torch.tensor([9, 4 * 7 + 3, 4 * 8, -1, 2, 4 * 39 + 3], dtype=torch.int32)
    qw, kw = torch.rand(dk, generator=g) + 0.5, torch.rand(dk, generator=g) + 0.5
    cs = ops.rope_cos_sin(rd, 256, 10000.0, None) if rd else None
    kc = torch.zeros(NB, G, bs, dk, dtype=dtype)
    vc = torch.zeros(NB, G, bs, dv, dtype=dtype)
    x = qkv.clone().to(device)
    kcd, vcd = kc.to(device), vc.to(device)
    mix.qknorm_rope_cache(x, pos.to(device), slots.to(device), qw.to(device), kw.to(device), 1e-3,
                          None if cs is None else cs.to(device), H, G, dk, dv, kcd, vcd)
    q = orc.unit_rms(qkv[:, :H * dk].double().view(T, H, dk), qw, 1e-3)
    k = orc.unit_rms(qkv[:, H * dk:(H + G) * dk].double().view(T, G, dk), kw, 1e-3)
    if rd:
        fr = orc.rotary_freqs(10000.0, rd)
        q, k = orc.rotate_pairs(q, pos.tolist(), fr), orc.rotate_pairs(k, pos.tolist(), fr)
    tol = 2e-5 if dtype == torch.float32 else 4e-2
    close(x.cpu()[:, :H * dk], q.reshape(T, -1), tol)
    assert torch.equal(x.cpu()[:, H * dk:], qkv[:, H * dk:])           # k, v, gate columns untouched
    v = qkv[:, (H + G) * dk:(H + G) * dk + G * dv].view(T, G, dv)
    for t in range(T):
        s = int(slots[t])
        if s < 0:
            continue
        close(kcd.cpu()[s // bs, :, s % bs], k[t], tol)
        assert torch.equal(vcd.cpu()[s // bs, :, s % bs], v[t])
    used = {int(s) for s in slots if s >= 0}
    flat = kcd.cpu().permute(0, 2, 1, 3).reshape(NB * bs, -1)
    assert all(flat[i].abs().sum() == 0 for i in range(NB * bs) if i not in used)   # nothing else written


def _paged(seq_k, seq_v, bs, NB, perm_seed):
    """Scatter one sequence's keys / values [n, G, d] into shuffled pages; returns caches + table."""
    n, G, dk = seq_k.shape
    dv = seq_v.shape[2]
    nb = (n + bs - 1) // bs
    g = torch.Generator().manual_seed(perm_seed)
    pages = (torch.randperm(NB - 1, generator=g)[:nb] + 1).tolist()
    kc = torch.randn(NB, G, bs, dk, generator=g).to(seq_k.dtype)       # stale values in unused slots
    vc = torch.randn(NB, G, bs, dv, generator=g).to(seq_v.dtype)
    for j in range(n):
        kc[pages[j // bs], :, j % bs] = seq_k[j]
        vc[pages[j // bs], :, j % bs] = seq_v[j]
    return kc, vc, pages


def _attn_oracle(q, k, v, p, H, G, scale, chunk, gate=None):
    keys = [j for j in range(k.shape[0]) if orc.visible(p, j, chunk)]
    out = []
    for h in range(H):
        s = torch.stack([(q[h].double() * k[j, h // (H // G)].double()).sum() * scale for j in keys])
        w = torch.softmax(s, 0)
        out.append(sum(w[i] * v[j, h // (H // G)].double() for i, j in enumerate(keys)))
    o = torch.cat(out)
    return o * torch.sigmoid(gate.double()) if gate is not None else o


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", ["decode", "prompt"])
def test_masked_attention_edges_with_a_standout_key(device, dtype, rows):
    """One key carries a score far above the rest and a value nothing else has: the output must
    show it exactly when the key is inside the query's block — just inside and just outside every
    edge, at page borders, at the first positions, and far back among hundreds (no mask)."""
    H, G, dk, dv, bs, NB = 4, 2, 16, 24, 4, 120
    g = torch.Generator().manual_seed(5)
    n = 330
    cases = []   # (chunk, query position, standout key)
    for chunk in (7, 16):
        for p in (chunk * 3, chunk * 3 + 1, chunk * 4 - 1, chunk * 5 + 2):
            first = p // chunk * chunk
            cases += [(chunk, p, first), (chunk, p, first - 1), (chunk, p, p)]
    cases += [(0, 329, 2), (0, 300, 0), (9, 0, 0), (9, 1, 0), (9, 1, 1), (64, 320, 320 - 64), (64, 329, 320)]
    for ci, (chunk, p, star) in enumerate(cases):
        k = torch.randn(n, G, dk, generator=g)
        v = torch.randn(n, G, dv, generator=g)
        q = torch.randn(H, dk, generator=g)
        if star >= 0:
            for gg in range(G):
                k[star, gg] = q[gg * (H // G)] * 3.0                     # dominant score for that group's heads
            v[star] = 50.0
        k, v, q = k.to(dtype), v.to(dtype), q.to(dtype)
        gate = torch.randn(H * dv, generator=g).to(dtype)
        kc, vc, pages = _paged(k, v, bs, NB, ci)
        bt = torch.zeros(2, NB, dtype=torch.int32)
        bt[1, :len(pages)] = torch.tensor(pages, dtype=torch.int32)
        if rows == "decode":      # row 1 of a 2-row decode batch (row 0: another sequence at position 0)
            qq = torch.stack([torch.zeros(H * dk, dtype=dtype), q.reshape(-1)])
            gt = torch.stack([torch.zeros(H * dv, dtype=dtype), gate])
            pos = torch.tensor([0, p], dtype=torch.int32)
            bt[0, 0] = pages[0]
            cu, row = None, 1
        else:                     # last row of a 3-token portion of sequence 1, behind a 2-token portion of sequence 0
            if p < 2:
                continue
            qq = torch.zeros(5, H * dk, dtype=dtype)
            qq[4] = q.reshape(-1)
            gt = torch.zeros(5, H * dv, dtype=dtype)
            gt[4] = gate
            pos = torch.tensor([0, 1, p - 2, p - 1, p], dtype=torch.int32)
            bt[0, 0] = pages[0]
            cu, row = torch.tensor([0, 2, 5], dtype=torch.int32), 4
        out = mix.masked_attn_rows(qq.to(device), kc.to(device), vc.to(device), bt.to(device),
                                   None if cu is None else cu.to(device), pos.to(device), H, G, 0.7, chunk,
                                   gt.to(device)).cpu()[row]
        want = _attn_oracle(q, k[:p + 1], v[:p + 1], p, H, G, 0.7, chunk, gate)
        close(out, want, 2e-4 if dtype == torch.float32 else 0.35)
        seen = orc.visible(p, star, chunk)
        ungated = out.double() / torch.sigmoid(gate.double())
        assert (ungated.abs().max() > 25.0) == seen, (chunk, p, star)


@pytest.mark.gpu
@pytest.mark.parametrize("hd", [64, 128])
def test_masked_prefill_mfma_edges(hd):
    """The MFMA prompt kernel (bf16, equal key / value size): portions that start inside a block,
    blocks that straddle 64-key tiles and 128-row query tiles, a standout key just inside and
    just outside the block of chosen rows, against the oracle and the row-wise kernel."""
    dev = "cuda"
    H, G, bs, NB = 4, 2, 16, 64
    g = torch.Generator().manual_seed(7)
    for chunk, ctx, ql in ((48, 300, 300), (120, 500, 137), (64, 256, 200), (200, 333, 5), (0, 260, 150), (1000, 400, 399)):
        k = torch.randn(ctx, G, hd, generator=g)
        v = torch.randn(ctx, G, hd, generator=g)
        q = torch.randn(ql, H, hd, generator=g) * 0.5
        probe = [ql - 1, ql // 2, 0]
        for r in probe:                 # a standout key just outside row r's block (or at its start)
            p = ctx - ql + r
            first = p // chunk * chunk if chunk else 0
            star = first - 1 if (r != ql // 2 and first > 0) else first
            k[star] = q[r, 0] * 4.0
            v[star] = 30.0
        k, v, q = k.bfloat16(), v.bfloat16(), q.bfloat16()
        gate = torch.randn(ql, H * hd, generator=g).bfloat16()
        kc, vc, pages = _paged(k, v, bs, NB, chunk)
        bt = torch.zeros(1, NB, dtype=torch.int32)
        bt[0, :len(pages)] = torch.tensor(pages, dtype=torch.int32)
        cu = torch.tensor([0, ql], dtype=torch.int32).to(dev)
        cl = torch.tensor([ctx], dtype=torch.int32).to(dev)
        args = (q.reshape(ql, -1).to(dev), kc.to(dev), vc.to(dev), bt.to(dev), cu)
        out = mix.paged_prefill_masked(*args, cl, H, G, 0.2, chunk, gate.to(dev)).cpu()
        pos = torch.arange(ctx - ql, ctx, dtype=torch.int32).to(dev)
        rows = mix.masked_attn_rows(*args, pos, H, G, 0.2, chunk, gate.to(dev)).cpu()
        close(out, rows, 0.3)
        for r in sorted(set(probe + [1, ql - 2, min(ql - 1, 127), min(ql - 1, 128)])):
            p = ctx - ql + r
            close(out[r], _attn_oracle(q[r], k[:p + 1], v[:p + 1], p, H, G, 0.2, chunk, gate[r]), 0.3)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_glu_and_softcap(device, dtype):
    g = torch.Generator().manual_seed(4)
    gu = (torch.randn(3, 2 * 37, generator=g) * 4).to(dtype)           # both clamps active
    lim = 1.3
    a, u = gu[:, :37].double().clamp(max=lim), gu[:, 37:].double().clamp(-lim, lim)
    want = a * torch.sigmoid(1.702 * a) * (u + 1)
    close(mix.glu_clamped(gu.to(device), lim).cpu(), want, 1e-5 if dtype == torch.float32 else 3e-2)
    x = (torch.randn(2, 50, generator=g) * 20).to(dtype)
    close(mix.scale_softcap(x.to(device), 1.7, 11.0).cpu(), 11.0 * torch.tanh(x.double() * 1.7 / 11.0), 1e-4)
    close(mix.scale_softcap(x.to(device), 0.5, 0.0).cpu(), x.double() * 0.5, 1e-5)


# ----------------------------------------------------------------------------------- model
@pytest.mark.parametrize("device", DEVICES)
def test_whole_prompt_every_layer(device):
    eng = engine(small_cfg(), device)
    t = toks(37, 1)
    eng.model.capture_layers = (0, 1, 2)
    got = eng.feed([("a", t, list(range(len(t))))])[0]
    want, streams = oracle_logits(eng, t)
    for i, s in enumerate(streams):
        close(eng.model.captured[i].cpu(), s, 2e-4)
    eng.model.capture_layers = ()
    close(got, want, 3e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_portions_and_token_by_token_equal_whole(device):
    cfg = small_cfg()
    t = toks(45, 2)
    want, _ = oracle_logits(engine(cfg, device), t)
    for cuts in ([], [2, 3, 2, 7, 5, 2, 16, 2], [44], [1, 1, 40]):      # [] = every token alone
        eng = engine(cfg, device)
        close(feed_all(eng, "r", t, cuts), want, 3e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(device):
    cfg = small_cfg()
    for n in (1, 2, 3):
        eng = engine(cfg, device)
        t = toks(n, 10 + n)
        close(eng.feed([("x", t, list(range(n)))])[0], oracle_logits(eng, t)[0], 3e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_across_blocks(device):
    eng = engine(small_cfg(), device)
    t = toks(3 * 16 + 5, 3)                                             # past three blocks of the widest layer
    close(feed_all(eng, "d", t, [4]), oracle_logits(eng, t)[0], 3e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_equals_each_alone_and_pages_are_reused(device):
    cfg = small_cfg()
    seqs = {"a": toks(30, 4), "b": toks(9, 5), "c": toks(21, 6), "d": toks(14, 7), "e": toks(26, 8)}
    alone = {}
    for k, t in seqs.items():
        alone[k] = oracle_logits(engine(cfg, "cpu"), t)[0]
    eng = engine(cfg, device, num_blocks=24)          # 23 usable pages of 4 tokens: fewer than all sequences need
    got = {k: [] for k in seqs}
    plan = [   # (entries: id -> count), ended ids
        ({"a": 6, "b": 1}, []), ({"a": 2, "b": 3, "c": 5}, []), ({"a": 1, "b": 1, "c": 1}, []),
        ({"a": 21, "b": 4}, ["a", "b"]),                       # a, b done: their pages return
        ({"c": 1, "d": 14}, ["d"]), ({"c": 2, "e": 20}, []), ({"c": 12, "e": 1}, ["c"]),
        ({"e": 1}, []), ({"e": 4}, ["e"]),
    ]
    at = {k: 0 for k in seqs}
    free0 = eng.pool.num_free
    for entries, end in plan:
        batch = []
        for k, n in entries.items():
            part = seqs[k][at[k]:at[k] + n]
            batch.append((k, part, list(range(len(part)))))
            at[k] += n
        for (k, _p, _w), lg in zip(batch, eng.feed(batch, end)):
            got[k].append(lg)
    assert at == {k: len(t) for k, t in seqs.items()}
    assert eng.pool.num_free == free0 and eng.pool.stats["allocs"] > free0        # pages came back and were reused
    for k in seqs:
        close(torch.cat(got[k], 0), alone[k], 3e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_portions_match_whole(device):
    """bf16 projections: how a prompt is cut changes the logits only by rounding."""
    cfg = small_cfg()
    t = toks(40, 9)
    whole = feed_all(engine(cfg, device, torch.bfloat16), "w", t, [40])
    parts = feed_all(engine(cfg, device, torch.bfloat16), "p", t, [3, 2, 9, 2])
    want = oracle_logits(engine(cfg, "cpu", torch.bfloat16), t)[0]
    scale = want.std().item()
    assert (whole.double() - want).pow(2).mean().sqrt().item() < 0.05 * scale
    assert (parts.double() - whole.double()).pow(2).mean().sqrt().item() < 0.05 * scale


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(device):
    cfg = small_cfg()
    eng = engine(cfg, device, graphs=(device == "cuda"))
    prompts = [toks(11, 20), toks(3, 21), toks(18, 22)]
    reqs = eng.generate(prompts, SamplingParams(max_tokens=7, temperature=0.0, ignore_eos=True))
    P, C = orc.from_model(eng.model)
    for p, r in zip(prompts, reqs):
        seq = list(p)
        for _ in range(7):
            lg = orc.forward(seq, P, C)[0][-1]
            top2 = lg.topk(2).values
            if (top2[0] - top2[1]).item() < 1e-3:      # a near tie is no test of the model
                break
            seq.append(int(lg.argmax()))
        n = len(seq) - len(p)
        assert r.output[:n] == seq[len(p):]


@pytest.mark.gpu
def test_mfma_prompt_path_in_the_model():
    """Equal 64- and 128-dim heads in bf16 take the MFMA prompt kernel: the model's logits with
    it, with the row-wise kernel instead, and cut into portions agree within bf16 rounding, and
    follow the oracle."""
    cfg = BebovikConfig(name="m", vocab_size=200, hidden_size=128, layers=[
        LayerSpec("attention", AttentionSpec(4, 2, 64, 64, 0.125, RotarySpec(10000.0, 32, None), "chunk", 48), GluSpec(256, 2.0)),
        LayerSpec("attention", AttentionSpec(2, 1, 128, 128, 0.09, RotarySpec(10000.0, 128, None), "chunk", 200), GluSpec(128, 2.0)),
    ], embedding_scale=2.0, logit_scale=1.0, logit_softcap=20.0, max_position=1024)
    t = toks(300, 30, 200)
    mk = lambda: engine(cfg, "cuda", torch.bfloat16, num_blocks=64, bs=16, max_len=512)     # noqa: E731
    a = feed_all(mk(), "a", t, [300])
    b = feed_all(mk(), "b", t, [130, 2, 77, 64])
    mix.MASKED_PREFILL = False
    try:
        c = feed_all(mk(), "c", t, [300])
    finally:
        mix.MASKED_PREFILL = True
    want = oracle_logits(engine(cfg, "cpu", torch.bfloat16, bs=16, num_blocks=8), t[:80])[0]
    scale = want.std().item()
    rms = lambda x, y: (x.double() - y.double()).pow(2).mean().sqrt().item()      # noqa: E731
    assert rms(a, c) < 0.05 * scale and rms(a, b) < 0.05 * scale
    assert rms(a[:80], want) < 0.06 * scale


def _layer(H, G, dk, dv, rd, chunk, ff, sc=None, base=10000.0, lim=1.2):
    return LayerSpec("attention", AttentionSpec(H, G, dk, dv, dk ** -0.5, RotarySpec(base, rd, sc), "chunk", chunk),
                     GluSpec(ff, lim) if ff else None)


def _ungated(layer):
    layer.mixer.out_gate = False
    return layer


_SC = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 32}
GEOMETRIES = {
    # heads of 64 and 128 (the MFMA prompt kernel in bf16 on a GPU) under block sizes that are no multiple of a
    # page or a key tile; a block longer than any sequence; a rotary of one pair
    "equal-64-128-odd-blocks": (96, 128, [_layer(4, 2, 64, 64, 32, 37, 160, _SC), _layer(2, 1, 128, 128, 128, 50, 0),
                                          _layer(8, 1, 64, 64, 2, 1000, 96)]),
    # 8 and 16 query heads per kv head, key size != value size, sizes that are multiples of 8 but not of 16
    "wide-groups": (70, 64, [_layer(8, 1, 32, 16, 16, 9, 64), _layer(16, 1, 16, 32, 8, 20, 0, _SC),
                             _layer(6, 3, 96, 40, 48, 33, 72)]),
    # a block of ONE position (every token sees only itself), a width that is no multiple of 4, odd-ish head sizes
    "block-of-one": (33, 50, [_layer(2, 1, 36, 12, 36, 1, 30), _layer(2, 2, 10, 6, 4, 3, 0), _layer(1, 1, 64, 128, 64, 64, 20)]),
    "wide-heads": (50, 256, [_layer(2, 1, 256, 256, 64, 24, 512, _SC, 500000.0), _layer(4, 4, 128, 64, 128, 17, 0)]),
    "no-feed-forward": (40, 64, [_layer(4, 2, 16, 16, 16, 11, 0), _layer(4, 1, 8, 24, 8, 40, 0)]),
    "no-output-gate": (40, 64, [_ungated(_layer(4, 2, 16, 16, 8, 11, 48)), _layer(2, 1, 64, 64, 64, 40, 0),
                                _ungated(_layer(2, 1, 64, 64, 32, 23, 0))]),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-5), (torch.bfloat16, 0.06)])
@pytest.mark.parametrize("name", list(GEOMETRIES))
def test_other_geometries_mixed_batches(device, dtype, tol, name):
    """Sizes, head ratios, block sizes and layer orders unlike the small configuration's, each run
    as three unequal requests in mixed steps (portions beside decode rows, pages reused) in a pool
    of 13 pages of 16 tokens, against the oracle."""
    vocab, W, layers = GEOMETRIES[name]
    cfg = BebovikConfig(name="g", vocab_size=vocab, hidden_size=W, layers=layers, embedding_scale=2.5, logit_scale=0.7,
                        logit_softcap=9.0, norm_eps=1e-5, max_position=512)
    eng = engine(cfg, device, dtype, num_blocks=14, bs=16, seed=11, max_len=192)
    seqs = {"a": toks(75, 70, vocab), "b": toks(31, 71, vocab), "c": toks(58, 72, vocab)}
    P, C = orc.from_model(eng.model)
    got, at = {k: [] for k in seqs}, {k: 0 for k in seqs}
    plan = [({"a": 40}, []), ({"a": 1, "b": 2}, []), ({"a": 1, "b": 1, "c": 17}, []), ({"a": 30, "b": 27, "c": 1}, []),
            ({"a": 1, "b": 1, "c": 2}, ["b"]), ({"a": 1, "c": 37}, []), ({"a": 1, "c": 1}, ["a", "c"])]
    for entries, end in plan:
        batch = []
        for k, n in entries.items():
            part = seqs[k][at[k]:at[k] + n]
            batch.append((k, part, list(range(len(part)))))
            at[k] += n
        for (k, _p, _w), lg in zip(batch, eng.feed(batch, end)):
            got[k].append(lg)
    for k, t in seqs.items():
        assert at[k] == len(t)
        want = orc.forward(t, P, C)[0]
        d = torch.cat(got[k], 0).double() - want
        d = d - d.mean(-1, keepdim=True)
        assert (d.pow(2).mean(-1).sqrt() / want.std()).max().item() < tol


# ----------------------------------------------------------------------------------- files, CLI
def _design_json(cfg: BebovikConfig) -> dict:
    lay = []
    for l in cfg.layers:
        m = l.mixer
        lay.append({"type": "attention",
                    "mixer": {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                              "mask": {"size": m.mask_size},
                              "rot": {"base": m.rot.base, "dims": m.rot.dims, "scaling": m.rot.scaling}},
                    "mlp": None if l.mlp is None else {"kind": "dense", "ff": l.mlp.ff, "limit": l.mlp.limit}})
    return {"architecture": "Bebovik", "vocab": cfg.vocab_size, "width": cfg.hidden_size, "layers": lay,
            "embedding": {"scale": cfg.embedding_scale}, "logit_scale": cfg.logit_scale,
            "logit_softcap": cfg.logit_softcap, "norm": {"eps": cfg.norm_eps}}


def _save_design(model, cfg, path):
    from safetensors.torch import save_file
    sd = {}
    for _n, t in model.tensors():          # the file stores bf16: round the fp32 parameters first
        t.copy_(t.bfloat16())

    def norm(name, n):
        sd[name], sd[name + ".b"], sd[name + ".alpha"] = n.w.bfloat16(), n.b.bfloat16(), n.alpha.reshape(()).bfloat16()

    sd["embed"], sd["head"] = model.embed.bfloat16(), model.head.bfloat16()
    norm("embed.norm", model.embed_norm)
    norm("final.norm", model.final_norm)
    for i, L in enumerate(model.layers):
        m, p = L.spec.mixer, f"l{i}."
        a, b, d = m.q_size, m.k_size, m.v_size
        w = L.qkvg.bfloat16()
        sd[p + "mix.q"], sd[p + "mix.k"], sd[p + "mix.v"], sd[p + "mix.g"] = w[:a], w[a:a + b], w[a + b:a + b + d], w[a + b + d:]
        sd[p + "mix.o"] = L.o.bfloat16()
        sd[p + "mix.q.norm"], sd[p + "mix.k.norm"] = L.q_norm.bfloat16(), L.k_norm.bfloat16()
        norm(p + "norm1", L.norm1)
        norm(p + "norm1b", L.norm1b)
        sd[p + "ls1"] = L.ls1.bfloat16()
        if L.gate_up is not None:
            ff = L.spec.mlp.ff
            sd[p + "mlp.gate"], sd[p + "mlp.up"], sd[p + "mlp.down"] = L.gate_up[:ff].bfloat16(), L.gate_up[ff:].bfloat16(), L.down.bfloat16()
            norm(p + "norm2", L.norm2)
            norm(p + "norm2b", L.norm2b)
            sd[p + "ls2"] = L.ls2.bfloat16()
    os.makedirs(path, exist_ok=True)
    save_file({k: v.contiguous().cpu() for k, v in sd.items()}, os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(_design_json(cfg), f)


def test_config_and_checkpoint_layout(tmp_path):
    cfg = small_cfg()
    src = engine(cfg, "cpu", torch.bfloat16).model        # bf16 weights: the file stores bf16
    d = str(tmp_path / "ckpt")
    _save_design(src, cfg, d)
    got = get_config(d)
    assert isinstance(got, BebovikConfig) and got.num_layers == 3 and got.layers[1].mlp is None
    assert [(l.mixer.heads, l.mixer.kv_heads, l.mixer.dim, l.mixer.vdim, l.mixer.mask_size) for l in got.layers] == \
        [(4, 2, 16, 8, 8), (2, 2, 12, 20, 5), (3, 1, 8, 8, 16)]
    assert got.layers[0].mixer.rot.scaling["original"] == 64 and got.layers[1].mixer.rot.scaling is None
    eng = LLMEngine(EngineConfig(model=d, device="cpu", dtype=torch.float32, block_size=4, num_blocks=32, max_num_seqs=2,
                                 max_model_len=128, max_num_batched_tokens=128, enable_prefix_caching=False, use_graphs=False))
    assert eng.model.load_info["tensors"] > 0
    t = toks(19, 40)
    close(eng.feed([("a", t, list(range(19)))])[0], oracle_logits(eng, t)[0], 3e-4)
    for (n1, a), (n2, b) in zip(src.tensors(), eng.model.tensors()):
        assert n1 == n2 and torch.equal(a.float(), b.float())


@pytest.mark.parametrize("device", DEVICES)
def test_trace_runner_cli(tmp_path, device):
    cfg = small_cfg()
    src = engine(cfg, "cpu", torch.bfloat16)
    d = str(tmp_path / "ckpt")
    _save_design(src.model, cfg, d)
    t1, t2 = toks(20, 50), toks(7, 51)
    steps = [
        {"step": 0, "entries": [{"id": "u", "tokens": t1[:9], "want": [0, 8]}, {"id": "v", "tokens": t2[:1], "want": []}], "end": []},
        {"step": 1, "entries": [{"id": "v", "tokens": t2[1:2], "want": [0]}], "end": []},
        {"step": 2, "entries": [{"id": "v", "tokens": t2[2:], "want": [4]}, {"id": "u", "tokens": t1[9:10], "want": [0]}], "end": ["v"]},
        {"step": 3, "entries": [{"id": "u", "tokens": t1[10:], "want": []}], "end": ["u"]},
    ]
    out = str(tmp_path / "out")
    r = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", "float32", "--out", out,
                        "--max-tokens", "64", "--device", device],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2", "done 3"]
    assert not os.path.exists(os.path.join(out, "3.f32"))
    import numpy as np
    ref = engine(cfg, "cpu")
    ref.model.copy_from(src.model)
    w1, w2 = oracle_logits(ref, t1)[0], oracle_logits(ref, t2)[0]
    rd = lambda n: torch.from_numpy(np.fromfile(os.path.join(out, f"{n}.f32"), dtype="<f4").reshape(-1, cfg.vocab_size).copy())  # noqa: E731
    close(rd(0), w1[[0, 8]], 3e-4)
    close(rd(1), w2[[1]], 3e-4)
    close(rd(2), torch.cat([w2[[6]], w1[[9]]]), 3e-4)


def test_worker_engine_serves_a_checkpoint_dir(tmp_path):
    """The worker's native engine picks the model class from config.json and generates through
    the same LLMEngine (chat template, tokenizer fallback, prefix caching on by default)."""
    sys.path.insert(0, os.path.join(ROOT, "worker"))
    from engines.llm_native import NativeLLMEngine
    cfg = small_cfg()
    d = str(tmp_path / "ckpt")
    _save_design(engine(cfg, "cpu", torch.bfloat16).model, cfg, d)
    e = NativeLLMEngine({"model_id": d, "device": "cpu", "max_model_len": 128, "max_num_batched_tokens": 128,
                         "num_blocks": 64, "max_num_seqs": 4})
    e.load_model()
    assert type(e.engine.model).__name__ == "BebovikModel"
    out = e.batch_inference([{"messages": [{"role": "user", "content": "hi"}], "max_tokens": 5, "temperature": 0.0}])
    assert out[0]["usage"]["completion_tokens"] == 5


@pytest.mark.parametrize("device", DEVICES)
def test_prefix_cache_hit_generates_the_same_tokens(device):
    cfg = small_cfg()
    eng = LLMEngine(EngineConfig(model="bebovik-test", device=device, dtype=torch.float32, block_size=4, num_blocks=64,
                                 max_num_seqs=4, max_model_len=128, max_num_batched_tokens=128, enable_prefix_caching=True,
                                 use_graphs=False, seed=3), model_cfg=cfg)
    p = toks(30, 60)
    sp = SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True)
    a = eng.generate([p], sp)[0]
    b = eng.generate([p + [5, 6]], sp)[0]
    c = eng.generate([p], sp)[0]
    assert c.num_cached >= 24 and b.num_cached >= 24 and a.num_cached == 0
    assert c.output == a.output
    fresh = engine(cfg, device)
    assert fresh.generate([p + [5, 6]], sp)[0].output == b.output


def test_bench_arch_compare_option_runs():
    """`bench.py --arch-compare` (tiny size, CPU): one JSON line with a row per model and phase numbers."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--arch-compare", "bebovik", "--arch-sizes", "tiny",
                        "--prompt-len", "40", "--concurrency", "2", "--steps", "2", "--warmup", "1",
                        "--max-batched-tokens", "128"], capture_output=True, text=True, timeout=600,
                       env={**os.environ, "CUDA_VISIBLE_DEVICES": "", "HIP_VISIBLE_DEVICES": ""})
    assert r.returncode == 0, r.stderr[-2000:]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    assert [x["model"] for x in out["rows"]] == ["bebovik", "llama"]
    assert all(x["prefill_tok_s"] > 0 and x["decode_tok_s"] > 0 for x in out["rows"])
