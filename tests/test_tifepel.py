"""Tifepel in the framework against the plain float64 oracle (tests/tifepel_oracle.py): every
mechanism alone, then the model through the engine's scheduler, block pool, state slots and step —
whole prompts, token-by-token decoding, portions down to two tokens, unequal batches, reused pages
and slots, distance-bucket edges and far keys, first tokens, long decoding, other geometries, greedy
generation, the checkpoint layout and the trace runner.  The same tests run the CPU reference ops
here and the HIP kernels on a GPU box."""
import copy
import json
import math
import os
import subprocess
import sys

import pytest
import torch

import tifepel_oracle as orc
from dgi.engine import EngineConfig, LLMEngine
from dgi.kv.state_pool import OutOfSlots, StatePool
from dgi.models.config import (AttentionSpec, LayerSpec, Mamba2Spec, MoeSpec, TifepelConfig, distance_bucket,
                               get_config)
from dgi.ops import mix, moe, recur
from dgi.sched.request import SamplingParams

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F64 = torch.float64
I32 = torch.int32


def attn(heads, kv, dim, vdim, scale, coef, every, rows, far):
    return AttentionSpec(heads, kv, dim, vdim, scale, None, out_gate=False, qk_norm_weight=False, q_temp_coef=coef,
                         q_temp_every=every, bias_rows=rows, bias_max=far)


def small_cfg(**kw) -> TifepelConfig:
    """Four layers that differ in everything: key size != value size, heads == kv heads, an odd
    bias table, Mamba-2 with groups == heads and with one norm group, experts with and without
    identity routes / shared expert, top == 1 and top == all routes, a layer without feed-forward;
    layers 1-2 run twice."""
    args = dict(name="t", vocab_size=53, hidden_size=32, layers=[
        LayerSpec("attention", attn(4, 2, 8, 12, 0.3, 0.4, 8, 10, 24.0), MoeSpec(3, 2, 2, 20, 16)),
        LayerSpec("mamba2", Mamba2Spec(4, 8, 12, 2, 3, 2), MoeSpec(4, 0, 1, 12, 0)),
        LayerSpec("attention", attn(2, 2, 12, 8, 0.25, 0.2, 5, 7, 30.0), None),
        LayerSpec("mamba2", Mamba2Spec(2, 20, 18, 2, 4, 1), MoeSpec(2, 1, 3, 8, 8)),
    ], streams=2, canon_taps=3, bigram_buckets=29, bigram_mul_prev=5, bigram_mul_cur=3, loop_start=1, loop_stop=3,
        loop_times=2, norm_eps=1e-5, max_position=512)
    args.update(kw)
    return TifepelConfig(**args)


def engine(cfg, device, dtype=torch.float32, num_blocks=96, bs=4, seed=3, max_len=256, seqs=4, graphs=False):
    return LLMEngine(EngineConfig(model="tifepel-test", device=device, dtype=dtype, block_size=bs, num_blocks=num_blocks,
                                  max_num_seqs=seqs, max_model_len=max_len, max_num_batched_tokens=max_len,
                                  enable_prefix_caching=True, use_graphs=graphs, token_align=0, decode_lookahead=graphs,
                                  seed=seed, graph_buckets=(1, 2, 4) if graphs else None), model_cfg=copy.deepcopy(cfg))


def toks(n, seed=0, vocab=53):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def config_dict(cfg: TifepelConfig) -> dict:
    """The design's config.json for ``cfg``."""
    layers = []
    for l in cfg.layers:
        m = l.mixer
        if l.type == "attention":
            mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                     "q_temp": {"coef": m.q_temp_coef, "every": m.q_temp_every}, "bias_max": m.bias_max}
        else:
            mixer = {"heads": m.heads, "vdim": m.vdim, "state": m.state, "groups": m.groups, "conv": m.conv,
                     "norm_groups": m.norm_groups}
        f = l.mlp
        mlp = None if f is None else {"kind": "moe", "expert": {"ff": f.ff},
                                      "router": {"experts": f.experts, "identity": f.identity, "top": f.top},
                                      "shared": {"ff": f.shared_ff} if f.shared_ff else None}
        layers.append({"type": l.type, "mixer": mixer, "mlp": mlp})
    return {"architecture": "Tifepel", "vocab": cfg.vocab_size, "width": cfg.hidden_size, "streams": cfg.streams,
            "canon": {"taps": cfg.canon_taps}, "norm": {"eps": cfg.norm_eps}, "max_positions": cfg.max_position,
            "embedding": {"bigram": {"buckets": cfg.bigram_buckets, "mul_prev": cfg.bigram_mul_prev,
                                     "mul_cur": cfg.bigram_mul_cur}},
            "loop": {"start": cfg.loop_start, "stop": cfg.loop_stop, "times": cfg.loop_times}, "layers": layers}


def params(model) -> dict:
    """The model's weights under the checkpoint's tensor names (CPU, model dtype)."""
    P = {"embed": model.embed, "bigram": model.bigram, "pos": model.pos, "head": model.head, "final.norm": model.final_norm}
    for i, L in enumerate(model.layers):
        p = f"l{i}."
        m, f = L.spec.mixer, L.spec.mlp
        for q in ("1", "2") if f is not None else ("1",):
            P[p + "norm" + q] = getattr(L, "norm" + q)
            P[p + "canon" + q] = getattr(L, "canon" + q)
            P[p + "rg" + q] = getattr(L, "rg" + q)
            P[f"{p}rg{q}.b"] = getattr(L, f"rg{q}_b")
            for k in ("in", "out", "mix"):
                P[f"{p}hc{q}.{k}"] = getattr(L, f"hc{q}_{k}")
        if L.spec.type == "attention":
            a, b = m.q_size, m.q_size + m.k_size
            P[p + "mix.q"], P[p + "mix.k"], P[p + "mix.v"] = L.qkv[:a], L.qkv[a:b], L.qkv[b:]
            P[p + "mix.rel"] = L.rel
        else:
            for key, t in (("in", L.in_proj), ("conv", L.conv), ("conv.b", L.conv_b), ("dt_bias", L.dt_bias),
                           ("A_log", L.a_log), ("D", L.d_skip), ("norm", L.mnorm)):
                P[p + "mix." + key] = t
        P[p + "mix.o"] = L.o
        if f is not None:
            P[p + "mlp.router"], P[p + "mlp.correction"] = L.router, L.correction
            for e in range(f.experts):
                P[f"{p}mlp.e{e}.gate"], P[f"{p}mlp.e{e}.up"] = L.gate_up[e, :f.ff], L.gate_up[e, f.ff:]
                P[f"{p}mlp.e{e}.down"] = L.down[e]
            if f.shared_ff:
                P[p + "mlp.shared.gate"] = L.shared_gate_up[:f.shared_ff]
                P[p + "mlp.shared.up"] = L.shared_gate_up[f.shared_ff:]
                P[p + "mlp.shared.down"] = L.shared_down
    return {k: v.detach().cpu().contiguous() for k, v in P.items() if v is not None}


def oracle_logits(eng, tokens, layers_out=None):
    P = {k: v.to(F64) for k, v in params(eng.model).items()}
    return orc.forward(P, config_dict(eng.model_cfg), tokens, layers_out)


def feed_all(eng, rid, tokens, cuts):
    """Feed `tokens` in portions of the given sizes (the rest one by one); logits of every position."""
    out, at = [], 0
    for n in list(cuts) + [1] * len(tokens):
        if at >= len(tokens):
            break
        part = tokens[at:at + n]
        out.append(eng.feed([(rid, part, list(range(len(part))))])[0])
        at += len(part)
    return torch.cat(out, 0)


def close(a, b, tol):
    assert a.shape == b.shape
    err = (a.double().cpu() - b.double().cpu()).abs().max().item()
    assert err <= tol, f"max abs difference {err} > {tol}"


def seq_meta(lens, starts, slots, device):
    pos, rs, r0 = [], [], [0]
    for i, (n, s) in enumerate(zip(lens, starts)):
        pos += list(range(s, s + n))
        rs += [i] * n
        r0.append(r0[-1] + n)
    mk = lambda x: torch.tensor(x, dtype=I32, device=device)   # noqa: E731
    return mk(pos), mk(rs), mk(r0), mk(slots)


# ----------------------------------------------------------------------------------- mechanisms
def test_distance_bucket_edges():
    # first half: one row per distance; then logarithmic up to `far`; everything beyond in the last row
    assert [distance_bucket(n, 12, 90.0) for n in range(6)] == list(range(6))
    assert distance_bucket(6, 12, 90.0) == 6 and distance_bucket(89, 12, 90.0) == 11
    assert distance_bucket(90, 12, 90.0) == 11 and distance_bucket(5000, 12, 90.0) == 11
    assert [distance_bucket(n, 16, 128.0) for n in (15, 16, 31, 32, 63, 64, 127, 128)] == [9, 10, 11, 12, 13, 14, 15, 15]
    for rows, far in ((12, 90.0), (7, 30.0), (10, 24.0)):            # same rule as the oracle's, odd tables too
        assert all(distance_bucket(n, rows, far) == orc.distance_bucket(n, rows, far) for n in range(200))
        rel = torch.randn(rows, 3)
        t = mix.distance_bias_table(rel, far)
        for n in (0, rows // 2 - 1, rows // 2, int(far) - 1, int(far), 10 * int(far)):
            assert torch.equal(t[min(n, t.shape[0] - 1)], rel[distance_bucket(n, rows, far)])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_streams(device, dtype):
    g = torch.Generator().manual_seed(1)
    V, W, S, nb = 40, 72, 3, 17
    lens, starts, slots = [1, 1, 5, 3], [6, 0, 0, 2], [2, 4, 1, 3]
    pos, rs, r0, sl = seq_meta(lens, starts, slots, device)
    T = sum(lens)
    ids = torch.randint(0, V, (T,), generator=g, dtype=I32)
    E, Bg, Pt = (torch.randn(n, W, generator=g).to(dtype) for n in (V, nb + 1, 16))
    prev = torch.tensor([0, 9, 11, 13, 15, 0], dtype=I32)
    pv = prev.clone().to(device)
    xs = recur.embed_streams(ids.to(device), pos, rs, r0, sl, pv, E.to(device), Bg.to(device), Pt.to(device), nb, 7, 3, S)
    assert xs.dtype == torch.float32 and xs.shape == (S, T, W)
    P = {"embed": E.double(), "bigram": Bg.double(), "pos": Pt.double()}
    cfg = {"embedding": {"bigram": {"buckets": nb, "mul_prev": 7, "mul_cur": 3}}}
    at = 0
    for n, s, slot in zip(lens, starts, slots):
        # the oracle embeds whole sequences: give it the missing prefix, with the state's token last
        prefix = [0] * (s - 1) + [int(prev[slot])] if s else []
        want = orc.embed(P, cfg, prefix + ids[at:at + n].tolist())[s:]
        for k in range(S):
            close(xs[k, at:at + n], want, 1e-5)
        assert int(pv[slot]) == int(ids[at + n - 1])
        at += n


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("S,W", [(1, 40), (2, 64), (4, 300)])
def test_hyper_connection_update_and_norm(device, dtype, S, W):
    g = torch.Generator().manual_seed(2)
    T = 9
    xs = torch.randn(S, T, W, generator=g) * 2
    y, gate = (torch.randn(T, W, generator=g).to(dtype) for _ in range(2))
    gb, nw = torch.randn(W, generator=g), torch.randn(W, generator=g)
    mx, oc, inn = torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g)
    x = xs.clone().to(device)
    h32, hd = recur.hc_mix_norm(x, y.to(device), gate.to(device), gb.to(device), mx.to(device), oc.to(device),
                                inn.to(device), nw.to(device), 1e-5, dtype)
    yy = y.double() * torch.sigmoid(gate.double() + gb.double())
    want = torch.einsum("st,sxw->txw", mx.double(), xs.double()) + oc.double()[:, None, None] * yy
    close(x, want, 2e-5)
    hw = orc.layer_norm((inn.double()[:, None, None] * want).sum(0), nw.double(), 1e-5)
    close(h32, hw, 5e-5)
    assert hd.dtype == dtype
    close(hd, hw, 5e-5 if dtype == torch.float32 else 4e-2)
    # update only / read-out only
    x2 = xs.clone().to(device)
    assert recur.hc_mix_norm(x2, y.to(device), None, None, mx.to(device), oc.to(device), None, None, 1e-5, dtype) == (None, None)
    close(x2, torch.einsum("st,sxw->txw", mx.double(), xs.double()) + oc.double()[:, None, None] * y.double(), 2e-5)
    h3, _ = recur.hc_mix_norm(x2, None, None, None, None, None, inn.to(device), nw.to(device), 1e-5, dtype)
    close(h3, orc.layer_norm((inn.double()[:, None, None] * x2.double().cpu()).sum(0), nw.double(), 1e-5), 5e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps,act,residual", [(4, 0, True), (3, 1, False), (1, 0, True), (2, 1, True), (6, 0, False)])
@pytest.mark.parametrize("C,pad,off", [(37, 6, 3), (40, 8, 4)])        # odd channels / the four-channel vector path
def test_causal_conv_portions(device, taps, act, residual, C, pad, off):
    """A sequence cut into portions of 1, 2, taps - 1, taps and more rows, another one beside it,
    slots that held other data before: equal to the whole-sequence convolution."""
    g = torch.Generator().manual_seed(3)
    n = 23
    w = torch.randn(C, taps, generator=g)
    b = torch.randn(C, generator=g) if act else None
    xa, xb = torch.randn(n, C + pad, generator=g), torch.randn(n, C + pad, generator=g)   # wider rows: a column slice
    tail = torch.randn(5, max(taps - 1, 0), C).to(device) * 100 if taps > 1 else None     # stale slot contents
    want = {}
    for name, x in (("a", xa), ("b", xb)):
        o = orc.causal_taps(x[:, off:off + C].double(), w.double(), None if b is None else b.double())
        o = orc.silu(o) if act else o
        want[name] = o + x[:, off:off + C].double() if residual else o
    cuts = [1, 1, 2, max(taps - 1, 1), taps, 5, 1, n]
    at_a = at_b = 0
    got_a, got_b = [], []
    for i, c in enumerate(cuts):
        na, nb_ = min(c, n - at_a), (min(3, n - at_b) if i % 2 == 0 else 0)
        lens, starts, slots, rows = [], [], [], []
        if nb_:
            lens.append(nb_), starts.append(at_b), slots.append(4), rows.append(xb[at_b:at_b + nb_])
        if na:
            lens.append(na), starts.append(at_a), slots.append(2), rows.append(xa[at_a:at_a + na])
        if not lens:
            break
        pos, rs, r0, sl = seq_meta(lens, starts, slots, device)
        x = torch.cat(rows, 0).to(device)[:, off:off + C]
        out = recur.causal_conv(x, w.to(device), None if b is None else b.to(device), tail, pos, rs, r0, sl, act=act,
                                residual=residual, out_dtype=torch.float32)
        if nb_:
            got_b.append(out[:nb_])
        if na:
            got_a.append(out[nb_:])
        at_a, at_b = at_a + na, at_b + nb_
    close(torch.cat(got_a, 0), want["a"][:at_a], 1e-4)
    close(torch.cat(got_b, 0), want["b"][:at_b], 1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("taps,dtype", [(4, torch.float32), (3, torch.bfloat16), (2, torch.float32)])
def test_causal_conv_large_step_walks_rows(taps, dtype):
    """Steps of 2048 rows and more let a thread walk several consecutive rows with the window in registers:
    sequences that start inside a walk, one-row sequences, continued portions with their tails, a fresh one."""
    g = torch.Generator().manual_seed(11)
    C = 40
    lens, starts, slots = [1000, 1, 700, 3, 397, 5], [0, 9, 50, 0, 2, 1], [1, 2, 3, 4, 5, 6]
    T = sum(lens)
    assert T >= 2048
    x = torch.randn(T, C + 8, generator=g).to(dtype)
    w, b = torch.randn(C, taps, generator=g), torch.randn(C, generator=g)
    tail = torch.randn(8, taps - 1, C, generator=g)
    pos, rs, r0, sl = seq_meta(lens, starts, slots, "cpu")
    t_ref = tail.clone()
    want = recur.causal_conv_ref(x[:, 4:4 + C], w, b, t_ref, pos, r0, sl, 1, True, torch.float32)
    t_gpu = tail.clone().cuda()
    got = recur.causal_conv(x.cuda()[:, 4:4 + C], w.cuda(), b.cuda(), t_gpu, pos.cuda(), rs.cuda(), r0.cuda(), sl.cuda(),
                            act=1, residual=True, out_dtype=torch.float32)
    close(got, want, 1e-4)
    close(t_gpu[slots], t_ref[slots], 1e-6)


def mamba_parts(g, heads, dv, N, G, T, dtype):
    inner = heads * dv
    xbc = torch.randn(T, inner + 2 * G * N, generator=g)
    dt_raw = (torch.randn(T, heads + 2, generator=g) * 2).to(dtype)
    return xbc, dt_raw, torch.randn(heads, generator=g), torch.randn(heads, generator=g) * 0.5 - 1, torch.randn(heads, generator=g)


def oracle_scan(xbc, dt_raw, dt_bias, a_log, d_skip, heads, dv, N, G):
    """The recurrence of tifepel_oracle.mamba2 on given x | B | C and step sizes (fp64, one sequence)."""
    T = xbc.shape[0]
    inner = heads * dv
    x = xbc[:, :inner].double().view(T, heads, dv)
    Bm, Cm = xbc[:, inner:inner + G * N].double().view(T, G, N), xbc[:, inner + G * N:].double().view(T, G, N)
    dt = torch.nn.functional.softplus(dt_raw.double() + dt_bias.double(), threshold=1e9)
    y = torch.zeros(T, heads, dv, dtype=F64)
    for h in range(heads):
        S = torch.zeros(N, dv, dtype=F64)
        for t in range(T):
            S = torch.exp(-torch.exp(a_log[h].double()) * dt[t, h]) * S + dt[t, h] * torch.outer(Bm[t, h // (heads // G)], x[t, h])
            y[t, h] = S.T @ Cm[t, h // (heads // G)] + d_skip[h].double() * x[t, h]
    return y.reshape(T, inner)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("geom", [(4, 24, 20, 2), (2, 16, 64, 1), (3, 40, 130, 3), (1, 5, 3, 1)])
def test_ssm_scan_portions_and_slots(device, dtype, geom):
    """Whole sequence == portions of 1, 2, 7, ... rows through a slot that held another state before,
    with a second sequence in the same step; large positive / negative step-size inputs."""
    heads, dv, N, G = geom
    g = torch.Generator().manual_seed(4)
    n = 40
    xa, da, dt_bias, a_log, d_skip = mamba_parts(g, heads, dv, N, G, n, dtype)
    xb, db = mamba_parts(g, heads, dv, N, G, n, dtype)[:2]
    da[3], da[4] = 30.0, -30.0                     # softplus without overflow and without a clamp
    want_a = oracle_scan(xa, da[:, 1:1 + heads], dt_bias, a_log, d_skip, heads, dv, N, G)
    want_b = oracle_scan(xb, db[:, 1:1 + heads], dt_bias, a_log, d_skip, heads, dv, N, G)
    state = torch.randn(6, heads, dv, N).to(device) * 50
    at_a = at_b = 0
    got_a, got_b = [], []
    for i, c in enumerate([1, 1, 2, 7, 1, 13, n]):
        na, nb_ = min(c, n - at_a), (min(5, n - at_b) if i % 2 else 0)
        lens, starts, slots, xr, dr = [], [], [], [], []
        for cnt, at, slot, x, d in ((na, at_a, 3, xa, da), (nb_, at_b, 5, xb, db)):
            if cnt:
                lens.append(cnt), starts.append(at), slots.append(slot), xr.append(x[at:at + cnt]), dr.append(d[at:at + cnt])
        if not lens:
            break
        pos, _rs, r0, sl = seq_meta(lens, starts, slots, device)
        y = recur.ssm_scan(torch.cat(xr, 0).to(device), torch.cat(dr, 0).to(device)[:, 1:1 + heads], dt_bias.to(device),
                           a_log.to(device), d_skip.to(device), state, pos, r0, sl, heads, dv, N, G)
        if na:
            got_a.append(y[:na])
        if nb_:
            got_b.append(y[na:])
        at_a, at_b = at_a + na, at_b + nb_
    scale = max(1.0, want_a.abs().max().item())
    close(torch.cat(got_a, 0), want_a[:at_a], 2e-5 * scale)
    close(torch.cat(got_b, 0), want_b[:at_b], 2e-5 * max(1.0, want_b.abs().max().item()))


@pytest.mark.gpu
@pytest.mark.parametrize("geom", [(4, 24, 20, 2), (2, 16, 130, 1)])
def test_chunked_scan_equals_one_pass(geom, monkeypatch):
    """The chunk-parallel form (local chunk states, serial pass over them, outputs per chunk) against
    the oracle: portions that end inside a chunk, a one-row sequence beside them, a continued sequence
    whose slot holds its state, and a fresh one whose slot holds garbage."""
    heads, dv, N, G = geom
    monkeypatch.setattr(recur, "SCAN_CHUNK", 16)
    g = torch.Generator().manual_seed(9)
    n = 150
    xa, da, dt_bias, a_log, d_skip = mamba_parts(g, heads, dv, N, G, n, torch.float32)
    xb, db = mamba_parts(g, heads, dv, N, G, n, torch.float32)[:2]
    want_a = oracle_scan(xa, da[:, 1:1 + heads], dt_bias, a_log, d_skip, heads, dv, N, G)
    want_b = oracle_scan(xb, db[:, 1:1 + heads], dt_bias, a_log, d_skip, heads, dv, N, G)
    state = torch.randn(6, heads, dv, N).cuda() * 50
    par = [t.cuda() for t in (dt_bias, a_log, d_skip)]
    # step 1: a[0:70] (fresh) beside b[0:1]; step 2: a[70:150] (continued) beside b[1:131]
    for (a0, a1, b0, b1) in ((0, 70, 0, 1), (70, 150, 1, 131)):
        pos, _rs, r0, sl = seq_meta([a1 - a0, b1 - b0], [a0, b0], [2, 4], "cuda")
        x = torch.cat([xa[a0:a1], xb[b0:b1]], 0).cuda()
        d = torch.cat([da[a0:a1], db[b0:b1]], 0).cuda()[:, 1:1 + heads]
        y = recur.ssm_scan(x, d, *par, state, pos, r0, sl, heads, dv, N, G, chunked=True)
        close(y[: a1 - a0], want_a[a0:a1], 3e-5 * max(1.0, want_a.abs().max().item()))
        close(y[a1 - a0:], want_b[b0:b1], 3e-5 * max(1.0, want_b.abs().max().item()))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_scan_remembers_a_far_token(device, dtype):
    """One input 300 tokens back, a slow decay: the state still carries it (and a wrong or lost state
    would not): the output at the end equals the closed form."""
    heads, dv, N, G, n = 1, 4, 3, 1, 301
    xbc = torch.zeros(n, dv + 2 * N)
    xbc[0, :dv] = torch.tensor([1.0, -2.0, 3.0, 0.5])
    xbc[0, dv] = 2.0                               # B_0 = (2, 0, 0)
    xbc[-1, dv + N] = 1.0                          # C_last = (1, 0, 0)
    dt_raw = torch.full((n, 1), -2.0).to(dtype)
    a_log = torch.tensor([-4.0])
    state = torch.randn(3, heads, dv, N).to(device)
    pos, _rs, r0, sl = seq_meta([200], [0], [1], device)
    args = (torch.zeros(1).to(device), a_log.to(device), torch.zeros(1).to(device), state)
    recur.ssm_scan(xbc[:200].to(device), dt_raw[:200].to(device), *args, pos, r0, sl, heads, dv, N, G)
    out = []
    for t in range(200, n):                        # then token by token
        pos, _rs, r0, sl = seq_meta([1], [t], [1], device)
        out.append(recur.ssm_scan(xbc[t:t + 1].to(device), dt_raw[t:t + 1].to(device), *args, pos, r0, sl, heads, dv, N, G))
    dt = math.log1p(math.exp(-2.0))
    want = xbc[0, :dv].double() * 2.0 * dt * math.exp(-math.exp(-4.0) * dt * (n - 1))
    assert want.abs().max() > 0.05
    close(out[-1][0], want, 1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_group_norm_and_silu_mul(device, dtype):
    g = torch.Generator().manual_seed(5)
    T, C = 7, 96
    tol = 2e-5 if dtype == torch.float32 else 4e-2
    for pad, off in ((5, 2), (16, 8)):                 # an unaligned column slice, and the aligned one-pass path
        y, zw, w = torch.randn(T, C, generator=g) * 3, torch.randn(T, C + pad, generator=g).to(dtype), torch.randn(C, generator=g)
        z = zw[:, off:off + C]
        for groups in (1, 3, 96):
            got = recur.gated_group_norm(y.to(device), zw.to(device)[:, off:off + C], w.to(device), groups, 1e-4, dtype)
            gv = (y.double() * orc.silu(z.double())).view(T, groups, C // groups)
            close(got, orc.unit_rms(gv, 1e-4).reshape(T, C) * w.double(), tol)
    y, zw, w = torch.randn(3, 4096, generator=g), torch.randn(3, 4096, generator=g).to(dtype), torch.randn(4096, generator=g)
    got = recur.gated_group_norm(y.to(device), zw.to(device), w.to(device), 1, 1e-4, dtype)       # eight chunks a thread
    close(got, orc.unit_rms((y.double() * orc.silu(zw.double())).view(3, 1, 4096), 1e-4).reshape(3, 4096) * w.double(), tol)
    for I in (25, 32):                                 # scalar path and the four-column vector path
        gu = torch.randn(T, 2 * I, generator=g).to(dtype)
        close(moe.silu_mul(gu.to(device)), orc.silu(gu[:, :I].double()) * gu[:, I:].double(), tol)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("geom", [(4, 2, 8, 12), (2, 2, 12, 8), (3, 1, 10, 6), (8, 2, 40, 72)])
def test_attention_temperature_bias_and_edges(device, dtype, geom):
    """q/k unit norm + query temperature + paged write, then biased attention, against the oracle:
    a bias table with large entries, so one wrong bucket at an edge (rows / 2, `far`, beyond) or one
    wrong temperature step would change the output visibly; decode rows and prompt rows, keys across
    page borders and hundreds back."""
    H, G, dk, dv = geom
    g = torch.Generator().manual_seed(6)
    n, bs, rows, far, eps, scale = 150, 4, 10, 40.0, 1e-4, 0.35
    qt = (0.5, 16)
    qkv = torch.randn(n, (H + G) * dk + G * dv + 2, generator=g).to(dtype)
    rel = torch.randn(rows, H, generator=g) * 4
    NB = n // bs + 3
    perm = torch.randperm(NB - 1, generator=g)[: (n + bs - 1) // bs] + 1          # scattered pages
    bt = perm.to(I32).view(1, -1)
    pos = torch.arange(n, dtype=I32)
    slots = (bt[0, pos.long() // bs] * bs + pos % bs).to(I32)
    kc, vc = torch.zeros(NB, G, bs, dk, dtype=dtype).to(device), torch.zeros(NB, G, bs, dv, dtype=dtype).to(device)
    x = qkv.clone().to(device)
    ones = torch.ones(dk).to(device)
    mix.qknorm_rope_cache(x, pos.to(device), slots.to(device), ones, ones, eps, None, H, G, dk, dv, kc, vc, q_temp=qt)
    # oracle: the same attention on explicit q, k, v
    q = orc.unit_rms(qkv[:, :H * dk].double().view(n, H, dk), eps)
    k = orc.unit_rms(qkv[:, H * dk:(H + G) * dk].double().view(n, G, dk), eps)
    v = qkv[:, (H + G) * dk:(H + G) * dk + G * dv].double().view(n, G, dv)
    q = q * torch.tensor([1 + qt[0] * math.log((p + 1) // qt[1] + 1) for p in range(n)], dtype=F64)[:, None, None]
    tol = 3e-5 if dtype == torch.float32 else 6e-2
    close(x[:, :H * dk], q.reshape(n, H * dk), tol)
    want = torch.zeros(n, H, dv, dtype=F64)
    for h in range(H):
        for i in range(n):
            s = (k[: i + 1, h // (H // G)] @ q[i, h]) * scale
            s = s + torch.stack([rel[orc.distance_bucket(i - j, rows, far), h] for j in range(i + 1)]).double()
            want[i, h] = torch.softmax(s, 0) @ v[: i + 1, h // (H // G)]
    want = want.reshape(n, H * dv)
    db = mix.distance_bias_table(rel, far).to(device)
    cu = torch.tensor([0, n], dtype=I32, device=device)
    got = mix.masked_attn_rows(x, kc, vc, bt.to(device), cu, pos.to(device), H, G, scale, 0, None, dist_bias=db)
    close(got, want, tol)
    dec = [0, 1, rows // 2 - 1, rows // 2, int(far) - 1, int(far), int(far) + 1, n - 1]     # as decode rows
    got = mix.masked_attn_rows(x[dec].contiguous(), kc, vc, bt.to(device).repeat(len(dec), 1), None,
                               pos[dec].contiguous().to(device), H, G, scale, 0, None, dist_bias=db)
    close(got, want[dec], tol)


@pytest.mark.gpu
@pytest.mark.parametrize("hd,H,G", [(64, 4, 2), (128, 8, 2)])
def test_mfma_prompt_attention_with_distance_bias(hd, H, G):
    """Prompt portions on the MFMA flash kernel (bf16 heads of 64 / 128 dims): a portion on top of a
    cached prefix and a fresh prompt in one launch, a bias table that ends inside a 64-key tile and
    one longer than the context, against the row-wise reference (fp32 math on the same bf16 cache)."""
    from dgi import ops
    g = torch.Generator().manual_seed(8)
    bs, NB = 16, 64
    lens, ctxs = [200, 77], [333, 77]              # rows of this step, context including them
    T = sum(lens)
    q = torch.randn(T, H * hd, generator=g).to(torch.bfloat16)
    kc = torch.randn(NB, G, bs, hd, generator=g).to(torch.bfloat16)
    vc = torch.randn(NB, G, bs, hd, generator=g).to(torch.bfloat16)
    bt = torch.zeros(2, 24, dtype=I32)
    bt[0, :21] = torch.arange(1, 22, dtype=I32)
    bt[1, :5] = torch.arange(30, 35, dtype=I32)
    cu = torch.tensor([0, 200, 277], dtype=I32)
    ctx = torch.tensor(ctxs, dtype=I32)
    pos = torch.cat([torch.arange(133, 333), torch.arange(0, 77)]).to(I32)
    scale = hd ** -0.5
    for rows, far in ((12, 100.0), (16, 1000.0)):
        db = mix.distance_bias_table(torch.randn(rows, H, generator=g) * 2, far)
        want = mix.masked_attn_rows_ref(q, kc, vc, bt, cu, pos, H, G, scale, 0, None, db)
        tl = ops.prefill_tiles(cu.tolist(), context_lens=ctx.tolist(), tile=128)
        got = mix.paged_prefill_masked(q.cuda(), kc.cuda(), vc.cuda(), bt.cuda(), cu.cuda(), ctx.cuda(), H, G, scale, 0, None,
                                       tiles=torch.tensor(tl, dtype=I32).cuda(), dist_bias=db.cuda())
        close(got, want, 3e-2)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,I,top", [(5, 6, 3, 3), (70, 6, 3, 3), (9, 4, 0, 1), (40, 2, 2, 4), (3, 70, 0, 8), (2, 16, 2, 3), (300, 3, 1, 2)])
def test_moe_routing_and_experts(device, dtype, T, E, I, top):
    g = torch.Generator().manual_seed(7)
    W, ff = 48, 20
    h = torch.randn(T, W, generator=g).to(dtype)
    logits = torch.randn(T, E + I, generator=g) * 2
    corr = torch.randn(E + I, generator=g) * 0.5            # a selection bias large enough to change the choice
    idx, wts = moe.moe_route(logits.to(device), corr.to(device), top)
    s = torch.softmax(logits.double(), -1)
    want_idx = torch.topk(s + corr.double(), top, -1).indices
    assert not torch.equal(want_idx, torch.topk(s, top, -1).indices) or top == E + I
    assert torch.equal(idx.cpu().long(), want_idx)
    close(wts, torch.gather(s, 1, want_idx), 1e-6)           # plain scores, not renormalised
    gu = (torch.randn(E, 2 * ff, W, generator=g) * W ** -0.5).to(dtype)
    dn = (torch.randn(E, W, ff, generator=g) * ff ** -0.5).to(dtype)
    sh = torch.randn(T, W, generator=g).to(dtype)
    P = {"router": torch.zeros(E + I, W, dtype=F64)}
    for e in range(E):
        P[f"e{e}.gate"], P[f"e{e}.up"], P[f"e{e}.down"] = gu[e, :ff].double(), gu[e, ff:].double(), dn[e].double()
    want = sh.double().clone()
    for t in range(T):
        for e, wt in zip(want_idx[t].tolist(), torch.gather(s, 1, want_idx)[t].tolist()):
            want[t] += wt * (h[t].double() if e >= E else orc.glu_expert(P, f"e{e}.", h[t].double()))
    tol = 5e-5 if dtype == torch.float32 else 8e-2
    for shared in (sh, None):
        got = moe.moe_experts(h.to(device), idx, wts, gu.to(device), dn.to(device), None if shared is None else shared.to(device))
        close(got, want if shared is not None else want - sh.double(), tol)


def test_state_pool_slots():
    pool = StatePool(2, {"a": ((3,), torch.float32), "n": ((), torch.int32)})
    assert pool["a"].shape == (3, 3) and pool["n"].shape == (3,)
    s1, s2 = pool.allocate(), pool.allocate()
    assert {s1, s2} == {1, 2} and pool.num_free == 0
    with pytest.raises(OutOfSlots):
        pool.allocate()
    pool.free(s1)
    with pytest.raises(RuntimeError):
        pool.free(s1)
    assert pool.allocate() == s1


# ----------------------------------------------------------------------------------- the model
@pytest.mark.parametrize("device", DEVICES)
def test_layer_streams_match_oracle(device):
    eng = engine(small_cfg(), device)
    t = toks(19, 1)
    runs = eng.model_cfg.layer_runs
    assert runs == [0, 1, 2, 1, 2, 3]
    eng.model.capture_layers = tuple(range(len(runs)))
    got = eng.feed([("a", t, list(range(len(t))))], ["a"])[0]
    eng.model.capture_layers = ()
    lo = []
    want = oracle_logits(eng, t, lo)
    for r in range(len(runs)):
        close(eng.model.captured[r], lo[r], 2e-4 * max(1.0, lo[r].abs().max().item()))
    close(got, want, 3e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("variant", ["base", "one_stream", "no_loop", "wide_taps", "loop3", "all_mamba", "all_attention"])
def test_whole_decode_and_portions_match_oracle(device, variant):
    """Whole prompt, token by token, and portions of several sizes (down to two tokens, across pages):
    all equal the oracle; other stream counts, tap counts and loop settings too."""
    kw = {"base": {}, "one_stream": {"streams": 1, "canon_taps": 1}, "no_loop": {"loop_times": 1},
          "wide_taps": {"canon_taps": 5, "streams": 3}, "loop3": {"loop_start": 0, "loop_stop": 1, "loop_times": 3},
          "all_mamba": {"layers": [l for l in small_cfg().layers if l.type == "mamba2"], "loop_start": 0, "loop_stop": 2},
          "all_attention": {"layers": [l for l in small_cfg().layers if l.type == "attention"], "loop_start": 1,
                            "loop_stop": 2}}[variant]
    eng = engine(small_cfg(**kw), device)
    t = toks(45, 2)
    want = oracle_logits(eng, t)
    close(eng.feed([("w", t, list(range(len(t))))], ["w"])[0], want, 3e-4)
    for name, cuts in (("d", [1]), ("p", [2, 2, 7, 3, 16, 2, 5]), ("q", [30, 2]), ("r", [1, 13])):
        got = feed_all(eng, name, t, cuts)
        eng.feed([], [name])
        close(got, want, 3e-4)
    assert eng.pool.num_used == 0 and eng.state_pool.num_free == 4


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_unequal_batches_reuse_pages_and_slots(device, dtype):
    """Six requests of different lengths through four slots and a pool too small for all of them:
    portions beside single tokens, requests sitting steps out, pages and slots used again — every
    position equals the request run alone."""
    eng = engine(small_cfg(), device, dtype=dtype, num_blocks=40, bs=4)
    solo = engine(small_cfg(), device, dtype=dtype)
    solo.model.copy_from(eng.model)
    lens = {"a": 41, "b": 7, "c": 30, "d": 2, "e": 23, "f": 35}
    seqs = {k: toks(n, 10 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: solo.feed([(k, v, list(range(len(v))))], [k])[0] for k, v in seqs.items()}
    plan = [[("a", 5), ("b", 2)], [("a", 1), ("b", 1), ("c", 9), ("d", 2)], [("a", 17), ("c", 1)],
            [("b", 4), ("c", 2), ("a", 1), ("e", 3)], [("e", 20), ("a", 17)], [("c", 18), ("f", 6)],
            [("f", 1), ("c", 0)], [("f", 28)]]
    at = {k: 0 for k in seqs}
    got = {k: [] for k in seqs}
    for step in plan:
        entries, end = [], []
        for k, n in step:
            part = seqs[k][at[k]:at[k] + n]
            entries.append((k, part, list(range(len(part)))))
            at[k] += n
            if at[k] == len(seqs[k]):
                end.append(k)
        for k, out in zip([e[0] for e in entries], eng.feed(entries, end)):
            got[k].append(out)
    assert at == lens and eng.pool.num_used == 0 and eng.state_pool.num_free == 4
    assert eng.state_pool.stats["allocs"] == 6
    tol = 2e-4 if dtype == torch.float32 else 0.25
    for k in seqs:
        close(torch.cat(got[k], 0), want[k], tol)
    if dtype == torch.float32:
        close(want["a"], oracle_logits(solo, seqs["a"]), 3e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_and_long_decoding(device):
    eng = engine(small_cfg(), device, max_len=256)
    t = toks(140, 5)
    want = oracle_logits(eng, t)
    close(eng.feed([("one", t[:1], [0])], ["one"])[0], want[:1], 2e-4)            # a sequence of one token
    got = feed_all(eng, "x", t, [3])                                              # 137 single-token steps
    close(got, want, 4e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(device):
    eng = engine(small_cfg(), device, max_len=128)
    prompts = [toks(9, 20), toks(17, 21), toks(3, 22)]
    reqs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    assert eng.scheduler.radix is None                   # state-carrying models never resume from shared pages
    P = {k: v.to(F64) for k, v in params(eng.model).items()}
    cd = config_dict(eng.model_cfg)
    for p, r in zip(prompts, reqs):
        seq = list(p)
        for tok in r.output:
            lg = orc.forward(P, cd, seq)[-1]
            top2 = torch.topk(lg, 2).values
            assert tok == int(lg.argmax()) or (top2[0] - top2[1]) < 1e-3
            seq.append(tok)
    assert eng.pool.num_used == 0 and eng.state_pool.num_free == 4


@pytest.mark.gpu
def test_graph_decode_equals_eager_decode():
    """Decode steps replayed as hipGraphs (state slots in the staging image, padded rows on the reserved
    slot, decode lookahead) produce the tokens of the eager engine; replays follow each other with
    eager prompt steps between them."""
    cfg = small_cfg()
    eager, graph = engine(cfg, "cuda", max_len=128), engine(cfg, "cuda", max_len=128, graphs=True)
    graph.model.copy_from(eager.model)
    prompts = [toks(9, 60), toks(17, 61), toks(3, 62)]
    sp = SamplingParams(max_tokens=14, temperature=0.0, ignore_eos=True)
    want = [r.output for r in eager.generate(prompts, sp)]
    for _ in range(2):                                       # a second batch reuses slots and replays again
        assert [r.output for r in graph.generate(prompts, sp)] == want
    assert graph.runner.graphs is not None and graph.runner.graphs.captured
    assert graph.state_pool.num_free == 4 and graph.pool.num_used == 0


@pytest.mark.gpu
def test_mfma_prompt_path_in_the_model(monkeypatch):
    """Layers whose bf16 heads are 64 / 128 wide take the MFMA prompt kernel: same logits as the
    row-wise kernel on the same engine (portions on top of cached tokens, two prompts in one step);
    no experts, so nothing can flip a routing decision."""
    cfg = TifepelConfig(name="t", vocab_size=53, hidden_size=64, layers=[
        LayerSpec("attention", attn(4, 2, 64, 64, 0.125, 0.3, 16, 10, 40.0), None),
        LayerSpec("mamba2", Mamba2Spec(2, 16, 16, 1, 4, 1), None),
        LayerSpec("attention", attn(2, 1, 128, 128, 0.09, 0.0, 0, 8, 200.0), None),
    ], streams=2, canon_taps=4, bigram_buckets=29, bigram_mul_prev=5, bigram_mul_cur=3, max_position=512)
    a, b = toks(200, 70), toks(90, 71)

    def run():
        eng = engine(cfg, "cuda", dtype=torch.bfloat16, num_blocks=64, bs=16, max_len=512)
        out = [eng.feed([("a", a[:150], list(range(150)))]),
               eng.feed([("a", a[150:], list(range(50))), ("b", b, list(range(90)))], ["a", "b"])]
        return torch.cat([o for step in out for o in step], 0)

    assert mix.masked_prefill_available()
    fast = run()
    monkeypatch.setattr(mix, "MASKED_PREFILL", False)
    slow = run()
    close(fast, slow, 0.06 * max(1.0, slow.abs().max().item()))


def test_preempted_sequence_recomputes_its_state():
    """A pool too small for two growing sequences: one is preempted, gives its slot back, and is
    recomputed from position 0 — its tokens equal the undisturbed run."""
    cfg = small_cfg()
    big = engine(cfg, "cpu", max_len=128)
    ref = big.generate([toks(20, 30), toks(22, 31)], SamplingParams(max_tokens=20, temperature=0.0, ignore_eos=True))
    tight = engine(cfg, "cpu", num_blocks=18, bs=4, max_len=128)
    tight.model.copy_from(big.model)
    got = tight.generate([toks(20, 30), toks(22, 31)], SamplingParams(max_tokens=20, temperature=0.0, ignore_eos=True))
    assert tight.scheduler.num_preemptions > 0
    assert [r.output for r in got] == [r.output for r in ref]


def write_checkpoint(eng, path):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config_dict(eng.model_cfg), f)
    save_file({k: (v.to(torch.int32) if v.dtype == torch.int64 else v.to(torch.bfloat16)).contiguous()
               for k, v in params(eng.model).items()}, os.path.join(path, "model.safetensors"))


def test_checkpoint_layout_and_trace_runner(tmp_path):
    """config.json + safetensors in the design's naming -> registry, loader, engine; the replay
    command writes the logits of the wanted places, step by step."""
    src = engine(small_cfg(), "cpu", dtype=torch.bfloat16)          # bf16 weights survive the file bit for bit
    ck = str(tmp_path / "model")
    write_checkpoint(src, ck)
    cfg = get_config(ck)
    assert isinstance(cfg, TifepelConfig) and cfg.layer_runs == [0, 1, 2, 1, 2, 3]
    eng = LLMEngine(EngineConfig(model=ck, device="cpu", dtype=torch.float32, block_size=4, num_blocks=64, max_num_seqs=4,
                                 max_model_len=128, max_num_batched_tokens=128, use_graphs=False, token_align=0))
    assert eng.model_cfg.layers[0].mixer.bias_rows == 10 and eng.model_cfg.layers[2].mixer.bias_rows == 7
    t = toks(21, 40)
    want = oracle_logits(eng, t)
    close(eng.feed([("a", t, list(range(len(t))))], ["a"])[0], want, 3e-4)
    out = tmp_path / "out"
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": t[:6], "want": [0, 5]}, {"id": "y", "tokens": t[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": t[6:7], "want": [0]}], "end": ["y"]},
             {"step": 2, "entries": [{"id": "x", "tokens": t[7:], "want": [13]}], "end": ["x"]}]
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", ck, "--dtype", "float32", "--out",
                        str(out), "--max-tokens", "64", "--device", "cpu"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    import numpy as np
    for step, rows in ((0, [0, 5]), (1, [6]), (2, [20])):
        got = torch.from_numpy(np.fromfile(str(out / f"{step}.f32"), dtype="<f4").reshape(len(rows), -1))
        close(got, want[rows], 3e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_kernels_match_the_reference_ops_on_a_prompt_batch(dtype):
    """The HIP kernels against the CPU reference ops through the same engine code, over a batch of
    portions and decode rows: fp32 within rounding at every position; bf16 at the typical position
    (one expert choice that flips on a close call moves a whole row, so rows are judged by their median)."""
    cfg = small_cfg()
    cpu, gpu = engine(cfg, "cpu", dtype=dtype), engine(cfg, "cuda", dtype=dtype)
    cpu.model.copy_from(gpu.model)
    a, b = toks(50, 50), toks(33, 51)
    for eng in (cpu, gpu):
        eng.out = [eng.feed([("a", a[:40], list(range(40))), ("b", b[:2], [0, 1])]),
                   eng.feed([("a", a[40:41], [0]), ("b", b[2:], list(range(31)))]),
                   eng.feed([("a", a[41:], list(range(9)))], ["a", "b"])]
    x = torch.cat([u for o in cpu.out for u in o], 0)
    y = torch.cat([v for o in gpu.out for v in o], 0).cpu()
    if dtype == torch.float32:
        close(y, x, 3e-4)
    else:
        assert (y - x).abs().amax(1).median().item() < 0.1
