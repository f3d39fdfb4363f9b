"""Plain whole-sequence Tifepel in float64: the oracle of tests/test_tifepel.py.

One function per mechanism, written from the design's equations (see the model's docstring in
``dgi/models/tifepel.py`` for the notation); no cache, no batching, no state carried between calls
and no code shared with the product path.  ``P`` is a dict name -> float64 tensor in the checkpoint
naming (``l<i>.mix.q`` ...), ``cfg`` the parsed ``config.json`` dictionary.
"""
import math

import torch

F = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def embed(P, cfg, tokens):
    """Token row + bigram row + learned position row."""
    bg = cfg["embedding"]["bigram"]
    nb = int(bg["buckets"])
    rows = []
    for p, t in enumerate(tokens):
        if p == 0:
            r = nb
        else:
            r = (tokens[p - 1] * int(bg["mul_prev"]) + t * int(bg["mul_cur"])) % nb
        rows.append(P["embed"][t] + P["bigram"][r] + P["pos"][p])
    return torch.stack(rows)


def causal_taps(h, w, bias=None):
    """out_t = sum_j w[:, j] * h_(t - taps + 1 + j) (+ bias), zeros before the start.  h [T, C], w [C, taps]."""
    T, C = h.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    if bias is not None:
        out = out + bias
    return out


def distance_bucket(n, B, D):
    half = B // 2
    if n < half:
        return n
    return min(B - 1, half + int(math.floor(math.log(n / half) / math.log(D / half) * (B - half))))


def attention(P, pre, m, h, eps):
    T = h.shape[0]
    H, G, dk, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ P[pre + "q"].T).view(T, H, dk)
    k = (h @ P[pre + "k"].T).view(T, G, dk)
    v = (h @ P[pre + "v"].T).view(T, G, dv)
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    qt = m.get("q_temp")
    if qt:
        for p in range(T):
            q[p] = q[p] * (1 + float(qt["coef"]) * math.log((p + 1) // int(qt["every"]) + 1))
    rel = P[pre + "rel"]
    B = rel.shape[0]
    out = torch.zeros(T, H, dv, dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        for i in range(T):
            s = (k[: i + 1, g] @ q[i, hd]) * float(m["scale"])
            for j in range(i + 1):
                s[j] += rel[distance_bucket(i - j, B, float(m["bias_max"])), hd]
            out[i, hd] = torch.softmax(s, 0) @ v[: i + 1, g]
    return out.reshape(T, H * dv) @ P[pre + "o"].T


def mamba2(P, pre, m, h, eps):
    T = h.shape[0]
    nh, dv, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    inner = nh * dv
    u = h @ P[pre + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner: 2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_taps(xbc, P[pre + "conv"], P[pre + "conv.b"]))
    x = xbc[:, :inner].view(T, nh, dv)
    Bm = xbc[:, inner: inner + G * N].view(T, G, N)
    Cm = xbc[:, inner + G * N:].view(T, G, N)
    dt = torch.nn.functional.softplus(dt + P[pre + "dt_bias"], threshold=1e9)
    A = -torch.exp(P[pre + "A_log"])
    y = torch.zeros(T, nh, dv, dtype=F)
    for hd in range(nh):
        g = hd // (nh // G)
        S = torch.zeros(N, dv, dtype=F)
        for t in range(T):
            S = torch.exp(A[hd] * dt[t, hd]) * S + dt[t, hd] * torch.outer(Bm[t, g], x[t, hd])
            y[t, hd] = S.T @ Cm[t, g] + P[pre + "D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    ng = int(m["norm_groups"])
    y = unit_rms(y.view(T, ng, inner // ng), eps).reshape(T, inner) * P[pre + "norm"]
    return y @ P[pre + "o"].T


def glu_expert(P, pre, h):
    return (silu(h @ P[pre + "gate"].T) * (h @ P[pre + "up"].T)) @ P[pre + "down"].T


def moe(P, pre, f, h):
    r = f["router"]
    E, I, top = int(r["experts"]), int(r.get("identity") or 0), int(r["top"])
    s = torch.softmax(h @ P[pre + "router"].T, -1)
    choice = s + P[pre + "correction"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in torch.topk(choice[t], top).indices.tolist():
            out[t] += s[t, e] * (h[t] if e >= E else glu_expert(P, f"{pre}e{e}.", h[t]))
    if f.get("shared"):
        out = out + glu_expert(P, pre + "shared.", h)
    return out


def layer_runs(cfg):
    """Layer indices in execution order (the looped span repeated)."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    a, b, k = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    return list(range(a)) + list(range(a, b)) * k + list(range(b, n))


def sublayer(P, cfg, li, q, xs, fn):
    """Hyper-connected, gated sublayer q (1 mixer, 2 feed-forward) on the streams xs [S, T, W]."""
    eps = float(cfg["norm"]["eps"])
    p = f"l{li}."
    hc = f"{p}hc{q}."
    u = (P[hc + "in"][:, None, None] * xs).sum(0)
    h = layer_norm(u, P[f"{p}norm{q}"], eps)
    gate = torch.sigmoid(h @ P[f"{p}rg{q}"].T + P[f"{p}rg{q}.b"])
    y = fn(h + causal_taps(h, P[f"{p}canon{q}"])) * gate
    return torch.einsum("st,sxw->txw", P[hc + "mix"], xs) + P[hc + "out"][:, None, None] * y


def forward(P, cfg, tokens, layers_out=None):
    """fp64 logits [T, V]; ``layers_out`` (a list) receives the summed streams after every layer run."""
    eps = float(cfg["norm"]["eps"])
    x = embed(P, cfg, tokens)
    xs = x.unsqueeze(0).repeat(int(cfg["streams"]), 1, 1)
    for li in layer_runs(cfg):
        e = cfg["layers"][li]
        pre = f"l{li}.mix."
        m = e["mixer"]
        mixer = {"attention": attention, "mamba2": mamba2}[e["type"]]
        xs = sublayer(P, cfg, li, 1, xs, lambda h: mixer(P, pre, m, h, eps))
        if e.get("mlp") is not None:
            xs = sublayer(P, cfg, li, 2, xs, lambda h: moe(P, f"l{li}.mlp.", e["mlp"], h))
        if layers_out is not None:
            layers_out.append(xs.sum(0))
    return layer_norm(xs.sum(0), P["final.norm"], eps) @ P["head"].T
