"""A plain, slow Bebovik written from the design's equations (float64, whole sequences, no
cache, no batching): the oracle the framework's Bebovik path is tested against.  One function
per mechanism; nothing here imports the product code.

Notation: x is a [T, W] stream; a layer is x += ls1 * N1b(Mix(N1(x))), x += ls2 * N2b(FF(N2(x))).
"""
import math

import torch

F64 = torch.float64


def dyt(x, alpha, w, b):
    """Dynamic-Tanh norm: tanh(alpha x) w + b."""
    return torch.tanh(alpha.to(F64) * x) * w.to(F64) + b.to(F64)


def unit_rms(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w.to(F64)


def rotary_freqs(base, dims, scaling=None):
    """f_i = base^(-2i/dims); wavelength-dependent rescale (factor, low, high, original)."""
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if scaling:
        o, lo, hi, fac = scaling["original"], scaling["low"], scaling["high"], scaling["factor"]
        out = []
        for fi in f:
            lam = 2 * math.pi / fi
            if lam < o / hi:
                out.append(fi)
            elif lam > o / lo:
                out.append(fi / fac)
            else:
                s = (o / lam - lo) / (hi - lo)
                out.append((1 - s) * fi / fac + s * fi)
        f = out
    return torch.tensor(f, dtype=F64)


def rotate_pairs(x, pos, freqs):
    """Pairs (2i, 2i+1) of the first 2*len(freqs) dims of x [T, heads, d] turn by pos * f_i."""
    rd = 2 * len(freqs)
    out = x.clone()
    for t in range(x.shape[0]):
        for i in range(rd // 2):
            a = float(pos[t]) * float(freqs[i])
            c, s = math.cos(a), math.sin(a)
            u, v = x[t, :, 2 * i].clone(), x[t, :, 2 * i + 1].clone()
            out[t, :, 2 * i] = u * c - v * s
            out[t, :, 2 * i + 1] = v * c + u * s
    return out


def visible(i, j, chunk):
    """Key j for query i: causal, and in the same block of `chunk` positions (0: causal only)."""
    return j <= i and (chunk <= 0 or i // chunk == j // chunk)


def attention_mixer(h, p, m, eps, pos0=0):
    """h [T, W] -> [T, W].  p: the layer's tensors; m: dict(heads, kv_heads, dim, vdim, scale,
    rot_dims, base, scaling, chunk)."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ p["q"].to(F64).T).view(T, H, dk)
    k = (h @ p["k"].to(F64).T).view(T, G, dk)
    v = (h @ p["v"].to(F64).T).view(T, G, dv)
    q, k = unit_rms(q, p["q_norm"], eps), unit_rms(k, p["k_norm"], eps)
    if m["rot_dims"]:
        fr = rotary_freqs(m["base"], m["rot_dims"], m["scaling"])
        pos = list(range(pos0, pos0 + T))
        q, k = rotate_pairs(q, pos, fr), rotate_pairs(k, pos, fr)
    o = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        keys = [j for j in range(T) if visible(i, j, m["chunk"])]
        for hh in range(H):
            g = hh // (H // G)
            s = torch.stack([(q[i, hh] * k[j, g]).sum() * m["scale"] for j in keys])
            w = torch.softmax(s, 0)
            o[i, hh] = sum(w[n] * v[j, g] for n, j in enumerate(keys))
    o = o.reshape(T, H * dv)
    if p["g"].numel():                      # output gate from the mixer's own input
        o = o * torch.sigmoid(h @ p["g"].to(F64).T)
    return o @ p["o"].to(F64).T


def feed_forward(h, p, limit):
    g = torch.clamp(h @ p["gate"].to(F64).T, max=limit)
    u = torch.clamp(h @ p["up"].to(F64).T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ p["down"].to(F64).T


def forward(tokens, P, C):
    """Logits [T, V] (float64) of the whole sequence.  P: tensors by plain names, C: constants."""
    x = P["embed"].to(F64)[torch.tensor(tokens)] * C["embedding_scale"]
    x = dyt(x, *P["embed_norm"])
    streams = []
    for L, m in zip(P["layers"], C["layers"]):
        x = x + dyt(attention_mixer(dyt(x, *L["norm1"]), L, m, C["eps"]), *L["norm1b"]) * L["ls1"].to(F64)
        if m["ff"]:
            x = x + dyt(feed_forward(dyt(x, *L["norm2"]), L, m["limit"]), *L["norm2b"]) * L["ls2"].to(F64)
        streams.append(x.clone())
    lg = dyt(x, *P["final_norm"]) @ P["head"].to(F64).T * C["logit_scale"]
    cap = C["logit_softcap"]
    return (cap * torch.tanh(lg / cap) if cap > 0 else lg), streams


def from_model(model):
    """Plain tensors and constants of a framework model object (read, not computed)."""
    c = model.cfg
    P = {"embed": model.embed.float().cpu(), "head": model.head.float().cpu(), "layers": []}
    n3 = lambda n: tuple(t.float().cpu() for t in (n.alpha, n.w, n.b))      # noqa: E731
    P["embed_norm"], P["final_norm"] = n3(model.embed_norm), n3(model.final_norm)
    C = {"embedding_scale": c.embedding_scale, "logit_scale": c.logit_scale, "logit_softcap": c.logit_softcap,
         "eps": c.norm_eps, "layers": []}
    for L in model.layers:
        m = L.spec.mixer
        w = L.qkvg.float().cpu()
        a, b, d = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
        lay = {"q": w[:a], "k": w[a:a + b], "v": w[a + b:a + b + d], "g": w[a + b + d:], "o": L.o.float().cpu(),
               "q_norm": L.q_norm.cpu(), "k_norm": L.k_norm.cpu(), "norm1": n3(L.norm1), "norm1b": n3(L.norm1b),
               "ls1": L.ls1.cpu()}
        ff = 0
        if L.gate_up is not None:
            ff = L.spec.mlp.ff
            gu = L.gate_up.float().cpu()
            lay.update(gate=gu[:ff], up=gu[ff:], down=L.down.float().cpu(), norm2=n3(L.norm2), norm2b=n3(L.norm2b),
                       ls2=L.ls2.cpu())
        P["layers"].append(lay)
        C["layers"].append({"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                            "rot_dims": m.rot.dims if m.rot else 0, "base": m.rot.base if m.rot else 0.0,
                            "scaling": m.rot.scaling if m.rot else None,
                            "chunk": m.mask_size if m.mask_kind == "chunk" else 0, "ff": ff,
                            "limit": L.spec.mlp.limit if ff else 0.0})
    return P, C
