"""Mixture-of-experts feed-forward ops (``dgi/_C_mix.so``): routing, expert evaluation, combine.

Routing is fp32: scores s = softmax(logits) over all routes (real experts, then identity
experts), the ``top`` routes by s + selection bias are taken and weighed by s itself (not
renormalised).  A real expert e is W_down[e] (silu(W_gate[e] h) * (W_up[e] h)); an identity
route returns h.  Expert weights are stacked: ``gate_up`` [E, 2 ff, W] (gate rows, then up rows)
and ``down`` [E, W, ff].

Two evaluation paths on the GPU, same result up to summation order:

* few rows (decode steps, and every step inside a captured graph; no host round trip): when the step's
  (token, route) pairs are at least as many as the experts, all experts run as one batched vendor GEMM
  over the step's rows and the combine kernel picks each token's routes; with fewer pairs, workgroups own
  (expert, output tile) and walk the pairs that chose the expert, so only the chosen experts' rows stream
  from the stacked weights;
* many rows (prompt portions): pairs are sorted by expert, every expert with tokens runs the
  vendor GEMM over its contiguous segment, and a combine kernel gathers each token's routes in
  their fixed order (deterministic, no atomics).

CPU tensors run ``*_ref`` (fp32), the oracle of the kernel tests.
"""
from __future__ import annotations

import os

import torch

from dgi.ops.mix import _call, _native

# rows up to which the expert-major kernels evaluate the experts (above: sorted segments + GEMMs)
EXPERT_MAJOR_ROWS = int(os.environ.get("DGI_MOE_EXPERT_MAJOR_ROWS", "64"))


def silu_mul_ref(gu: torch.Tensor) -> torch.Tensor:
    I = gu.shape[-1] // 2
    g = gu[..., :I].float()
    return (g * torch.sigmoid(g) * gu[..., I:].float()).to(gu.dtype)


def silu_mul(gu: torch.Tensor) -> torch.Tensor:
    """silu(g) * u over fused [gate | up] rows."""
    if _native(gu):
        out = torch.empty(gu.shape[0], gu.shape[1] // 2, dtype=gu.dtype, device=gu.device)
        _call("glu_silu", out, gu)
        return out
    return silu_mul_ref(gu)


def moe_route_ref(logits, correction, top):
    s = torch.softmax(logits.float(), -1)
    idx = torch.topk(s + correction, top, dim=-1).indices
    return idx.to(torch.int32), torch.gather(s, 1, idx)


def moe_route(logits: torch.Tensor, correction: torch.Tensor, top: int):
    """fp32 ``logits`` [T, R] -> (routes [T, top] int32 ordered by falling s + correction,
    weights [T, top] fp32 = the plain softmax scores of those routes)."""
    if _native(logits):
        T = logits.shape[0]
        idx = torch.empty(T, top, dtype=torch.int32, device=logits.device)
        w = torch.empty(T, top, dtype=torch.float32, device=logits.device)
        _call("moe_route", idx, w, logits, correction)
        return idx, w
    return moe_route_ref(logits, correction, top)


def moe_experts_ref(h, idx, wts, gate_up, down, shared):
    T, W = h.shape
    E = gate_up.shape[0]
    ff = down.shape[2]
    hf = h.float()
    out = torch.zeros(T, W) if shared is None else shared.float().clone()
    for t in range(T):
        for e, w in zip(idx[t].tolist(), wts[t].tolist()):
            if e >= E:
                out[t] += w * hf[t]
            else:
                gu = gate_up[e].float() @ hf[t]
                g, u = gu[:ff], gu[ff:]
                out[t] += w * (down[e].float() @ (g * torch.sigmoid(g) * u))
    return out.to(h.dtype)


def moe_experts(h, idx, wts, gate_up, down, shared=None) -> torch.Tensor:
    """sum_k wts[t, k] * route_{idx[t, k]}(h_t) (+ ``shared`` [T, W]) in h's dtype."""
    if not _native(h):
        return moe_experts_ref(h, idx, wts, gate_up, down, shared)
    T, W = h.shape
    E, ff = gate_up.shape[0], down.shape[2]
    top = idx.shape[1]
    out = torch.empty(T, W, dtype=h.dtype, device=h.device)
    if T <= EXPERT_MAJOR_ROWS or torch.cuda.is_current_stream_capturing():
        if T * top >= E:
            # a small step that touches (nearly) every expert anyway: all experts as one batched vendor GEMM
            # over the step's rows (weight-bandwidth bound either way; the extra FLOPs are free at these
            # sizes), then every token picks its routes' rows in the combine
            gu = torch.matmul(h.unsqueeze(0), gate_up.transpose(1, 2))                  # [E, T, 2 ff]
            act = silu_mul(gu.view(E * T, 2 * ff))
            ys = torch.bmm(act.view(E, T, ff), down.transpose(1, 2)).view(E * T, W)
            where = (idx * T + torch.arange(T, dtype=torch.int32, device=h.device)[:, None]).clamp_(0, E * T - 1)
            _call("moe_combine", out, ys, where, h, idx, wts, shared, E)
            return out
        mid = torch.empty(T * top, ff, dtype=torch.float32, device=h.device)
        ys = torch.empty(T * top, W, dtype=h.dtype, device=h.device)     # identity pairs' rows are never read
        _call("moe_expert_gate_up", mid, h, idx, gate_up)
        _call("moe_expert_down", ys, mid, idx, down)
        _call("moe_combine", out, ys, None, h, idx, wts, shared, E)
        return out
    from dgi import ops
    flat = idx.reshape(-1).long()
    order = torch.argsort(flat, stable=True)                       # pairs grouped by route
    counts = torch.bincount(flat, minlength=E).tolist()            # host: segment sizes
    xs = h.index_select(0, order // top)
    ys = torch.empty(T * top, W, dtype=h.dtype, device=h.device)   # identity segments are never read
    o = 0
    for e in range(E):
        c = counts[e]
        if c:
            act = silu_mul(ops.linear(xs[o:o + c], gate_up[e]))
            torch.matmul(act, down[e].t(), out=ys[o:o + c])
            o += c
    where = torch.empty_like(order)
    where[order] = torch.arange(order.numel(), device=order.device)
    _call("moe_combine", out, ys, where.to(torch.int32), h, idx, wts, shared, E)
    return out
