"""Ops of models that carry per-sequence state and several residual streams (``dgi/_C_mix.so``):
hashed-bigram + position embedding, hyper-connected stream mixing fused with the next layer norm,
causal convolutions over packed rows with their tails in state slots, the Mamba-2 selective scan
and its gated group norm.

Same rules as ``dgi.ops.mix``: GPU tensors run the HIP kernel (and raise if the library is
missing), CPU tensors the ``*_ref`` function in fp32, which is also the kernel tests' oracle.

Rows of a step are ``[decode rows | prompt portions]``; ``row_seq`` [T] names each row's sequence
of the step, ``seq_row0`` [n + 1] the first row of each sequence, ``seq_slots`` [n] its slot in the
state tensors (``dgi.kv.state_pool``).  A portion that starts at position 0 reads no state.
"""
from __future__ import annotations

import os
from typing import Optional

import torch

from dgi.ops.mix import _call, _native


def _seqs(positions, seq_row0, seq_slots):
    """(first row, end row, slot, first position) of every sequence of the step (host lists)."""
    r0 = seq_row0.tolist()
    sl = seq_slots.tolist()
    pos = positions.tolist()
    return [(r0[i], r0[i + 1], sl[i], pos[r0[i]] if r0[i + 1] > r0[i] else 0) for i in range(len(sl))]


# ----------------------------------------------------------------------------
# Embedding: token row + hashed bigram row + position row, copied into S streams
# ----------------------------------------------------------------------------

def embed_streams_ref(ids, positions, row_seq, seq_row0, seq_slots, prev_tok, embed, bigram, pos_table, buckets, mul_prev,
                      mul_cur, streams):
    T = ids.shape[0]
    x = embed[ids.long()].float()
    if pos_table is not None:
        x = x + pos_table[positions.long()].float()
    if bigram is not None:
        prev = torch.zeros(T, dtype=torch.long)
        prev[1:] = ids[:-1].long()
        rows = (prev * mul_prev + ids.long() * mul_cur) % buckets
        for r0, r1, slot, p0 in _seqs(positions, seq_row0, seq_slots):
            if r1 > r0:
                rows[r0] = buckets if p0 == 0 else (int(prev_tok[slot]) * mul_prev + int(ids[r0]) * mul_cur) % buckets
        x = x + bigram[rows].float()
    for r0, r1, slot, _p0 in _seqs(positions, seq_row0, seq_slots):
        if r1 > r0:
            prev_tok[slot] = int(ids[r1 - 1])
    return x.unsqueeze(0).repeat(streams, 1, 1).contiguous()


def embed_streams(ids, positions, row_seq, seq_row0, seq_slots, prev_tok, embed, bigram, pos_table, buckets: int,
                  mul_prev: int, mul_cur: int, streams: int) -> torch.Tensor:
    """fp32 streams [S, T, W], each embed[id] + bigram[(prev * mul_prev + id * mul_cur) mod buckets]
    + pos_table[position]; a sequence's first token takes bigram row ``buckets``.  The previous
    token of a portion's first row comes from ``prev_tok[slot]`` (int32), which then receives the
    portion's last token.  ``bigram`` / ``pos_table`` may be None."""
    if _native(embed):
        T, W = ids.shape[0], embed.shape[1]
        xs = torch.empty(streams, T, W, dtype=torch.float32, device=embed.device)
        _call("embed_streams", xs, ids, positions, row_seq, seq_row0, seq_slots, prev_tok, embed, bigram, pos_table,
              int(buckets), int(mul_prev), int(mul_cur))
        return xs
    return embed_streams_ref(ids, positions, row_seq, seq_row0, seq_slots, prev_tok, embed, bigram, pos_table, buckets,
                             mul_prev, mul_cur, streams)


# ----------------------------------------------------------------------------
# Hyper-connections: stream update of one sublayer + read-out and layer norm of the next
# ----------------------------------------------------------------------------

def hc_mix_norm_ref(xs, y, gate, gate_b, mix, out, in_next, norm_w, eps, dtype):
    if y is not None:
        yy = y.float()
        if gate is not None:
            yy = yy * torch.sigmoid(gate.float() + gate_b)
        new = torch.einsum("st,sxw->txw", mix, xs) + out[:, None, None] * yy
        xs.copy_(new)
    if in_next is None:
        return None, None
    u = (in_next[:, None, None] * xs).sum(0)
    mu = u.mean(-1, keepdim=True)
    var = ((u - mu) ** 2).mean(-1, keepdim=True)
    h = (u - mu) / torch.sqrt(var + eps) * norm_w
    return h, h if dtype == torch.float32 else h.to(dtype)


def hc_mix_norm(xs, y, gate, gate_b, mix, out, in_next, norm_w, eps: float, dtype):
    """One pass over the fp32 streams ``xs`` [S, T, W]:

    * with ``y`` [T, W] (a sublayer's output): x_t <- sum_s mix[s, t] x_s + out[t] * y * sigmoid(gate + gate_b)
      for all streams at once, in place (``gate`` None: no gate);
    * with ``in_next`` [S]: u = sum_s in_next[s] x_s and the weight-only layer norm
      h = (u - mean) / sqrt(var + eps) * norm_w, returned as (h fp32, h in ``dtype``) — the next
      sublayer's input (the second is the first when ``dtype`` is fp32)."""
    if _native(xs):
        S, T, W = xs.shape
        h32 = hd = None
        if in_next is not None:
            h32 = torch.empty(T, W, dtype=torch.float32, device=xs.device)
            hd = h32 if dtype == torch.float32 else torch.empty(T, W, dtype=dtype, device=xs.device)
        _call("hc_mix_norm", xs, y, gate, gate_b, mix, out, in_next, norm_w, float(eps), h32,
              None if hd is h32 else hd)
        return h32, hd
    return hc_mix_norm_ref(xs, y, gate, gate_b, mix, out, in_next, norm_w, eps, dtype)


# ----------------------------------------------------------------------------
# Causal convolution over packed rows, tails in state slots
# ----------------------------------------------------------------------------

def causal_conv_ref(x, w, bias, tail, positions, seq_row0, seq_slots, act, residual, out_dtype):
    T, C = x.shape
    taps = w.shape[1]
    xf = x.float()
    out = torch.zeros(T, C)
    for r0, r1, slot, p0 in _seqs(positions, seq_row0, seq_slots):
        n = r1 - r0
        if n == 0:
            continue
        hist = torch.zeros(taps - 1, C) if (p0 == 0 or taps == 1) else tail[slot].clone()
        if 0 < p0 < taps - 1:
            hist[: taps - 1 - p0] = 0          # before the sequence's start
        full = torch.cat([hist, xf[r0:r1]], 0)               # positions p0 - (taps - 1) ... p0 + n - 1
        acc = torch.zeros(n, C)
        for j in range(taps):
            acc += w[:, j] * full[j: j + n]
        if bias is not None:
            acc = acc + bias
        if act == 1:
            acc = acc * torch.sigmoid(acc)
        out[r0:r1] = acc + xf[r0:r1] if residual else acc
        if taps > 1:
            tail[slot] = full[n:]
    return out.to(out_dtype)


def causal_conv(x, w, bias, tail, positions, row_seq, seq_row0, seq_slots, act: int = 0, residual: bool = False,
                out_dtype=None) -> torch.Tensor:
    """Per-channel causal convolution over time of the packed rows ``x`` [T, C] (unit column
    stride; fp32 or the activation dtype): out_t = sum_j w[:, j] * x_(t - taps + 1 + j) (+ bias),
    zeros before position 0, ``act`` 1: SiLU, ``residual``: + x_t.  Inputs older than the portion come
    from ``tail`` [slots, taps - 1, C] (fp32, the sequence's last taps - 1 inputs), which is
    brought up to date afterwards.  fp32 math."""
    out_dtype = out_dtype or x.dtype
    if _native(x):
        out = torch.empty(x.shape[0], x.shape[1], dtype=out_dtype, device=x.device)
        _call("causal_conv", out, x, w, bias, tail, positions, row_seq, seq_row0, seq_slots, int(act), bool(residual))
        return out
    return causal_conv_ref(x, w, bias, tail, positions, seq_row0, seq_slots, act, residual, out_dtype)


# ----------------------------------------------------------------------------
# Mamba-2 selective scan and gated group norm
# ----------------------------------------------------------------------------

def ssm_scan_ref(xbc, dt_raw, dt_bias, a_log, d_skip, state, positions, seq_row0, seq_slots, heads, dv, N, G):
    T = xbc.shape[0]
    inner = heads * dv
    x = xbc[:, :inner].float().view(T, heads, dv)
    Bm = xbc[:, inner: inner + G * N].float().view(T, G, N).repeat_interleave(heads // G, 1)
    Cm = xbc[:, inner + G * N: inner + 2 * G * N].float().view(T, G, N).repeat_interleave(heads // G, 1)
    dt = torch.nn.functional.softplus(dt_raw.float() + dt_bias, threshold=1e9)      # [T, heads]
    dA = torch.exp(-torch.exp(a_log) * dt)
    y = torch.zeros(T, heads, dv)
    for r0, r1, slot, p0 in _seqs(positions, seq_row0, seq_slots):
        if r1 == r0:
            continue
        S = torch.zeros(heads, N, dv) if p0 == 0 else state[slot].transpose(1, 2).clone()
        for t in range(r0, r1):
            S = dA[t, :, None, None] * S + dt[t, :, None, None] * Bm[t, :, :, None] * x[t, :, None, :]
            y[t] = torch.einsum("hnv,hn->hv", S, Cm[t]) + d_skip[:, None] * x[t]
        state[slot] = S.transpose(1, 2)
    return y.reshape(T, inner)


SCAN_CHUNK = int(os.environ.get("DGI_SCAN_CHUNK", "128"))       # rows per chunk of the chunked scan (0: off)
SCAN_WS_BYTES = 512 << 20                                      # largest chunk-state workspace
SCAN_CHUNK_BELOW = int(os.environ.get("DGI_SCAN_CHUNK_BELOW", "512"))   # one-pass workgroups below which steps are chunked


def ssm_scan(xbc, dt_raw, dt_bias, a_log, d_skip, state, positions, seq_row0, seq_slots, heads: int, dv: int,
             N: int, G: int, chunked=None) -> torch.Tensor:
    """Mamba-2 recurrence over packed rows.  ``xbc`` [T, heads*dv + 2*G*N] fp32 = x | B | C (after the
    convolution), ``dt_raw`` [T, heads] the projected step sizes; per head h (group floor(h / (heads/G))):
    dt = softplus(dt_raw + dt_bias), S <- exp(-exp(a_log) dt) S + dt B x^T, y = S^T C + d_skip x, with
    S [N, dv] in fp32 read from / written to ``state`` [slots, heads, dv, N] (value-major; zero at position 0).
    Returns y [T, heads*dv] fp32.

    On the GPU a step with long portions of few sequences runs in chunks of ``SCAN_CHUNK`` rows in
    parallel (local chunk states, a serial pass over them, outputs from each chunk's incoming state)
    when the model is bf16 (``chunked`` None) — the same recurrence with its fp32 sums reassociated;
    fp32 models, short steps and steps with enough sequences to fill the chip run each sequence in one pass."""
    if _native(xbc):
        T, n_seq = xbc.shape[0], seq_slots.shape[0]
        y = torch.empty(T, heads * dv, dtype=torch.float32, device=xbc.device)
        longest = T - n_seq + 1                       # no portion is longer (every sequence has a row)
        L = SCAN_CHUNK
        if chunked is None:
            # worth twice the recurrence work only while one-pass workgroups (sequence x head x 16 columns)
            # cannot fill the chip: measured slower than one pass from 512 workgroups on
            chunked = dt_raw.dtype != torch.float32 and n_seq * heads * -(-dv // 16) < SCAN_CHUNK_BELOW
        if chunked and L > 0 and longest >= 4 * L:
            nch = -(-longest // L)
            if n_seq * nch * heads * dv * N * 4 <= SCAN_WS_BYTES:
                ws = torch.empty(n_seq * nch * heads * dv * N, dtype=torch.float32, device=xbc.device)
                wsd = torch.empty(n_seq * nch * heads, dtype=torch.float32, device=xbc.device)
                _call("ssm_scan", y, xbc, dt_raw, dt_bias, a_log, d_skip, state, positions, seq_row0, seq_slots,
                      heads, dv, N, G, ws, wsd, L, nch)
                return y
        _call("ssm_scan", y, xbc, dt_raw, dt_bias, a_log, d_skip, state, positions, seq_row0, seq_slots, heads, dv, N, G)
        return y
    return ssm_scan_ref(xbc, dt_raw, dt_bias, a_log, d_skip, state, positions, seq_row0, seq_slots, heads, dv, N, G)


def gated_group_norm_ref(y, z, w, groups, eps, dtype):
    T, C = y.shape
    zf = z.float()
    g = (y.float() * zf * torch.sigmoid(zf)).view(T, groups, C // groups)
    g = g / torch.sqrt(g.pow(2).mean(-1, keepdim=True) + eps)
    return (g.reshape(T, C) * w).to(dtype)


def gated_group_norm(y, z, w, groups: int, eps: float, dtype) -> torch.Tensor:
    """(y * silu(z)) divided by its root mean square in ``groups`` equal parts of a row, times w."""
    if _native(y):
        out = torch.empty(y.shape[0], y.shape[1], dtype=dtype, device=y.device)
        _call("gated_group_norm", out, y, z, w, int(groups), float(eps))
        return out
    return gated_group_norm_ref(y, z, w, groups, eps, dtype)
