"""Native Tifepel decoder for the MI355X runtime.

Notation (T rows of a step, W the width, S residual streams x_1..x_S, all fp32):

    embedding   e_t = E[tok_t] + Bg[(tok_(t-1) * a + tok_t * b) mod n] + P[pos_t]   (first token: Bg[n]);
                every stream starts as e
    sublayer q of a layer (q = 1 mixer, q = 2 feed-forward):
                u  = sum_s in_q[s] x_s
                h  = LN(u) * w_q                       weight-only layer norm
                g  = sigmoid(R_q h + r_q)              output gate, from h
                c  = h + conv_q(h)                     causal per-channel convolution over time
                y  = F_q(c) * g
                x_t <- sum_s mix_q[s, t] x_s + out_q[t] y      all streams at once
    logits      head(LN(sum_s x_s) * w_f)

F_1 is softmax attention without rotation — unit-RMS q and k per head, q scaled by a slowly growing
function of the position, a learned bias per (distance bucket, head) added to the scaled scores —
or a Mamba-2 mixer (input projection -> z | x | B | C | dt, causal convolution + SiLU over x | B | C,
the selective scan with an fp32 state per head, gate by silu(z), group RMS norm, output projection).
F_2 is a mixture of experts with identity routes and a shared expert (``dgi.ops.moe``).  A span of
layers may run several times with the same weights; every layer RUN has its own cache pages
(attention) or state (Mamba-2, convolution tails).

Per layer run the step executes (rows: decode rows first, then packed prompt portions)::

    hc_mix_norm (HIP)      previous sublayer's stream update + this sublayer's u, LN  -> h fp32 (+ bf16)
    gate GEMM              R h                                 (bias and sigmoid live in the next hc_mix_norm)
    causal_conv (HIP)      c = h + conv(h), tail in the sequence's state slot
    attention:  q|k|v GEMM -> qknorm_rope_cache (HIP: unit RMS, q temperature, paged K/V write)
                -> masked_attn_rows (HIP, distance bias; prompt rows of bf16 64 / 128-dim heads: the MFMA
                   flash kernel with the same bias) -> o GEMM
    mamba2:     in GEMM -> causal_conv (HIP, bias + SiLU, fp32 out) -> ssm_scan (HIP, fp32 state in the slot)
                -> gated_group_norm (HIP) -> o GEMM
    moe:        router GEMM (fp32) -> moe_route (HIP) -> experts (HIP pair kernels or sorted segment GEMMs)
                + shared expert (GEMM, silu_mul, GEMM)

Streams, norms, scores / softmax, the router, the scan (state, decays, step sizes) and the
convolutions are fp32 whatever ``dtype`` is; with bf16 the projections and expert GEMMs take bf16
inputs with fp32 accumulation.  Pages come from the engine's block pool (one page geometry per
attention run), everything else a sequence carries from ``dgi.kv.state_pool.StatePool``.
"""
from __future__ import annotations

from typing import Optional

import torch

from dgi import ops
from dgi.models.config import TifepelConfig
from dgi.ops import mix, moe, recur
from dgi.runtime.batch import AttnMeta


class TifepelLayerWeights:
    FIELDS = ("norm1", "norm2", "canon1", "canon2", "rg1", "rg1_b", "rg2", "rg2_b", "hc1_in", "hc1_out", "hc1_mix",
              "hc2_in", "hc2_out", "hc2_mix", "qkv", "o", "rel", "in_proj", "conv", "conv_b", "dt_bias", "a_log",
              "d_skip", "mnorm", "router", "correction", "gate_up", "down", "shared_gate_up", "shared_down")
    __slots__ = ("spec", "dist_bias") + FIELDS

    def __init__(self):
        for k in self.__slots__:
            setattr(self, k, None)

    def named(self):
        for k in self.FIELDS:
            t = getattr(self, k)
            if t is not None:
                yield k, t


class TifepelModel:
    """A Tifepel causal LM (all layers on one device)."""

    routes_gemms = False       # projections are plain vendor GEMMs: no start-up routing table

    def __init__(self, cfg: TifepelConfig, device: torch.device | str = "cpu", dtype=torch.bfloat16,
                 layer_start: int = 0, layer_end: Optional[int] = None, has_embed: Optional[bool] = None,
                 has_head: Optional[bool] = None, seed: int = 0, init: str = "random",
                 checkpoint: Optional[str] = None):
        if layer_start != 0 or (layer_end is not None and layer_end != cfg.num_layers):
            raise ValueError("Tifepel runs all its layers in one stage (a looped span cannot be cut)")
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.layer_start, self.layer_end = 0, cfg.num_layers
        self.has_embed = self.has_head = True
        self.num_local_layers = cfg.num_layers
        self.runs = cfg.layer_runs
        self.kv_cache = None
        self.kv_layers: list = []
        self.state = None
        self.layers: list[TifepelLayerWeights] = []
        self.embed = self.bigram = self.pos = self.head = self.final_norm = None
        self.capture_layers: tuple = ()
        self.captured: dict = {}
        self.layer_hook = None
        self.reduce = None
        self.mlp_pad = self.mlp_impl = self.proj_impl = self.fold_impl = None
        self.load_info: Optional[dict] = None
        if checkpoint:
            from dgi.models.weights import load_tifepel_checkpoint, tifepel_bias_rows
            tifepel_bias_rows(cfg, checkpoint)
        self._init_empty()
        if checkpoint:
            self.load_info = load_tifepel_checkpoint(self, checkpoint)
        elif init == "random":
            self._init_random(seed)
        self.finish_weights()
        # page-pool layer of every attention run
        self.kv_index = {}
        for r, li in enumerate(self.runs):
            if cfg.layers[li].type == "attention":
                self.kv_index[r] = len(self.kv_index)
        self._ones = torch.ones(cfg.streams, device=self.device)

    # ------------------------------------------------------------------ weights
    def _init_empty(self):
        c, dev, dt = self.cfg, self.device, self.dtype
        W, S, f32 = c.hidden_size, c.streams, torch.float32

        def e(*shape, dtype=dt):
            return torch.zeros(*shape, device=dev, dtype=dtype)

        for spec in c.layers:
            L = TifepelLayerWeights()
            L.spec = spec
            m = spec.mixer
            for q in ("1", "2") if spec.mlp is not None else ("1",):
                setattr(L, "norm" + q, torch.ones(W, device=dev))
                if c.canon_taps > 0:
                    setattr(L, "canon" + q, e(W, c.canon_taps, dtype=f32))
                setattr(L, f"rg{q}", e(W, W))
                setattr(L, f"rg{q}_b", e(W, dtype=f32))
                setattr(L, f"hc{q}_in", e(S, dtype=f32))
                setattr(L, f"hc{q}_out", e(S, dtype=f32))
                setattr(L, f"hc{q}_mix", e(S, S, dtype=f32))
            if spec.type == "attention":
                L.qkv = e(m.q_size + m.k_size + m.v_size, W)
                L.o = e(W, m.o_size)
                if m.bias_rows:
                    L.rel = e(max(m.bias_rows, 2), m.heads, dtype=f32)
            else:
                L.in_proj = e(m.in_size, W)
                L.conv = e(m.conv_channels, m.conv, dtype=f32)
                L.conv_b = e(m.conv_channels, dtype=f32)
                L.dt_bias, L.a_log, L.d_skip = e(m.heads, dtype=f32), e(m.heads, dtype=f32), e(m.heads, dtype=f32)
                L.mnorm = torch.ones(m.inner, device=dev)
                L.o = e(W, m.inner)
            f = spec.mlp
            if f is not None:
                L.router = e(f.routes, W, dtype=f32)
                L.correction = e(f.routes, dtype=f32)
                L.gate_up = e(f.experts, 2 * f.ff, W)
                L.down = e(f.experts, W, f.ff)
                if f.shared_ff:
                    L.shared_gate_up = e(2 * f.shared_ff, W)
                    L.shared_down = e(W, f.shared_ff)
            self.layers.append(L)
        self.embed = e(c.vocab_size, W)
        if c.bigram_buckets > 0:
            self.bigram = e(c.bigram_buckets + 1, W)
        self.pos = e(c.max_position, W)
        self.final_norm = torch.ones(W, device=dev)
        self.head = e(c.vocab_size, W)

    def _init_random(self, seed: int):
        """Deterministic per-tensor values drawn on the CPU (the same on every device)."""
        c = self.cfg
        W, S = c.hidden_size, c.streams
        gen = torch.Generator()

        def fill(t, std, mean=0.0):
            if t is not None:
                t.copy_((torch.randn(t.shape, generator=gen) * std + mean).to(t.dtype))

        for li, L in enumerate(self.layers):
            gen.manual_seed(seed * 1000003 + li * 7919 + 1)
            for q in ("1", "2"):
                fill(getattr(L, "norm" + q), 0.1, 1.0)
                fill(getattr(L, "canon" + q), 0.2)
                fill(getattr(L, "rg" + q), W ** -0.5)
                fill(getattr(L, f"rg{q}_b"), 0.2, 0.5)
                fill(getattr(L, f"hc{q}_in"), 0.1, 1.0 / S)
                fill(getattr(L, f"hc{q}_out"), 0.1, 0.5)
                mx = getattr(L, f"hc{q}_mix")
                if mx is not None:
                    mx.copy_(0.8 * torch.eye(S) + torch.randn(S, S, generator=gen) * 0.1)
            fill(L.qkv, W ** -0.5)
            fill(L.o, L.o.shape[1] ** -0.5)
            fill(L.rel, 0.5)
            fill(L.in_proj, W ** -0.5)
            fill(L.conv, 0.3)
            fill(L.conv_b, 0.1)
            fill(L.dt_bias, 0.5, -1.0)
            fill(L.a_log, 0.3, -0.5)
            fill(L.d_skip, 0.2, 0.5)
            fill(L.mnorm, 0.1, 1.0)
            fill(L.router, W ** -0.5 * 2)
            fill(L.correction, 0.05)
            fill(L.gate_up, W ** -0.5)
            if L.down is not None:
                fill(L.down, L.down.shape[2] ** -0.5)
            fill(L.shared_gate_up, W ** -0.5)
            if L.shared_down is not None:
                fill(L.shared_down, L.shared_down.shape[1] ** -0.5)
        gen.manual_seed(seed * 1000003 + 17)
        fill(self.embed, 1.0)
        fill(self.bigram, 0.5)
        fill(self.pos, 0.3)
        fill(self.head, W ** -0.5)
        fill(self.final_norm, 0.1, 1.0)

    def finish_weights(self) -> None:
        """Derived tables (after the weights are in place): the distance-bias rows by distance."""
        for L in self.layers:
            if L.rel is not None:
                L.dist_bias = mix.distance_bias_table(L.rel, L.spec.mixer.bias_max)

    def tensors(self):
        for i, L in enumerate(self.layers):
            for k, t in L.named():
                yield f"layers.{i}.{k}", t
        for k in ("embed", "bigram", "pos", "final_norm", "head"):
            t = getattr(self, k)
            if t is not None:
                yield k, t

    def copy_from(self, other: "TifepelModel") -> "TifepelModel":
        src = dict(other.tensors())
        for name, t in self.tensors():
            if name in src:
                t.copy_(src[name])
        self.finish_weights()
        return self

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for _n, t in self.tensors())

    # ------------------------------------------------------------------ cache and state
    def state_fields(self) -> dict:
        """What one sequence carries besides pages: name -> (shape, dtype) per layer run."""
        c = self.cfg
        f32 = torch.float32
        fields = {"prev_tok": ((), torch.int32)}
        for r, li in enumerate(self.runs):
            spec = c.layers[li]
            if c.canon_taps > 1:
                fields[f"canon1.{r}"] = ((c.canon_taps - 1, c.hidden_size), f32)
                if spec.mlp is not None:
                    fields[f"canon2.{r}"] = ((c.canon_taps - 1, c.hidden_size), f32)
            if spec.type == "mamba2":
                m = spec.mixer
                if m.conv > 1:
                    fields[f"conv.{r}"] = ((m.conv - 1, m.conv_channels), f32)
                fields[f"ssm.{r}"] = ((m.heads, m.vdim, m.state), f32)
        return fields

    def attach_cache(self, pool, state_pool=None) -> None:
        """Bind the engine's block pool (``kv_layers[i]`` = pages of attention run i) and state pool."""
        self.kv_cache = pool.kv
        self.kv_layers = pool.layers
        if state_pool is not None:
            self.state = state_pool

    # ------------------------------------------------------------------ forward
    def _attention(self, r: int, L, c: torch.Tensor, meta: AttnMeta) -> torch.Tensor:
        m = L.spec.mixer
        qkv = ops.linear(c, L.qkv)
        kc, vc = self.kv_layers[self.kv_index[r]]
        mix.qknorm_rope_cache(qkv, meta.positions, meta.slot_mapping, self._unit(m.dim), self._unit(m.dim),
                              self.cfg.norm_eps, None, m.heads, m.kv_heads, m.dim, m.vdim, kc, vc,
                              q_temp=(m.q_temp_coef, m.q_temp_every))
        out = torch.empty(qkv.shape[0], m.o_size, device=qkv.device, dtype=qkv.dtype)
        nd = meta.num_decode
        if nd > 0:
            mix.masked_attn_rows(qkv[:nd], kc, vc, meta.dec_block_tables, None, meta.positions[:nd], m.heads,
                                 m.kv_heads, m.scale, 0, None, out=out[:nd], dist_bias=L.dist_bias)
        if meta.num_prefill_tokens > 0:
            if (qkv.is_cuda and qkv.dtype == torch.bfloat16 and m.dim == m.vdim and m.dim in (64, 128)
                    and qkv.shape[1] % 8 == 0 and mix.masked_prefill_available()):
                # MFMA flash kernel (bf16 heads of 64 / 128 dims); other geometries and fp32: the row-wise kernel
                mix.paged_prefill_masked(qkv[nd:], kc, vc, meta.pre_block_tables, meta.pre_cu_seqlens,
                                         meta.pre_context_lens, m.heads, m.kv_heads, m.scale, 0, None,
                                         tiles=meta.pre_tiles, out=out[nd:], dist_bias=L.dist_bias)
            else:
                mix.masked_attn_rows(qkv[nd:], kc, vc, meta.pre_block_tables, meta.pre_cu_seqlens, meta.positions[nd:],
                                     m.heads, m.kv_heads, m.scale, 0, None, out=out[nd:], dist_bias=L.dist_bias)
        return ops.linear(out, L.o)

    def _unit(self, n: int) -> torch.Tensor:
        t = getattr(self, "_unit_w", None)
        if t is None or t.shape[0] < n:
            t = self._unit_w = torch.ones(max(n, 64), device=self.device)
        return t[:n]

    def _mamba2(self, r: int, L, c: torch.Tensor, meta: AttnMeta) -> torch.Tensor:
        m = L.spec.mixer
        st = self.state
        u = ops.linear(c, L.in_proj)                                  # z | x | B | C | dt
        inner, cc = m.inner, m.conv_channels
        tail = st[f"conv.{r}"] if m.conv > 1 else None
        xbc = recur.causal_conv(u[:, inner: inner + cc], L.conv, L.conv_b, tail, meta.positions, meta.row_seq,
                                meta.seq_row0, meta.seq_slots, act=1, residual=False, out_dtype=torch.float32)
        y = recur.ssm_scan(xbc, u[:, inner + cc:], L.dt_bias, L.a_log, L.d_skip, st[f"ssm.{r}"], meta.positions,
                           meta.seq_row0, meta.seq_slots, m.heads, m.vdim, m.state, m.groups)
        g = recur.gated_group_norm(y, u[:, :inner], L.mnorm, m.norm_groups, self.cfg.norm_eps, self.dtype)
        return ops.linear(g, L.o)

    def _moe(self, L, c: torch.Tensor) -> torch.Tensor:
        f = L.spec.mlp
        logits = torch.nn.functional.linear(c.float(), L.router)
        idx, wts = moe.moe_route(logits, L.correction, f.top)
        shared = None
        if L.shared_gate_up is not None:
            shared = ops.linear(moe.silu_mul(ops.linear(c, L.shared_gate_up)), L.shared_down)
        return moe.moe_experts(c, idx, wts, L.gate_up, L.down, shared)

    def _canon(self, h32, w, name: str, meta: AttnMeta) -> torch.Tensor:
        """The sublayer's input c = h + conv(h) in the GEMM dtype (no convolution: h)."""
        taps = self.cfg.canon_taps
        if taps <= 0:
            return h32 if self.dtype == torch.float32 else h32.to(self.dtype)
        tail = self.state[name] if taps > 1 else None
        return recur.causal_conv(h32, w, None, tail, meta.positions, meta.row_seq, meta.seq_row0, meta.seq_slots,
                                 act=0, residual=True, out_dtype=self.dtype)

    def forward_layers(self, xs: torch.Tensor, meta: AttnMeta) -> torch.Tensor:
        """Run every layer run on the fp32 streams ``xs`` [S, T, W] (updated in place)."""
        c, dt = self.cfg, self.dtype
        eps = c.norm_eps
        pend = None                # (y, gate, gate bias, mix, out) of the sublayer whose update is due
        for r, li in enumerate(self.runs):
            L = self.layers[li]
            for q in ("1", "2") if L.spec.mlp is not None else ("1",):
                h32, hd = recur.hc_mix_norm(xs, *(pend or (None, None, None, None, None)),
                                            getattr(L, f"hc{q}_in"), getattr(L, "norm" + q), eps, dt)
                gate = ops.linear(hd, getattr(L, "rg" + q))
                cin = self._canon(h32, getattr(L, "canon" + q), f"canon{q}.{r}", meta)
                if q == "2":
                    y = self._moe(L, cin)
                elif L.spec.type == "attention":
                    y = self._attention(r, L, cin, meta)
                else:
                    y = self._mamba2(r, L, cin, meta)
                if self.reduce is not None:
                    self.reduce(y)
                pend = (y, gate, getattr(L, f"rg{q}_b"), getattr(L, f"hc{q}_mix"), getattr(L, f"hc{q}_out"))
            if self.capture_layers and r in self.capture_layers:
                recur.hc_mix_norm(xs, *pend, None, None, eps, dt)
                pend = None
                self.captured[r] = xs.sum(0)
            if self.layer_hook is not None:
                self.layer_hook(li)
        if pend is not None:
            recur.hc_mix_norm(xs, *pend, None, None, eps, dt)
        return xs

    def embed_tokens(self, input_ids: torch.Tensor, meta: AttnMeta) -> torch.Tensor:
        c = self.cfg
        return recur.embed_streams(input_ids.to(torch.int32), meta.positions, meta.row_seq, meta.seq_row0, meta.seq_slots,
                                   self.state["prev_tok"], self.embed, self.bigram, self.pos, c.bigram_buckets,
                                   c.bigram_mul_prev, c.bigram_mul_cur, c.streams)

    def forward(self, meta: AttnMeta, input_ids: Optional[torch.Tensor] = None,
                hidden: Optional[torch.Tensor] = None) -> torch.Tensor:
        """fp32 logits [n, V] of the step's logits rows."""
        if meta.seq_slots is None:
            raise RuntimeError("Tifepel needs the step's sequence tables (a runner built with a state pool)")
        xs = self.forward_layers(self.embed_tokens(input_ids, meta), meta)
        idx = meta.logits_indices
        if idx is not None:
            xs = xs.index_select(1, idx.long())
        return self.compute_logits(xs)

    def compute_logits(self, xs: torch.Tensor) -> torch.Tensor:
        _h32, hd = recur.hc_mix_norm(xs.contiguous(), None, None, None, None, None, self._ones, self.final_norm,
                                     self.cfg.norm_eps, self.dtype)
        return ops.linear(hd, self.head).float()
