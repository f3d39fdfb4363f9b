"""Native Bebovik decoder for the MI355X runtime.

A Bebovik layer is ``x += ls1 * norm1b(mixer(norm1(x)))`` then ``x += ls2 * norm2b(ff(norm2(x)))``
with Dynamic-Tanh norms (no row statistics), an fp32 residual stream, and per-layer geometry:
every layer names its own head counts, key / value sizes, rotary parameters, attention block
("chunk") size and feed-forward width (or no feed-forward).  The mixer is grouped-query softmax
attention with per-head RMS norm of q and k, interleaved partial rotary, a block mask counted from
position 0 of the sequence, and a sigmoid output gate computed from the mixer's input.

Per layer the step runs (T rows: decode rows first, then packed prompt portions, as in
``dgi.models.llama``)::

    [norm1 fused into the previous dyt_add]
    q|k|v|g GEMM (one fused weight, hipBLASLt)
    qknorm_rope_cache (HIP)   q, k normalised + rotated; k, v -> paged cache
    attention (HIP)           decode rows: row-wise kernel over the row's own block of keys;
                              prompt rows: MFMA flash kernel with the block mask where the geometry
                              allows (bf16, dk == dv in {64, 128}), else the row-wise kernel;
                              sigmoid(g) gate applied in the epilogue
    o GEMM
    dyt_add (HIP)             x += ls1 * norm1b(o);  y = norm2(x)          one pass
    gate|up GEMM -> glu_clamped (HIP) -> down GEMM
    dyt_add (HIP)             x += ls2 * norm2b(d);  y = next layer's norm1(x)

All norms, the stream, scores / softmax and rotary angles are fp32 whatever ``dtype`` is
(bf16: projections and activations in bf16 with fp32 accumulation; fp32: everything in fp32).
The KV cache is the engine's block pool with per-layer page shapes
(``BlockPool(layer_shapes=...)``); a model object may hold any contiguous layer range.
"""
from __future__ import annotations

from typing import Optional

import torch

from dgi import ops
from dgi.models.config import BebovikConfig
from dgi.ops import mix
from dgi.ops.mix import DytNorm
from dgi.runtime.batch import AttnMeta

GLU_ALPHA = 1.702          # sigmoid slope of the feed-forward's gate activation (fixed by the design)


class BebovikLayerWeights:
    __slots__ = ("spec", "norm1", "norm1b", "norm2", "norm2b", "qkvg", "o", "q_norm", "k_norm", "ls1", "ls2",
                 "gate_up", "down", "cos_sin")

    def named(self):
        """(name, tensor) of every weight of the layer."""
        for k in ("qkvg", "o", "q_norm", "k_norm", "ls1", "ls2", "gate_up", "down"):
            t = getattr(self, k)
            if t is not None:
                yield k, t
        for k in ("norm1", "norm1b", "norm2", "norm2b"):
            n = getattr(self, k)
            if n is not None:
                for s, t in n.tensors():
                    yield f"{k}.{s}", t


class BebovikModel:
    """Layer range [layer_start, layer_end) of a Bebovik causal LM."""

    routes_gemms = False       # no start-up GEMM routing table (dgi.runtime.gemm_pad is Llama-shaped)

    def __init__(self, cfg: BebovikConfig, device: torch.device | str = "cpu", dtype=torch.bfloat16,
                 layer_start: int = 0, layer_end: Optional[int] = None, has_embed: Optional[bool] = None,
                 has_head: Optional[bool] = None, seed: int = 0, init: str = "random",
                 checkpoint: Optional[str] = None):
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.layer_start = layer_start
        self.layer_end = cfg.num_layers if layer_end is None else layer_end
        self.has_embed = (layer_start == 0) if has_embed is None else has_embed
        self.has_head = (self.layer_end == cfg.num_layers) if has_head is None else has_head
        self.num_local_layers = self.layer_end - self.layer_start
        self.kv_cache = None
        self.kv_layers: list = []
        self.layers: list[BebovikLayerWeights] = []
        self.embed = self.head = None
        self.embed_norm = self.final_norm = None
        self.capture_layers: tuple = ()
        self.captured: dict = {}
        self.layer_hook = None
        self.reduce = None
        self.mlp_pad = self.mlp_impl = self.proj_impl = self.fold_impl = None
        self.load_info: Optional[dict] = None
        self._tables: dict = {}
        self._init_empty()
        if checkpoint:
            from dgi.models.weights import load_bebovik_checkpoint
            self.load_info = load_bebovik_checkpoint(self, checkpoint)
        elif init == "random":
            self._init_random(seed)
        for L in self.layers:
            L.cos_sin = self._rope_table(L.spec.mixer.rot)

    # ------------------------------------------------------------------ weights
    def _norm(self, W: int) -> DytNorm:
        dev = self.device
        return DytNorm(torch.ones(1, device=dev), torch.ones(W, device=dev), torch.zeros(W, device=dev))

    def _init_empty(self):
        c, dev, dt = self.cfg, self.device, self.dtype
        W = c.hidden_size
        for spec in c.layers[self.layer_start:self.layer_end]:
            m = spec.mixer
            L = BebovikLayerWeights()
            L.spec = spec
            L.norm1, L.norm1b = self._norm(W), self._norm(W)
            gate_rows = m.o_size if m.out_gate else 0
            L.qkvg = torch.empty(m.q_size + m.k_size + m.v_size + gate_rows, W, device=dev, dtype=dt)
            L.o = torch.empty(W, m.o_size, device=dev, dtype=dt)
            L.q_norm = torch.ones(m.dim, device=dev)
            L.k_norm = torch.ones(m.dim, device=dev)
            L.ls1 = torch.ones(W, device=dev)
            L.cos_sin = None
            if spec.mlp is not None:
                L.norm2, L.norm2b = self._norm(W), self._norm(W)
                L.gate_up = torch.empty(2 * spec.mlp.ff, W, device=dev, dtype=dt)
                L.down = torch.empty(W, spec.mlp.ff, device=dev, dtype=dt)
                L.ls2 = torch.ones(W, device=dev)
            else:
                L.norm2 = L.norm2b = L.gate_up = L.down = L.ls2 = None
            self.layers.append(L)
        if self.has_embed:
            self.embed = torch.empty(c.vocab_size, W, device=dev, dtype=dt)
            self.embed_norm = self._norm(W)
        if self.has_head:
            self.final_norm = self._norm(W)
            self.head = torch.empty(c.vocab_size, W, device=dev, dtype=dt)

    def _init_random(self, seed: int):
        """Deterministic per-layer seeds, drawn on the CPU so every device gets the same
        weights (a layer does not depend on how the model is cut into stages)."""
        c = self.cfg
        W = c.hidden_size
        gen = torch.Generator()

        def fill(t, std, mean=0.0):
            t.copy_((torch.randn(t.shape, generator=gen) * std + mean).to(t.dtype))

        def fill_norm(n: DytNorm):
            fill(n.alpha, 0.1, 0.8)
            fill(n.w, 0.1, 1.0)
            fill(n.b, 0.05)

        for li, L in zip(range(self.layer_start, self.layer_end), self.layers):
            gen.manual_seed(seed * 1000003 + li * 7919 + 1)
            for n in (L.norm1, L.norm1b, L.norm2, L.norm2b):
                if n is not None:
                    fill_norm(n)
            fill(L.qkvg, W ** -0.5)
            fill(L.o, L.o.shape[1] ** -0.5)
            fill(L.q_norm, 0.1, 1.0)
            fill(L.k_norm, 0.1, 1.0)
            fill(L.ls1, 0.05, 0.5)
            if L.gate_up is not None:
                fill(L.gate_up, W ** -0.5)
                fill(L.down, L.down.shape[1] ** -0.5)
                fill(L.ls2, 0.05, 0.5)
        if self.has_embed:
            gen.manual_seed(seed * 1000003 + 17)
            fill(self.embed, 1.0)
            fill_norm(self.embed_norm)
        if self.has_head:
            gen.manual_seed(seed * 1000003 + 23)
            fill(self.head, W ** -0.5)
            fill_norm(self.final_norm)

    def _rope_table(self, rot) -> Optional[torch.Tensor]:
        if rot is None or rot.dims <= 0:
            return None
        key = (rot.dims, rot.base, tuple(sorted((rot.scaling or {}).items())), self.cfg.max_position)
        t = self._tables.get(key)
        if t is None:
            t = self._tables[key] = ops.rope_cos_sin(rot.dims, self.cfg.max_position, rot.base, rot.scaling,
                                                     device=self.device)
        return t

    def tensors(self):
        for i, L in enumerate(self.layers):
            for k, t in L.named():
                yield f"layers.{self.layer_start + i}.{k}", t
        if self.embed is not None:
            yield "embed", self.embed
            for s, t in self.embed_norm.tensors():
                yield f"embed_norm.{s}", t
        if self.head is not None:
            yield "head", self.head
            for s, t in self.final_norm.tensors():
                yield f"final_norm.{s}", t

    def copy_from(self, other: "BebovikModel") -> "BebovikModel":
        src = dict(other.tensors())
        for name, t in self.tensors():
            if name in src:
                t.copy_(src[name])
        return self

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for _n, t in self.tensors())

    # ------------------------------------------------------------------ cache
    def attach_cache(self, pool) -> None:
        """Bind the engine's block pool: ``kv_layers[i]`` = (k pages, v pages) of local layer i."""
        self.kv_cache = pool.kv
        self.kv_layers = pool.layers

    # ------------------------------------------------------------------ forward
    @staticmethod
    def _mfma_prefill_ok(m, q: torch.Tensor, kc: torch.Tensor) -> bool:
        return (q.is_cuda and q.dtype == torch.bfloat16 and m.dim == m.vdim and m.dim in (64, 128)
                and mix.masked_prefill_available())

    def attention(self, li: int, qkvg: torch.Tensor, meta: AttnMeta) -> torch.Tensor:
        """Gated attention output [T, H * dv] of the fused projection rows [q | k | v | g]."""
        L = self.layers[li]
        m = L.spec.mixer
        kc, vc = self.kv_layers[li]
        mix.qknorm_rope_cache(qkvg, meta.positions, meta.slot_mapping, L.q_norm, L.k_norm, self.cfg.norm_eps,
                              L.cos_sin, m.heads, m.kv_heads, m.dim, m.vdim, kc, vc)
        T = qkvg.shape[0]
        g0 = m.q_size + m.k_size + m.v_size
        gate = qkvg[:, g0:g0 + m.o_size] if m.out_gate else None
        out = torch.empty(T, m.o_size, device=qkvg.device, dtype=qkvg.dtype)
        mask = m.mask_size if m.mask_kind == "chunk" else 0
        nd = meta.num_decode
        if nd > 0:
            mix.masked_attn_rows(qkvg[:nd], kc, vc, meta.dec_block_tables, None, meta.positions[:nd], m.heads,
                                 m.kv_heads, m.scale, mask, None if gate is None else gate[:nd], out=out[:nd])
        if meta.num_prefill_tokens > 0:
            if self._mfma_prefill_ok(m, qkvg, kc):
                mix.paged_prefill_masked(qkvg[nd:], kc, vc, meta.pre_block_tables, meta.pre_cu_seqlens,
                                         meta.pre_context_lens, m.heads, m.kv_heads, m.scale, mask,
                                         None if gate is None else gate[nd:], tiles=meta.pre_tiles, out=out[nd:])
            else:
                mix.masked_attn_rows(qkvg[nd:], kc, vc, meta.pre_block_tables, meta.pre_cu_seqlens,
                                     meta.positions[nd:], m.heads, m.kv_heads, m.scale, mask,
                                     None if gate is None else gate[nd:], out=out[nd:])
        return out

    def forward_layers(self, x: torch.Tensor, meta: AttnMeta, trim_last: Optional[torch.Tensor] = None):
        """Run the local layers on the fp32 stream ``x`` [T, W] (updated in place; returned).
        ``trim_last`` (row indices): after the last layer's attention — which has written every
        row's K/V — only those rows go through its o-proj and feed-forward; the returned stream
        holds just them."""
        dt = self.dtype
        n = len(self.layers)
        if n == 0:
            return x
        y = mix.dyt(x, self.layers[0].norm1, dt)
        for i, L in enumerate(self.layers):
            last = i == n - 1
            attn = self.attention(i, ops.linear(y, L.qkvg), meta)
            if last and trim_last is not None:
                attn = attn.index_select(0, trim_last)
                x = x.index_select(0, trim_last)
            h = ops.linear(attn, L.o)
            if self.reduce is not None:
                self.reduce(h)
            after = None if last else self.layers[i + 1].norm1
            if L.gate_up is not None:
                y = mix.dyt_add(x, h, L.norm1b, L.ls1, L.norm2)
                act = mix.glu_clamped(ops.linear(y, L.gate_up), L.spec.mlp.limit, GLU_ALPHA)
                d = ops.linear(act, L.down)
                if self.reduce is not None:
                    self.reduce(d)
                y = mix.dyt_add(x, d, L.norm2b, L.ls2, after)
            else:
                y = mix.dyt_add(x, h, L.norm1b, L.ls1, after)
            if self.capture_layers and (self.layer_start + i) in self.capture_layers:
                self.captured[self.layer_start + i] = x.clone()
            if self.layer_hook is not None:
                self.layer_hook(self.layer_start + i)
        return x

    def embed_tokens(self, input_ids: torch.Tensor) -> torch.Tensor:
        return mix.embed_dyt(input_ids, self.embed, self.cfg.embedding_scale, self.embed_norm)

    def forward(self, meta: AttnMeta, input_ids: Optional[torch.Tensor] = None,
                hidden: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Stage forward: fp32 logits [n, V] on the last stage (scaled and soft-capped), else the
        fp32 residual stream [T, W] for the next stage."""
        x = self.embed_tokens(input_ids) if self.has_embed else hidden.float().clone()
        idx = meta.logits_indices
        trim = (idx is not None and self.has_head and self.num_local_layers > 0 and not self.capture_layers
                and idx.shape[0] < x.shape[0])
        x = self.forward_layers(x, meta, trim_last=idx if trim else None)
        if not self.has_head:
            return x
        if idx is not None and not trim:
            x = x.index_select(0, idx)
        return self.compute_logits(x)

    def compute_logits(self, x: torch.Tensor) -> torch.Tensor:
        hn = mix.dyt(x.contiguous(), self.final_norm, self.dtype)
        return mix.scale_softcap(ops.linear(hn, self.head), self.cfg.logit_scale, self.cfg.logit_softcap)
