"""Native Depelix decoder for the MI355X runtime.

Notation (T rows of a step, W the width, x the fp32 residual stream, rms(v) = sqrt(mean(v^2) + eps)):

    embedding   x_t = E[tok_t] + Bg[(tok_(t-1) * a + tok_t * b) mod n]      (a sequence's first token: row Bg[n])
    layer i     x += Mix_i(x / rms(x) * n1)
                x += FF_i(x / rms(x) * n2)                                   (if the layer has a feed-forward)
                y  = P_i (gelu(G_i x) * S[tok_t, i * d : (i + 1) * d])       per-layer token input, d = side_dim
                x += y / rms(y) * ns
    logits      head(x / rms(x) * nf)

Mix is latent attention (``dgi.ops.latent``): the query goes through a normalised latent
(c_q = D_q h / rms * w, q = U_q c_q, per head ``dim`` unrotated + ``rot_dim`` rotated dims); keys and
values of all heads come from one normalised latent c = D_kv h / rms * w per token plus one rotated
key part shared by the heads, and only ``[c | rotated part]`` is cached.  Two layer kinds:

* ``latent_attention``: half-split rotary pairs (i, i + dims/2), a sliding window (a query sees
  itself and the ``mask_size - 1`` positions before it), one sigmoid output gate per head; a layer
  with ``kv_from = j`` has no D_kv and reads layer j's cached rows with its own U_k / U_v;
* ``latent_attention_2``: interleaved rotary pairs (2i, 2i + 1), causal, one sigmoid gate per
  output element.

FF is W_d gelu(W_u h) (tanh form) or a mixture of experts with sigmoid router scores (fp32), the
``top`` largest taken as they are, each weight multiplying its expert's INPUT, experts being clamped
sigmoid-GLUs (``dgi.ops.moe`` with ``score="sigmoid", act="clamped", weigh="input"``).

Per layer the step executes (rows: decode rows first, then packed prompt portions)::

    stream_add_norm (HIP)   previous sublayer's residual add (+ the token input's unit-RMS norm) + n1 norm
    D_q | D_kv | gate GEMM  one fused weight
    latent_prep (HIP)       c_q norm; c norm + rotary of the key part -> the paged cache row
    U_q GEMM
    rows (decode rows, short portions, fp32):  q_nope -> latent space by a batched GEMM over heads (the key
                            up-projection folded into the query) -> latent_attn_rows (HIP: MFMA for bf16, window /
                            causal, rotates the query's rotated part) on the cached rows themselves -> U_v batched GEMM
    long portions (bf16, dim + rot_dim == vdim in {64, 128}):  pages expanded into per-head keys [U_k c | r] and
                            values U_v c (two GEMMs) -> rotate_heads (HIP) -> MFMA flash kernel with window / causal mask
    gate_heads (HIP: head gate / element gate, heads side by side) -> o GEMM
    stream_add_norm (HIP)   x += mix, n2 norm
    dense: up GEMM -> gelu_tanh (HIP) -> down GEMM;  moe: router GEMM (fp32) -> moe_route (HIP) -> experts
    stream_add_norm (HIP)   x += ff (-> bf16 copy of x) ; G GEMM -> gelu_tanh x gathered token row (HIP) -> P GEMM

The stream, every norm, rotary angles, scores / softmax and the router are fp32 whatever ``dtype``
is; with bf16 the projections and activations are bf16 with fp32 accumulation.  Pages come from the
engine's block pool (one page geometry per layer that owns a latent), the previous token of the
bigram hash from ``dgi.kv.state_pool.StatePool``.
"""
from __future__ import annotations

import os
from typing import Optional

import torch

from dgi import ops
from dgi.models.config import DepelixConfig
from dgi.ops import latent, mix, moe, recur
from dgi.runtime.batch import AttnMeta

GLU_ALPHA = 1.702          # sigmoid slope of the experts' gate activation (fixed by the design)
# prompt rows of a step from which the MFMA prompt path (keys and values expanded per head) replaces the
# row-wise kernel, where the geometry allows it (DGI_LATENT_MFMA_ROWS; a huge value switches it off)
MFMA_PROMPT_ROWS = int(os.environ.get("DGI_LATENT_MFMA_ROWS", "64"))


class DepelixLayerWeights:
    FIELDS = ("norm1", "norm2", "in_proj", "dq_norm", "dkv_norm", "uq", "uk", "uv", "o", "up", "down", "router",
              "gate_up", "side_gate", "side_proj", "side_norm")
    __slots__ = ("spec", "cos_sin") + FIELDS

    def __init__(self):
        for k in self.__slots__:
            setattr(self, k, None)

    def named(self):
        for k in self.FIELDS:
            t = getattr(self, k)
            if t is not None:
                yield k, t


class DepelixModel:
    """A Depelix causal LM (all layers on one device)."""

    routes_gemms = False       # projections are plain vendor GEMMs: no start-up routing table

    def __init__(self, cfg: DepelixConfig, device: torch.device | str = "cpu", dtype=torch.bfloat16,
                 layer_start: int = 0, layer_end: Optional[int] = None, has_embed: Optional[bool] = None,
                 has_head: Optional[bool] = None, seed: int = 0, init: str = "random",
                 checkpoint: Optional[str] = None):
        if layer_start != 0 or (layer_end is not None and layer_end != cfg.num_layers):
            raise ValueError("Depelix runs all its layers in one stage (layers may read an earlier layer's cache rows)")
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.layer_start, self.layer_end = 0, cfg.num_layers
        self.has_embed = self.has_head = True
        self.num_local_layers = cfg.num_layers
        self.kv_cache = None
        self.kv_layers: list = []
        self.state = None
        self.layers: list[DepelixLayerWeights] = []
        self.embed = self.bigram = self.side_embed = self.head = self.final_norm = None
        self.capture_layers: tuple = ()
        self.captured: dict = {}
        self.layer_hook = None
        self.reduce = None
        self.mlp_pad = self.mlp_impl = self.proj_impl = self.fold_impl = None
        self.load_info: Optional[dict] = None
        self._tables: dict = {}
        # page-pool layer of every layer that owns a latent; the others index their source's
        self.kv_index = {li: n for n, li in enumerate(cfg.kv_owners)}
        self._init_empty()
        if checkpoint:
            from dgi.models.weights import load_depelix_checkpoint
            self.load_info = load_depelix_checkpoint(self, checkpoint)
        elif init == "random":
            self._init_random(seed)
        self.finish_weights()

    # ------------------------------------------------------------------ weights
    def _init_empty(self):
        c, dev, dt = self.cfg, self.device, self.dtype
        W, f32 = c.hidden_size, torch.float32

        def e(*shape, dtype=dt):
            return torch.zeros(*shape, device=dev, dtype=dtype)

        for spec in c.layers:
            L = DepelixLayerWeights()
            L.spec = spec
            m = spec.mixer
            own = m.kv_from is None
            L.norm1 = torch.ones(W, device=dev)
            L.in_proj = e(m.q_rank + (m.cache_dim if own else 0) + m.gate_rows, W)     # D_q | D_kv | gate
            L.dq_norm = torch.ones(m.q_rank, device=dev)
            if own:
                L.dkv_norm = torch.ones(m.kv_rank, device=dev)
            L.uq = e(m.q_size, m.q_rank)
            L.uk = e(m.heads, m.dim, m.kv_rank)
            L.uv = e(m.heads, m.vdim, m.kv_rank)
            L.o = e(W, m.o_size)
            f = spec.mlp
            if f is not None:
                L.norm2 = torch.ones(W, device=dev)
                if f.kind == "dense":
                    L.up, L.down = e(f.ff, W), e(W, f.ff)
                else:
                    L.router = e(f.experts, W, dtype=f32)
                    L.gate_up = e(f.experts, 2 * f.ff, W)
                    L.down = e(f.experts, W, f.ff)
            if c.side_dim > 0:
                L.side_gate, L.side_proj = e(c.side_dim, W), e(W, c.side_dim)
                L.side_norm = torch.ones(W, device=dev)
            self.layers.append(L)
        self.embed = e(c.vocab_size, W)
        if c.bigram_buckets > 0:
            self.bigram = e(c.bigram_buckets + 1, W)
        if c.side_dim > 0:
            self.side_embed = e(c.vocab_size, c.side_dim * c.num_layers)
        self.final_norm = torch.ones(W, device=dev)
        self.head = e(c.vocab_size, W)

    def _init_random(self, seed: int):
        """Deterministic per-tensor values drawn on the CPU (the same on every device)."""
        c = self.cfg
        W = c.hidden_size
        gen = torch.Generator()

        def fill(t, std, mean=0.0):
            if t is not None:
                t.copy_((torch.randn(t.shape, generator=gen) * std + mean).to(t.dtype))

        for li, L in enumerate(self.layers):
            gen.manual_seed(seed * 1000003 + li * 7919 + 1)
            m = L.spec.mixer
            for n in (L.norm1, L.norm2, L.dq_norm, L.dkv_norm):
                fill(n, 0.1, 1.0)
            fill(L.side_norm, 0.05, 0.3)
            fill(L.in_proj, W ** -0.5)
            fill(L.uq, m.q_rank ** -0.5)
            fill(L.uk, m.kv_rank ** -0.5)
            fill(L.uv, m.kv_rank ** -0.5)
            fill(L.o, m.o_size ** -0.5)
            fill(L.up, W ** -0.5)
            fill(L.router, W ** -0.5 * 2)
            fill(L.gate_up, W ** -0.5)
            if L.down is not None:
                fill(L.down, L.down.shape[-1] ** -0.5)
            fill(L.side_gate, W ** -0.5)
            fill(L.side_proj, max(1, c.side_dim) ** -0.5)
        gen.manual_seed(seed * 1000003 + 17)
        fill(self.embed, 1.0)
        fill(self.bigram, 0.5)
        fill(self.side_embed, 1.0)
        fill(self.head, W ** -0.5)
        fill(self.final_norm, 0.1, 1.0)

    def _rope_table(self, rot) -> Optional[torch.Tensor]:
        if rot is None or rot.dims <= 0:
            return None
        key = (rot.dims, rot.base, self.cfg.max_position)
        t = self._tables.get(key)
        if t is None:
            t = self._tables[key] = ops.rope_cos_sin(rot.dims, self.cfg.max_position, rot.base, rot.scaling,
                                                     device=self.device)
        return t

    def finish_weights(self) -> None:
        """Derived tables (after the weights are in place): rotary cos / sin by position."""
        for L in self.layers:
            L.cos_sin = self._rope_table(L.spec.mixer.rot)

    def tensors(self):
        for i, L in enumerate(self.layers):
            for k, t in L.named():
                yield f"layers.{i}.{k}", t
        for k in ("embed", "bigram", "side_embed", "final_norm", "head"):
            t = getattr(self, k)
            if t is not None:
                yield k, t

    def copy_from(self, other: "DepelixModel") -> "DepelixModel":
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
        """What one sequence carries besides pages: the previous token (bigram hash)."""
        return {"prev_tok": ((), torch.int32)}

    def attach_cache(self, pool, state_pool=None) -> None:
        """Bind the engine's block pool (``kv_layers[n]`` = pages of the n-th layer that owns a
        latent; the value half of a page is empty) and the state pool."""
        self.kv_cache = pool.kv
        self.kv_layers = pool.layers
        if state_pool is not None:
            self.state = state_pool

    # ------------------------------------------------------------------ forward
    def _attention(self, li: int, L, h: torch.Tensor, meta: AttnMeta) -> torch.Tensor:
        m = L.spec.mixer
        own = m.kv_from is None
        cache = self.kv_layers[self.kv_index[li if own else m.kv_from]][0]
        inter = m.rot is not None and m.rot.layout == "interleaved"
        proj = ops.linear(h, L.in_proj)
        cq = latent.latent_prep(proj, m.q_rank, m.kv_rank, m.rot_dim, L.dq_norm, L.dkv_norm, self.cfg.norm_eps,
                                meta.positions, meta.slot_mapping, L.cos_sin, inter, cache if own else None)
        q = ops.linear(cq, L.uq)
        T, H, kr = q.shape[0], m.heads, m.kv_rank
        nd = meta.num_decode
        g0 = m.q_rank + (m.cache_dim if own else 0)
        gate = proj[:, g0:g0 + m.gate_rows] if m.gate_rows else None
        if meta.num_prefill_tokens >= MFMA_PROMPT_ROWS and self._mfma_prompt_ok(m, q):
            return ops.linear(self._attention_mfma_prompt(L, m, q, gate, cache, meta, inter), L.o)
        # unrotated query part of every head through its key up-projection: [H, T, dim] x [H, dim, kr]
        q_lat = torch.bmm(q.view(T, H, m.qk_dim)[:, :, :m.dim].transpose(0, 1), L.uk)
        o_lat = torch.empty(H, T, kr, device=q.device, dtype=q.dtype)
        if nd > 0:
            latent.latent_attn_rows(q[:nd], q_lat[:, :nd], cache, meta.dec_block_tables, None, meta.positions[:nd], H,
                                    m.dim, m.rot_dim, kr, m.scale, m.window, L.cos_sin, inter, out=o_lat[:, :nd],
                                    max_keys=meta.dec_block_tables.shape[1] * cache.shape[2])
        if meta.num_prefill_tokens > 0:
            latent.latent_attn_rows(q[nd:], q_lat[:, nd:], cache, meta.pre_block_tables, meta.pre_cu_seqlens,
                                    meta.positions[nd:], H, m.dim, m.rot_dim, kr, m.scale, m.window, L.cos_sin, inter,
                                    out=o_lat[:, nd:])
        ov = torch.bmm(o_lat, L.uv.transpose(1, 2))                       # weighted latent sums -> head values
        return ops.linear(latent.gate_heads(ov, gate, m.gate == "head"), L.o)

    @staticmethod
    def _mfma_prompt_ok(m, q: torch.Tensor) -> bool:
        return (q.is_cuda and q.dtype == torch.bfloat16 and m.qk_dim == m.vdim and m.vdim in (64, 128)
                and mix.masked_prefill_available() and not torch.cuda.is_current_stream_capturing())

    def _attention_mfma_prompt(self, L, m, q, gate, cache, meta: AttnMeta, inter: bool) -> torch.Tensor:
        """Gated head outputs [T, H * vdim] of a step with prompt portions, on the MFMA flash kernel: the
        portions' pages are expanded once into per-head keys [U_k c | r] and values U_v c (two GEMMs over
        the cached latents: the explicit form costs (dim + rot_dim + vdim) MACs per query, key and head
        instead of the 2 kv_rank + rot_dim of the folded form), laid out as pages of their own; the step's
        decode rows still run the folded row-wise kernel on the cached latents."""
        T, H, kr, dv = q.shape[0], m.heads, m.kv_rank, m.vdim
        nd = meta.num_decode
        out = torch.empty(T, H * dv, device=q.device, dtype=q.dtype)
        per_head = m.gate == "head"
        if nd > 0:
            q_lat = torch.bmm(q[:nd].view(nd, H, m.qk_dim)[:, :, :m.dim].transpose(0, 1), L.uk)
            o_lat = torch.empty(H, nd, kr, device=q.device, dtype=q.dtype)
            latent.latent_attn_rows(q[:nd], q_lat, cache, meta.dec_block_tables, None, meta.positions[:nd], H, m.dim,
                                    m.rot_dim, kr, m.scale, m.window, L.cos_sin, inter, out=o_lat,
                                    max_keys=meta.dec_block_tables.shape[1] * cache.shape[2])
            latent.gate_heads(torch.bmm(o_lat, L.uv.transpose(1, 2)), None if gate is None else gate[:nd], per_head,
                              out=out[:nd])
        bt = meta.pre_block_tables
        Bp, mb = bt.shape
        bs = cache.shape[2]
        rows = cache.view(cache.shape[0], bs, m.cache_dim).index_select(0, bt.reshape(-1).long())    # [P, bs, kr + rd]
        npg = Bp * mb
        lat = rows.view(npg * bs, m.cache_dim)[:, :kr]
        kt = torch.empty(npg, H, bs, m.qk_dim, device=q.device, dtype=q.dtype)
        kt[..., :m.dim] = ops.linear(lat, L.uk.view(H * m.dim, kr)).view(npg, bs, H, m.dim).permute(0, 2, 1, 3)
        kt[..., m.dim:] = rows[:, None, :, kr:]
        vt = ops.linear(lat, L.uv.view(H * dv, kr)).view(npg, bs, H, dv).permute(0, 2, 1, 3).contiguous()
        qp = q[nd:]
        if L.cos_sin is not None:
            latent.rotate_heads(qp, meta.positions[nd:], L.cos_sin, inter, H, m.qk_dim, m.dim)
        own_bt = torch.arange(npg, dtype=torch.int32, device=q.device).view(Bp, mb)
        att = mix.paged_prefill_masked(qp, kt, vt, own_bt, meta.pre_cu_seqlens, meta.pre_context_lens, H, H, m.scale, 0,
                                       None if per_head or gate is None else gate[nd:], tiles=meta.pre_tiles,
                                       window=m.window, out=out[nd:] if not per_head else None)
        if per_head:
            latent.gate_heads(att.view(T - nd, H, dv).transpose(0, 1), None if gate is None else gate[nd:], True, out=out[nd:])
        return out

    def _ff(self, L, h: torch.Tensor) -> torch.Tensor:
        f = L.spec.mlp
        if f.kind == "dense":
            return ops.linear(latent.gelu_tanh(ops.linear(h, L.up)), L.down)
        logits = torch.nn.functional.linear(h.float(), L.router)
        idx, wts = moe.moe_route(logits, None, f.top, score=f.score)
        return moe.moe_experts(h, idx, wts, L.gate_up, L.down, None, act=f.act, limit=f.limit, alpha=GLU_ALPHA,
                               weigh=f.weigh)

    def forward_layers(self, x: torch.Tensor, meta: AttnMeta, ids: torch.Tensor) -> torch.Tensor:
        """Run every layer on the fp32 stream ``x`` [T, W] (updated in place)."""
        c, dt = self.cfg, self.dtype
        eps = c.norm_eps
        pend = (None, None)            # (y, post-norm weight) of the sublayer whose residual add is due
        for li, L in enumerate(self.layers):
            h = latent.stream_add_norm(x, *pend, L.norm1, eps, dt)
            y = self._attention(li, L, h, meta)
            if self.reduce is not None:
                self.reduce(y)
            if L.spec.mlp is not None:
                h = latent.stream_add_norm(x, y, None, L.norm2, eps, dt)
                y = self._ff(L, h)
                if self.reduce is not None:
                    self.reduce(y)
            pend = (y, None)
            if L.side_gate is not None:
                # the token input reads the stream itself: finish the add, then gate a slice of the token's row
                xb = latent.stream_add_norm(x, y, None, None, eps, None if dt == torch.float32 else dt)
                g = latent.gelu_tanh(ops.linear(x if xb is None else xb, L.side_gate), self.side_embed, ids,
                                     li * c.side_dim)
                pend = (ops.linear(g, L.side_proj), L.side_norm)
            if self.capture_layers and li in self.capture_layers:
                latent.stream_add_norm(x, *pend, None, eps, None)
                pend = (None, None)
                self.captured[li] = x.clone()
            if self.layer_hook is not None:
                self.layer_hook(li)
        if pend[0] is not None:
            latent.stream_add_norm(x, *pend, None, eps, None)
        return x

    def embed_tokens(self, ids: torch.Tensor, meta: AttnMeta) -> torch.Tensor:
        c = self.cfg
        return recur.embed_streams(ids, meta.positions, meta.row_seq, meta.seq_row0, meta.seq_slots,
                                   self.state["prev_tok"], self.embed, self.bigram, None, c.bigram_buckets,
                                   c.bigram_mul_prev, c.bigram_mul_cur, 1)[0]

    def forward(self, meta: AttnMeta, input_ids: Optional[torch.Tensor] = None,
                hidden: Optional[torch.Tensor] = None) -> torch.Tensor:
        """fp32 logits [n, V] of the step's logits rows."""
        if meta.seq_slots is None:
            raise RuntimeError("Depelix needs the step's sequence tables (a runner built with a state pool)")
        ids = input_ids.to(torch.int32)
        x = self.forward_layers(self.embed_tokens(ids, meta), meta, ids)
        idx = meta.logits_indices
        if idx is not None:
            x = x.index_select(0, idx.long())
        return self.compute_logits(x)

    def compute_logits(self, x: torch.Tensor) -> torch.Tensor:
        hn = latent.stream_add_norm(x.contiguous(), None, None, self.final_norm, self.cfg.norm_eps, self.dtype)
        return ops.linear(hn, self.head).float()
