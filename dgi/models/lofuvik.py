"""Native Lofuvik decoder for the MI355X runtime.

Notation (T rows of a step, W the width, x the fp32 residual stream, rms(v) = sqrt(mean(v^2) + eps)):

    embedding   x_t = E[tok_t]                         (e = this x, kept for repeated passes)
    layer       h = x / rms(x) * n1;   x += Mix(h) + FF(h)      both sublayers read the same h
    logits      head(x / rms(x) * nf)

A span of layers runs several times with the same weights; every layer RUN has its own cache pages or
state, and every pass but the first begins with x += e.  Mix is one of

* ``wkv`` — RWKV-style time mixing: r, k, v, g and the decay input each read their own blend
  h + (h' - h) mu of the current and the previous token's h; the decay w = exp(-exp(W2 tanh(W1 .) + w0))
  is per key channel; per head o = (S + diag(u) k v^T)^T r, S <- diag(w) S + k v^T; o / rms(o) per head,
  times a weight, times silu(g), then the output projection;
* ``delta`` — gated delta rule: q, k (shared by groups of value heads) and v through a short causal
  convolution + SiLU, q and k made unit vectors, per head a decay g = exp(-exp(A) softplus(a + dt)) and a
  write strength beta = sigmoid(b): S <- g S, S += k (beta (v - S^T k))^T, o = S^T q; o / rms(o) per head
  times a weight shared by the heads, times silu(gate);
* ``parallel`` — softmax attention (RMS norm over the whole q and the whole k projection, half-split
  rotary with ramp-scaled frequencies, soft-capped scores, a learned sink logit per head in the
  denominator, sigmoid output gate) beside a matrix memory (``dgi.ops.linrec.mlstm_scan``, sigmoid output
  gate); the result is the mean of the two branch outputs, each RMS-normed over W with its own weight.

FF is a mixture of experts: fp32 router logits with a bias, the ``top`` largest taken, weights the
softmax over those, gated-SiLU experts (``dgi.ops.moe``).

Per layer run the step executes (rows: decode rows first, then packed prompt portions)::

    stream_add_norm (HIP)   the previous layer's x += mix + ff and this layer's norm -> h
    side GEMM (fp32)        router logits | the recurrence's gate projections, one fp32 GEMM on h
    wkv:      token_shift (HIP: five blends, previous row from the state slot) -> r|k|v|g batched GEMM,
              decay GEMMs (fp32) -> linear_scan (HIP, mode wkv) -> head_norm_gate (HIP) -> o GEMM
    delta:    q|k|v|g GEMM -> causal_conv (HIP, SiLU, tail in the slot) -> linear_scan (HIP, mode delta)
              -> head_norm_gate (HIP) -> o GEMM
    parallel: one GEMM for both branches -> qk_prep (HIP: full-width q / k norm, rotary, paged K/V write)
              -> masked_attn_rows (HIP; bf16 heads of 64 / 128: the MFMA prompt kernel), sink + cap + gate
              fused -> o GEMM;  linear_scan (HIP, mode mlstm) -> head_norm_gate (HIP) -> o GEMM;
              rms_pair_mean (HIP)
    moe:      moe_route (HIP) -> experts (HIP pair kernels, one batched GEMM, or sorted segment GEMMs)

The stream, every norm, rotary angles, scores / softmax, the router, and all that enters a recurrence
besides q / k / v (decays, gates, unit norms, states) are fp32 whatever ``dtype`` is; with bf16 the large
projections and expert GEMMs take bf16 inputs with fp32 accumulation.  Pages come from the engine's block
pool (one page geometry per attention run), states from ``dgi.kv.state_pool.StatePool``.
"""
from __future__ import annotations

from typing import Optional

import torch

from dgi import ops
from dgi.models.config import LofuvikConfig
from dgi.ops import latent, linrec, mix, moe, recur
from dgi.runtime.batch import AttnMeta

SHIFT_BLENDS = ("r", "k", "v", "g", "w")      # order of the time-mixing blends (and of ``mu``)


class LofuvikLayerWeights:
    FIELDS = ("norm1", "side", "side_b", "gate_up", "down",
              "in_proj", "conv", "a_log", "dt_bias", "mnorm", "o",
              "mu", "rkvg", "w1", "w2", "w0", "bonus",
              "q_norm", "k_norm", "sink", "o_right", "rnorm", "out_left", "out_right")
    __slots__ = ("spec", "cos_sin") + FIELDS

    def __init__(self):
        for k in self.__slots__:
            setattr(self, k, None)

    def named(self):
        for k in self.FIELDS:
            t = getattr(self, k)
            if t is not None:
                yield k, t


def side_rows(spec) -> int:
    """Rows of a layer's fp32 side projection after the router's: the recurrence's gate projections."""
    if spec.type == "delta":
        return 2 * spec.mixer.heads                # write strength | step size
    if spec.type == "parallel":
        return 2 * spec.mixer.right.heads          # input gate | forget gate
    return 0


class LofuvikModel:
    """A Lofuvik causal LM (all layers on one device)."""

    routes_gemms = False       # projections are plain vendor GEMMs: no start-up routing table

    def __init__(self, cfg: LofuvikConfig, device: torch.device | str = "cpu", dtype=torch.bfloat16,
                 layer_start: int = 0, layer_end: Optional[int] = None, has_embed: Optional[bool] = None,
                 has_head: Optional[bool] = None, seed: int = 0, init: str = "random",
                 checkpoint: Optional[str] = None):
        if layer_start != 0 or (layer_end is not None and layer_end != cfg.num_layers):
            raise ValueError("Lofuvik runs all its layers in one stage (a looped span cannot be cut)")
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
        self.layers: list[LofuvikLayerWeights] = []
        self.embed = self.head = self.final_norm = None
        self.capture_layers: tuple = ()
        self.captured: dict = {}
        self.layer_hook = None
        self.reduce = None
        self.mlp_pad = self.mlp_impl = self.proj_impl = self.fold_impl = None
        self.load_info: Optional[dict] = None
        self._tables: dict = {}
        if checkpoint:
            from dgi.models.weights import lofuvik_checkpoint_shapes
            lofuvik_checkpoint_shapes(cfg, checkpoint)
        self._init_empty()
        if checkpoint:
            from dgi.models.weights import load_lofuvik_checkpoint
            self.load_info = load_lofuvik_checkpoint(self, checkpoint)
        elif init == "random":
            self._init_random(seed)
        self.finish_weights()
        # page-pool layer of every attention run
        self.kv_index = {}
        for r, li in enumerate(self.runs):
            if cfg.layers[li].type == "parallel":
                self.kv_index[r] = len(self.kv_index)

    # ------------------------------------------------------------------ weights
    def _init_empty(self):
        c, dev, dt = self.cfg, self.device, self.dtype
        W, f32 = c.hidden_size, torch.float32

        def e(*shape, dtype=dt):
            return torch.zeros(*shape, device=dev, dtype=dtype)

        for spec in c.layers:
            L = LofuvikLayerWeights()
            L.spec = spec
            m, f = spec.mixer, spec.mlp
            L.norm1 = torch.ones(W, device=dev)
            n_side = (f.routes if f is not None else 0) + side_rows(spec)
            if n_side:
                L.side, L.side_b = e(n_side, W, dtype=f32), e(n_side, dtype=f32)
            if f is not None:
                L.gate_up, L.down = e(f.experts, 2 * f.ff, W), e(f.experts, W, f.ff)
            if spec.type == "wkv":
                if m.decay_rank <= 0:
                    raise ValueError("Lofuvik: a wkv layer needs decay_rank (read from the checkpoint, or given)")
                L.mu = e(len(SHIFT_BLENDS), W, dtype=f32)
                L.rkvg = e(4, m.inner, W)
                L.w1, L.w2, L.w0 = e(m.decay_rank, W, dtype=f32), e(m.inner, m.decay_rank, dtype=f32), e(m.inner, dtype=f32)
                L.bonus = e(m.inner, dtype=f32)
                L.mnorm = torch.ones(m.inner, device=dev)
                L.o = e(W, m.inner)
            elif spec.type == "delta":
                L.in_proj = e(m.conv_channels + m.inner, W)                    # q | k | v | gate
                L.conv = e(m.conv_channels, m.conv, dtype=f32)
                L.a_log, L.dt_bias = e(m.heads, dtype=f32), e(m.heads, dtype=f32)
                L.mnorm = torch.ones(m.vdim, device=dev)
                L.o = e(W, m.inner)
            else:
                a, r = m.left, m.right
                # attention q | k | v | gate, then memory q | k | v | gate: one GEMM for both branches
                L.in_proj = e(a.q_size + a.k_size + a.v_size + a.o_size + 2 * r.qk_size + 2 * r.inner, W)
                L.q_norm, L.k_norm = torch.ones(a.q_size, device=dev), torch.ones(a.k_size, device=dev)
                L.sink = e(a.heads, dtype=f32)
                L.o = e(W, a.o_size)
                L.o_right = e(W, r.inner)
                L.rnorm = torch.ones(r.inner, device=dev)
                L.out_left, L.out_right = torch.ones(W, device=dev), torch.ones(W, device=dev)
            self.layers.append(L)
        self.embed = e(c.vocab_size, W)
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
            for n in (L.norm1, L.mnorm, L.rnorm, L.q_norm, L.k_norm, L.out_left, L.out_right):
                fill(n, 0.1, 1.0)
            fill(L.side, W ** -0.5 * 2)
            fill(L.side_b, 0.3)
            if L.spec.type == "delta":                 # the delta rule's gate projections have no bias
                L.side_b[L.spec.mlp.routes if L.spec.mlp is not None else 0:].zero_()
            fill(L.gate_up, W ** -0.5)
            if L.down is not None:
                fill(L.down, L.down.shape[-1] ** -0.5)
            fill(L.in_proj, W ** -0.5)
            fill(L.conv, 0.4)
            fill(L.a_log, 0.5, -1.0)
            fill(L.dt_bias, 0.5, -1.0)
            fill(L.o, L.o.shape[1] ** -0.5)
            if L.o_right is not None:
                fill(L.o_right, L.o_right.shape[1] ** -0.5)
            if L.mu is not None:
                L.mu.copy_(torch.rand(L.mu.shape, generator=gen))
            fill(L.rkvg, W ** -0.5)
            fill(L.w1, W ** -0.5)
            if L.w2 is not None:
                fill(L.w2, L.w2.shape[1] ** -0.5)
            fill(L.w0, 0.7, -1.5)
            fill(L.bonus, 0.3, 0.3)
            fill(L.sink, 1.0)
        gen.manual_seed(seed * 1000003 + 17)
        fill(self.embed, 1.0)
        fill(self.head, W ** -0.5)
        fill(self.final_norm, 0.1, 1.0)

    def _rope_table(self, rot) -> Optional[torch.Tensor]:
        if rot is None or rot.dims <= 0:
            return None
        sc = rot.scaling or {}
        key = (rot.dims, rot.base, tuple(sorted(sc.items())), self.cfg.max_position)
        t = self._tables.get(key)
        if t is None:
            t = self._tables[key] = ops.rope_cos_sin(rot.dims, self.cfg.max_position, rot.base, rot.scaling,
                                                     device=self.device)
        return t

    def finish_weights(self) -> None:
        """Derived tables (after the weights are in place): rotary cos / sin by position."""
        for L in self.layers:
            if L.spec.type == "parallel":
                L.cos_sin = self._rope_table(L.spec.mixer.left.rot)

    def tensors(self):
        for i, L in enumerate(self.layers):
            for k, t in L.named():
                yield f"layers.{i}.{k}", t
        for k in ("embed", "final_norm", "head"):
            yield k, getattr(self, k)

    def copy_from(self, other: "LofuvikModel") -> "LofuvikModel":
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
        fields = {}
        for r, li in enumerate(self.runs):
            spec = c.layers[li]
            m = spec.mixer
            if spec.type == "wkv":
                fields[f"shift.{r}"] = ((c.hidden_size,), f32)
                fields[f"mem.{r}"] = ((m.heads, m.dim, m.dim), f32)
            elif spec.type == "delta":
                if m.conv > 1:
                    fields[f"conv.{r}"] = ((m.conv - 1, m.conv_channels), f32)
                fields[f"mem.{r}"] = ((m.heads, m.dim, m.vdim), f32)
            else:
                rr = m.right
                fields[f"mem.{r}"] = ((rr.heads, rr.dim, rr.vdim), f32)
                fields[f"nrm.{r}"] = ((rr.heads, rr.dim), f32)
                fields[f"max.{r}"] = ((rr.heads,), f32)
        return fields

    def attach_cache(self, pool, state_pool=None) -> None:
        """Bind the engine's block pool (``kv_layers[i]`` = pages of attention run i) and state pool."""
        self.kv_cache = pool.kv
        self.kv_layers = pool.layers
        if state_pool is not None:
            self.state = state_pool

    # ------------------------------------------------------------------ mixers
    def _wkv(self, r: int, L, h: torch.Tensor, side, meta: AttnMeta) -> torch.Tensor:
        m = L.spec.mixer
        st = self.state
        T = h.shape[0]
        xs = linrec.token_shift(h, L.mu, st[f"shift.{r}"], meta.positions, meta.row_seq, meta.seq_row0, meta.seq_slots,
                                self.dtype)                                             # [5, T, W]
        # one plain GEMM per blend (a skinny-row kernel at decode sizes): the vendor's batched bf16 product of these
        # four faulted at 32 rows x 2048 x 2048, so no batched call here
        rkvg = [ops.linear(xs[i], L.rkvg[i]) for i in range(4)]                         # 4 x [T, H*D]
        low = torch.tanh(torch.nn.functional.linear(xs[4].float(), L.w1))
        w_raw = torch.nn.functional.linear(low, L.w2)                                   # fp32 decay logits
        y = linrec.wkv_scan(rkvg[0], rkvg[1], rkvg[2], w_raw, L.w0, L.bonus, st[f"mem.{r}"], meta.positions,
                            meta.seq_row0, meta.seq_slots, m.heads, m.dim)
        g = linrec.head_norm_gate(y, rkvg[3], L.mnorm, m.heads, self.cfg.norm_eps, "silu", self.dtype)
        return ops.linear(g, L.o)

    def _delta(self, r: int, L, h: torch.Tensor, side, meta: AttnMeta) -> torch.Tensor:
        m = L.spec.mixer
        st = self.state
        u = ops.linear(h, L.in_proj)                                                    # q | k | v | gate
        cc, qk = m.conv_channels, m.qk_size
        tail = st[f"conv.{r}"] if m.conv > 1 else None
        qkv = recur.causal_conv(u[:, :cc], L.conv, None, tail, meta.positions, meta.row_seq, meta.seq_row0,
                                meta.seq_slots, act=1, residual=False, out_dtype=torch.float32)
        H = m.heads
        y = linrec.delta_scan(qkv[:, :qk], qkv[:, qk:2 * qk], qkv[:, 2 * qk:], side[:, :H], side[:, H:2 * H], L.a_log,
                              L.dt_bias, st[f"mem.{r}"], meta.positions, meta.seq_row0, meta.seq_slots, H, m.kv_heads,
                              m.dim, m.vdim)
        g = linrec.head_norm_gate(y, u[:, cc:], L.mnorm, H, self.cfg.norm_eps, "silu", self.dtype)
        return ops.linear(g, L.o)

    def _attention(self, r: int, L, a, u: torch.Tensor, meta: AttnMeta) -> torch.Tensor:
        """Gated head outputs [T, H * vdim] of the attention branch; ``u`` rows = q | k | v | gate | ..."""
        kc, vc = self.kv_layers[self.kv_index[r]]
        mix.qknorm_rope_cache(u, meta.positions, meta.slot_mapping, L.q_norm, L.k_norm, self.cfg.norm_eps, L.cos_sin,
                              a.heads, a.kv_heads, a.dim, a.vdim, kc, vc, span="full", layout="half")
        gate = u[:, a.q_size + a.k_size + a.v_size: a.q_size + a.k_size + a.v_size + a.o_size]
        out = torch.empty(u.shape[0], a.o_size, device=u.device, dtype=u.dtype)
        nd = meta.num_decode
        kw = dict(softcap=a.softcap, sinks=L.sink)
        if nd > 0:
            mix.masked_attn_rows(u[:nd], kc, vc, meta.dec_block_tables, None, meta.positions[:nd], a.heads, a.kv_heads,
                                 a.scale, 0, gate[:nd], out=out[:nd], **kw)
        if meta.num_prefill_tokens > 0:
            if (u.is_cuda and u.dtype == torch.bfloat16 and a.dim == a.vdim and a.dim in (64, 128)
                    and u.shape[1] % 8 == 0 and mix.masked_prefill_available()
                    and not torch.cuda.is_current_stream_capturing()):
                # MFMA flash kernel (bf16 heads of 64 / 128 dims); other geometries and fp32: the row-wise kernel
                mix.paged_prefill_masked(u[nd:], kc, vc, meta.pre_block_tables, meta.pre_cu_seqlens,
                                         meta.pre_context_lens, a.heads, a.kv_heads, a.scale, 0, gate[nd:],
                                         tiles=meta.pre_tiles, out=out[nd:], **kw)
            else:
                mix.masked_attn_rows(u[nd:], kc, vc, meta.pre_block_tables, meta.pre_cu_seqlens, meta.positions[nd:],
                                     a.heads, a.kv_heads, a.scale, 0, gate[nd:], out=out[nd:], **kw)
        return out

    def _parallel(self, r: int, L, h: torch.Tensor, side, meta: AttnMeta) -> torch.Tensor:
        a, rr = L.spec.mixer.left, L.spec.mixer.right
        st = self.state
        u = ops.linear(h, L.in_proj)
        left = ops.linear(self._attention(r, L, a, u, meta), L.o)
        c0 = a.q_size + a.k_size + a.v_size + a.o_size
        q, k = u[:, c0: c0 + rr.qk_size], u[:, c0 + rr.qk_size: c0 + 2 * rr.qk_size]
        v = u[:, c0 + 2 * rr.qk_size: c0 + 2 * rr.qk_size + rr.inner]
        z = u[:, c0 + 2 * rr.qk_size + rr.inner: c0 + 2 * rr.qk_size + 2 * rr.inner]
        H = rr.heads
        y = linrec.mlstm_scan(q, k, v, side[:, :H], side[:, H:2 * H], rr.gate_cap, st[f"mem.{r}"], st[f"nrm.{r}"],
                              st[f"max.{r}"], meta.positions, meta.seq_row0, meta.seq_slots, H, rr.dim, rr.vdim)
        g = linrec.head_norm_gate(y, z, L.rnorm, H, self.cfg.norm_eps, "sigmoid", self.dtype)
        right = ops.linear(g, L.o_right)
        return linrec.rms_pair_mean(left, right, L.out_left, L.out_right, self.cfg.norm_eps)

    def _moe(self, L, h: torch.Tensor, logits: torch.Tensor) -> torch.Tensor:
        f = L.spec.mlp
        idx, wts = moe.moe_route(logits, None, f.top, score=f.score)
        return moe.moe_experts(h, idx, wts, L.gate_up, L.down, None)

    # ------------------------------------------------------------------ forward
    def forward_layers(self, x: torch.Tensor, meta: AttnMeta) -> torch.Tensor:
        """Run every layer run on the fp32 stream ``x`` [T, W] (updated in place)."""
        c, dt = self.cfg, self.dtype
        eps = c.norm_eps
        starts = c.pass_starts
        x0 = x.clone() if starts else None        # the embedding output, added again before every repeated pass
        pend = (None, None)                       # (mixer output, feed-forward output) whose residual add is due
        mixers = {"wkv": self._wkv, "delta": self._delta, "parallel": self._parallel}
        for r, li in enumerate(self.runs):
            L = self.layers[li]
            if r in starts:
                latent.stream_add_norm(x, pend[0], None, None, eps, None, y2=pend[1])
                pend = (x0, None)
            h = latent.stream_add_norm(x, pend[0], None, L.norm1, eps, dt, y2=pend[1])
            f = L.spec.mlp
            side = None
            if L.side is not None:
                side = torch.nn.functional.linear(h if h.dtype == torch.float32 else h.float(), L.side, L.side_b)
            n_r = f.routes if f is not None else 0
            y = mixers[L.spec.type](r, L, h, None if side is None else side[:, n_r:], meta)
            y2 = self._moe(L, h, side[:, :n_r]) if f is not None else None
            if self.reduce is not None:
                self.reduce(y)
            pend = (y, y2)
            if self.capture_layers and r in self.capture_layers:
                latent.stream_add_norm(x, pend[0], None, None, eps, None, y2=pend[1])
                pend = (None, None)
                self.captured[r] = x.clone()
            if self.layer_hook is not None:
                self.layer_hook(li)
        if pend[0] is not None:
            latent.stream_add_norm(x, pend[0], None, None, eps, None, y2=pend[1])
        return x

    def embed_tokens(self, ids: torch.Tensor) -> torch.Tensor:
        return self.embed.index_select(0, ids.long()).float()

    def forward(self, meta: AttnMeta, input_ids: Optional[torch.Tensor] = None,
                hidden: Optional[torch.Tensor] = None) -> torch.Tensor:
        """fp32 logits [n, V] of the step's logits rows."""
        if meta.seq_slots is None:
            raise RuntimeError("Lofuvik needs the step's sequence tables (a runner built with a state pool)")
        x = self.forward_layers(self.embed_tokens(input_ids), meta)
        idx = meta.logits_indices
        if idx is not None:
            x = x.index_select(0, idx.long())
        return self.compute_logits(x)

    def compute_logits(self, x: torch.Tensor) -> torch.Tensor:
        hn = latent.stream_add_norm(x.contiguous(), None, None, self.final_norm, self.cfg.norm_eps, self.dtype)
        return ops.linear(hn, self.head).float()
