"""Mixer-block ops for models with fp32 residual streams and per-layer head geometry
(``dgi/_C_mix.so``, sources in ``dgi/csrc/mix``): Dynamic-Tanh norms, per-head q/k RMS norm +
interleaved rotary + paged KV write, row-wise masked attention, clamped GLU, soft-capped logits.

Same contract as the rest of ``dgi.ops``: the HIP kernel runs whenever the tensors are on the
GPU (and raises if the library is missing), the ``*_ref`` function — plain PyTorch, fp32 math —
runs on CPU tensors and is the oracle of the kernel tests.  Activations are bf16 or fp32; norm
parameters and the residual stream are fp32 in both.
"""
from __future__ import annotations

import os
from typing import Optional

import torch

_LIB = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "_C_mix.so")
_loaded = False


def load_native(required: bool = False) -> bool:
    """Load ``dgi/_C_mix.so`` once (built by ``python -m dgi.build mix``)."""
    global _loaded
    if _loaded:
        return True
    err = f"{_LIB} not built (run `python -m dgi.build mix`)"
    if os.path.exists(_LIB):
        try:
            torch.ops.load_library(_LIB)
            _loaded = True
            return True
        except Exception as e:  # pragma: no cover - depends on the box
            err = repr(e)
    if required:
        raise RuntimeError(f"dgi mixer kernels unavailable: {err}")
    return False


def _native(t: torch.Tensor) -> bool:
    if t.is_cuda:
        load_native(required=True)
        return True
    return False


def _call(name: str, *args) -> None:
    from dgi import ops
    getattr(torch.ops.dgi, name)(*args)
    if ops._DEBUG_SYNC:
        from dgi.utils.debug import after_op
        after_op(name, *args)


class DytNorm:
    """Parameters of one Dynamic-Tanh norm, y = tanh(alpha * x) * w + b (all fp32)."""
    __slots__ = ("alpha", "w", "b")

    def __init__(self, alpha: torch.Tensor, w: torch.Tensor, b: torch.Tensor):
        self.alpha, self.w, self.b = alpha, w, b

    def tensors(self):
        return (("alpha", self.alpha), ("w", self.w), ("b", self.b))


# ----------------------------------------------------------------------------
# Dynamic-Tanh norms
# ----------------------------------------------------------------------------

def dyt_ref(x: torch.Tensor, n: DytNorm, dtype: torch.dtype) -> torch.Tensor:
    return (torch.tanh(n.alpha * x.float()) * n.w + n.b).to(dtype)


def dyt(x: torch.Tensor, n: DytNorm, dtype: torch.dtype) -> torch.Tensor:
    """Norm of the fp32 stream ``x`` [T, W] -> [T, W] in ``dtype`` (the GEMM input)."""
    if _native(x):
        y = torch.empty(x.shape, dtype=dtype, device=x.device)
        _call("dyt", y, x, n.alpha, n.w, n.b)
        return y
    return dyt_ref(x, n, dtype)


def dyt_add_ref(res: torch.Tensor, h: torch.Tensor, post: DytNorm, ls: torch.Tensor,
                nxt: Optional[DytNorm] = None) -> Optional[torch.Tensor]:
    res.add_((torch.tanh(post.alpha * h.float()) * post.w + post.b) * ls)
    return None if nxt is None else dyt_ref(res, nxt, h.dtype)


def dyt_add(res: torch.Tensor, h: torch.Tensor, post: DytNorm, ls: torch.Tensor,
            nxt: Optional[DytNorm] = None) -> Optional[torch.Tensor]:
    """res += post(h) * ls in place (sublayer output norm, layer scale, residual add); with
    ``nxt`` also returns nxt(res) in h's dtype — the next sublayer's input, from the same pass."""
    if _native(res):
        y = torch.empty(res.shape, dtype=h.dtype, device=res.device) if nxt is not None else None
        _call("dyt_add", res, h, post.alpha, post.w, post.b, ls, y, *((nxt.alpha, nxt.w, nxt.b) if nxt else (None,) * 3))
        return y
    return dyt_add_ref(res, h, post, ls, nxt)


def embed_dyt_ref(ids: torch.Tensor, table: torch.Tensor, scale: float, n: DytNorm) -> torch.Tensor:
    ids = ids.long().clamp(0, table.shape[0] - 1)          # the kernel clamps too: no read outside the table
    return dyt_ref(table[ids].float() * scale, n, torch.float32)


def embed_dyt(ids: torch.Tensor, table: torch.Tensor, scale: float, n: DytNorm) -> torch.Tensor:
    """fp32 stream [T, W] = n(table[ids] * scale)."""
    if _native(table):
        res = torch.empty(ids.numel(), table.shape[1], dtype=torch.float32, device=table.device)
        _call("embed_dyt", res, ids.long().contiguous(), table, float(scale), n.alpha, n.w, n.b)
        return res
    return embed_dyt_ref(ids, table, scale, n)


# ----------------------------------------------------------------------------
# q/k norm + rotary + paged cache write
# ----------------------------------------------------------------------------

def _rot_pairs(x: torch.Tensor, cs: torch.Tensor) -> torch.Tensor:
    """Interleaved-pair rotation of the first rd = cs.shape[-1] dims of x [T, heads, d] (fp32)."""
    rd = cs.shape[-1]
    if rd == 0:
        return x
    c, s = cs[:, None, : rd // 2], cs[:, None, rd // 2:]
    u, v = x[..., 0:rd:2], x[..., 1:rd:2]
    r = torch.stack([u * c - v * s, v * c + u * s], dim=-1).flatten(-2)
    return torch.cat([r, x[..., rd:]], dim=-1)


def _rot_halves(x: torch.Tensor, cs: torch.Tensor) -> torch.Tensor:
    """Half-split rotation (pairs i, i + rd/2) of the first rd = cs.shape[-1] dims of x [T, heads, d] (fp32)."""
    rd = cs.shape[-1]
    if rd == 0:
        return x
    h = rd // 2
    c, s = cs[:, None, :h], cs[:, None, h:]
    u, v = x[..., :h], x[..., h:rd]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., rd:]], dim=-1)


def qknorm_rope_cache_ref(qkv, positions, slots, qw, kw, eps, cos_sin, H, G, dk, dv, k_cache, v_cache,
                          q_temp=None, span="head", layout="interleaved") -> None:
    T = qkv.shape[0]
    if T == 0:
        return
    bs = k_cache.shape[2]
    q = qkv[:, : H * dk].float()
    k = qkv[:, H * dk:(H + G) * dk].float()
    v = qkv[:, (H + G) * dk:(H + G) * dk + G * dv].view(T, G, dv)
    if span == "full":
        q = (q / torch.sqrt(q.pow(2).mean(-1, keepdim=True) + eps) * qw).view(T, H, dk)
        k = (k / torch.sqrt(k.pow(2).mean(-1, keepdim=True) + eps) * kw).view(T, G, dk)
    else:
        q, k = q.view(T, H, dk), k.view(T, G, dk)
        q = q / torch.sqrt(q.pow(2).mean(-1, keepdim=True) + eps) * qw
        k = k / torch.sqrt(k.pow(2).mean(-1, keepdim=True) + eps) * kw
    if q_temp is not None and q_temp[1] > 0:
        steps = torch.div(positions.long() + 1, int(q_temp[1]), rounding_mode="floor")
        q = q * (1.0 + float(q_temp[0]) * torch.log(steps.float() + 1.0))[:, None, None]
    if cos_sin is not None:
        cs = cos_sin[positions.long()]
        rot = _rot_halves if layout == "half" else _rot_pairs
        q, k = rot(q, cs), rot(k, cs)
    qkv[:, : H * dk] = q.reshape(T, H * dk).to(qkv.dtype)
    ok = slots >= 0
    if ok.any():
        s = slots[ok].long()
        k_cache[s // bs, :, s % bs] = k[ok].to(k_cache.dtype)
        v_cache[s // bs, :, s % bs] = v[ok]


def qknorm_rope_cache(qkv, positions, slots, qw, kw, eps: float, cos_sin, H: int, G: int, dk: int, dv: int,
                      k_cache, v_cache, q_temp=None, span: str = "head", layout: str = "interleaved") -> None:
    """Rows of ``qkv`` = [q: H*dk | k: G*dk | v: G*dv | ...]: per-head RMS norm (weights ``qw`` /
    ``kw`` [dk], eps inside the root) and interleaved rotary (``cos_sin`` [max_pos, rd], or None)
    of q in place and of k into ``k_cache`` [NB, G, bs, dk]; v into ``v_cache`` [NB, G, bs, dv]
    at ``slots`` (-1: not written).  ``q_temp`` = (coef, every): the normalised q of a row at
    position p is also multiplied by 1 + coef * ln(floor((p + 1) / every) + 1).
    ``span`` "full": the RMS runs over the whole q (and the whole k) projection of a row instead of
    per head, with weights ``qw`` [H*dk] / ``kw`` [G*dk].  ``layout`` "half": rotary pairs are
    (i, i + rd/2) inside a head instead of (2i, 2i+1)."""
    qt = (float(q_temp[0]), int(q_temp[1])) if q_temp is not None else (0.0, 0)
    if _native(qkv):
        if span == "head" and layout == "interleaved":
            _call("qknorm_rope_cache", qkv, positions, slots, qw, kw, float(eps), cos_sin, H, G, dk, dv, k_cache,
                  v_cache, qt[0], qt[1])
        else:
            if qt[1]:
                raise ValueError("qknorm_rope_cache: a query temperature needs span='head', layout='interleaved'")
            _call("qk_prep", qkv, positions, slots, qw, kw, float(eps), cos_sin, H, G, dk, dv, k_cache, v_cache,
                  span == "full", layout == "half")
    else:
        qknorm_rope_cache_ref(qkv, positions, slots, qw, kw, eps, cos_sin, H, G, dk, dv, k_cache, v_cache, qt, span,
                              layout)


# ----------------------------------------------------------------------------
# Row-wise masked attention
# ----------------------------------------------------------------------------

def distance_bias_table(rel: torch.Tensor, far: float) -> torch.Tensor:
    """fp32 bias by distance [n, H] from a bucketed table ``rel`` [rows, H]
    (``dgi.models.config.distance_bucket``): row d is the bias at distance d, the last row serves
    every distance beyond it (the buckets end at ``far``)."""
    from dgi.models.config import distance_bucket
    rows = rel.shape[0]
    n = max(int(-(-far // 1)), rows // 2) + 1
    idx = torch.tensor([distance_bucket(d, rows, far) for d in range(n)], dtype=torch.long, device=rel.device)
    return rel.float()[idx].contiguous()


def masked_attn_rows_ref(q, k_cache, v_cache, block_tables, cu_seqlens, positions, H, G, scale, mask, gate=None,
                         dist_bias=None, window=0, softcap=0.0, sinks=None):
    T = q.shape[0]
    bs, dk, dv = k_cache.shape[2], k_cache.shape[3], v_cache.shape[3]
    out = torch.zeros(T, H * dv, dtype=q.dtype, device=q.device)
    cu = cu_seqlens.tolist() if cu_seqlens is not None else None
    pos = positions.tolist()
    seq = 0
    for t in range(T):
        if cu is None:
            seq = t
        else:
            while cu[seq + 1] <= t:
                seq += 1
        p = pos[t]
        first = (p // mask) * mask if mask > 0 else (max(0, p - window + 1) if window > 0 else 0)
        keys = torch.arange(first, p + 1, device=q.device)
        blk = block_tables[seq][keys // bs].long()
        k = k_cache[blk, :, keys % bs].float()          # [n, G, dk]
        v = v_cache[blk, :, keys % bs].float()
        qt = q[t, : H * dk].float().view(G, H // G, dk)
        s = torch.einsum("ghd,ngd->ghn", qt, k) * scale
        if dist_bias is not None:
            d = (p - keys).clamp(max=dist_bias.shape[0] - 1)
            s = s + dist_bias[d].t().reshape(G, H // G, -1)
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        if sinks is not None:
            # the sink is one more logit in the denominator; it has no value
            s = torch.cat([s, sinks.float().reshape(G, H // G, 1)], dim=-1)
            pr = torch.softmax(s, dim=-1)[..., :-1]
        else:
            pr = torch.softmax(s, dim=-1)
        o = torch.einsum("ghn,ngd->ghd", pr, v).reshape(H * dv)
        if gate is not None:
            o = o * torch.sigmoid(gate[t, : H * dv].float())
        out[t] = o.to(q.dtype)
    return out


def masked_attn_rows(q, k_cache, v_cache, block_tables, cu_seqlens, positions, H: int, G: int, scale: float,
                     mask: int = 0, gate=None, out=None, dist_bias=None, softcap: float = 0.0, sinks=None) -> torch.Tensor:
    """Softmax attention of each row of ``q`` (position ``positions[t]``) over keys
    [floor(p / mask) * mask, p] of its sequence (``mask`` 0: [0, p]) read from the paged cache;
    rows map to ``block_tables`` rows through ``cu_seqlens`` (None: row i <-> table row i).
    ``gate``: the output is multiplied by sigmoid(gate) element by element.  ``dist_bias``
    [n, H] fp32: added to the scaled score of a key at distance d = p - j, row min(d, n - 1).
    ``softcap`` > 0: the (scaled, biased) score s becomes softcap * tanh(s / softcap).  ``sinks`` [H] fp32:
    exp(sinks[h]) joins head h's softmax denominator (a logit without a key or a value)."""
    if _native(q):
        if out is None:
            out = torch.empty(q.shape[0], H * v_cache.shape[3], dtype=q.dtype, device=q.device)
        _call("masked_attn_rows", out, q, k_cache, v_cache, block_tables, cu_seqlens, positions, H, G, float(scale),
              int(mask), gate, dist_bias, float(softcap), sinks)
        return out
    r = masked_attn_rows_ref(q, k_cache, v_cache, block_tables, cu_seqlens, positions, H, G, scale, mask, gate,
                             dist_bias, 0, softcap, sinks)
    if out is not None:
        out.copy_(r)
        return out
    return r


# ----------------------------------------------------------------------------
# MFMA prompt attention with a block mask (bf16, equal key / value size of 64 or 128)
# ----------------------------------------------------------------------------

MASKED_PREFILL = os.environ.get("DGI_MASKED_PREFILL", "1") == "1"   # 0: prompt rows on the row-wise kernel (A/B)


def masked_prefill_available() -> bool:
    """Whether prompt portions may take the MFMA kernel with a block mask and gate epilogue."""
    from dgi import ops
    return MASKED_PREFILL and ops.PREFILL_TILE == 128


def paged_prefill_masked(q, k_cache, v_cache, block_tables, cu_seqlens_q, context_lens, nh, nkv, scale,
                         mask: int = 0, gate=None, tiles=None, out=None, dist_bias=None, window: int = 0,
                         softcap: float = 0.0, sinks=None) -> torch.Tensor:
    """``paged_prefill`` with a block mask — a query at position p sees keys
    [floor(p / mask) * mask, p] (``mask`` 0: all keys up to p) — or a sliding window (``window`` > 0
    with ``mask`` 0: keys [max(0, p - window + 1), p]) and an optional sigmoid output
    gate (out *= sigmoid(gate)) and an optional distance bias (``dist_bias`` as in
    ``masked_attn_rows``), an optional score soft cap and per-head sink logits (``softcap`` / ``sinks``, as in
    ``masked_attn_rows``).  bf16, key size == value size in {64, 128} on the GPU
    (dgi/csrc/mix/masked_prefill.hip); the row-wise reference elsewhere."""
    from dgi import ops
    if _native(q):
        hd = k_cache.shape[-1]
        if out is None:
            out = torch.empty(q.shape[0], nh * hd, dtype=q.dtype, device=q.device)
        if tiles is None:
            tl = ops.prefill_tiles(cu_seqlens_q.tolist(), context_lens=context_lens.tolist(), tile=128)
            tiles = torch.tensor(tl if tl else [[0, 0]], dtype=torch.int32, device=q.device)[: len(tl)]
        if mask and window:
            raise ValueError("paged_prefill_masked: a block mask or a window, not both")
        _call("paged_prefill_masked", out, q, k_cache, v_cache, block_tables, cu_seqlens_q, context_lens, tiles,
              nh, nkv, float(scale), int(mask) if mask else -int(window), gate, dist_bias,      # the kernel takes a window as a negative mask
              float(softcap), sinks)
        return out
    cu = cu_seqlens_q.tolist()
    pos = torch.cat([torch.arange(int(context_lens[b]) - (cu[b + 1] - cu[b]), int(context_lens[b]), dtype=torch.int32)
                     for b in range(len(cu) - 1)]) if len(cu) > 1 else torch.zeros(0, dtype=torch.int32)
    r = masked_attn_rows_ref(q, k_cache, v_cache, block_tables, cu_seqlens_q, pos.to(q.device), nh, nkv, scale,
                             mask, gate, dist_bias, window, softcap, sinks)
    if out is not None:
        out.copy_(r)
        return out
    return r


# ----------------------------------------------------------------------------
# Activations / logits
# ----------------------------------------------------------------------------

def glu_clamped_ref(gu: torch.Tensor, limit: float, alpha: float = 1.702) -> torch.Tensor:
    I = gu.shape[-1] // 2
    g = gu[..., :I].float().clamp(max=limit)
    u = gu[..., I:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)


def glu_clamped(gu: torch.Tensor, limit: float, alpha: float = 1.702) -> torch.Tensor:
    """g * sigmoid(alpha g) * (u + 1) over the fused [gate | up] rows, gate clamped from above
    and up to [-limit, limit]."""
    if _native(gu):
        out = torch.empty(gu.shape[0], gu.shape[1] // 2, dtype=gu.dtype, device=gu.device)
        _call("glu_clamped", out, gu, float(limit), float(alpha))
        return out
    return glu_clamped_ref(gu, limit, alpha)


def scale_softcap_ref(x: torch.Tensor, scale: float, cap: float) -> torch.Tensor:
    v = x.float() * scale
    return cap * torch.tanh(v / cap) if cap > 0 else v


def scale_softcap(x: torch.Tensor, scale: float, cap: float) -> torch.Tensor:
    """fp32 logits = cap * tanh(x * scale / cap) (cap <= 0: x * scale)."""
    if _native(x):
        out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
        _call("scale_softcap", out, x, float(scale), float(cap))
        return out
    return scale_softcap_ref(x, scale, cap)
