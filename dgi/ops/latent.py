"""Ops of latent-attention models on an fp32 residual stream (``dgi/_C_mix.so``): residual add fused
with RMS norms, the latent projections' norm + rotary + paged cache write, row-wise attention over
cached latents (every head reads the same cached row as its key and its value), the per-head /
per-element output gate, and GELU activations with an optional gathered multiplier.

Latent attention in the form the kernels compute it.  Per token the cache holds one row
``[c | r]``: the normalised latent c (``kv_rank`` dims) and one rotated key part r (``rot_dim``
dims) shared by all heads.  Head h's key is ``[W_uk[h] c | r]`` and its value ``W_uv[h] c``, so

    score_h(i, j) = (q_nope_h(i) . W_uk[h] c_j + q_rot_h(i) . r_j) * scale
                  = ((W_uk[h]^T q_nope_h(i)) . c_j + q_rot_h(i) . r_j) * scale
    out_h(i)      = W_uv[h] (sum_j p_h(i, j) c_j)

i.e. with the query folded through W_uk ("q_lat", a batched GEMM over heads before the kernel) the
attention runs directly on the cached rows, and W_uv is applied once per query to the weighted
latent sum (a batched GEMM after the kernel).  In this form nothing per head is materialised per key;
long prompt portions may instead expand their pages into per-head keys and values for the MFMA
flash kernel (``dgi.models.depelix``), which costs fewer MACs per query and key.

Same rules as ``dgi.ops.mix``: GPU tensors run the HIP kernel (and raise if the library is
missing), CPU tensors the ``*_ref`` function in fp32, which is also the kernel tests' oracle.
"""
from __future__ import annotations

import math
import os
from typing import Optional

import torch

from dgi.ops.mix import _call, _native


# ----------------------------------------------------------------------------
# Residual stream: add (optionally unit-RMS normed and weighted) + next RMS norm
# ----------------------------------------------------------------------------

def _unit_rms(v: torch.Tensor, eps: float) -> torch.Tensor:
    return v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps)


def stream_add_norm_ref(x, y, post_w, next_w, eps, out_dtype, y2=None):
    if y is not None:
        v = y.float()
        if post_w is not None:
            v = _unit_rms(v, eps) * post_w
        if y2 is not None:
            v = v + y2.float()
        x.add_(v)
    if out_dtype is None:
        return None
    return (x if next_w is None else _unit_rms(x, eps) * next_w).to(out_dtype)


def stream_add_norm(x: torch.Tensor, y: Optional[torch.Tensor], post_w: Optional[torch.Tensor],
                    next_w: Optional[torch.Tensor], eps: float, out_dtype=None,
                    y2: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """One pass over the fp32 stream ``x`` [T, W] (updated in place): ``x += y`` — with ``post_w``:
    ``x += y / rms(y) * post_w`` — then, if ``out_dtype`` is given, returns ``x / rms(x) * next_w``
    (``next_w`` None: x itself) in that dtype, the next GEMM's input.  rms(v) = sqrt(mean(v^2) + eps).
    ``y2`` (needs ``y``): a second addend of the same step, ``x += y + y2`` (two sublayers that read
    the same input)."""
    if _native(x):
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device) if out_dtype is not None else None
        _call("stream_add_norm", x, y, post_w, next_w, float(eps), out, y2)
        return out
    return stream_add_norm_ref(x, y, post_w, next_w, eps, out_dtype, y2)


# ----------------------------------------------------------------------------
# Latent projections: norms, rotary, cache write
# ----------------------------------------------------------------------------

def rotate_ref(v: torch.Tensor, cs: torch.Tensor, dims: int, interleaved: bool) -> torch.Tensor:
    """Rotary on the first ``dims`` entries of the last axis of ``v`` [T, ..., d]; ``cs`` [T, dims] holds the
    row's cos (first half) and sin (second half)."""
    if dims <= 0:
        return v
    half = dims // 2
    shape = (cs.shape[0],) + (1,) * (v.dim() - 2) + (half,)
    c, s = cs[:, :half].reshape(shape), cs[:, half:].reshape(shape)
    if interleaved:
        a, b = v[..., 0:dims:2], v[..., 1:dims:2]
        r = torch.stack([a * c - b * s, b * c + a * s], dim=-1).flatten(-2)
    else:
        a, b = v[..., :half], v[..., half:dims]
        r = torch.cat([a * c - b * s, b * c + a * s], dim=-1)
    return torch.cat([r, v[..., dims:]], dim=-1)


def latent_prep_ref(proj, q_rank, kv_rank, rot_dim, dq_w, dkv_w, eps, positions, slots, cos_sin, interleaved, cache):
    T = proj.shape[0]
    cq = (_unit_rms(proj[:, :q_rank].float(), eps) * dq_w).to(proj.dtype)
    if cache is not None and T > 0:
        c = _unit_rms(proj[:, q_rank:q_rank + kv_rank].float(), eps) * dkv_w
        r = proj[:, q_rank + kv_rank:q_rank + kv_rank + rot_dim].float()
        if cos_sin is not None:
            r = rotate_ref(r, cos_sin[positions.long()], cos_sin.shape[1], interleaved)
        row = torch.cat([c, r], dim=-1).to(cache.dtype)
        ok = slots >= 0
        if ok.any():
            s = slots[ok].long()
            bs = cache.shape[2]
            cache[s // bs, 0, s % bs] = row[ok]
    return cq


def latent_prep(proj: torch.Tensor, q_rank: int, kv_rank: int, rot_dim: int, dq_w: torch.Tensor,
                dkv_w: Optional[torch.Tensor], eps: float, positions: torch.Tensor, slots: torch.Tensor,
                cos_sin: Optional[torch.Tensor], interleaved: bool, cache: Optional[torch.Tensor]) -> torch.Tensor:
    """Rows of ``proj`` = [query latent: q_rank | key/value latent: kv_rank | key part: rot_dim | ...].
    Returns the RMS-normed query latent times ``dq_w`` [T, q_rank] in proj's dtype; with ``cache``
    [NB, 1, bs, kv_rank + rot_dim] also writes, at ``slots`` (-1: not written), the RMS-normed
    latent times ``dkv_w`` followed by the key part rotated by the row's position (``cos_sin``
    [max_pos, dims]: first ``dims`` entries rotate — interleaved pairs (2i, 2i+1) or halves
    (i, i + dims/2) — the rest pass).  ``cache`` None (a layer that reads another layer's
    latent): the row has no latent columns and only the query side is computed."""
    if _native(proj):
        cq = torch.empty(proj.shape[0], q_rank, dtype=proj.dtype, device=proj.device)
        _call("latent_prep", cq, proj, int(q_rank), int(kv_rank if cache is not None else 0),
              int(rot_dim if cache is not None else 0), dq_w, dkv_w, float(eps), positions, slots, cos_sin,
              bool(interleaved), cache)
        return cq
    return latent_prep_ref(proj, q_rank, kv_rank, rot_dim, dq_w, dkv_w, eps, positions, slots, cos_sin, interleaved,
                           cache)


# ----------------------------------------------------------------------------
# Attention over cached latents
# ----------------------------------------------------------------------------

def latent_attn_rows_ref(o_lat, q, q_lat, cache, block_tables, cu_seqlens, positions, H, dim, rot_dim, kv_rank, scale,
                         window, cos_sin, interleaved):
    T = q.shape[0]
    bs = cache.shape[2]
    cu = cu_seqlens.tolist() if cu_seqlens is not None else None
    pos = positions.tolist()
    qr = q.float().view(T, H, dim + rot_dim)[:, :, dim:]
    if cos_sin is not None and T > 0:
        qr = rotate_ref(qr, cos_sin[positions.long()], cos_sin.shape[1], interleaved)
    seq = 0
    for t in range(T):
        if cu is None:
            seq = t
        else:
            while cu[seq + 1] <= t:
                seq += 1
        p = pos[t]
        first = max(0, p - window + 1) if window > 0 else 0
        keys = torch.arange(first, p + 1, device=q.device)
        blk = block_tables[seq][keys // bs].long()
        rows = cache[blk, 0, keys % bs].float()                   # [n, kv_rank + rot_dim]
        s = (q_lat[:, t].float() @ rows[:, :kv_rank].t() + qr[t] @ rows[:, kv_rank:].t()) * scale      # [H, n]
        o_lat[:, t] = (torch.softmax(s, dim=-1) @ rows[:, :kv_rank]).to(o_lat.dtype)


SPLIT_WAVES = int(os.environ.get("DGI_LATENT_SPLIT_WAVES", "4096"))     # (row, head, run) waves a small step is cut into


MFMA_ROWS = os.environ.get("DGI_LATENT_MFMA", "1") == "1"     # 0: bf16 rows on the element-wise kernel too (A/B)


def mfma_rows_ok(dtype, kv_rank: int, rot_dim: int) -> bool:
    """Whether ``latent_attn_rows`` takes its MFMA kernel: bf16, latent and latent + key part multiples
    of 16, at most 512 / 576 wide (accumulators and query fragments live in registers)."""
    return (MFMA_ROWS and dtype == torch.bfloat16 and kv_rank % 16 == 0 and (kv_rank + rot_dim) % 16 == 0
            and kv_rank <= 512 and kv_rank + rot_dim <= 576)


def split_runs(rows: int, heads: int, max_keys: int) -> int:
    """Runs of keys per row for a step of ``rows`` x ``heads`` over at most ``max_keys`` keys: 1 when
    the step fills the chip by itself or the bound is unknown, else enough for ``SPLIT_WAVES`` waves,
    every run at least two 64-key tiles long, 16 at most."""
    if max_keys <= 0 or rows <= 0 or rows * heads >= SPLIT_WAVES // 2:
        return 1
    return int(max(1, min(16, SPLIT_WAVES // (rows * heads), max_keys // 128)))


def latent_attn_rows(q: torch.Tensor, q_lat: torch.Tensor, cache: torch.Tensor, block_tables: torch.Tensor,
                     cu_seqlens: Optional[torch.Tensor], positions: torch.Tensor, H: int, dim: int, rot_dim: int,
                     kv_rank: int, scale: float, window: int, cos_sin: Optional[torch.Tensor], interleaved: bool,
                     out: torch.Tensor, max_keys: int = 0) -> torch.Tensor:
    """Softmax attention of every row over the cached rows ``[c | r]`` of its sequence
    (``cache`` [NB, 1, bs, kv_rank + rot_dim], pages by ``block_tables``; rows map to table rows
    through ``cu_seqlens``, None: row i <-> table row i).  Row t at position p sees keys
    [max(0, p - window + 1), p] (``window`` 0: [0, p]).  Head h's score of key j is
    ``(q_lat[h, t] . c_j + rot(q[t, h, dim:]) . r_j) * scale``: ``q_lat`` [H, T, kv_rank] is the
    unrotated query part folded through the key up-projection, ``q`` [T, H * (dim + rot_dim)] the
    query projection whose rotated part is rotated here by the row's position.  Writes the
    weighted latent sums ``out`` [H, T, kv_rank] (any strides with unit inner stride).  ``max_keys``: an
    upper bound of the keys a row sees, if the caller knows one — a step of few rows over many keys
    is then cut into several runs of keys per row (more workgroups than rows x heads) and combined."""
    if _native(q):
        T = q.shape[0]
        mfma = mfma_rows_ok(q.dtype, kv_rank, rot_dim)
        # the MFMA kernel's workgroups (16 heads, 4 waves) are best at about one per compute unit
        nsplit = split_runs(T, (H + 15) // 16 * 16 if mfma else H,
                            min(max_keys, window) if window > 0 and max_keys > 0 else max_keys)
        po = pm = None
        if nsplit > 1:
            po = torch.empty(nsplit * H * T * kv_rank, dtype=torch.float32, device=q.device)
            pm = torch.empty(nsplit * H * T * 2, dtype=torch.float32, device=q.device)
        _call("latent_attn_rows", out, q, q_lat, cache, block_tables, cu_seqlens, positions, int(H), int(dim),
              int(rot_dim), int(kv_rank), float(scale), int(window), cos_sin, bool(interleaved), nsplit, po, pm, mfma)
    else:
        latent_attn_rows_ref(out, q, q_lat, cache, block_tables, cu_seqlens, positions, H, dim, rot_dim, kv_rank, scale,
                             window, cos_sin, interleaved)
    return out


def gate_heads_ref(ov, gate, per_head):
    H, T, dv = ov.shape
    g = torch.sigmoid(gate.float())
    o = ov.float().permute(1, 0, 2)                                # [T, H, dv]
    o = o * (g[:, :, None] if per_head else g.view(T, H, dv))
    return o.reshape(T, H * dv).to(ov.dtype)


def gate_heads(ov: torch.Tensor, gate: Optional[torch.Tensor], per_head: bool,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Head outputs ``ov`` [H, T, dv] (any head / row strides) -> [T, H * dv] (heads side by side),
    multiplied by sigmoid(gate): ``gate`` [T, H] with ``per_head`` (one gate per head), else
    [T, H * dv]; None: no gate.  ``out``: contiguous rows to write."""
    H, T, dv = ov.shape
    if _native(ov):
        if out is None:
            out = torch.empty(T, H * dv, dtype=ov.dtype, device=ov.device)
        _call("gate_heads", out, ov, gate, bool(per_head))
        return out
    r = ov.permute(1, 0, 2).reshape(T, H * dv).contiguous() if gate is None else gate_heads_ref(ov, gate, per_head)
    if out is not None:
        out.copy_(r)
        return out
    return r


def rotate_heads(x: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor, interleaved: bool, H: int,
                 head_size: int, offset: int) -> torch.Tensor:
    """Rotary in place on ``cos_sin.shape[1]`` entries starting at ``offset`` inside each of the H heads
    (``head_size`` apart) of every row of ``x`` [T, >= H * head_size], by the row's position."""
    if _native(x):
        _call("rotate_heads", x, positions, cos_sin, bool(interleaved), int(H), int(head_size), int(offset))
        return x
    T, dims = x.shape[0], cos_sin.shape[1]
    if T:
        v = x[:, :H * head_size].view(T, H, head_size)
        r = rotate_ref(v[:, :, offset:offset + dims].float(), cos_sin[positions.long()], dims, interleaved)
        v[:, :, offset:offset + dims] = r.to(x.dtype)
    return x


# ----------------------------------------------------------------------------
# GELU (tanh form), optionally times a gathered table slice
# ----------------------------------------------------------------------------

_GELU_C = math.sqrt(2.0 / math.pi)


def gelu_tanh_ref(x: torch.Tensor, table=None, ids=None, col0: int = 0) -> torch.Tensor:
    z = x.float()
    y = 0.5 * z * (1.0 + torch.tanh(_GELU_C * (z + 0.044715 * z * z * z)))
    if table is not None:
        y = y * table[ids.long(), col0:col0 + x.shape[1]].float()
    return y.to(x.dtype)


def gelu_tanh(x: torch.Tensor, table: Optional[torch.Tensor] = None, ids: Optional[torch.Tensor] = None,
              col0: int = 0) -> torch.Tensor:
    """0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))) over ``x`` [T, n]; with ``table`` [V, C] and
    ``ids`` [T]: times ``table[ids[t], col0 : col0 + n]`` (a per-token input gathered in the same pass)."""
    if _native(x):
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _call("gelu_tanh", out, x, table, ids, int(col0))
        return out
    return gelu_tanh_ref(x, table, ids, col0)
