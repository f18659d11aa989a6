"""Mixture-of-experts feed-forward ops (``dgi/_C_mix.so``): routing, expert evaluation, combine.

Routing is fp32: scores s = softmax(logits) over all routes (real experts, then identity
experts) — or independent sigmoids (``score="sigmoid"``) — the ``top`` routes by s + selection bias
are taken and weighed by s itself (not renormalised).  A real expert e is
W_down[e] act(W_gate[e] x, W_up[e] x) with act(g, u) = silu(g) * u, or the clamped sigmoid-GLU
g' sigmoid(alpha g') (u' + 1), g' = min(g, limit), u' = clamp(u, +-limit) (``act="clamped"``); an
identity route returns h.  The route weight multiplies the expert's output, or
(``weigh="input"``) its input x = w h; since both projections are linear the kernels apply w to
the projections' results, W (w h) = w (W h), in fp32 before the clamps.  Expert weights are
stacked: ``gate_up`` [E, 2 ff, W] (gate rows, then up rows) and ``down`` [E, W, ff].

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


def glu_rows_ref(gu, act, limit, alpha, row_scale):
    I = gu.shape[-1] // 2
    g, u = gu[..., :I].float(), gu[..., I:].float()
    if row_scale is not None:
        g, u = g * row_scale[:, None], u * row_scale[:, None]
    if act == "clamped":
        g, u = g.clamp(max=limit), u.clamp(-limit, limit)
        return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)
    return (g * torch.sigmoid(g) * u).to(gu.dtype)


def glu_rows(gu: torch.Tensor, act: str = "silu", limit: float = 0.0, alpha: float = 1.702,
             row_scale: torch.Tensor = None) -> torch.Tensor:
    """Expert activation over fused [gate | up] rows [n, 2 ff]; ``row_scale`` [n] fp32 multiplies
    both halves first (a route weight on the expert's input, applied after the projection)."""
    if _native(gu):
        if act == "silu" and row_scale is None:
            return silu_mul(gu)
        out = torch.empty(gu.shape[0], gu.shape[1] // 2, dtype=gu.dtype, device=gu.device)
        _call("glu_rows", out, gu, 1 if act == "clamped" else 0, float(limit), float(alpha), row_scale)
        return out
    return glu_rows_ref(gu, act, limit, alpha, row_scale)


def moe_route_ref(logits, correction, top, score="softmax"):
    if score == "top_softmax":
        lf = logits.float()
        idx = torch.sort(lf, dim=-1, descending=True, stable=True).indices[:, :top]
        return idx.to(torch.int32), torch.softmax(torch.gather(lf, 1, idx), -1)
    s = torch.softmax(logits.float(), -1) if score == "softmax" else torch.sigmoid(logits.float())
    pick = s if correction is None else s + correction
    idx = torch.sort(pick, dim=-1, descending=True, stable=True).indices[:, :top]      # ties: the lowest index first
    return idx.to(torch.int32), torch.gather(s, 1, idx)


def moe_route(logits: torch.Tensor, correction, top: int, score: str = "softmax"):
    """fp32 ``logits`` [T, R] -> (routes [T, top] int32 ordered by falling s + correction,
    weights [T, top] fp32 = the plain scores of those routes); s = softmax over the routes, or
    sigmoid of each (``score="sigmoid"``); ``correction`` None: the choice is by s alone.  Ties
    go to the lowest index.  ``score="top_softmax"``: the ``top`` largest logits are taken and the
    weights are the softmax over those alone (no ``correction``)."""
    if _native(logits):
        T = logits.shape[0]
        idx = torch.empty(T, top, dtype=torch.int32, device=logits.device)
        w = torch.empty(T, top, dtype=torch.float32, device=logits.device)
        if score == "top_softmax" and correction is not None:
            raise ValueError("moe_route: top_softmax takes no selection bias")
        _call("moe_route", idx, w, logits, correction, {"softmax": 0, "sigmoid": 1, "top_softmax": 2}[score])
        return idx, w
    return moe_route_ref(logits, correction, top, score)


def moe_experts_ref(h, idx, wts, gate_up, down, shared, act="silu", limit=0.0, alpha=1.702, weigh="output"):
    T, W = h.shape
    E = gate_up.shape[0]
    ff = down.shape[2]
    hf = h.float()
    out = torch.zeros(T, W) if shared is None else shared.float().clone()
    for t in range(T):
        for e, w in zip(idx[t].tolist(), wts[t].tolist()):
            if e >= E:
                out[t] += w * hf[t]
                continue
            w_in, w_out = (w, 1.0) if weigh == "input" else (1.0, w)
            gu = (gate_up[e].float() @ hf[t]) * w_in
            g, u = gu[:ff], gu[ff:]
            if act == "clamped":
                g, u = g.clamp(max=limit), u.clamp(-limit, limit)
                mid = g * torch.sigmoid(alpha * g) * (u + 1.0)
            else:
                mid = g * torch.sigmoid(g) * u
            out[t] += w_out * (down[e].float() @ mid)
    return out.to(h.dtype)


def moe_experts(h, idx, wts, gate_up, down, shared=None, act: str = "silu", limit: float = 0.0, alpha: float = 1.702,
                weigh: str = "output") -> torch.Tensor:
    """sum_k route_{idx[t, k]}(h_t) weighed by wts[t, k] on the output or (``weigh="input"``) on the
    expert's input (+ ``shared`` [T, W]) in h's dtype; ``act`` / ``limit`` / ``alpha``: the experts'
    activation (``glu_rows``)."""
    if not _native(h):
        return moe_experts_ref(h, idx, wts, gate_up, down, shared, act, limit, alpha, weigh)
    T, W = h.shape
    E, ff = gate_up.shape[0], down.shape[2]
    top = idx.shape[1]
    plain = act == "silu" and weigh == "output"
    w_in = wts if weigh == "input" else None             # weights applied inside the activation
    w_out = None if weigh == "input" else wts            # weights applied by the combine (None: 1)
    out = torch.empty(T, W, dtype=h.dtype, device=h.device)
    if T <= EXPERT_MAJOR_ROWS or torch.cuda.is_current_stream_capturing():
        if T * top >= E:
            # a small step that touches (nearly) every expert anyway: all experts as one batched vendor GEMM
            # over the step's rows (weight-bandwidth bound either way; the extra FLOPs are free at these
            # sizes), then every token picks its routes' rows in the combine
            gu = torch.matmul(h.unsqueeze(0), gate_up.transpose(1, 2))                  # [E, T, 2 ff]
            where = (idx * T + torch.arange(T, dtype=torch.int32, device=h.device)[:, None]).clamp_(0, E * T - 1)
            rs = None
            if w_in is not None:      # the weight of pair (t, e) at row e * T + t; rows nobody chose are never read
                rs = torch.ones(E * T, dtype=torch.float32, device=h.device)
                rs.index_put_((where.reshape(-1).long(),), w_in.reshape(-1))
            act_rows = silu_mul(gu.view(E * T, 2 * ff)) if plain else glu_rows(gu.view(E * T, 2 * ff), act, limit, alpha, rs)
            ys = torch.bmm(act_rows.view(E, T, ff), down.transpose(1, 2)).view(E * T, W)
            _call("moe_combine", out, ys, where, h, idx, w_out, shared, E)
            return out
        mid = torch.empty(T * top, ff, dtype=torch.float32, device=h.device)
        ys = torch.empty(T * top, W, dtype=h.dtype, device=h.device)     # identity pairs' rows are never read
        _call("moe_expert_gate_up", mid, h, idx, gate_up, w_in, 1 if act == "clamped" else 0, float(limit), float(alpha))
        _call("moe_expert_down", ys, mid, idx, down)
        _call("moe_combine", out, ys, None, h, idx, w_out, shared, E)
        return out
    from dgi import ops
    flat = idx.reshape(-1).long()
    order = torch.argsort(flat, stable=True)                       # pairs grouped by route
    counts = torch.bincount(flat, minlength=E).tolist()            # host: segment sizes
    xs = h.index_select(0, order // top)
    rs = w_in.reshape(-1)[order].contiguous() if w_in is not None else None
    ys = torch.empty(T * top, W, dtype=h.dtype, device=h.device)   # identity segments are never read
    o = 0
    for e in range(E):
        c = counts[e]
        if c:
            gu = ops.linear(xs[o:o + c], gate_up[e])
            a = silu_mul(gu) if plain else glu_rows(gu, act, limit, alpha, None if rs is None else rs[o:o + c])
            torch.matmul(a, down[e].t(), out=ys[o:o + c])
            o += c
    where = torch.empty_like(order)
    where[order] = torch.arange(order.numel(), device=order.device)
    _call("moe_combine", out, ys, where.to(torch.int32), h, idx, w_out, shared, E)
    return out
