"""Ops of mixers that carry a matrix state per head from token to token (``dgi/_C_mix.so``):
RWKV-style time mixing, the gated delta rule and the matrix memory of xLSTM, plus the small ops
around them (blends with the previous token's input, per-head RMS norm with an output gate, the
mean of two width-normed branches).

All three recurrences keep S [dk, dv] per (sequence, head) in fp32 and differ in the update:

    wkv     o_t = (S + diag(u) k v^T)^T r          S <- diag(w) S + k v^T          w per key channel
    delta   S <- g S;  S += k (beta (v - S^T k))^T  o_t = S^T q                    g, beta per head
    mlstm   m' = max(f + m, i);  S <- e^(f+m-m') S + e^(i-m') k v^T  (n likewise with k alone)
            o_t = S^T q / (max(|n . q|, e^(-m')) + 1e-6)

Everything that enters a recurrence besides q / k / v themselves (decays, gates, unit norms,
stabiliser) is fp32 whatever the activation dtype.  States live in ``dgi.kv.state_pool`` slots
([slots, heads, dk, dv] fp32); a portion that starts at position 0 reads no state.

Same rules as ``dgi.ops.mix``: GPU tensors run the HIP kernel (and raise if the library is
missing), CPU tensors the ``*_ref`` function in fp32, which is also the kernel tests' oracle.
Rows of a step are ``[decode rows | prompt portions]``; ``seq_row0`` [n + 1] holds the first row of
each sequence of the step, ``seq_slots`` [n] its state slot, ``row_seq`` [T] each row's sequence.
"""
from __future__ import annotations

from typing import Optional

import torch

from dgi.ops.mix import _call, _native
from dgi.ops.recur import _seqs


# ----------------------------------------------------------------------------
# Blends of the current and the previous token's input
# ----------------------------------------------------------------------------

def token_shift_ref(h, mu, tail, positions, seq_row0, seq_slots, out_dtype):
    T, W = h.shape
    hf = h.float()
    prev = torch.zeros(T, W)
    prev[1:] = hf[:-1]
    for r0, r1, slot, p0 in _seqs(positions, seq_row0, seq_slots):
        if r1 == r0:
            continue
        prev[r0] = 0.0 if p0 == 0 else tail[slot]
        tail[slot] = hf[r1 - 1]
    return (hf[None] + (prev - hf)[None] * mu[:, None, :]).to(out_dtype)


def token_shift(h, mu, tail, positions, row_seq, seq_row0, seq_slots, out_dtype=None) -> torch.Tensor:
    """out[s] = h + (h' - h) * mu[s] for each of the n blends ``mu`` [n, W] (fp32), h' being the previous
    token's row of ``h`` [T, W]: the row above inside a portion, ``tail[slot]`` ([slots, W] fp32) for a
    portion's first row, zeros at position 0.  ``tail`` then receives each portion's last row.
    Returns [n, T, W] in ``out_dtype`` (default h's)."""
    out_dtype = out_dtype or h.dtype
    if _native(h):
        out = torch.empty(mu.shape[0], h.shape[0], h.shape[1], dtype=out_dtype, device=h.device)
        _call("token_shift", out, h, mu, tail, positions, row_seq, seq_row0, seq_slots)
        return out
    return token_shift_ref(h, mu, tail, positions, seq_row0, seq_slots, out_dtype)


# ----------------------------------------------------------------------------
# The recurrences
# ----------------------------------------------------------------------------

def _heads(x, n, d):
    return x.float().reshape(x.shape[0], n, d)


def wkv_scan_ref(r, k, v, w_raw, w0, u, state, positions, seq_row0, seq_slots, H, D):
    T = r.shape[0]
    rr, kk, vv = _heads(r, H, D), _heads(k, H, D), _heads(v, H, D)
    dec = torch.exp(-torch.exp(w_raw.float() + w0)).reshape(T, H, D)
    uu = u.reshape(H, D)
    y = torch.zeros(T, H, D)
    for r0, r1, slot, p0 in _seqs(positions, seq_row0, seq_slots):
        if r1 == r0:
            continue
        S = torch.zeros(H, D, D) if p0 == 0 else state[slot].clone()
        for t in range(r0, r1):
            kv = kk[t, :, :, None] * vv[t, :, None, :]
            y[t] = torch.einsum("hkv,hk->hv", S + uu[:, :, None] * kv, rr[t])
            S = dec[t, :, :, None] * S + kv
        state[slot] = S
    return y.reshape(T, H * D)


def wkv_scan(r, k, v, w_raw, w0, u, state, positions, seq_row0, seq_slots, H: int, D: int) -> torch.Tensor:
    """RWKV-style recurrence over packed rows.  ``r`` / ``k`` / ``v`` [T, H*D] (rows may be strided),
    ``w_raw`` [T, H*D] the projected decay logits, ``w0`` [H*D] their offset, ``u`` [H*D] the bonus:
    per head w = exp(-exp(w_raw + w0)), o = (S + diag(u) k v^T)^T r, S <- diag(w) S + k v^T with
    S [D, D] from / to ``state`` [slots, H, D, D].  Returns o [T, H*D] fp32."""
    if _native(r):
        y = torch.empty(r.shape[0], H * D, dtype=torch.float32, device=r.device)
        _call("linear_scan", y, 0, r, k, v, w_raw, None, w0, u, state, None, None, positions, seq_row0, seq_slots,
              H, H, D, D, 0.0)
        return y
    return wkv_scan_ref(r, k, v, w_raw, w0, u, state, positions, seq_row0, seq_slots, H, D)


def delta_scan_ref(q, k, v, b_raw, a_raw, a_log, dt_bias, state, positions, seq_row0, seq_slots, H, G, D, V):
    T = q.shape[0]
    qq, kk, vv = _heads(q, G, D), _heads(k, G, D), _heads(v, H, V)
    qq = qq / torch.sqrt(qq.pow(2).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    kk = kk / torch.sqrt(kk.pow(2).sum(-1, keepdim=True) + 1e-6)
    qq, kk = qq.repeat_interleave(H // G, 1), kk.repeat_interleave(H // G, 1)
    beta = torch.sigmoid(b_raw.float())
    dec = torch.exp(-torch.exp(a_log) * torch.nn.functional.softplus(a_raw.float() + dt_bias, threshold=1e9))
    y = torch.zeros(T, H, V)
    for r0, r1, slot, p0 in _seqs(positions, seq_row0, seq_slots):
        if r1 == r0:
            continue
        S = torch.zeros(H, D, V) if p0 == 0 else state[slot].clone()
        for t in range(r0, r1):
            S = dec[t, :, None, None] * S
            uu = beta[t, :, None] * (vv[t] - torch.einsum("hkv,hk->hv", S, kk[t]))
            S = S + kk[t, :, :, None] * uu[:, None, :]
            y[t] = torch.einsum("hkv,hk->hv", S, qq[t])
        state[slot] = S
    return y.reshape(T, H * V)


def delta_scan(q, k, v, b_raw, a_raw, a_log, dt_bias, state, positions, seq_row0, seq_slots, H: int, G: int, D: int,
               V: int) -> torch.Tensor:
    """Gated delta rule over packed rows.  ``q`` / ``k`` [T, G*D] and ``v`` [T, H*V] (after convolution and
    SiLU; value head h uses q/k head floor(h / (H/G))), ``b_raw`` / ``a_raw`` [T, H] fp32 the projected write
    strength and step size.  Per head: q, k -> unit vectors (x / sqrt(sum x^2 + 1e-6)), q *= D^-1/2,
    beta = sigmoid(b_raw), g = exp(-exp(a_log) softplus(a_raw + dt_bias)); S <- g S; S += k (beta (v - S^T k))^T;
    o = S^T q with S [D, V] from / to ``state`` [slots, H, D, V].  Returns o [T, H*V] fp32."""
    if _native(q):
        y = torch.empty(q.shape[0], H * V, dtype=torch.float32, device=q.device)
        _call("linear_scan", y, 1, q, k, v, b_raw, a_raw, a_log, dt_bias, state, None, None, positions, seq_row0,
              seq_slots, H, G, D, V, 0.0)
        return y
    return delta_scan_ref(q, k, v, b_raw, a_raw, a_log, dt_bias, state, positions, seq_row0, seq_slots, H, G, D, V)


def mlstm_scan_ref(q, k, v, i_raw, f_raw, cap, state, norm, mx, positions, seq_row0, seq_slots, H, D, V):
    T = q.shape[0]
    qq, kk, vv = _heads(q, H, D) * D ** -0.5, _heads(k, H, D), _heads(v, H, V)
    ig = cap * torch.tanh(i_raw.float() / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh(f_raw.float() / cap))
    y = torch.zeros(T, H, V)
    for r0, r1, slot, p0 in _seqs(positions, seq_row0, seq_slots):
        if r1 == r0:
            continue
        if p0 == 0:
            S, n, m = torch.zeros(H, D, V), torch.zeros(H, D), torch.zeros(H)
        else:
            S, n, m = state[slot].clone(), norm[slot].clone(), mx[slot].clone()
        for t in range(r0, r1):
            new = torch.maximum(fg[t] + m, ig[t])
            a, b = torch.exp(fg[t] + m - new), torch.exp(ig[t] - new)
            S = a[:, None, None] * S + b[:, None, None] * kk[t, :, :, None] * vv[t, :, None, :]
            n = a[:, None] * n + b[:, None] * kk[t]
            m = new
            den = torch.maximum((n * qq[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
            y[t] = torch.einsum("hkv,hk->hv", S, qq[t]) / den[:, None]
        state[slot], norm[slot], mx[slot] = S, n, m
    return y.reshape(T, H * V)


def mlstm_scan(q, k, v, i_raw, f_raw, cap: float, state, norm, mx, positions, seq_row0, seq_slots, H: int, D: int,
               V: int) -> torch.Tensor:
    """Matrix-memory recurrence over packed rows.  ``q`` / ``k`` [T, H*D], ``v`` [T, H*V], ``i_raw`` /
    ``f_raw`` [T, H] fp32 the projected gates (bias included).  Per head: i = cap tanh(i_raw / cap),
    f = logsigmoid(cap tanh(f_raw / cap)), m' = max(f + m, i), S <- e^(f + m - m') S + e^(i - m') k v^T,
    n likewise with k alone, o = S^T q' / (max(|n . q'|, e^(-m')) + 1e-6), q' = q D^-1/2; S, n, m from / to
    ``state`` [slots, H, D, V], ``norm`` [slots, H, D], ``mx`` [slots, H] (all zero at position 0).
    Returns o [T, H*V] fp32."""
    if _native(q):
        y = torch.empty(q.shape[0], H * V, dtype=torch.float32, device=q.device)
        _call("linear_scan", y, 2, q, k, v, i_raw, f_raw, None, None, state, norm, mx, positions, seq_row0, seq_slots,
              H, H, D, V, float(cap))
        return y
    return mlstm_scan_ref(q, k, v, i_raw, f_raw, cap, state, norm, mx, positions, seq_row0, seq_slots, H, D, V)


# ----------------------------------------------------------------------------
# Per-head RMS norm, weight, output gate
# ----------------------------------------------------------------------------

def head_norm_gate_ref(y, z, w, heads, eps, act, dtype):
    T, C = y.shape
    v = y.float().view(T, heads, C // heads)
    v = (v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, C)
    v = v * (w if w.numel() == C else w.repeat(C // w.numel()))
    zf = z.float()
    return (v * (zf * torch.sigmoid(zf) if act == "silu" else torch.sigmoid(zf))).to(dtype)


def head_norm_gate(y, z, w, heads: int, eps: float, act: str, dtype) -> torch.Tensor:
    """Rows of ``y`` [T, C] (fp32): each of the ``heads`` equal parts divided by its root mean square
    (eps inside the root), times ``w`` (C entries, or C / heads entries shared by the heads), times
    silu(z) or sigmoid(z) (``act``; ``z`` [T, C], rows may be strided).  Returns [T, C] in ``dtype``."""
    if _native(y):
        out = torch.empty(y.shape[0], y.shape[1], dtype=dtype, device=y.device)
        _call("head_norm_gate", out, y, z, w, int(heads), float(eps), 1 if act == "sigmoid" else 0)
        return out
    return head_norm_gate_ref(y, z, w, heads, eps, act, dtype)


# ----------------------------------------------------------------------------
# Mean of two branches, each RMS-normed over the width
# ----------------------------------------------------------------------------

def rms_pair_mean_ref(a, b, wa, wb, eps):
    af, bf = a.float(), b.float()
    af = af / torch.sqrt(af.pow(2).mean(-1, keepdim=True) + eps) * wa
    bf = bf / torch.sqrt(bf.pow(2).mean(-1, keepdim=True) + eps) * wb
    return 0.5 * (af + bf)


def rms_pair_mean(a, b, wa, wb, eps: float) -> torch.Tensor:
    """0.5 * (a / rms(a) * wa + b / rms(b) * wb) per row, fp32 [T, W]; rms(v) = sqrt(mean(v^2) + eps)."""
    if _native(a):
        out = torch.empty(a.shape, dtype=torch.float32, device=a.device)
        _call("rms_pair_mean", out, a, b, wa, wb, float(eps))
        return out
    return rms_pair_mean_ref(a, b, wa, wb, eps)
