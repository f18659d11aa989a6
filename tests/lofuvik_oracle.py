"""Plain float64 Lofuvik: whole sequences, token by token, one function per mechanism.

Nothing here is shared with ``dgi``: no cache, no state slots, no batching, no kernels.  A model
is (``cfg``, ``w``): the dictionary of the design's ``config.json`` and a name -> float64 tensor
map with the checkpoint's tensor names.  ``forward`` returns the logits of every position and,
on request, the residual stream after every layer run.

Notation: W width, T tokens, h the layer's normed input, rms(v) = sqrt(mean(v^2) + eps).
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(v, eps):
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def lin(w, x):
    return x @ w.T


# ------------------------------------------------------------------ rotary
def yarn_tables(rot: dict, n_pos: int):
    """cos / sin [n_pos, dims / 2] of the rotated pairs (i, i + dims / 2)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    i = torch.arange(half, dtype=F64)
    f = base ** (-2.0 * i / dims)
    mult = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def turn_dim(turns):
            return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

        lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
        hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
        f = f / factor * ramp + f * (1 - ramp)
        mult = 0.1 * math.log(factor) + 1.0
    a = torch.arange(n_pos, dtype=F64)[:, None] * f[None, :]
    return torch.cos(a) * mult, torch.sin(a) * mult


def rotate_half(x, cos, sin):
    """x [T, heads, d]; the first 2 * cos.shape[1] dims of every head rotate."""
    half = cos.shape[1]
    u, v = x[..., :half], x[..., half:2 * half]
    c, s = cos[:, None, :], sin[:, None, :]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], -1)


# ------------------------------------------------------------------ mixers
def wkv_core(r, k, v, dec, u):
    """r, k, v, dec [T, H, D], u [H, D] -> o [T, H, D]; the bonus u replaces the state for the current token."""
    T, H, D = r.shape
    S = torch.zeros(H, D, D, dtype=F64)          # [head, key channel, value channel]
    out = torch.zeros(T, H, D, dtype=F64)
    for t in range(T):
        kv = k[t, :, :, None] * v[t, :, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S + u[:, :, None] * kv, r[t])
        S = dec[t, :, :, None] * S + kv
    return out


def wkv_mixer(w, p, m, h, eps):
    T = h.shape[0]
    H, D = int(m["heads"]), int(m["dim"])
    prev = torch.cat([torch.zeros(1, h.shape[1], dtype=F64), h[:-1]], 0)

    def mixed(s):
        return h + (prev - h) * w[p + "mu." + s]

    r = lin(w[p + "r"], mixed("r")).view(T, H, D)
    k = lin(w[p + "k"], mixed("k")).view(T, H, D)
    v = lin(w[p + "v"], mixed("v")).view(T, H, D)
    gate = silu(lin(w[p + "g"], mixed("g")))
    dec = torch.exp(-torch.exp(lin(w[p + "w2"], torch.tanh(lin(w[p + "w1"], mixed("w")))) + w[p + "w0"])).view(T, H, D)
    out = wkv_core(r, k, v, dec, w[p + "u"].view(H, D))
    o = rms_unit(out, eps).reshape(T, H * D) * w[p + "norm"] * gate
    return lin(w[p + "o"], o)


def causal_conv_silu(x, taps_w):
    """x [T, C], taps_w [C, taps] with the last column on the current token."""
    T, C = x.shape
    taps = taps_w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F64), x], 0)
    acc = torch.zeros(T, C, dtype=F64)
    for j in range(taps):
        acc = acc + pad[j:j + T] * taps_w[:, j]
    return silu(acc)


def unit_vectors(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def delta_core(q, k, v, beta, dec):
    """q, k [T, H, D] (already unit vectors, q scaled), v [T, H, V], beta, dec [T, H] -> o [T, H, V]."""
    T, H, D = q.shape
    V = v.shape[2]
    S = torch.zeros(H, D, V, dtype=F64)
    out = torch.zeros(T, H, V, dtype=F64)
    for t in range(T):
        S = dec[t, :, None, None] * S
        u = beta[t, :, None] * (v[t] - torch.einsum("hkv,hk->hv", S, k[t]))
        S = S + k[t, :, :, None] * u[:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S, q[t])
    return out


def delta_mixer(w, p, m, h, eps):
    T = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = causal_conv_silu(lin(w[p + "q"], h), w[p + "q.conv"]).view(T, G, D)
    k = causal_conv_silu(lin(w[p + "k"], h), w[p + "k.conv"]).view(T, G, D)
    v = causal_conv_silu(lin(w[p + "v"], h), w[p + "v.conv"]).view(T, H, V)
    q = unit_vectors(q) * D ** -0.5
    k = unit_vectors(k)
    rep = H // G
    q, k = q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1)
    beta = torch.sigmoid(lin(w[p + "b"], h))
    dec = torch.exp(-torch.exp(w[p + "A_log"]) * softplus(lin(w[p + "a"], h) + w[p + "dt_bias"]))
    out = delta_core(q, k, v, beta, dec)
    o = (rms_unit(out, eps) * w[p + "norm"]).reshape(T, H * V) * silu(lin(w[p + "g"], h))
    return lin(w[p + "o"], o)


def sink_attention_core(q, k, v, scale, cap, sink):
    """q [T, H, D], k [T, G, D], v [T, G, V], sink [H] or None -> causal softmax attention [T, H, V]; the
    sink is a logit of its own in the denominator (no key, no value, not scaled, not capped)."""
    T, H, _ = q.shape
    rep = H // k.shape[1]
    k, v = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    if cap > 0:
        s = cap * torch.tanh(s / cap)
    s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), -math.inf)
    top = s.max(-1).values
    if sink is not None:
        top = torch.maximum(top, sink[:, None])
    e = torch.exp(s - top[..., None])
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink[:, None] - top)[..., None]
    return torch.einsum("hij,jhd->ihd", e / den, v)


def sink_attention(w, p, m, h, eps):
    T = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = rms_unit(lin(w[p + "q"], h), eps) * w[p + "q.norm"]
    k = rms_unit(lin(w[p + "k"], h), eps) * w[p + "k.norm"]
    v = lin(w[p + "v"], h).view(T, G, V)
    q, k = q.view(T, H, D), k.view(T, G, D)
    rot = m.get("rot")
    if rot and int(rot["dims"]) > 0:
        cos, sin = yarn_tables(rot, T)
        q, k = rotate_half(q, cos, sin), rotate_half(k, cos, sin)
    o = sink_attention_core(q, k, v, float(m["scale"]), float(m.get("softcap") or 0.0), w[p + "sink"]).reshape(T, H * V)
    return lin(w[p + "o"], o * torch.sigmoid(lin(w[p + "g"], h)))


def capped_gates(i_raw, f_raw, cap):
    """Log input gate and log forget gate from the projections (bias included)."""
    return cap * torch.tanh(i_raw / cap), torch.nn.functional.logsigmoid(cap * torch.tanh(f_raw / cap))


def mlstm_core(q, k, v, ig, fg):
    """q (already scaled), k [T, H, D], v [T, H, V], log gates ig, fg [T, H] -> o [T, H, V]."""
    T, H, D = q.shape
    V = v.shape[2]
    S = torch.zeros(H, D, V, dtype=F64)
    n = torch.zeros(H, D, dtype=F64)
    mx = torch.zeros(H, dtype=F64)               # the running maximum starts at 0
    out = torch.zeros(T, H, V, dtype=F64)
    for t in range(T):
        new = torch.maximum(fg[t] + mx, ig[t])
        a, b = torch.exp(fg[t] + mx - new), torch.exp(ig[t] - new)
        S = a[:, None, None] * S + b[:, None, None] * k[t, :, :, None] * v[t, :, None, :]
        n = a[:, None] * n + b[:, None] * k[t]
        mx = new
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        out[t] = torch.einsum("hkv,hk->hv", S, q[t]) / den[:, None]
    return out


def mlstm_mixer(w, p, m, h, eps):
    T = h.shape[0]
    H, D, V = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    cap = float(m["gate_cap"])
    q = lin(w[p + "q"], h).view(T, H, D) * D ** -0.5
    k = lin(w[p + "k"], h).view(T, H, D)
    v = lin(w[p + "v"], h).view(T, H, V)
    ig, fg = capped_gates(lin(w[p + "i"], h) + w[p + "i.b"], lin(w[p + "f"], h) + w[p + "f.b"], cap)
    out = mlstm_core(q, k, v, ig, fg)
    o = rms_unit(out, eps).reshape(T, H * V) * w[p + "norm"] * torch.sigmoid(lin(w[p + "g"], h))
    return lin(w[p + "o"], o)


def parallel_mixer(w, p, m, h, eps):
    a = rms_unit(sink_attention(w, p + "left.", m["left"], h, eps), eps) * w[p + "left.out"]
    b = rms_unit(mlstm_mixer(w, p + "right.", m["right"], h, eps), eps) * w[p + "right.out"]
    return 0.5 * (a + b)


MIXERS = {"wkv": wkv_mixer, "delta": delta_mixer, "parallel": parallel_mixer}


# ------------------------------------------------------------------ feed-forward
def route_top(z, top):
    """The `top` largest logits of every row and the softmax over those alone."""
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, -1)


def moe_ff(w, p, f, h):
    E, top = int(f["router"]["experts"]), int(f["router"]["top"])
    idx, wt = route_top(lin(w[p + "router"], h) + w[p + "router.b"], top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            assert e < E
            mid = silu(lin(w[f"{p}e{e}.gate"], h[t])) * lin(w[f"{p}e{e}.up"], h[t])
            out[t] += wt[t, j] * lin(w[f"{p}e{e}.down"], mid)
    return out


# ------------------------------------------------------------------ model
def layer_runs(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop") or {}
    a, b, times = int(lp.get("start") or 0), int(lp.get("stop") or 0), int(lp.get("times") or 1)
    if times <= 1 or b <= a:
        return [(i, False) for i in range(n)]
    runs = [(i, False) for i in range(a)]
    for r in range(times):
        runs += [(i, r > 0 and i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg, w, tokens, want_layers=False):
    eps = float(cfg["norm"]["eps"])
    x0 = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0.clone()
    streams = []
    for li, add_embed in layer_runs(cfg):
        if add_embed:
            x = x + x0
        e = cfg["layers"][li]
        p = f"l{li}."
        h = rms_unit(x, eps) * w[p + "norm1"]
        y = MIXERS[e["type"]](w, p + "mix.", e["mixer"], h, eps)
        if e.get("mlp") is not None:
            y = y + moe_ff(w, p + "mlp.", e["mlp"], h)
        x = x + y
        streams.append(x.clone())
    logits = lin(w["head"], rms_unit(x, eps) * w["final.norm"])
    return (logits, torch.stack(streams)) if want_layers else logits
