"""Plain whole-sequence Depelix in float64: the oracle of tests/test_depelix.py.

One function per mechanism, written from the design's equations (the notation is that of the
model's docstring in ``dgi/models/depelix.py``); no cache, no batching, no state carried between
calls and no code shared with the product path.  ``P`` is a dict name -> float64 tensor in the
checkpoint naming (``l<i>.mix.dq`` ...), ``cfg`` the parsed ``config.json`` dictionary.  Keys and
values are formed explicitly per head (nothing is folded into the queries) and every query takes
its visible keys by an explicit slice.
"""
import math

import torch

F = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def embed(P, cfg, tokens):
    """Token row + hashed bigram row (the extra last row for a sequence's first token)."""
    rows = []
    bg = (cfg.get("embedding") or {}).get("bigram")
    for p, t in enumerate(tokens):
        x = P["embed"][t].clone()
        if bg:
            nb = int(bg["buckets"])
            r = nb if p == 0 else (tokens[p - 1] * int(bg["mul_prev"]) + t * int(bg["mul_cur"])) % nb
            x = x + P["bigram"][r]
        rows.append(x)
    return torch.stack(rows)


def rotate(v, pos, dims, base, interleaved):
    """Rotary position on the first ``dims`` entries of the vector ``v`` at position ``pos``."""
    out = v.clone()
    half = dims // 2
    for i in range(half):
        a = pos * base ** (-2.0 * i / dims)
        i0, i1 = (2 * i, 2 * i + 1) if interleaved else (i, i + half)
        c, s = math.cos(a), math.sin(a)
        out[i0] = v[i0] * c - v[i1] * s
        out[i1] = v[i1] * c + v[i0] * s
    return out


def latent_kv(P, pre, m, h, eps, interleaved):
    """(latent c [T, kv_rank], rotated shared key part [T, rot_dim]) of the layer whose tensors start with ``pre``."""
    r = int(m["kv_rank"])
    d = h @ P[pre + "mix.dkv"].T
    c = rms_norm(d[:, :r], P[pre + "mix.dkv.norm"], eps)
    rot = m["rot"]
    kr = torch.stack([rotate(d[t, r:], t, int(rot["dims"]), float(rot["base"]), interleaved) for t in range(d.shape[0])])
    return c, kr


def latent_attention(P, pre, m, h, eps, kind, shared=None):
    """One latent-attention mixer on the whole sequence ``h`` [T, W].  ``kind`` is the layer type;
    ``shared`` = (c, kr) of the layer named by ``kv_from``.  Returns (output, (c, kr))."""
    second = kind == "latent_attention_2"
    T = h.shape[0]
    H, dn, dr, dv = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
    rot = m["rot"]
    cq = rms_norm(h @ P[pre + "mix.dq"].T, P[pre + "mix.dq.norm"], eps)
    q = (cq @ P[pre + "mix.uq"].T).view(T, H, dn + dr)
    c, kr = shared if shared is not None else latent_kv(P, pre, m, h, eps, second)
    kn = (c @ P[pre + "mix.uk"].T).view(T, H, dn)
    v = (c @ P[pre + "mix.uv"].T).view(T, H, dv)
    window = int((m.get("mask") or {}).get("size") or 0)
    g = torch.sigmoid(h @ P[pre + "mix.g"].T)
    out = torch.zeros(T, H * dv, dtype=F)
    for i in range(T):
        lo = 0
        if window > 0:
            lo = max(0, i - window + 1)
        for hh in range(H):
            qn = q[i, hh, :dn]
            qr = rotate(q[i, hh, dn:], i, int(rot["dims"]), float(rot["base"]), second)
            s = (kn[lo:i + 1, hh] @ qn + kr[lo:i + 1] @ qr) * float(m["scale"])     # keys lo .. i, nothing else
            p = torch.softmax(s, 0)
            o = (p[:, None] * v[lo:i + 1, hh]).sum(0)
            if second:
                o = o * g[i, hh * dv:(hh + 1) * dv]
            else:
                o = o * g[i, hh]
            out[i, hh * dv:(hh + 1) * dv] = o
    return out @ P[pre + "mix.o"].T, (c, kr)


def dense_ff(P, pre, h):
    return gelu_tanh(h @ P[pre + "mlp.up"].T) @ P[pre + "mlp.down"].T


def route(z, top):
    """Chosen experts and their weights from router logits ``z`` [E]: sigmoid scores, the ``top``
    largest, weights = those scores as they are."""
    s = torch.sigmoid(z)
    order = sorted(range(z.shape[0]), key=lambda e: (-float(s[e]), e))[:top]
    return order, [s[e] for e in order]


def expert(P, pre, e, x, limit):
    g = torch.clamp(x @ P[f"{pre}mlp.e{e}.gate"].T, max=limit)
    u = torch.clamp(x @ P[f"{pre}mlp.e{e}.up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ P[f"{pre}mlp.e{e}.down"].T


def moe_ff(P, pre, f, h):
    top, limit = int(f["router"]["top"]), float(f["expert"]["limit"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        es, ws = route(h[t] @ P[pre + "mlp.router"].T, top)
        for e, w in zip(es, ws):
            out[t] += expert(P, pre, e, w * h[t], limit)          # the weight scales the expert's INPUT
    return out


def token_side(P, cfg, pre, li, x, tokens, eps):
    """Per-layer token input added to the stream after the feed-forward."""
    d = int(cfg["token_side"]["dim"])
    e = P["side.embed"][torch.tensor(tokens)][:, li * d:(li + 1) * d]
    y = (gelu_tanh(x @ P[pre + "side.gate"].T) * e) @ P[pre + "side.proj"].T
    return x + unit_rms(y, eps) * P[pre + "side.norm"]


def forward(P, cfg, tokens, return_layers=False):
    """Logits [T, vocab] of a whole sequence (and the stream after every layer)."""
    eps = float(cfg["norm"]["eps"])
    x = embed(P, cfg, tokens)
    kept, streams = {}, []
    for li, L in enumerate(cfg["layers"]):
        pre = f"l{li}."
        m = L["mixer"]
        h = rms_norm(x, P[pre + "norm1"], eps)
        src = m.get("kv_from")
        y, kept[li] = latent_attention(P, pre, m, h, eps, L["type"], None if src is None else kept[int(src)])
        x = x + y
        f = L.get("mlp")
        if f is not None:
            h = rms_norm(x, P[pre + "norm2"], eps)
            x = x + (dense_ff(P, pre, h) if f.get("kind", "dense") == "dense" else moe_ff(P, pre, f, h))
        if cfg.get("token_side"):
            x = token_side(P, cfg, pre, li, x, tokens, eps)
        streams.append(x.clone())
    logits = rms_norm(x, P["final.norm"], eps) @ P["head"].T
    return (logits, streams) if return_layers else logits
