"""Depelix in the framework against the plain float64 oracle (tests/depelix_oracle.py): every
mechanism alone, then the model through the engine's scheduler, block pool, state slots and step —
whole prompts, token-by-token decoding, portions down to two tokens, unequal batches, reused pages
and slots, keys just inside / outside every window, at page borders and far away, first tokens,
long decoding past the windows, other geometries, greedy generation, the checkpoint layout and the
trace runner.  The same tests run the CPU reference ops here and the HIP kernels on a GPU box."""
import copy
import json
import math
import os
import subprocess
import sys

import pytest
import torch

import depelix_oracle as orc
from dgi.engine import EngineConfig, LLMEngine
from dgi.models.config import (DenseSpec, DepelixConfig, LatentAttentionSpec, LayerSpec, MoeSpec, RotarySpec, get_config)
from dgi.ops import latent, moe
from dgi.sched.request import SamplingParams

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F64 = torch.float64
I32 = torch.int32


def la(kind, heads, dim, rot_dim, vdim, kv_rank, q_rank, window=0, kv_from=None, dims=None, base=100.0, scale=None):
    first = kind == 1
    return LatentAttentionSpec(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale or (dim + rot_dim) ** -0.5,
                               RotarySpec(base, rot_dim if dims is None else dims, None, "half" if first else "interleaved"),
                               "window" if window else "causal", window, "head" if first else "elem", kv_from)


def experts(n, top, ff, limit):
    return MoeSpec(n, 0, top, ff, score="sigmoid", act="clamped", limit=limit, weigh="input", selection_bias=False)


T1, T2 = "latent_attention", "latent_attention_2"


def small_cfg(**kw) -> DepelixConfig:
    """Six layers that differ in everything: unrotated / rotated / value sizes all different, windows of
    5 and 9, a windowed layer reading another's latent (with its own head count and window), a causal
    layer whose key part rotates only in part, experts with top 2 of 5 and top = all, dense widths, a
    layer without feed-forward; latent + key part of 16 (vector kernel) and of 14 / 11 (element-wise)."""
    args = dict(name="t", vocab_size=53, hidden_size=32, layers=[
        LayerSpec(T1, la(1, 3, 8, 4, 6, 12, 10, window=5), DenseSpec(40)),
        LayerSpec(T1, la(1, 2, 6, 4, 10, 12, 7, window=9, kv_from=0), experts(5, 2, 12, 0.8)),
        LayerSpec(T2, la(2, 4, 4, 6, 5, 8, 9, dims=4), None),
        LayerSpec(T1, la(1, 1, 5, 2, 3, 9, 6, window=3), experts(3, 3, 8, 1.5)),
        LayerSpec(T2, la(2, 2, 8, 4, 8, 12, 16), DenseSpec(24)),
        LayerSpec(T1, la(1, 5, 3, 2, 4, 9, 5, window=17, kv_from=3), experts(4, 1, 6, 0.5)),
    ], side_dim=6, bigram_buckets=29, bigram_mul_prev=5, bigram_mul_cur=3, norm_eps=1e-5, max_position=512)
    args.update(kw)
    return DepelixConfig(**args)


def engine(cfg, device, dtype=torch.float32, num_blocks=96, bs=4, seed=3, max_len=256, seqs=4, graphs=False):
    return LLMEngine(EngineConfig(model="depelix-test", device=device, dtype=dtype, block_size=bs, num_blocks=num_blocks,
                                  max_num_seqs=seqs, max_model_len=max_len, max_num_batched_tokens=max_len,
                                  enable_prefix_caching=True, use_graphs=graphs, token_align=0, decode_lookahead=graphs,
                                  seed=seed, graph_buckets=(1, 2, 4) if graphs else None), model_cfg=copy.deepcopy(cfg))


def toks(n, seed=0, vocab=53):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def config_dict(cfg: DepelixConfig) -> dict:
    """The design's config.json for ``cfg``."""
    layers = []
    for l in cfg.layers:
        m = l.mixer
        mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                 "q_rank": m.q_rank, "scale": m.scale, "rot": {"base": m.rot.base, "dims": m.rot.dims}}
        if m.window:
            mixer["mask"] = {"size": m.window}
        if m.kv_from is not None:
            mixer["kv_from"] = m.kv_from
        f = l.mlp
        if f is None:
            mlp = None
        elif f.kind == "dense":
            mlp = {"kind": "dense", "ff": f.ff}
        else:
            mlp = {"kind": "moe", "expert": {"ff": f.ff, "limit": f.limit}, "router": {"experts": f.experts, "top": f.top}}
        layers.append({"type": l.type, "mixer": mixer, "mlp": mlp})
    d = {"architecture": "Depelix", "vocab": cfg.vocab_size, "width": cfg.hidden_size, "norm": {"eps": cfg.norm_eps},
         "layers": layers}
    if cfg.bigram_buckets:
        d["embedding"] = {"bigram": {"buckets": cfg.bigram_buckets, "mul_prev": cfg.bigram_mul_prev,
                                     "mul_cur": cfg.bigram_mul_cur}}
    if cfg.side_dim:
        d["token_side"] = {"dim": cfg.side_dim}
    return d


def params(model) -> dict:
    """The model's weights under the checkpoint's tensor names (CPU, model dtype)."""
    P = {"embed": model.embed, "bigram": model.bigram, "side.embed": model.side_embed, "head": model.head,
         "final.norm": model.final_norm}
    for i, L in enumerate(model.layers):
        p = f"l{i}."
        m, f = L.spec.mixer, L.spec.mlp
        P[p + "norm1"], P[p + "norm2"] = L.norm1, L.norm2
        r = m.q_rank
        P[p + "mix.dq"] = L.in_proj[:r]
        if m.kv_from is None:
            P[p + "mix.dkv"] = L.in_proj[r:r + m.cache_dim]
            r += m.cache_dim
        P[p + "mix.g"] = L.in_proj[r:]
        P[p + "mix.dq.norm"], P[p + "mix.dkv.norm"] = L.dq_norm, L.dkv_norm
        P[p + "mix.uq"], P[p + "mix.o"] = L.uq, L.o
        P[p + "mix.uk"] = L.uk.reshape(m.heads * m.dim, m.kv_rank)
        P[p + "mix.uv"] = L.uv.reshape(m.heads * m.vdim, m.kv_rank)
        if f is not None and f.kind == "dense":
            P[p + "mlp.up"], P[p + "mlp.down"] = L.up, L.down
        elif f is not None:
            P[p + "mlp.router"] = L.router
            for e in range(f.experts):
                P[f"{p}mlp.e{e}.gate"], P[f"{p}mlp.e{e}.up"] = L.gate_up[e, :f.ff], L.gate_up[e, f.ff:]
                P[f"{p}mlp.e{e}.down"] = L.down[e]
        P[p + "side.gate"], P[p + "side.proj"], P[p + "side.norm"] = L.side_gate, L.side_proj, L.side_norm
    return {k: v.detach().cpu().contiguous() for k, v in P.items() if v is not None}


def oracle_logits(eng, tokens, layers=False):
    P = {k: v.to(F64) for k, v in params(eng.model).items()}
    return orc.forward(P, config_dict(eng.model_cfg), tokens, layers)


def feed_all(eng, rid, tokens, cuts):
    """Feed `tokens` in portions of the given sizes (the rest one by one); logits of every position."""
    out, at = [], 0
    for n in list(cuts) + [1] * len(tokens):
        if at >= len(tokens):
            break
        part = tokens[at:at + n]
        out.append(eng.feed([(rid, part, list(range(len(part))))])[0])
        at += len(part)
    return torch.cat(out, 0)


def close(a, b, tol):
    assert a.shape == b.shape
    err = (a.double().cpu() - b.double().cpu()).abs().max().item()
    assert err <= tol, f"max abs difference {err} > {tol}"


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64) * scale


# ----------------------------------------------------------------------------------- mechanisms
def test_config_reads_every_size_and_rejects_bad_sharing():
    d = config_dict(small_cfg())
    c = DepelixConfig.from_dict(d)
    assert [l.mixer.kv_from for l in c.layers] == [None, 0, None, None, None, 3]
    assert c.kv_owners == [0, 2, 3, 4] and c.kv_layer_shapes() == [(1, 16, 0), (1, 14, 0), (1, 11, 0), (1, 16, 0)]
    assert [l.mixer.window for l in c.layers] == [5, 9, 0, 3, 0, 17]
    assert c.layers[1].mixer.gate == "head" and c.layers[2].mixer.gate == "elem" and c.layers[2].mixer.rot.dims == 4
    assert c.layers[0].mixer.rot.layout == "half" and c.layers[2].mixer.rot.layout == "interleaved"
    assert c.layers[1].mlp.top == 2 and c.layers[1].mlp.limit == 0.8 and c.layers[2].mlp is None
    bad = copy.deepcopy(d)
    bad["layers"][1]["mixer"]["kv_from"] = 1
    with pytest.raises(ValueError):
        DepelixConfig.from_dict(bad)
    bad = copy.deepcopy(d)
    bad["layers"][5]["mixer"]["kv_from"] = 1          # layer 1 holds no latent of its own
    with pytest.raises(ValueError):
        DepelixConfig.from_dict(bad)
    bad = copy.deepcopy(d)
    bad["layers"][0]["type"] = "attention"
    with pytest.raises(ValueError):
        DepelixConfig.from_dict(bad)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W", [37, 64, 1024, 2052])
def test_stream_add_norm(device, dtype, W):
    """Residual add, add of a unit-RMS normed and weighted input, the next norm, and the plain copy."""
    T, eps = 5, 1e-3
    x0, y = rnd(T, W, seed=1), rnd(T, W, seed=2, scale=3.0).to(dtype)
    pw, nw = rnd(W, seed=3) + 1, rnd(W, seed=4) + 1
    dev = lambda t, d=torch.float32: t.to(d).to(device)   # noqa: E731
    tol = 1e-5 if dtype == torch.float32 else 0.008       # bf16: relative to the largest value
    for post, nxt, has_y, out in ((None, nw, True, True), (pw, nw, True, True), (pw, None, True, False),
                                  (None, None, True, True), (None, nw, False, True)):
        x = dev(x0)
        got = latent.stream_add_norm(x, dev(y, dtype) if has_y else None, None if post is None else dev(post),
                                     None if nxt is None else dev(nxt), eps, dtype if out else None)
        want_x = x0.clone()
        if has_y:
            yy = y.to(F64)
            want_x = want_x + (yy if post is None else orc.unit_rms(yy, eps) * post)
        close(x, want_x, 1e-5)
        if out:
            want = want_x if nxt is None else orc.rms_norm(want_x, nxt, eps)
            close(got.float(), want, tol * max(1.0, want.abs().max().item()))
        else:
            assert got is None


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kr,rd,dims,inter,qr,extra", [(12, 4, 4, False, 10, 3), (8, 6, 4, True, 10, 3), (9, 2, 2, False, 10, 3),
                                                       (64, 32, 32, True, 10, 3), (64, 32, 32, False, 24, 8), (24, 8, 8, True, 2056, 0)])
def test_latent_prep_norms_rotates_and_writes_pages(device, dtype, kr, rd, dims, inter, qr, extra):
    """Query latent norm; latent norm + rotary of the key part into scattered page slots; rows with slot -1
    are not written; a layer without a latent of its own computes the query side only."""
    from dgi import ops
    T, eps, bs = 7, 1e-4, 4
    proj = rnd(T, qr + kr + rd + extra, seed=5).to(dtype)
    dqw, dkw = rnd(qr, seed=6) + 1, rnd(kr, seed=7) + 1
    pos = torch.tensor([0, 1, 2, 30, 31, 32, 200], dtype=I32)
    slots = torch.tensor([9, 10, 11, 4, -1, 21, 0], dtype=I32)
    cs = ops.rope_cos_sin(dims, 256, 50.0)
    cache = torch.zeros(8, 1, bs, kr + rd, dtype=dtype)
    cache_d = cache.to(device)
    cq = latent.latent_prep(proj.to(device), qr, kr, rd, dqw.float().to(device), dkw.float().to(device), eps,
                            pos.to(device), slots.to(device), cs.to(device), inter, cache_d)
    tol = 1e-5 if dtype == torch.float32 else 0.03
    p64 = proj.to(F64)
    close(cq.float(), orc.rms_norm(p64[:, :qr], dqw, eps), tol)
    flat = cache_d.cpu().float().view(-1, kr + rd)
    for t in range(T):
        if slots[t] < 0:
            continue
        want = torch.cat([orc.rms_norm(p64[t, qr:qr + kr], dkw, eps), orc.rotate(p64[t, qr + kr:qr + kr + rd], int(pos[t]), dims, 50.0, inter)])
        close(flat[int(slots[t])], want, tol)
    written = {int(s) for s in slots if s >= 0}
    assert all(flat[s].abs().sum() == 0 for s in range(flat.shape[0]) if s not in written)
    cq2 = latent.latent_prep(proj[:, :qr + extra].contiguous().to(device), qr, kr, rd, dqw.float().to(device), None, eps,
                             pos.to(device), slots.to(device), cs.to(device), inter, None)
    close(cq2.float(), cq.float(), 0)


def attend_plain(qn, qr, c, r, uk, window, scale, p):
    """Head outputs in latent space for ONE query at position p, keys formed explicitly per head:
    qn [H, dim], qr [H, rd] (already rotated), c [N, kr], r [N, rd], uk [H, dim, kr] -> [H, kr]."""
    lo = max(0, p - window + 1) if window else 0
    out = []
    for h in range(qn.shape[0]):
        k = c[lo:p + 1] @ uk[h].T                                # [n, dim] unrotated keys of this head
        s = (k @ qn[h] + r[lo:p + 1] @ qr[h]) * scale
        out.append(torch.softmax(s, 0) @ c[lo:p + 1])
    return torch.stack(out)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,dim,rd,kr,window,inter", [(3, 8, 4, 12, 5, False), (2, 4, 6, 8, 0, True), (5, 6, 2, 9, 17, False),
                                                      (6, 16, 8, 24, 64, True), (17, 8, 8, 64, 33, False),
                                                      (4, 16, 16, 32, 70, False), (19, 8, 32, 64, 0, True), (16, 24, 16, 144, 129, True)])
def test_latent_attention_rows_edges_and_far_keys(device, dtype, H, dim, rd, kr, window, inter):
    """Decode rows and prompt rows over scattered pages.  One key is made to dominate a head's scores (its
    latent is a large multiple of the folded query) and placed just inside the window, just outside it, at
    page borders, at positions 0 / 1 and hundreds back: seeing it or not changes the output completely."""
    from dgi import ops
    N, bs, scale = 300, 4, 0.3
    g = torch.Generator().manual_seed(11)
    c = rnd(N, kr, seed=12, scale=0.5)
    r = rnd(N, rd, seed=13, scale=0.5)
    uk = rnd(H, dim, kr, seed=14, scale=kr ** -0.5)
    cs = ops.rope_cos_sin(rd, 512, 100.0)
    nblk = (N + bs - 1) // bs
    perm = (torch.randperm(nblk, generator=g) + 1).to(I32)          # scattered pages, page 0 unused
    queries = [299, 298, 297, 255, 256, 1, 0, 64, 65, 130]
    w = window or 10 ** 6
    placed = {}
    for qi, p in enumerate(queries):
        # the dominating key for query qi: alternately just inside / just outside its window, or far back / at page borders
        cand = [p - w + 1, p - w, p - (p % bs), p - (p % bs) - 1, 0, 1, p - 250, p]
        j = cand[qi % len(cand)]
        if 0 <= j <= p and j not in placed.values() and all(abs(j - q) > 0 for q in queries):
            placed[p] = j
    q = rnd(len(queries), H * (dim + rd), seed=15).to(dtype)
    qf = q.to(F64).view(len(queries), H, dim + rd)
    q_lat = torch.einsum("thd,hdk->htk", qf[:, :, :dim], uk)                 # the fold, in float64
    for p, j in placed.items():
        qi = queries.index(p)
        v = q_lat[qi % H, qi]
        c[j] = v / v.norm() * 40.0                                           # head (qi % H) of query qi locks onto key j
    cache = torch.zeros(nblk + 1, 1, bs, kr + rd, dtype=dtype)
    row = torch.cat([c, r], 1).to(dtype)
    for j in range(N):
        cache[int(perm[j // bs]), 0, j % bs] = row[j]
    cq, rq = row[:, :kr].to(F64), row[:, kr:].to(F64)                        # what the cache holds
    want = torch.stack([attend_plain(qf[i, :, :dim], torch.stack([orc.rotate(qf[i, h, dim:], p, rd, 100.0, inter) for h in range(H)]),
                                     cq, rq, uk, window, scale, p) for i, p in enumerate(queries)], 1)       # [H, T, kr]
    ql = q_lat.to(dtype).to(device)
    pos = torch.tensor(queries, dtype=I32, device=device)
    tol = 2e-5 if dtype == torch.float32 else 0.12
    # decode rows: one block-table row per query
    tables = perm[None, :].repeat(len(queries), 1).contiguous().to(device)
    out = torch.full((H, len(queries), kr), 7.0, dtype=dtype, device=device)
    latent.latent_attn_rows(q.to(device), ql, cache.to(device), tables, None, pos, H, dim, rd, kr, scale, window,
                            cs.to(device), inter, out)
    if dtype == torch.float32:
        close(out, want, tol)
    else:       # bf16 queries: the folded query was rounded; judge against the same rounded inputs
        want = torch.stack([attend_plain_folded(ql[:, i].cpu().to(F64), torch.stack([orc.rotate(qf[i, h, dim:], p, rd, 100.0, inter) for h in range(H)]),
                                                cq, rq, window, scale, p) for i, p in enumerate(queries)], 1)
        close(out.float(), want, tol)
    # few rows over many keys: every row's keys cut into runs (several workgroups per row and head), then combined
    assert latent.split_runs(len(queries), H, N) > 1
    out3 = torch.zeros(H, len(queries), kr, dtype=dtype, device=device)
    latent.latent_attn_rows(q.to(device), ql, cache.to(device), tables, None, pos, H, dim, rd, kr, scale, window,
                            cs.to(device), inter, out3, max_keys=N)
    close(out3.float(), out.float(), 1e-5 if dtype == torch.float32 else 1e-2)
    # a folded query that sits at an odd offset inside a wider buffer (no 16-byte accesses possible)
    wide = torch.zeros(H, len(queries), kr + 6, dtype=dtype, device=device)
    wide[:, :, 3:kr + 3] = ql
    out4 = torch.zeros(H, len(queries), kr, dtype=dtype, device=device)
    latent.latent_attn_rows(q.to(device), wide[:, :, 3:kr + 3], cache.to(device), tables, None, pos, H, dim, rd, kr, scale,
                            window, cs.to(device), inter, out4)
    close(out4.float(), out.float(), 1e-5 if dtype == torch.float32 else 1e-2)
    # the same rows as portions of two sequences that share the pages (rows map to tables through cu_seqlens)
    order = sorted(range(len(queries)), key=lambda i: queries[i])
    idx = torch.tensor(order)
    cu = torch.tensor([0, 4, len(queries)], dtype=I32, device=device)
    out2 = torch.zeros(H, len(queries), kr, dtype=dtype, device=device)
    latent.latent_attn_rows(q[idx].to(device), ql[:, idx.to(device)].contiguous(), cache.to(device), tables[:2].contiguous(), cu,
                            pos[idx.to(device)].contiguous(), H, dim, rd, kr, scale, window, cs.to(device), inter, out2)
    close(out2.float(), out.float()[:, idx.to(device)], 1e-6 if dtype == torch.float32 else 1e-2)
    # seeing the dominating key or not decides the output: inside -> the output is (nearly) that key's latent
    for p, j in placed.items():
        qi = queries.index(p)
        lo = max(0, p - window + 1) if window else 0
        o = out.float()[qi % H, qi].cpu().to(F64)
        hit = (o - cq[j]).norm() < 0.05 * cq[j].norm()
        assert hit == (lo <= j <= p), (p, j, lo)


def attend_plain_folded(ql, qr, c, r, window, scale, p):
    lo = max(0, p - window + 1) if window else 0
    return torch.stack([torch.softmax((c[lo:p + 1] @ ql[h] + r[lo:p + 1] @ qr[h]) * scale, 0) @ c[lo:p + 1]
                        for h in range(ql.shape[0])])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gate_heads_and_gelu(device, dtype):
    tol = 1e-6 if dtype == torch.float32 else 0.03
    for H, T, dv in ((3, 5, 7), (5, 4, 16)):                    # element-wise and 16-byte paths
        ov = rnd(H, T + 2, dv, seed=20).to(dtype)[:, 1:T + 1]   # a strided [H, T, dv] view
        o = ov.to(F64).permute(1, 0, 2)
        for per_head in (True, False):
            n = H if per_head else H * dv
            gate = rnd(T, n + 8, seed=21).to(dtype)[:, 8 * (dv == 16):][:, :n]      # gate columns inside a wider row
            got = latent.gate_heads(ov.to(device), gate.to(device), per_head)
            sg = torch.sigmoid(gate.to(F64))
            close(got.float(), (o * (sg[:, :, None] if per_head else sg.view(T, H, dv))).reshape(T, H * dv), tol)
        close(latent.gate_heads(ov.to(device), None, True).float(), o.reshape(T, H * dv), tol)
    T = 5
    for n in (6, 64):
        x = rnd(T, n, seed=22, scale=2.0).to(dtype)
        close(latent.gelu_tanh(x.to(device)).float(), orc.gelu_tanh(x.to(F64)), tol)
        table = rnd(11, 3 * n, seed=23).to(dtype)
        ids = torch.tensor([3, 0, 10, 3, 7], dtype=I32)
        got = latent.gelu_tanh(x.to(device), table.to(device), ids.to(device), n)
        close(got.float(), orc.gelu_tanh(x.to(F64)) * table.to(F64)[ids.long(), n:2 * n], 2 * tol)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,top", [(5, 6, 2), (70, 6, 3), (9, 4, 1), (40, 3, 3), (3, 70, 8), (2, 16, 1), (300, 5, 2)])
def test_sigmoid_routing_and_clamped_experts(device, dtype, T, E, top):
    """Sigmoid scores, the `top` largest as they are, each weight on its expert's input; clamps that bite;
    top = 1 and top = all experts; every evaluation path of the GPU op (few pairs, batched, sorted segments)."""
    W, ff, limit = 24, 12, 0.6
    h = rnd(T, W, seed=30).to(dtype)
    router = rnd(E, W, seed=31, scale=0.5)
    gu = rnd(E, 2 * ff, W, seed=32, scale=0.4).to(dtype)
    dn = rnd(E, W, ff, seed=33, scale=0.3).to(dtype)
    logits = (h.to(F64) @ router.T).float()
    idx, wts = moe.moe_route(logits.to(device), None, top, score="sigmoid")
    P = {"mlp.router": router}
    for e in range(E):
        P[f"mlp.e{e}.gate"], P[f"mlp.e{e}.up"], P[f"mlp.e{e}.down"] = gu[e, :ff].to(F64), gu[e, ff:].to(F64), dn[e].to(F64)
    for t in range(T):
        es, ws = orc.route(logits[t].to(F64), top)
        assert idx[t].tolist() == es
        close(wts[t].cpu(), torch.stack(ws).float(), 1e-6)
    got = moe.moe_experts(h.to(device), idx, wts, gu.to(device), dn.to(device), None, act="clamped", limit=limit,
                          alpha=1.702, weigh="input")
    want = orc.moe_ff(P, "", {"router": {"top": top}, "expert": {"limit": limit}}, h.to(F64))
    clamped = sum(int(((h[t].to(F64) * w) @ P[f"mlp.e{e}.gate"].T > limit).sum()) for t in range(min(T, 5))
                  for e, w in zip(*orc.route(logits[t].to(F64), top)))
    assert clamped > 0                                               # the limit is reached somewhere
    close(got.float(), want, 2e-5 if dtype == torch.float32 else 0.06)


def test_route_ties_go_to_the_lowest_index():
    z = torch.tensor([[0.5, 2.0, 2.0, -1.0, 2.0]])
    idx, w = moe.moe_route(z, None, 2, score="sigmoid")
    assert idx.tolist() == [[1, 2]] and abs(float(w[0, 0]) - 1 / (1 + math.exp(-2.0))) < 1e-6


# ----------------------------------------------------------------------------------- the model in the engine
@pytest.mark.parametrize("device", DEVICES)
def test_layer_streams_match_oracle(device):
    eng = engine(small_cfg(), device)
    t = toks(23, 1)
    eng.model.capture_layers = tuple(range(6))
    got = eng.feed([("a", t, list(range(len(t))))], ["a"])[0]
    want, streams = oracle_logits(eng, t, True)
    for i, s in enumerate(streams):
        close(eng.model.captured[i], s, 2e-4)
    close(got, want, 3e-4)


VARIANTS = {
    "base": {},
    "no_side_no_bigram": {"side_dim": 0, "bigram_buckets": 0},
    "one_layer": {"layers": [LayerSpec(T1, la(1, 1, 1, 2, 1, 1, 1, window=1), None)]},          # sizes of one, a window of one
    "all_causal": {"layers": [LayerSpec(T2, la(2, 2, 8, 4, 8, 12, 16), experts(2, 2, 8, 5.0)),
                              LayerSpec(T2, la(2, 3, 2, 4, 4, 12, 4, kv_from=0), DenseSpec(8))]},
    "vector_sizes": {"layers": [LayerSpec(T1, la(1, 4, 16, 8, 16, 24, 32, window=11), DenseSpec(64)),
                                LayerSpec(T1, la(1, 8, 8, 8, 8, 24, 16, window=6, kv_from=0), experts(8, 1, 16, 1.0)),
                                LayerSpec(T2, la(2, 2, 16, 16, 24, 48, 32), DenseSpec(32))], "hidden_size": 64},
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("variant", list(VARIANTS))
def test_whole_decode_and_portions_match_oracle(device, variant):
    """Whole prompt, token by token, and portions of several sizes (down to two tokens, across pages and
    windows): all equal the oracle; other layer orders and sizes too."""
    eng = engine(small_cfg(**VARIANTS[variant]), device)
    t = toks(45, 2)
    want = oracle_logits(eng, t)
    close(eng.feed([("w", t, list(range(len(t))))], ["w"])[0], want, 3e-4)
    for name, cuts in (("d", [1]), ("p", [2, 2, 7, 3, 16, 2, 5]), ("q", [30, 2]), ("r", [1, 13])):
        got = feed_all(eng, name, t, cuts)
        eng.feed([], [name])
        close(got, want, 3e-4)
    assert eng.pool.num_used == 0 and eng.state_pool.num_free == 4


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_unequal_batches_reuse_pages_and_slots(device, dtype):
    """Six requests of different lengths through four slots and a pool too small for all of them:
    portions beside single tokens, requests sitting steps out, pages and slots used again — every
    position equals the request run alone."""
    eng = engine(small_cfg(), device, dtype=dtype, num_blocks=40, bs=4)
    solo = engine(small_cfg(), device, dtype=dtype)
    solo.model.copy_from(eng.model)
    lens = {"a": 41, "b": 7, "c": 30, "d": 2, "e": 23, "f": 35}
    seqs = {k: toks(n, 10 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: solo.feed([(k, v, list(range(len(v))))], [k])[0] for k, v in seqs.items()}
    plan = [[("a", 5), ("b", 2)], [("a", 1), ("b", 1), ("c", 9), ("d", 2)], [("a", 17), ("c", 1)],
            [("b", 4), ("c", 2), ("a", 1), ("e", 3)], [("e", 20), ("a", 17)], [("c", 18), ("f", 6)],
            [("f", 1), ("c", 0)], [("f", 28)]]
    at = {k: 0 for k in seqs}
    got = {k: [] for k in seqs}
    for step in plan:
        entries, end = [], []
        for k, n in step:
            part = seqs[k][at[k]:at[k] + n]
            entries.append((k, part, list(range(len(part)))))
            at[k] += n
            if at[k] == len(seqs[k]):
                end.append(k)
        for k, out in zip([e[0] for e in entries], eng.feed(entries, end)):
            got[k].append(out)
    assert at == lens and eng.pool.num_used == 0 and eng.state_pool.num_free == 4
    assert eng.state_pool.stats["allocs"] == 6
    if dtype == torch.float32:
        for k in seqs:
            close(torch.cat(got[k], 0), want[k], 2e-4)
        close(want["a"], oracle_logits(solo, seqs["a"]), 3e-4)
    else:       # an expert choice that flips on a close call moves a whole row: rows are judged by their median
        for k in seqs:
            assert (torch.cat(got[k], 0) - want[k]).abs().amax(1).median().item() < 0.1


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_and_long_decoding(device):
    """A sequence of one token; 137 single-token steps, far past every window (17 at most) and over many pages."""
    eng = engine(small_cfg(), device, max_len=256)
    t = toks(140, 5)
    want = oracle_logits(eng, t)
    close(eng.feed([("one", t[:1], [0])], ["one"])[0], want[:1], 2e-4)
    got = feed_all(eng, "x", t, [3])
    close(got, want, 4e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_a_key_at_the_window_edge_decides_the_logits(device):
    """One layer, window 6, weights set so that the query locks onto one earlier token's latent: the logits at
    position p follow that token while it is inside the window (prompt rows and decode rows) and change when
    it falls out — and both match the oracle."""
    cfg = small_cfg(layers=[LayerSpec(T1, la(1, 2, 4, 2, 4, 6, 6, window=6, scale=6.0), None)], side_dim=0, bigram_buckets=0)
    eng = engine(cfg, device, bs=4)
    t = toks(30, 9)
    want = oracle_logits(eng, t)
    close(eng.feed([("w", t, list(range(30)))], ["w"])[0], want, 5e-4)
    close(feed_all(eng, "d", t, [9, 2]), want, 5e-4)
    # with such a sharp softmax a window that is one token off cannot hide: compare against the oracle run on a
    # configuration whose window is one longer / shorter, which must differ clearly
    for other in (5, 7):
        d = config_dict(eng.model_cfg)
        d["layers"][0]["mixer"]["mask"]["size"] = other
        P = {k: v.to(F64) for k, v in params(eng.model).items()}
        off = orc.forward(P, d, t)
        assert (off - want)[8:].abs().max() > 0.05


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(device):
    eng = engine(small_cfg(), device, max_len=128)
    prompts = [toks(9, 20), toks(17, 21), toks(3, 22)]
    reqs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    P = {k: v.to(F64) for k, v in params(eng.model).items()}
    cd = config_dict(eng.model_cfg)
    for p, r in zip(prompts, reqs):
        seq = list(p)
        for tok in r.output:
            lg = orc.forward(P, cd, seq)[-1]
            top2 = torch.topk(lg, 2).values
            assert tok == int(lg.argmax()) or (top2[0] - top2[1]) < 1e-3
            seq.append(tok)
    assert eng.pool.num_used == 0 and eng.state_pool.num_free == 4


@pytest.mark.gpu
def test_graph_decode_equals_eager_decode():
    """Decode steps replayed as hipGraphs produce the tokens of the eager engine; replays follow each other
    with eager prompt steps between them, slots and pages reused by a second batch."""
    cfg = small_cfg()
    eager, graph = engine(cfg, "cuda", max_len=128), engine(cfg, "cuda", max_len=128, graphs=True)
    graph.model.copy_from(eager.model)
    prompts = [toks(9, 60), toks(17, 61), toks(3, 62)]
    sp = SamplingParams(max_tokens=14, temperature=0.0, ignore_eos=True)
    want = [r.output for r in eager.generate(prompts, sp)]
    for _ in range(2):
        assert [r.output for r in graph.generate(prompts, sp)] == want
    assert graph.runner.graphs is not None and graph.runner.graphs.captured
    assert graph.state_pool.num_free == 4 and graph.pool.num_used == 0


def test_preempted_sequence_is_recomputed():
    cfg = small_cfg()
    big = engine(cfg, "cpu", max_len=128)
    sp = SamplingParams(max_tokens=20, temperature=0.0, ignore_eos=True)
    ref = big.generate([toks(20, 30), toks(22, 31)], sp)
    tight = engine(cfg, "cpu", num_blocks=18, bs=4, max_len=128)
    tight.model.copy_from(big.model)
    got = tight.generate([toks(20, 30), toks(22, 31)], sp)
    assert tight.scheduler.num_preemptions > 0
    assert [r.output for r in got] == [r.output for r in ref]


def write_checkpoint(eng, path):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config_dict(eng.model_cfg), f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in params(eng.model).items()},
              os.path.join(path, "model.safetensors"))


def test_checkpoint_layout_and_trace_runner(tmp_path):
    """config.json + safetensors in the design's naming -> registry, loader, engine; the replay
    command writes the logits of the wanted places, step by step."""
    src = engine(small_cfg(), "cpu", dtype=torch.bfloat16)          # bf16 weights survive the file bit for bit
    ck = str(tmp_path / "model")
    write_checkpoint(src, ck)
    cfg = get_config(ck)
    assert isinstance(cfg, DepelixConfig) and cfg.kv_owners == [0, 2, 3, 4]
    eng = LLMEngine(EngineConfig(model=ck, device="cpu", dtype=torch.float32, block_size=4, num_blocks=64, max_num_seqs=4,
                                 max_model_len=128, max_num_batched_tokens=128, use_graphs=False, token_align=0))
    assert eng.model.load_info["tensors"] == len(params(src.model))
    t = toks(21, 40)
    want = oracle_logits(eng, t)
    close(eng.feed([("a", t, list(range(len(t))))], ["a"])[0], want, 3e-4)
    out = tmp_path / "out"
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": t[:6], "want": [0, 5]}, {"id": "y", "tokens": t[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": t[6:7], "want": [0]}], "end": ["y"]},
             {"step": 2, "entries": [{"id": "x", "tokens": t[7:], "want": [13]}], "end": ["x"]}]
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", ck, "--dtype", "float32", "--out",
                        str(out), "--max-tokens", "64", "--device", "cpu"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    import numpy as np
    for step, rows in ((0, [0, 5]), (1, [6]), (2, [20])):
        got = torch.from_numpy(np.fromfile(str(out / f"{step}.f32"), dtype="<f4").reshape(len(rows), -1))
        close(got, want[rows], 3e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("variant", ["base", "vector_sizes"])
def test_kernels_match_the_reference_ops_on_a_prompt_batch(dtype, variant):
    """The HIP kernels against the CPU reference ops through the same engine code, over a batch of
    portions and decode rows: fp32 within rounding at every position; bf16 at the typical position."""
    cfg = small_cfg(**VARIANTS[variant])
    cpu, gpu = engine(cfg, "cpu", dtype=dtype), engine(cfg, "cuda", dtype=dtype)
    cpu.model.copy_from(gpu.model)
    a, b = toks(50, 50), toks(33, 51)
    for eng in (cpu, gpu):
        eng.out = [eng.feed([("a", a[:40], list(range(40))), ("b", b[:2], [0, 1])]),
                   eng.feed([("a", a[40:41], [0]), ("b", b[2:], list(range(31)))]),
                   eng.feed([("a", a[41:], list(range(9)))], ["a", "b"])]
    x = torch.cat([u for o in cpu.out for u in o], 0)
    y = torch.cat([v for o in gpu.out for v in o], 0).cpu()
    if dtype == torch.float32:
        close(y, x, 3e-4)
    else:
        assert (y - x).abs().amax(1).median().item() < 0.1


def test_bench_arch_compare_option_runs():
    """`bench.py --arch-compare depelix` (tiny size, CPU): one JSON line with a row per model and phase numbers."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--arch-compare", "depelix", "--arch-sizes", "tiny",
                        "--prompt-len", "40", "--concurrency", "2", "--steps", "2", "--warmup", "1",
                        "--max-batched-tokens", "128"], capture_output=True, text=True, timeout=600,
                       env={**os.environ, "CUDA_VISIBLE_DEVICES": "", "HIP_VISIBLE_DEVICES": ""})
    assert r.returncode == 0, r.stderr[-2000:]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    assert [x["model"] for x in out["rows"]] == ["depelix", "llama"]
    assert all(x["prefill_tok_s"] > 0 and x["decode_tok_s"] > 0 for x in out["rows"])


@pytest.mark.gpu
@pytest.mark.parametrize("hd,H,window", [(64, 4, 100), (128, 2, 64), (128, 3, 1), (64, 2, 300)])
def test_mfma_prompt_kernel_with_a_sliding_window(hd, H, window):
    """The MFMA prompt kernel with a sliding window against the row-wise reference: two portions on top of cached
    tokens, windows that end inside 64-key tiles and span several, a dominating key just inside / outside."""
    from dgi.ops import mix
    bs, G = 16, H
    g = torch.Generator().manual_seed(7)
    lens, ctx = [200, 77], [330, 77]
    nblk = sum((c + bs - 1) // bs for c in ctx)
    kc = (torch.randn(nblk + 1, G, bs, hd, generator=g) * 0.5).to(torch.bfloat16)
    vc = (torch.randn(nblk + 1, G, bs, hd, generator=g) * 0.5).to(torch.bfloat16)
    q = (torch.randn(sum(lens), H * hd, generator=g) * 0.5).to(torch.bfloat16)
    perm = (torch.randperm(nblk, generator=g) + 1).tolist()
    mb = max((c + bs - 1) // bs for c in ctx)
    bt = torch.zeros(2, mb, dtype=I32)
    at = 0
    for b, c in enumerate(ctx):
        n = (c + bs - 1) // bs
        bt[b, :n] = torch.tensor(perm[at:at + n], dtype=I32)
        at += n
    # row 150 of the first portion sits at position 280: its window starts at 280 - window + 1
    p = 280
    for j, scale in ((p - window + 1, 6.0), (p - window, 9.0)):
        if j >= 0:
            kc[int(bt[0, j // bs]), 0, j % bs] = (q[150, :hd].float() * scale).to(torch.bfloat16)
    cu = torch.tensor([0, lens[0], sum(lens)], dtype=I32)
    cl = torch.tensor(ctx, dtype=I32)
    want = mix.paged_prefill_masked(q, kc, vc, bt, cu, cl, H, G, 0.2, 0, None, window=window)            # CPU: row-wise reference
    got = mix.paged_prefill_masked(q.cuda(), kc.cuda(), vc.cuda(), bt.cuda(), cu.cuda(), cl.cuda(), H, G, 0.2, 0, None,
                                   window=window)
    close(got.float(), want.float(), 0.03)


@pytest.mark.gpu
def test_mfma_prompt_path_in_the_model(monkeypatch):
    """Layers whose bf16 heads are 64 / 128 wide (unrotated + rotated = value size) take the MFMA prompt kernel
    on expanded keys and values: same logits as the row-wise kernel on the cached latents (portions on top of
    cached tokens, two prompts and a decode row in one step, windows shorter than the prompt, a shared latent)."""
    from dgi.models import depelix as dm
    cfg = DepelixConfig(name="t", vocab_size=53, hidden_size=64, layers=[
        LayerSpec(T1, la(1, 4, 32, 32, 64, 40, 48, window=70), DenseSpec(64)),
        LayerSpec(T1, la(1, 2, 96, 32, 128, 40, 32, window=33, kv_from=0), None),
        LayerSpec(T2, la(2, 3, 96, 32, 128, 24, 32), DenseSpec(64)),
        LayerSpec(T2, la(2, 2, 32, 32, 64, 24, 32, kv_from=2), None),
    ], side_dim=8, bigram_buckets=29, bigram_mul_prev=5, bigram_mul_cur=3, max_position=512)
    a, b, c = toks(200, 70), toks(90, 71), toks(40, 72)

    def run():
        eng = engine(cfg, "cuda", dtype=torch.bfloat16, num_blocks=64, bs=16, max_len=512)
        out = [eng.feed([("a", a[:150], list(range(150))), ("c", c[:39], [38])]),
               eng.feed([("a", a[150:], list(range(50))), ("b", b, list(range(90))), ("c", c[39:], [0])], ["a", "b", "c"])]
        return torch.cat([o for step in out for o in step], 0)

    calls = []
    real = dm.DepelixModel._attention_mfma_prompt
    monkeypatch.setattr(dm.DepelixModel, "_attention_mfma_prompt", lambda self, *a, **k: (calls.append(1), real(self, *a, **k))[1])
    fast = run()
    assert len(calls) == 8                                   # every layer of both steps
    monkeypatch.setattr(dm, "MFMA_PROMPT_ROWS", 1 << 30)
    slow = run()
    assert len(calls) == 8
    close(fast, slow, 0.06 * max(1.0, slow.abs().max().item()))


def test_worker_engine_serves_a_checkpoint_dir(tmp_path):
    """The worker's native engine picks the model class from config.json and generates through the same LLMEngine."""
    sys.path.insert(0, os.path.join(ROOT, "worker"))
    from engines.llm_native import NativeLLMEngine
    d = str(tmp_path / "ckpt")
    write_checkpoint(engine(small_cfg(vocab_size=300), "cpu", torch.bfloat16), d)
    e = NativeLLMEngine({"model_id": d, "device": "cpu", "max_model_len": 128, "max_num_batched_tokens": 128,
                         "num_blocks": 64, "max_num_seqs": 4})
    e.load_model()
    assert type(e.engine.model).__name__ == "DepelixModel"
    out = e.batch_inference([{"messages": [{"role": "user", "content": "hi"}], "max_tokens": 5, "temperature": 0.0}])
    assert out[0]["usage"]["completion_tokens"] == 5
