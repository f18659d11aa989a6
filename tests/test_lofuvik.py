"""Lofuvik in the framework against the plain float64 oracle (tests/lofuvik_oracle.py): every
mechanism alone, then the model through the engine's scheduler, block pool, state slots and step —
whole prompts, token-by-token decoding, portions down to two tokens, unequal batches, reused pages
and slots, far keys and far memories, page borders, first tokens, long decoding, other geometries,
greedy generation, the checkpoint layout and the trace runner.  The same tests run the CPU reference
ops here and the HIP kernels on a GPU box."""
import copy
import json
import math
import os
import subprocess
import sys

import pytest
import torch

import lofuvik_oracle as orc
from dgi import ops
from dgi.engine import EngineConfig, LLMEngine
from dgi.models.config import (AttentionSpec, DeltaSpec, LayerSpec, LofuvikConfig, MlstmSpec, MoeSpec, ParallelSpec,
                               RotarySpec, WkvSpec, get_config)
from dgi.ops import latent, linrec, mix, moe
from dgi.sched.request import SamplingParams

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F64 = torch.float64
I32 = torch.int32
RAMP = {"factor": 3.0, "original": 40, "fast": 6.0, "slow": 1.5}


def experts(n, top, ff):
    return MoeSpec(n, 0, top, ff, score="top_softmax", selection_bias=False, router_bias=True)


def left(heads, kv, dim, vdim, scale, rot_dims, cap=8.0, scaling=RAMP, base=100.0):
    return AttentionSpec(heads, kv, dim, vdim, scale, RotarySpec(base, rot_dims, scaling, "half") if rot_dims else None,
                         out_gate=True, qk_norm="full", softcap=cap, sink=True)


def small_cfg(**kw) -> LofuvikConfig:
    """Five layers that differ in everything: partial and full rotation, with and without frequency
    scaling, heads == kv heads and 3 query heads per kv head, key size != value size, one tap and five,
    top == 1 and top == all experts, a layer without feed-forward; layers 1-3 run twice."""
    args = dict(name="t", vocab_size=53, hidden_size=32, layers=[
        LayerSpec("delta", DeltaSpec(4, 2, 6, 10, 3), experts(3, 2, 20)),
        LayerSpec("parallel", ParallelSpec(left(6, 2, 8, 12, 0.4, 6), MlstmSpec(2, 10, 6, 4.0)), experts(4, 1, 12)),
        LayerSpec("wkv", WkvSpec(2, 12, 5), None),
        LayerSpec("parallel", ParallelSpec(left(2, 2, 12, 8, 0.3, 12, cap=3.0, scaling=None), MlstmSpec(3, 4, 20, 9.0)),
                  experts(2, 2, 8)),
        LayerSpec("delta", DeltaSpec(3, 3, 20, 4, 5), experts(5, 3, 6)),
    ], loop_start=1, loop_stop=4, loop_times=2, norm_eps=1e-5, max_position=512)
    args.update(kw)
    return LofuvikConfig(**args)


def engine(cfg, device, dtype=torch.float32, num_blocks=96, bs=4, seed=3, max_len=256, seqs=4, graphs=False):
    return LLMEngine(EngineConfig(model="lofuvik-test", device=device, dtype=dtype, block_size=bs, num_blocks=num_blocks,
                                  max_num_seqs=seqs, max_model_len=max_len, max_num_batched_tokens=max_len,
                                  enable_prefix_caching=True, use_graphs=graphs, token_align=0, decode_lookahead=graphs,
                                  seed=seed, graph_buckets=(1, 2, 4) if graphs else None), model_cfg=copy.deepcopy(cfg))


def toks(n, seed=0, vocab=53):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def rot_dict(rot):
    return None if rot is None else {"base": rot.base, "dims": rot.dims, "scaling": rot.scaling}


def config_dict(cfg: LofuvikConfig) -> dict:
    """The design's config.json for ``cfg``."""
    layers = []
    for l in cfg.layers:
        m = l.mixer
        if l.type == "wkv":
            mixer = {"heads": m.heads, "dim": m.dim}
        elif l.type == "delta":
            mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "conv": m.conv}
        else:
            a, r = m.left, m.right
            mixer = {"left": {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale,
                              "softcap": a.softcap, "rot": rot_dict(a.rot) or {"base": 10000.0, "dims": 0}},
                     "right": {"heads": r.heads, "dim": r.dim, "vdim": r.vdim, "gate_cap": r.gate_cap}}
        f = l.mlp
        mlp = None if f is None else {"kind": "moe", "expert": {"ff": f.ff}, "router": {"experts": f.experts, "top": f.top}}
        layers.append({"type": l.type, "mixer": mixer, "mlp": mlp})
    return {"architecture": "Lofuvik", "vocab": cfg.vocab_size, "width": cfg.hidden_size, "norm": {"eps": cfg.norm_eps},
            "loop": {"start": cfg.loop_start, "stop": cfg.loop_stop, "times": cfg.loop_times}, "layers": layers}


def params(model) -> dict:
    """The model's weights under the checkpoint's tensor names (CPU, model dtype)."""
    P = {"embed": model.embed, "head": model.head, "final.norm": model.final_norm}
    for i, L in enumerate(model.layers):
        p, x = f"l{i}.", f"l{i}.mix."
        m, f = L.spec.mixer, L.spec.mlp
        P[p + "norm1"] = L.norm1
        r0 = 0
        if f is not None:
            r0 = f.routes
            P[p + "mlp.router"], P[p + "mlp.router.b"] = L.side[:r0], L.side_b[:r0]
            for e in range(f.experts):
                P[f"{p}mlp.e{e}.gate"], P[f"{p}mlp.e{e}.up"] = L.gate_up[e, :f.ff], L.gate_up[e, f.ff:]
                P[f"{p}mlp.e{e}.down"] = L.down[e]
        if L.spec.type == "wkv":
            for j, s in enumerate(("r", "k", "v", "g", "w")):
                P[x + "mu." + s] = L.mu[j]
            for j, s in enumerate(("r", "k", "v", "g")):
                P[x + s] = L.rkvg[j]
            for key, t in (("w1", L.w1), ("w2", L.w2), ("w0", L.w0), ("u", L.bonus.view(m.heads, m.dim)), ("norm", L.mnorm),
                           ("o", L.o)):
                P[x + key] = t
        elif L.spec.type == "delta":
            H, qk = m.heads, m.qk_size
            P[x + "q"], P[x + "k"], P[x + "v"], P[x + "g"] = (L.in_proj[:qk], L.in_proj[qk:2 * qk],
                                                              L.in_proj[2 * qk:2 * qk + m.inner], L.in_proj[2 * qk + m.inner:])
            P[x + "q.conv"], P[x + "k.conv"], P[x + "v.conv"] = L.conv[:qk], L.conv[qk:2 * qk], L.conv[2 * qk:]
            P[x + "b"], P[x + "a"] = L.side[r0:r0 + H], L.side[r0 + H:r0 + 2 * H]
            for key, t in (("A_log", L.a_log), ("dt_bias", L.dt_bias), ("norm", L.mnorm), ("o", L.o)):
                P[x + key] = t
        else:
            a, r = m.left, m.right
            c = 0
            for key, rows in (("left.q", a.q_size), ("left.k", a.k_size), ("left.v", a.v_size), ("left.g", a.o_size),
                              ("right.q", r.qk_size), ("right.k", r.qk_size), ("right.v", r.inner), ("right.g", r.inner)):
                P[x + key] = L.in_proj[c:c + rows]
                c += rows
            H = r.heads
            P[x + "right.i"], P[x + "right.f"] = L.side[r0:r0 + H], L.side[r0 + H:r0 + 2 * H]
            P[x + "right.i.b"], P[x + "right.f.b"] = L.side_b[r0:r0 + H], L.side_b[r0 + H:r0 + 2 * H]
            for key, t in (("left.q.norm", L.q_norm), ("left.k.norm", L.k_norm), ("left.sink", L.sink), ("left.o", L.o),
                           ("left.out", L.out_left), ("right.o", L.o_right), ("right.norm", L.rnorm),
                           ("right.out", L.out_right)):
                P[x + key] = t
    return {k: v.detach().cpu().contiguous() for k, v in P.items()}


def oracle_logits(eng, tokens, layers=False):
    P = {k: v.to(F64) for k, v in params(eng.model).items()}
    return orc.forward(config_dict(eng.model_cfg), P, tokens, layers)


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


def seq_meta(lens, starts, slots, device):
    pos, rs, r0 = [], [], [0]
    for i, (n, s) in enumerate(zip(lens, starts)):
        pos += list(range(s, s + n))
        rs += [i] * n
        r0.append(r0[-1] + n)
    mk = lambda x: torch.tensor(x, dtype=I32, device=device)   # noqa: E731
    return mk(pos), mk(rs), mk(r0), mk(slots)


def portions(n, cuts, other_n=0, other_every=2):
    """(count of sequence a, count of sequence b) per step: a in the given cuts then whole, b five rows now and then."""
    at_a = at_b = 0
    for i, c in enumerate(list(cuts) + [n]):
        na = min(c, n - at_a)
        nb = min(5, other_n - at_b) if (other_n and i % other_every) else 0
        if na or nb:
            yield at_a, na, at_b, nb
        at_a, at_b = at_a + na, at_b + nb


# ----------------------------------------------------------------------------------- mechanisms
def test_configuration_from_the_file_form():
    cfg = small_cfg()
    back = LofuvikConfig.from_dict(config_dict(cfg))
    assert back.layer_runs == [0, 1, 2, 3, 1, 2, 3, 4] and back.pass_starts == {4}
    assert back.kv_layer_shapes() == [(2, 8, 12), (2, 12, 8), (2, 8, 12), (2, 12, 8)]
    assert back.layers[1].mixer.left.rot.dims == 6 and back.layers[1].mixer.left.rot.layout == "half"
    assert back.layers[3].mixer.left.rot.scaling is None and back.layers[2].mlp is None
    assert back.layers[2].mixer.decay_rank == 0          # only the checkpoint's shapes give it
    with pytest.raises(ValueError):
        d = config_dict(cfg)
        d["layers"][0]["type"] = "other"
        LofuvikConfig.from_dict(d)
    with pytest.raises(ValueError):
        d = config_dict(cfg)
        d["layers"][0]["mixer"]["kv_heads"] = 3
        LofuvikConfig.from_dict(d)


@pytest.mark.parametrize("scaling", [None, RAMP, {"factor": 8.0, "original": 16, "fast": 32.0, "slow": 1.0},
                                     {"factor": 1.0, "original": 4096, "fast": 4.0, "slow": 4.0}])
@pytest.mark.parametrize("dims,base", [(6, 100.0), (16, 10000.0), (2, 7.0)])
def test_rotary_table_with_ramp_scaling(scaling, dims, base):
    cos, sin = orc.yarn_tables({"dims": dims, "base": base, "scaling": scaling}, 300)
    t = ops.rope_cos_sin(dims, 300, base, scaling)
    close(t[:, :dims // 2], cos, 2e-6)
    close(t[:, dims // 2:], sin, 2e-6)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W", [40, 300])
def test_token_shift_portions(device, dtype, W):
    """Blends with the previous token's row: whole == portions of 1, 2, 7 rows through a slot that held
    another sequence before, with a second sequence in the same step; zeros before position 0."""
    g = torch.Generator().manual_seed(1)
    n = 30
    ha, hb = torch.randn(n, W, generator=g).to(dtype), torch.randn(n, W, generator=g).to(dtype)
    mu = torch.rand(5, W, generator=g)

    def want(h):
        hf = h.to(F64)
        prev = torch.cat([torch.zeros(1, W, dtype=F64), hf[:-1]], 0)
        return hf[None] + (prev - hf)[None] * mu.to(F64)[:, None, :]

    tail = (torch.randn(6, W, generator=g) * 50).to(device)
    got_a, got_b = [], []
    for at_a, na, at_b, nb in portions(n, [1, 1, 2, 7, 1, 13], n):
        lens, starts, slots, rows = [], [], [], []
        for cnt, at, slot, h in ((na, at_a, 3, ha), (nb, at_b, 5, hb)):
            if cnt:
                lens.append(cnt), starts.append(at), slots.append(slot), rows.append(h[at:at + cnt])
        pos, rs, r0, sl = seq_meta(lens, starts, slots, device)
        y = linrec.token_shift(torch.cat(rows, 0).to(device), mu.to(device), tail, pos, rs, r0, sl, torch.float32)
        got_a.append(y[:, :na])
        got_b.append(y[:, na:])
    close(torch.cat(got_a, 1), want(ha), 1e-5)
    gb = torch.cat(got_b, 1)
    close(gb, want(hb)[:, :gb.shape[1]], 1e-5)


def scan_inputs(g, mode, H, G, D, V, n, dtype):
    q, k = torch.randn(n, G * D, generator=g).to(dtype), torch.randn(n, G * D, generator=g).to(dtype)
    v = torch.randn(n, H * V, generator=g).to(dtype)
    if mode == "wkv":
        return q, k, v, torch.randn(n, H * D, generator=g) * 1.5 - 1.0, None
    return q, k, v, torch.randn(n, H, generator=g) * 2, torch.randn(n, H, generator=g) * 2


def scan_oracle(mode, q, k, v, a1, a2, par, H, G, D, V):
    n = q.shape[0]
    q, k, v = q.to(F64), k.to(F64), v.to(F64)
    if mode == "wkv":
        dec = torch.exp(-torch.exp(a1.to(F64) + par["w0"].to(F64))).view(n, H, D)
        return orc.wkv_core(q.view(n, H, D), k.view(n, H, D), v.view(n, H, D), dec, par["u"].to(F64).view(H, D)).reshape(n, -1)
    if mode == "delta":
        qq = (orc.unit_vectors(q.view(n, G, D)) * D ** -0.5).repeat_interleave(H // G, 1)
        kk = orc.unit_vectors(k.view(n, G, D)).repeat_interleave(H // G, 1)
        dec = torch.exp(-torch.exp(par["a_log"].to(F64)) * orc.softplus(a2.to(F64) + par["dt_bias"].to(F64)))
        return orc.delta_core(qq, kk, v.view(n, H, V), torch.sigmoid(a1.to(F64)), dec).reshape(n, -1)
    ig, fg = orc.capped_gates(a1.to(F64), a2.to(F64), par["cap"])
    return orc.mlstm_core(q.view(n, H, D) * D ** -0.5, k.view(n, H, D), v.view(n, H, V), ig, fg).reshape(n, -1)


def scan_call(mode, q, k, v, a1, a2, par, st, pos, r0, sl, H, G, D, V):
    dev = q.device
    if mode == "wkv":
        return linrec.wkv_scan(q, k, v, a1, par["w0"].to(dev), par["u"].to(dev), st["S"], pos, r0, sl, H, D)
    if mode == "delta":
        return linrec.delta_scan(q, k, v, a1, a2, par["a_log"].to(dev), par["dt_bias"].to(dev), st["S"], pos, r0, sl, H, G, D, V)
    return linrec.mlstm_scan(q, k, v, a1, a2, par["cap"], st["S"], st["n"], st["m"], pos, r0, sl, H, D, V)


def scan_params(g, mode, H, D):
    if mode == "wkv":
        return {"w0": torch.randn(H * D, generator=g) * 0.7 - 1.5, "u": torch.randn(H * D, generator=g) * 0.5}
    if mode == "delta":
        return {"a_log": torch.randn(H, generator=g) * 0.5 - 1.0, "dt_bias": torch.randn(H, generator=g) * 0.5 - 1.0}
    return {"cap": 5.0}


SCAN_GEOMS = [("wkv", 2, 2, 12, 12), ("wkv", 3, 3, 64, 64), ("wkv", 1, 1, 5, 5), ("wkv", 2, 2, 130, 130),
              ("delta", 4, 2, 6, 10), ("delta", 3, 3, 20, 4), ("delta", 2, 1, 128, 64), ("delta", 6, 2, 16, 70),
              ("mlstm", 2, 2, 10, 6), ("mlstm", 3, 3, 4, 20), ("mlstm", 2, 2, 64, 128), ("mlstm", 1, 1, 300, 17),
              ("delta", 2, 1, 48, 40), ("mlstm", 2, 2, 100, 33), ("wkv", 2, 2, 40, 40)]


@pytest.mark.gpu
@pytest.mark.parametrize("heads", [6, 48, 64])
@pytest.mark.parametrize("mode", ["wkv", "delta", "mlstm"])
def test_recurrences_prompt_steps_of_every_grid_size(mode, heads):
    """A prompt step picks its thread layout by the number of workgroups (sequences x heads x column blocks): five
    sequences of nine rows with few, many and very many heads take the three layouts; each continues a state."""
    H, G, D, V, n, ns = heads, heads // 2, 64, 64, 9, 5
    g = torch.Generator().manual_seed(heads)
    par = scan_params(g, mode, H, D)
    st = {"S": torch.randn(ns + 1, H, D, V, generator=g) * 0.3, "n": torch.randn(ns + 1, H, D, generator=g) * 0.3,
          "m": torch.randn(ns + 1, H, generator=g).abs()}
    if mode != "delta":
        G = H
    ins = [scan_inputs(g, mode, H, G, D, V, n, torch.float32) for _ in range(ns)]
    cat = [None if ins[0][j] is None else torch.cat([x[j] for x in ins], 0) for j in range(5)]
    out = {}
    for device in ("cpu", "cuda"):
        pos, rs, r0, sl = seq_meta([n] * ns, [3] * ns, list(range(1, ns + 1)), device)
        sd = {k: v.clone().to(device) for k, v in st.items()}
        y = scan_call(mode, *[None if c is None else c.to(device) for c in cat], par, sd, pos, r0, sl, H, G, D, V)
        out[device] = [y.cpu()] + [sd[k].cpu() for k in ("S", "n", "m")]
    for a, b in zip(out["cuda"], out["cpu"]):
        scale = b.abs().max().clamp(min=1.0)
        close(a / scale, b / scale, 2e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("geom", SCAN_GEOMS, ids=lambda x: "-".join(map(str, x)))
def test_recurrences_portions_and_slots(device, dtype, geom):
    """Whole sequence == portions of 1, 2, 7, ... rows through a slot that held another state before, with a
    second sequence in the same step; strided row views; extreme gate inputs."""
    mode, H, G, D, V = geom
    if mode == "wkv":
        V = D
    g = torch.Generator().manual_seed(4)
    n = 37
    qa, ka, va, a1a, a2a = scan_inputs(g, mode, H, G, D, V, n, dtype)
    qb, kb, vb, a1b, a2b = scan_inputs(g, mode, H, G, D, V, n, dtype)
    if mode != "wkv":
        a1a[3], a1a[4], a2a[5], a2a[6] = 40.0, -40.0, 40.0, -40.0        # gates without overflow
    par = scan_params(g, mode, H, D)
    want_a = scan_oracle(mode, qa, ka, va, a1a, a2a, par, H, G, D, V)
    want_b = scan_oracle(mode, qb, kb, vb, a1b, a2b, par, H, G, D, V)
    st = {"S": (torch.randn(6, H, D, V, generator=g) * 50).to(device), "n": (torch.randn(6, H, D, generator=g) * 50).to(device),
          "m": (torch.randn(6, H, generator=g) * 50).to(device)}
    got_a, got_b = [], []
    for at_a, na, at_b, nb in portions(n, [1, 1, 2, 7, 1, 9, 3], n):
        lens, starts, slots, parts = [], [], [], [[] for _ in range(5)]
        for cnt, at, slot, src in ((na, at_a, 3, (qa, ka, va, a1a, a2a)), (nb, at_b, 5, (qb, kb, vb, a1b, a2b))):
            if cnt:
                lens.append(cnt), starts.append(at), slots.append(slot)
                for lst, t in zip(parts, src):
                    lst.append(None if t is None else t[at:at + cnt])
        pos, _rs, r0, sl = seq_meta(lens, starts, slots, device)
        # q | k | v as views of one wider row buffer, gate inputs as views of another (the model's layout)
        qkv = torch.cat([torch.cat(parts[0], 0), torch.cat(parts[1], 0), torch.cat(parts[2], 0)], 1).to(device)
        c1, c2 = G * D, 2 * G * D
        if mode == "wkv":
            a1, a2 = torch.cat(parts[3], 0).to(device), None
        else:
            side = torch.cat([torch.zeros(sum(lens), 3), torch.cat(parts[3], 0), torch.cat(parts[4], 0)], 1).to(device)
            a1, a2 = side[:, 3:3 + H], side[:, 3 + H:]
        y = scan_call(mode, qkv[:, :c1], qkv[:, c1:c2], qkv[:, c2:], a1, a2, par, st, pos, r0, sl, H, G, D, V)
        got_a.append(y[:na])
        got_b.append(y[na:])
    for got, want in ((torch.cat(got_a, 0), want_a), (torch.cat(got_b, 0), want_b)):
        close(got, want[:got.shape[0]], 3e-5 * max(1.0, want.abs().max().item()))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("mode", ["wkv", "delta", "mlstm"])
def test_recurrences_remember_a_far_token(device, mode):
    """One early token writes a large value under a key that only the last query asks for, hundreds of
    tokens later, through slow decays and many decode steps: a lost or reset state shows at once."""
    H, D, V = 2, 8, 8
    n, far = 400, 7
    g = torch.Generator().manual_seed(9)
    q, k, v = torch.zeros(n, H * D), torch.zeros(n, H * D), torch.randn(n, H * V, generator=g) * 0.1
    k[:, 1::D] = 1.0                                  # every token writes under channel 1 of each head
    k[far] = 0.0
    k[far, 0::D] = 1.0                                # ... but the far token under channel 0
    v[far] = 5.0
    q[:, 1::D] = 1.0
    q[n - 1] = 0.0
    q[n - 1, 0::D] = 1.0                              # only the last query reads channel 0
    if mode == "wkv":
        a1, a2 = torch.full((n, H * D), -9.0), None   # decay exp(-exp(-9 - 1.5)) per step
    elif mode == "delta":
        a1, a2 = torch.full((n, H), 3.0), torch.full((n, H), -12.0)
    else:
        a1, a2 = torch.zeros(n, H), torch.full((n, H), 12.0)
    par = scan_params(g, mode, H, D)
    want = scan_oracle(mode, q, k, v, a1, a2, par, H, H, D, V)
    assert want[n - 1].abs().min() > 0.05             # the far value is what the last query reads
    st = {"S": torch.zeros(3, H, D, V, device=device), "n": torch.zeros(3, H, D, device=device),
          "m": torch.zeros(3, H, device=device)}
    out, at = [], 0
    for c in [50, 2, 200] + [1] * 148:
        pos, _rs, r0, sl = seq_meta([c], [at], [2], device)
        sl_ = slice(at, at + c)
        out.append(scan_call(mode, q[sl_].to(device), k[sl_].to(device), v[sl_].to(device), a1[sl_].to(device),
                             None if a2 is None else a2[sl_].to(device), par, st, pos, r0, sl, H, H, D, V))
        at += c
    assert at == n
    close(torch.cat(out, 0), want, 2e-4 * max(1.0, want.abs().max().item()))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_head_norm_gate_and_branch_mean(device, dtype):
    g = torch.Generator().manual_seed(2)
    for H, dv, shared, act in ((3, 20, False, "silu"), (4, 10, True, "silu"), (2, 130, False, "sigmoid"), (1, 7, True, "sigmoid")):
        y = torch.randn(9, H * dv, generator=g) * 3
        zz = torch.randn(9, H * dv + 5, generator=g).to(dtype)
        w = torch.randn(dv if shared else H * dv, generator=g)
        z = zz[:, 5:]
        v = orc.rms_unit(y.to(F64).view(9, H, dv), 1e-5).reshape(9, -1) * (w.repeat(H) if shared else w).to(F64)
        zf = z.to(F64)
        want = v * (orc.silu(zf) if act == "silu" else torch.sigmoid(zf))
        got = linrec.head_norm_gate(y.to(device), zz.to(device)[:, 5:], w.to(device), H, 1e-5, act, torch.float32)
        close(got, want, 2e-5)
    for W in (32, 300, 1000):
        a, b = (torch.randn(7, W, generator=g) * 4).to(dtype), torch.randn(7, W, generator=g).to(dtype)
        wa, wb = torch.randn(W, generator=g), torch.randn(W, generator=g)
        want = 0.5 * (orc.rms_unit(a.to(F64), 1e-5) * wa.to(F64) + orc.rms_unit(b.to(F64), 1e-5) * wb.to(F64))
        close(linrec.rms_pair_mean(a.to(device), b.to(device), wa.to(device), wb.to(device), 1e-5), want, 2e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W", [40, 1024])
def test_stream_add_with_two_addends(device, dtype, W):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(6, W, generator=g)
    y, y2 = torch.randn(6, W, generator=g), torch.randn(6, W, generator=g).to(dtype)
    w = torch.randn(W, generator=g)
    xs = x.clone().to(device)
    out = latent.stream_add_norm(xs, y.to(device), None, w.to(device), 1e-5, torch.float32, y2=y2.to(device))
    want = x.to(F64) + y.to(F64) + y2.to(F64)
    close(xs, want, 1e-5)
    close(out, orc.rms_unit(want, 1e-5) * w.to(F64), 2e-5)


def paged(seq_lens, G, dk, dv, bs, dtype, device, g):
    """Scattered block tables for the given sequences in a pool with spare pages."""
    nb = [-(-n // bs) for n in seq_lens]
    perm = torch.randperm(sum(nb) + 5, generator=g) + 1
    bt = torch.zeros(len(seq_lens), max(nb), dtype=I32)
    at = 0
    for i, n in enumerate(nb):
        bt[i, :n] = perm[at:at + n].to(I32)
        at += n
    kc = torch.zeros(sum(nb) + 7, G, bs, dk, dtype=dtype, device=device)
    vc = torch.zeros(sum(nb) + 7, G, bs, dv, dtype=dtype, device=device)
    return bt, kc, vc


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("geom", [(6, 2, 8, 12, 6), (2, 2, 12, 8, 12), (3, 1, 10, 6, 0), (4, 4, 64, 64, 32), (9, 1, 16, 24, 8)])
def test_full_width_norm_rotary_and_cache_write(device, dtype, geom):
    """q / k normed over the whole projection, half-split rotation of the first dims, K / V rows at scattered
    slots, a row that is not written."""
    H, G, dk, dv, rd = geom
    g = torch.Generator().manual_seed(5)
    T, bs = 11, 4
    row = torch.randn(T, (H + G) * dk + G * dv + 9, generator=g).to(dtype)
    qw, kw = torch.randn(H * dk, generator=g), torch.randn(G * dk, generator=g)
    pos = torch.randint(0, 200, (T,), generator=g).to(I32)
    slots = (torch.randperm(40, generator=g)[:T]).to(I32)
    slots[4] = -1
    rot = {"dims": rd, "base": 100.0, "scaling": RAMP}
    cs = ops.rope_cos_sin(rd, 256, 100.0, RAMP).to(device) if rd else None
    rf = row.to(F64)
    q = (orc.rms_unit(rf[:, :H * dk], 1e-5) * qw.to(F64)).view(T, H, dk)
    k = (orc.rms_unit(rf[:, H * dk:(H + G) * dk], 1e-5) * kw.to(F64)).view(T, G, dk)
    if rd:
        cos, sin = orc.yarn_tables(rot, 256)
        q, k = orc.rotate_half(q, cos[pos.long()], sin[pos.long()]), orc.rotate_half(k, cos[pos.long()], sin[pos.long()])
    kc = torch.zeros(10, G, bs, dk, dtype=dtype, device=device)
    vc = torch.zeros(10, G, bs, dv, dtype=dtype, device=device)
    buf = row.clone().to(device)
    mix.qknorm_rope_cache(buf, pos.to(device), slots.to(device), qw.to(device), kw.to(device), 1e-5, cs, H, G, dk, dv, kc, vc,
                          span="full", layout="half")
    tol = 3e-5 if dtype == torch.float32 else 0.06
    close(buf[:, :H * dk], q.reshape(T, -1), tol * max(1.0, q.abs().max().item()))
    assert torch.equal(buf[:, H * dk:].cpu(), row[:, H * dk:])                  # everything but q untouched
    for t in range(T):
        s = int(slots[t])
        if s < 0:
            continue
        close(kc[s // bs, :, s % bs], k[t], tol * max(1.0, k.abs().max().item()))
        assert torch.equal(vc[s // bs, :, s % bs].cpu().reshape(-1), row[t, (H + G) * dk:(H + G) * dk + G * dv])
    assert kc.float().abs().sum(dim=(1, 3)).flatten().count_nonzero().item() == T - 1     # the skipped row wrote nothing


ATT_GEOMS = [(6, 2, 8, 12), (2, 2, 12, 8), (3, 1, 10, 6), (8, 2, 40, 72), (9, 1, 16, 24), (4, 2, 64, 64)]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("geom", ATT_GEOMS)
def test_attention_with_cap_and_sink(device, dtype, geom):
    """Rows over scattered pages against the oracle: a key made to stand out for one head 250 positions
    back, at page borders and at positions 0 and 1; sinks from negligible to dominating; a cap that
    saturates the standout score; decode rows and prompt rows (portions on top of cached keys)."""
    H, G, dk, dv = geom
    g = torch.Generator().manual_seed(6)
    n, bs = 300, 16
    q = torch.randn(n, H, dk, generator=g).to(dtype)
    k = torch.randn(n, G, dk, generator=g).to(dtype)
    v = torch.randn(n, G, dv, generator=g).to(dtype)
    rows = [299, 298, 297, 270, 17, 16, 15, 1, 0]
    targets = {299: 49, 298: 48, 297: 47, 270: 0, 17: 1, 16: 16, 15: 15}          # query row -> key it must find
    for i, (r, j) in enumerate(targets.items()):
        h = i % H
        q[r, h] = k[j, h // (H // G)] * (6.0 if i % 2 else 1.5)                   # scores of ~6 |k|^2: beyond the cap, or within it
    sink = torch.linspace(-6.0, 9.0, H)
    scale, cap = 0.3, 7.0
    want = orc.sink_attention_core(q.to(F64), k.to(F64), v.to(F64), scale, cap, sink.to(F64))
    bt, kc, vc = paged([n], G, dk, dv, bs, dtype, device, g)
    for j in range(n):
        b = int(bt[0, j // bs])
        kc[b, :, j % bs], vc[b, :, j % bs] = k[j].to(device), v[j].to(device)
    tol = 3e-5 if dtype == torch.float32 else 0.03
    pos = torch.tensor(rows, dtype=I32, device=device)
    qd = q[rows].reshape(len(rows), H * dk).to(device)
    gate = torch.randn(len(rows), H * dv, generator=g).to(dtype)
    got = mix.masked_attn_rows(qd, kc, vc, bt.repeat(len(rows), 1).to(device), None, pos, H, G, scale, 0, gate.to(device),
                               softcap=cap, sinks=sink.to(device))
    close(got, want[rows].reshape(len(rows), -1) * torch.sigmoid(gate.to(F64)), tol * max(1.0, want.abs().max().item()))
    # a portion of 41 rows on top of 259 cached keys, through cu_seqlens
    p0 = 259
    cu = torch.tensor([0, n - p0], dtype=I32, device=device)
    got = mix.masked_attn_rows(q[p0:].reshape(n - p0, H * dk).to(device), kc, vc, bt.to(device), cu,
                               torch.arange(p0, n, dtype=I32, device=device), H, G, scale, 0, None, softcap=cap,
                               sinks=sink.to(device))
    close(got, want[p0:].reshape(n - p0, -1), tol * max(1.0, want.abs().max().item()))
    # the sink alone: the denominator grows, the output shrinks by exactly that factor
    no_sink = orc.sink_attention_core(q.to(F64), k.to(F64), v.to(F64), scale, cap, None)
    assert (want[299, H - 1].abs().sum() < 0.7 * no_sink[299, H - 1].abs().sum())


@pytest.mark.gpu
@pytest.mark.parametrize("hd,H,G", [(64, 4, 2), (128, 8, 2)])
def test_mfma_prompt_attention_with_cap_and_sink(hd, H, G):
    """The MFMA prompt kernel with soft cap, sinks and gate against the oracle: two portions, one on top of
    cached keys that end inside a 64-key tile, rows past the 128-row tile border."""
    g = torch.Generator().manual_seed(8)
    dev, bs = "cuda", 16
    lens, cached = [200, 90], [150, 0]
    sink = torch.linspace(-3.0, 6.0, H)
    scale, cap = hd ** -0.5, 5.0
    bt, kc, vc = paged(lens, G, hd, hd, bs, torch.bfloat16, dev, g)
    qs, wants, gates = [], [], []
    for i, (n, c) in enumerate(zip(lens, cached)):
        q = (torch.randn(n, H, hd, generator=g) * 1.5).bfloat16()
        k, v = (torch.randn(n, G, hd, generator=g) * 1.5).bfloat16(), torch.randn(n, G, hd, generator=g).bfloat16()
        q[n - 1, 0] = k[3, 0] * 4                        # a far key beyond the cap
        for j in range(n):
            b = int(bt[i, j // bs])
            kc[b, :, j % bs], vc[b, :, j % bs] = k[j].to(dev), v[j].to(dev)
        gate = torch.randn(n - c, H * hd, generator=g).bfloat16()
        w = orc.sink_attention_core(q.to(F64), k.to(F64), v.to(F64), scale, cap, sink.to(F64))[c:].reshape(n - c, -1)
        wants.append(w * torch.sigmoid(gate.to(F64)))
        qs.append(q[c:].reshape(n - c, -1))
        gates.append(gate)
    cu = torch.tensor([0, lens[0] - cached[0], lens[0] - cached[0] + lens[1] - cached[1]], dtype=I32, device=dev)
    got = mix.paged_prefill_masked(torch.cat(qs, 0).to(dev), kc, vc, bt.to(dev), cu, torch.tensor(lens, dtype=I32, device=dev),
                                   H, G, scale, 0, torch.cat(gates, 0).to(dev), softcap=cap, sinks=sink.to(dev))
    close(got, torch.cat(wants, 0), 0.03)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("T,E,top", [(5, 6, 3), (70, 6, 2), (9, 4, 1), (40, 3, 3), (3, 70, 8), (300, 12, 4)])
def test_routing_by_the_largest_logits(device, T, E, top):
    """The `top` largest logits (bias included), weights = softmax over those alone, also when they lie far
    below zero or far apart; ties go to the lowest index."""
    g = torch.Generator().manual_seed(7)
    z = torch.randn(T, E, generator=g) * 3
    z[0] -= 200.0                                      # a softmax over all routes would still be fine; over none it is not
    z[1, 0] += 120.0                                   # one route far above the rest
    if T > 2 and E > 2:
        z[2, 1] = z[2, 2] = z[2].max() + 1.0           # a tie at the top
    idx, w = moe.moe_route(z.to(device), None, top, score="top_softmax")
    widx, ww = orc.route_top(z.to(F64), top)
    order = torch.sort(z.to(F64), dim=-1, descending=True, stable=True).indices[:, :top]
    assert torch.equal(idx.cpu().long(), order)
    assert torch.equal(torch.sort(idx.cpu().long(), -1).values, torch.sort(widx, -1).values)
    close(w, torch.softmax(torch.gather(z.to(F64), 1, order), -1), 1e-6)
    close(w.sum(-1), torch.ones(T, dtype=F64), 1e-6)


# ----------------------------------------------------------------------------------- the model
@pytest.mark.parametrize("device", DEVICES)
def test_layer_streams_match_oracle(device):
    eng = engine(small_cfg(), device)
    t = toks(19, 1)
    runs = eng.model_cfg.layer_runs
    assert runs == [0, 1, 2, 3, 1, 2, 3, 4]
    eng.model.capture_layers = tuple(range(len(runs)))
    got = eng.feed([("a", t, list(range(len(t))))], ["a"])[0]
    eng.model.capture_layers = ()
    want, streams = oracle_logits(eng, t, True)
    for r in range(len(runs)):
        close(eng.model.captured[r], streams[r], 2e-4 * max(1.0, streams[r].abs().max().item()))
    close(got, want, 3e-4)


VARIANTS = {
    "base": {},
    "no_loop": {"loop_times": 1},
    "loop3_first": {"loop_start": 0, "loop_stop": 1, "loop_times": 3},
    "loop_all": {"loop_start": 0, "loop_stop": 5, "loop_times": 2},
    "recurrent_only": {"layers": [small_cfg().layers[i] for i in (0, 2, 4)], "loop_start": 1, "loop_stop": 3},
    "attention_only": {"layers": [small_cfg().layers[i] for i in (1, 3)], "loop_start": 0, "loop_stop": 1},
    "ones": {"layers": [LayerSpec("delta", DeltaSpec(1, 1, 1, 1, 1), experts(1, 1, 1)),
                        LayerSpec("parallel", ParallelSpec(left(1, 1, 2, 1, 1.0, 2, cap=0.0), MlstmSpec(1, 1, 1, 1.0)), None),
                        LayerSpec("wkv", WkvSpec(1, 1, 1), experts(2, 2, 3))], "loop_times": 1},
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("variant", list(VARIANTS))
def test_whole_decode_and_portions_match_oracle(device, variant):
    """Whole prompt, token by token, and portions of several sizes (down to two tokens, across pages):
    all equal the oracle; other layer orders, loop spans and sizes of one too."""
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
    else:
        # bf16: one expert choice that flips on a close call moves a whole row, so rows are judged by their median
        for k in seqs:
            assert (torch.cat(got[k], 0) - want[k]).abs().amax(1).median().item() < 0.25


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_and_long_decoding(device):
    eng = engine(small_cfg(), device, max_len=256)
    t = toks(140, 5)
    want = oracle_logits(eng, t)
    close(eng.feed([("one", t[:1], [0])], ["one"])[0], want[:1], 2e-4)            # a sequence of one token
    close(eng.feed([("two", t[:2], [0, 1])], ["two"])[0], want[:2], 2e-4)
    got = feed_all(eng, "x", t, [3])                                              # 137 single-token steps
    close(got, want, 5e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_attention_branch_finds_a_far_key_through_the_model(device):
    """One layer, attention beside the memory, sharp scores: the last token's query is made to match one key
    hundreds of positions back, in prompt portions and in decoding; the oracle agrees only if rotation,
    pages and the sink are right at that distance."""
    cfg = LofuvikConfig(name="t", vocab_size=53, hidden_size=16, layers=[
        LayerSpec("parallel", ParallelSpec(left(2, 1, 8, 8, 3.0, 4, cap=50.0), MlstmSpec(1, 4, 4, 6.0)), None)],
        norm_eps=1e-5, max_position=512)
    eng = engine(cfg, device, max_len=400, num_blocks=120)
    t = toks(330, 8)
    want = oracle_logits(eng, t)
    got = torch.cat([eng.feed([("a", t[:257], list(range(257)))])[0], feed_all(eng, "a", t[257:], [2, 40])], 0)
    close(got, want, 5e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(device):
    eng = engine(small_cfg(), device, max_len=128)
    prompts = [toks(9, 20), toks(17, 21), toks(3, 22)]
    reqs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    assert eng.scheduler.radix is None                   # state-carrying models never resume from shared pages
    P = {k: v.to(F64) for k, v in params(eng.model).items()}
    cd = config_dict(eng.model_cfg)
    for p, r in zip(prompts, reqs):
        seq = list(p)
        for tok in r.output:
            lg = orc.forward(cd, P, seq)[-1]
            top2 = torch.topk(lg, 2).values
            assert tok == int(lg.argmax()) or (top2[0] - top2[1]) < 1e-3
            seq.append(tok)
    assert eng.pool.num_used == 0 and eng.state_pool.num_free == 4


@pytest.mark.gpu
def test_graph_decode_equals_eager_decode():
    """Decode steps replayed as hipGraphs (state slots in the staging image, padded rows on the reserved
    slot) produce the tokens of the eager engine; replays follow each other with eager prompt steps
    between them."""
    cfg = small_cfg()
    eager, graph = engine(cfg, "cuda", max_len=128), engine(cfg, "cuda", max_len=128, graphs=True)
    graph.model.copy_from(eager.model)
    prompts = [toks(9, 60), toks(17, 61), toks(3, 62)]
    sp = SamplingParams(max_tokens=14, temperature=0.0, ignore_eos=True)
    want = [r.output for r in eager.generate(prompts, sp)]
    for _ in range(2):                                       # a second batch reuses slots and replays again
        assert [r.output for r in graph.generate(prompts, sp)] == want
    assert graph.runner.graphs is not None and graph.runner.graphs.captured
    assert graph.state_pool.num_free == 4 and graph.pool.num_used == 0


@pytest.mark.gpu
def test_mfma_prompt_path_in_the_model(monkeypatch):
    """Attention branches whose bf16 heads are 64 / 128 wide take the MFMA prompt kernel: same logits as the
    row-wise kernel on the same engine (portions on top of cached tokens, two prompts in one step); no
    experts, so nothing can flip a routing decision."""
    cfg = LofuvikConfig(name="t", vocab_size=53, hidden_size=64, layers=[
        LayerSpec("parallel", ParallelSpec(left(4, 2, 64, 64, 0.125, 32), MlstmSpec(2, 16, 16, 8.0)), None),
        LayerSpec("delta", DeltaSpec(2, 1, 16, 16, 4), None),
        LayerSpec("parallel", ParallelSpec(left(2, 1, 128, 128, 0.09, 128, cap=20.0, scaling=None), MlstmSpec(1, 8, 32, 8.0)), None),
    ], max_position=512)
    a, b = toks(200, 70), toks(90, 71)

    def run():
        eng = engine(cfg, "cuda", dtype=torch.bfloat16, num_blocks=64, bs=16, max_len=512)
        out = [eng.feed([("a", a[:150], list(range(150)))]),
               eng.feed([("a", a[150:], list(range(50))), ("b", b, list(range(90)))], ["a", "b"])]
        return torch.cat([o for step in out for o in step], 0)

    assert mix.masked_prefill_available()
    fast = run()
    monkeypatch.setattr(mix, "MASKED_PREFILL", False)
    slow = run()
    close(fast, slow, 0.06 * max(1.0, slow.abs().max().item()))


def test_preempted_sequence_recomputes_its_state():
    """A pool too small for two growing sequences: one is preempted, gives its slot back, and is
    recomputed from position 0 — its tokens equal the undisturbed run."""
    cfg = small_cfg()
    big = engine(cfg, "cpu", max_len=128)
    ref = big.generate([toks(20, 30), toks(22, 31)], SamplingParams(max_tokens=20, temperature=0.0, ignore_eos=True))
    tight = engine(cfg, "cpu", num_blocks=18, bs=4, max_len=128)
    tight.model.copy_from(big.model)
    got = tight.generate([toks(20, 30), toks(22, 31)], SamplingParams(max_tokens=20, temperature=0.0, ignore_eos=True))
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
    for L in src.model.layers:                                      # ... also those the model keeps in fp32
        for _k, t in L.named():
            t.copy_(t.to(torch.bfloat16).to(t.dtype))
    ck = str(tmp_path / "model")
    write_checkpoint(src, ck)
    cfg = get_config(ck)
    assert isinstance(cfg, LofuvikConfig) and cfg.layer_runs == [0, 1, 2, 3, 1, 2, 3, 4]
    eng = LLMEngine(EngineConfig(model=ck, device="cpu", dtype=torch.float32, block_size=4, num_blocks=64, max_num_seqs=4,
                                 max_model_len=128, max_num_batched_tokens=128, use_graphs=False, token_align=0))
    assert eng.model_cfg.layers[2].mixer.decay_rank == 5              # from the tensor's shape
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


def test_preset_and_registry():
    cfg = get_config("lofuvik-tiny")
    assert isinstance(cfg, LofuvikConfig) and cfg.layer_runs == [0, 1, 0, 1, 2, 3]
    eng = LLMEngine(EngineConfig(model="lofuvik-tiny", device="cpu", dtype=torch.float32, num_blocks=32, max_num_seqs=2,
                                 max_model_len=128, use_graphs=False))
    assert type(eng.model).__name__ == "LofuvikModel" and eng.state_pool is not None
    r = eng.generate([toks(5, 1, 512)], SamplingParams(max_tokens=4, temperature=0.0, ignore_eos=True))
    assert len(r[0].output) == 4


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_kernels_match_the_reference_ops_on_a_prompt_batch(dtype):
    """The HIP kernels against the CPU reference ops through the same engine code, over a batch of
    portions and decode rows: fp32 within rounding at every position; bf16 at the typical position
    (one expert choice that flips on a close call moves a whole row, so rows are judged by their median)."""
    cfg = small_cfg()
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
