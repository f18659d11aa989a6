"""Time of the matrix-state mixer kernels (dgi.ops.linrec and the attention kernels' cap / sink options) beside the
like kernels of the other state-carrying family, at the layer shapes of a 1B-class decoder: a decode step of 32 rows
at position 2000 and a prompt step of 2 x 2048 rows.  One JSON line per kernel: time, the bytes it has to move (or
the multiply-adds of a recurrence), achieved TB/s (GFLOP/s).  Each kernel's name is printed before it runs.

    python scripts/linrec_bench.py [--width 2048] [--iters 20]
"""
import argparse
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import torch

from dgi import ops
from dgi.ops import latent, linrec, mix, recur

ap = argparse.ArgumentParser()
ap.add_argument("--width", type=int, default=2048)
ap.add_argument("--iters", type=int, default=20)
ap.add_argument("--only", default="", help="comma separated kernel groups: scan, rows, prep, attn")
args = ap.parse_args()
W, IT = args.width, args.iters
dev = "cuda"
bf, f32, i32 = torch.bfloat16, torch.float32, torch.int32
only = set(args.only.split(",")) if args.only else None


def timed(name, fn, work, unit="TB/s"):
    print(f"# {name}", flush=True)
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(IT):
        fn()
    torch.cuda.synchronize()
    us = (time.perf_counter() - t0) / IT * 1e6
    rate = work / us / 1e6 if unit == "TB/s" else work / us / 1e3
    print(json.dumps({"kernel": name, "us": round(us, 1), "work": work, "rate": round(rate, 2), "unit": unit}), flush=True)


def seqs(n_seq, rows, start):
    pos = torch.arange(start, start + rows, dtype=i32).repeat(n_seq)
    rs = torch.arange(n_seq, dtype=i32).repeat_interleave(rows)
    r0 = torch.arange(0, n_seq * rows + 1, rows, dtype=i32)
    sl = torch.arange(1, n_seq + 1, dtype=i32)
    return pos.to(dev), rs.to(dev), r0.to(dev), sl.to(dev)


STEPS = {"decode": (32, 1, 2000), "prompt": (2, 2048, 0)}        # sequences, rows each, first position
H, D = W // 64, 64                                               # recurrent heads of 64 x 64

if only is None or "scan" in only:
    for step, (ns, rows, start) in STEPS.items():
        T = ns * rows
        pos, rs, r0, sl = seqs(ns, rows, start)
        state = torch.zeros(33, H, D, D, device=dev)
        nrm, mx = torch.zeros(33, H, D, device=dev), torch.zeros(33, H, device=dev)
        u = torch.randn(T, 4 * H * D, device=dev, dtype=bf)
        q, k, v = u[:, :H * D], u[:, H * D:2 * H * D], u[:, 2 * H * D:3 * H * D]
        gates = torch.randn(T, 2 * H, device=dev)
        sb = 2 * ns * H * D * D * 4                               # state in + out
        fl = 2 * T * H * D * D                                    # multiply-adds of one pass over S, x2 flops
        wr, w0, bonus = torch.randn(T, H * D, device=dev), torch.randn(H * D, device=dev) - 1.5, torch.randn(H * D, device=dev)
        timed(f"linear_scan wkv {step}", lambda: linrec.wkv_scan(q, k, v, wr, w0, bonus, state, pos, r0, sl, H, D),
              sb if rows == 1 else 2 * fl, "TB/s" if rows == 1 else "GFLOP/s")
        qf = torch.randn(T, 2 * (H // 2) * D + H * D, device=dev)
        c1 = (H // 2) * D
        al, dtb = torch.randn(H, device=dev) - 1, torch.randn(H, device=dev) - 1
        timed(f"linear_scan delta {step}",
              lambda: linrec.delta_scan(qf[:, :c1], qf[:, c1:2 * c1], qf[:, 2 * c1:], gates[:, :H], gates[:, H:], al, dtb, state,
                                        pos, r0, sl, H, H // 2, D, D), sb if rows == 1 else 2 * fl, "TB/s" if rows == 1 else "GFLOP/s")
        timed(f"linear_scan mlstm {step}",
              lambda: linrec.mlstm_scan(q, k, v, gates[:, :H], gates[:, H:], 15.0, state, nrm, mx, pos, r0, sl, H, D, D),
              sb if rows == 1 else 2 * fl, "TB/s" if rows == 1 else "GFLOP/s")
        # the like kernel: the Mamba-2 scan of a layer of the same width (inner 2 W, heads of 64, state 128, 8 groups)
        mh, mv, N, G = 2 * W // 64, 64, 128, 8
        xbc = torch.randn(T, mh * mv + 2 * G * N, device=dev)
        dtr = torch.randn(T, mh, device=dev, dtype=bf)
        mstate = torch.zeros(33, mh, mv, N, device=dev)
        z1 = torch.randn(mh, device=dev)
        timed(f"ssm_scan {step}", lambda: recur.ssm_scan(xbc, dtr, z1, z1 - 1, z1, mstate, pos, r0, sl, mh, mv, N, G, chunked=False),
              2 * ns * mh * mv * N * 4 if rows == 1 else 2 * 2 * T * mh * mv * N, "TB/s" if rows == 1 else "GFLOP/s")

if only is None or "rows" in only:
    T = 4096
    pos, rs, r0, sl = seqs(2, 2048, 0)
    y = torch.randn(T, W, device=dev)
    zz = torch.randn(T, 2 * W, device=dev, dtype=bf)
    wn = torch.randn(W, device=dev)
    timed("head_norm_gate", lambda: linrec.head_norm_gate(y, zz[:, W:], wn, H, 1e-6, "silu", bf), T * W * (4 + 2 + 2))
    y2, z2, w2 = torch.randn(T, 2 * W, device=dev), torch.randn(T, 2 * W, device=dev, dtype=bf), torch.randn(2 * W, device=dev)
    timed("gated_group_norm (like)", lambda: recur.gated_group_norm(y2, z2, w2, 1, 1e-6, bf), T * 2 * W * (4 + 2 + 2))
    h = torch.randn(T, W, device=dev, dtype=bf)
    mu = torch.rand(5, W, device=dev)
    tail = torch.zeros(33, W, device=dev)
    timed("token_shift", lambda: linrec.token_shift(h, mu, tail, pos, rs, r0, sl, bf), T * W * (2 + 5 * 2))
    h32, cw, ctail = torch.randn(T, W, device=dev), torch.randn(W, 4, device=dev), torch.zeros(33, 3, W, device=dev)
    timed("causal_conv (like)", lambda: recur.causal_conv(h32, cw, None, ctail, pos, rs, r0, sl, act=0, residual=True, out_dtype=bf),
          T * W * (4 + 2))
    a, b = torch.randn(T, W, device=dev, dtype=bf), torch.randn(T, W, device=dev, dtype=bf)
    timed("rms_pair_mean", lambda: linrec.rms_pair_mean(a, b, wn, wn, 1e-6), T * W * (2 + 2 + 4))
    x = torch.randn(T, W, device=dev)
    timed("stream_add_norm two addends", lambda: latent.stream_add_norm(x, y, None, wn, 1e-6, bf, y2=a), T * W * (4 + 4 + 4 + 2 + 2))
    timed("stream_add_norm (like)", lambda: latent.stream_add_norm(x, a, None, wn, 1e-6, bf), T * W * (4 + 4 + 2 + 2))

AH, AG, AD = max(2, W // 128), max(1, W // 256), 128             # attention 16 / 8 heads of 128 at W = 2048
bs = 16
if only is None or "prep" in only:
    T = 4096
    pos, rs, r0, sl = seqs(2, 2048, 0)
    pages = 2 * 2048 // bs + 1
    kc = torch.zeros(pages, AG, bs, AD, device=dev, dtype=bf)
    vc = torch.zeros(pages, AG, bs, AD, device=dev, dtype=bf)
    slots = (torch.arange(T, dtype=i32) + bs).to(dev)
    row = torch.randn(T, (2 * AH + 2 * AG) * AD, device=dev, dtype=bf)
    cs = ops.rope_cos_sin(AD, 4096, 500000.0, {"factor": 8.0, "original": 8192, "fast": 32.0, "slow": 1.0}, device=dev)
    qw, kw = torch.randn(AH * AD, device=dev), torch.randn(AG * AD, device=dev)
    byt = T * ((AH + AG) * AD * 2 * 2 + AG * AD * 2 * 2)
    timed("qk_prep full-width norm, half rotary", lambda: mix.qknorm_rope_cache(row, pos, slots, qw, kw, 1e-6, cs, AH, AG, AD, AD, kc, vc,
                                                                                 span="full", layout="half"), byt)
    timed("qknorm_rope_cache per head, interleaved (like)",
          lambda: mix.qknorm_rope_cache(row, pos, slots, qw[:AD], kw[:AD], 1e-6, cs, AH, AG, AD, AD, kc, vc), byt)

if only is None or "attn" in only:
    ctx, nseq = 2048, 32
    per = ctx // bs
    pages = nseq * per + 1
    kc = torch.randn(pages, AG, bs, AD, device=dev, dtype=bf)
    vc = torch.randn(pages, AG, bs, AD, device=dev, dtype=bf)
    bt = (torch.arange(nseq * per, dtype=i32).view(nseq, per) + 1).to(dev)
    sink = torch.randn(AH, device=dev)
    q = torch.randn(nseq, 2 * AH * AD, device=dev, dtype=bf)
    dpos = torch.full((nseq,), 1999, dtype=i32, device=dev)
    kvb = nseq * 2000 * AG * AD * 2 * 2
    timed("masked_attn_rows decode, cap + sink + gate",
          lambda: mix.masked_attn_rows(q, kc, vc, bt, None, dpos, AH, AG, 0.09, 0, q[:, AH * AD:], softcap=30.0, sinks=sink), kvb)
    timed("masked_attn_rows decode, gate (like)", lambda: mix.masked_attn_rows(q, kc, vc, bt, None, dpos, AH, AG, 0.09, 0, q[:, AH * AD:]), kvb)
    T = 2 * 2048
    qp = torch.randn(T, 2 * AH * AD, device=dev, dtype=bf)
    cu = torch.tensor([0, 2048, 4096], dtype=i32, device=dev)
    cl = torch.tensor([2048, 2048], dtype=i32, device=dev)
    fl = 2 * 2 * AH * AD * 2048 * 2048                            # causal: half of 2 x (QK^T + PV)
    tl = ops.prefill_tiles(cu.tolist(), context_lens=cl.tolist(), tile=128)
    tiles = torch.tensor(tl, dtype=i32, device=dev)
    timed("paged_prefill_masked, cap + sink + gate",
          lambda: mix.paged_prefill_masked(qp, kc, vc, bt[:2], cu, cl, AH, AG, 0.09, 0, qp[:, AH * AD:], tiles=tiles, softcap=30.0,
                                           sinks=sink), fl, "GFLOP/s")
    timed("paged_prefill_masked, gate (like)", lambda: mix.paged_prefill_masked(qp, kc, vc, bt[:2], cu, cl, AH, AG, 0.09, 0, qp[:, AH * AD:],
                                                                                 tiles=tiles), fl, "GFLOP/s")
