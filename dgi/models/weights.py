"""Checkpoint loading for the native runtime: HF safetensors -> dgi weight layout.

The reference serves real checkpoints through ``AutoModelForCausalLM.from_pretrained``
(worker/engines/llm.py:14-41) and loads a layer range per pipeline worker
(worker/distributed/model_shard.py:61-148).  Here the dgi model (any layer range,
any tensor-parallel rank) reads exactly the bytes it owns:

* shards are opened with ``safetensors.safe_open`` (memory-mapped, nothing
  is unpickled) and read tensor by tensor through ``get_slice``, so a
  pipeline stage touches only its own layers and a TP rank only its rows /
  columns of each projection — there is never a full CPU copy of the model;
* each slice lands directly in its place inside the fused device weights
  (q|k|v -> ``qkv``, gate|up -> ``gate_up``; GLM's already fused
  ``gate_up_proj`` is split per TP rank);
* tensors are cast to the model dtype on the way (fp32 / fp16 checkpoints
  load into bf16 weights).

``resolve_checkpoint`` finds a local checkpoint for a model id: an explicit
path, a directory given as the model id, or an offline Hugging Face cache
snapshot (``local_files_only`` — no network is ever used).
"""
from __future__ import annotations

import json
import os
from typing import Iterable, Optional

import torch


def _has_safetensors(d: str) -> bool:
    return os.path.isdir(d) and any(f.endswith(".safetensors") for f in os.listdir(d))


def resolve_checkpoint(model_id: Optional[str], model_path: Optional[str] = None) -> Optional[str]:
    """Directory holding ``config.json`` + ``*.safetensors`` for this model, or None
    (None means: random-init weights of the preset architecture)."""
    for cand in (model_path, model_id):
        if cand and os.path.isdir(cand) and _has_safetensors(cand):
            return cand
    if model_path:
        raise FileNotFoundError(f"model_path {model_path!r} has no *.safetensors files")
    if model_id and "/" in model_id and not os.path.exists(model_id):
        try:  # offline HF cache lookup only
            from huggingface_hub import snapshot_download

            d = snapshot_download(model_id, local_files_only=True, allow_patterns=["*.json", "*.safetensors"])
            if _has_safetensors(d):
                return d
        except Exception:
            return None
    return None


class CheckpointReader:
    """Name -> shard map over the safetensors files of one checkpoint directory."""

    def __init__(self, path: str):
        from safetensors import safe_open

        self.path = path
        self._open = safe_open
        idx = os.path.join(path, "model.safetensors.index.json")
        self.where: dict[str, str] = {}
        if os.path.exists(idx):
            with open(idx) as f:
                for name, fn in json.load(f)["weight_map"].items():
                    self.where[name] = os.path.join(path, fn)
        else:
            for fn in sorted(os.listdir(path)):
                if fn.endswith(".safetensors"):
                    full = os.path.join(path, fn)
                    with safe_open(full, framework="pt", device="cpu") as f:
                        for name in f.keys():
                            self.where[name] = full
        self._handles: dict[str, object] = {}
        self.bytes_read = 0

    def __contains__(self, name: str) -> bool:
        return name in self.where

    def names(self) -> Iterable[str]:
        return self.where.keys()

    def _h(self, name: str):
        fn = self.where[name]
        h = self._handles.get(fn)
        if h is None:
            h = self._handles[fn] = self._open(fn, framework="pt", device="cpu")
        return h

    def read(self, name: str, rows: Optional[tuple] = None, cols: Optional[tuple] = None) -> torch.Tensor:
        """Tensor ``name`` (optionally rows [a, b) / cols [a, b) only) as a CPU tensor."""
        sl = self._h(name).get_slice(name)
        if rows is None and cols is None:
            t = sl[:] if len(sl.get_shape()) else self._h(name).get_tensor(name)     # 0-dim: no slicing
        elif cols is None:
            t = sl[rows[0]:rows[1]]
        elif rows is None:
            t = sl[:, cols[0]:cols[1]]
        else:
            t = sl[rows[0]:rows[1], cols[0]:cols[1]]
        self.bytes_read += t.numel() * t.element_size()
        return t

    def close(self) -> None:
        self._handles.clear()


def _put(dst: torch.Tensor, src: torch.Tensor) -> None:
    if tuple(dst.shape) != tuple(src.shape):
        raise ValueError(f"checkpoint tensor shape {tuple(src.shape)} != model slot {tuple(dst.shape)}")
    dst.copy_(src.to(dst.dtype), non_blocking=False)


def load_checkpoint(model, path: str, tp_rank: int = 0, tp: int = 1) -> dict:
    """Fill a ``LlamaModel`` (created with ``init="empty"``) from an HF checkpoint.

    ``model.cfg`` is the LOCAL config (per-rank heads / intermediate for TP);
    ``full`` is the checkpoint's.  Returns {"tensors": n, "bytes": b}."""
    model.norms_folded = False
    rd = CheckpointReader(path)
    c = model.cfg
    full = getattr(model, "full_cfg", c)
    hd = full.head_dim
    ql, kl = c.num_heads * hd, c.num_kv_heads * hd
    Il = c.intermediate_size
    q_rows = (tp_rank * ql, (tp_rank + 1) * ql)
    kv_rows = (tp_rank * kl, (tp_rank + 1) * kl)
    i_rows = (tp_rank * Il, (tp_rank + 1) * Il)
    n = 0
    for i, li in enumerate(range(model.layer_start, model.layer_end)):
        L = model.layers[i]
        p = f"model.layers.{li}."
        a = p + "self_attn."
        _put(L.qkv[:ql], rd.read(a + "q_proj.weight", rows=q_rows))
        _put(L.qkv[ql:ql + kl], rd.read(a + "k_proj.weight", rows=kv_rows))
        _put(L.qkv[ql + kl:], rd.read(a + "v_proj.weight", rows=kv_rows))
        n += 3
        if L.qkv_bias is not None:
            _put(L.qkv_bias[:ql], rd.read(a + "q_proj.bias", rows=q_rows))
            _put(L.qkv_bias[ql:ql + kl], rd.read(a + "k_proj.bias", rows=kv_rows))
            _put(L.qkv_bias[ql + kl:], rd.read(a + "v_proj.bias", rows=kv_rows))
            n += 3
        _put(L.o, rd.read(a + "o_proj.weight", cols=q_rows) if tp > 1 else rd.read(a + "o_proj.weight"))
        m = p + "mlp."
        if m + "gate_up_proj.weight" in rd:        # GLM-4: fused [gate; up]
            I = full.intermediate_size
            _put(L.gate_up[:Il], rd.read(m + "gate_up_proj.weight", rows=i_rows))
            _put(L.gate_up[Il:], rd.read(m + "gate_up_proj.weight", rows=(I + i_rows[0], I + i_rows[1])))
        else:
            _put(L.gate_up[:Il], rd.read(m + "gate_proj.weight", rows=i_rows))
            _put(L.gate_up[Il:], rd.read(m + "up_proj.weight", rows=i_rows))
        _put(L.down, rd.read(m + "down_proj.weight", cols=i_rows) if tp > 1 else rd.read(m + "down_proj.weight"))
        _put(L.in_norm, rd.read(p + "input_layernorm.weight"))
        _put(L.post_norm, rd.read(p + "post_attention_layernorm.weight"))
        n += 6
    if model.embed is not None:
        _put(model.embed, rd.read("model.embed_tokens.weight"))
        n += 1
    if model.has_head:
        _put(model.norm, rd.read("model.norm.weight"))
        n += 1
        if model.lm_head is not model.embed:
            if "lm_head.weight" in rd:
                _put(model.lm_head, rd.read("lm_head.weight"))
            else:   # tied checkpoint served by an untied slot (last stage without the embedding)
                _put(model.lm_head, rd.read("model.embed_tokens.weight"))
            n += 1
    out = {"tensors": n, "bytes": rd.bytes_read, "path": path}
    rd.close()
    return out


def load_bebovik_checkpoint(model, path: str) -> dict:
    """Fill a ``BebovikModel`` from the design's safetensors layout: ``embed`` / ``head``,
    norms as ``<name>`` (weight), ``<name>.b`` and the scalar ``<name>.alpha``, and per layer i
    ``l<i>.mix.{q,k,v,g,o}`` (stored [out, in]), ``l<i>.mix.{q,k}.norm``, ``l<i>.mlp.{gate,up,down}``,
    ``l<i>.ls1`` / ``ls2``.  q | k | v | g land in the fused projection weight and gate | up in the
    fused feed-forward weight; only the model's own layer range is read.  Norm parameters,
    layer scales and q/k norm weights are kept in fp32."""
    rd = CheckpointReader(path)
    n = 0

    def put(dst, name):
        nonlocal n
        src = rd.read(name)
        _put(dst, src.reshape(dst.shape) if src.numel() == dst.numel() and src.dim() != dst.dim() else src)
        n += 1

    def put_norm(norm, name):
        put(norm.w, name)
        put(norm.b, name + ".b")
        put(norm.alpha, name + ".alpha")

    for i, li in enumerate(range(model.layer_start, model.layer_end)):
        L = model.layers[i]
        m = L.spec.mixer
        p = f"l{li}."
        r = 0
        for key, rows in (("q", m.q_size), ("k", m.k_size), ("v", m.v_size), ("g", m.o_size if m.out_gate else 0)):
            if rows:
                put(L.qkvg[r:r + rows], p + "mix." + key)
            r += rows
        put(L.o, p + "mix.o")
        put(L.q_norm, p + "mix.q.norm")
        put(L.k_norm, p + "mix.k.norm")
        put_norm(L.norm1, p + "norm1")
        put_norm(L.norm1b, p + "norm1b")
        put(L.ls1, p + "ls1")
        if L.gate_up is not None:
            ff = L.spec.mlp.ff
            put(L.gate_up[:ff], p + "mlp.gate")
            put(L.gate_up[ff:], p + "mlp.up")
            put(L.down, p + "mlp.down")
            put_norm(L.norm2, p + "norm2")
            put_norm(L.norm2b, p + "norm2b")
            put(L.ls2, p + "ls2")
    if model.embed is not None:
        put(model.embed, "embed")
        put_norm(model.embed_norm, "embed.norm")
    if model.has_head:
        put(model.head, "head")
        put_norm(model.final_norm, "final.norm")
    out = {"tensors": n, "bytes": rd.bytes_read, "path": path}
    rd.close()
    return out


def tifepel_bias_rows(cfg, path: str) -> None:
    """Set every attention layer's ``bias_rows`` from the shape of its distance-bias table in the
    checkpoint (the configuration file gives only the distance at which the buckets end)."""
    rd = CheckpointReader(path)
    for i, l in enumerate(cfg.layers):
        if l.type == "attention" and l.mixer.bias_rows:
            l.mixer.bias_rows = int(rd._h(f"l{i}.mix.rel").get_slice(f"l{i}.mix.rel").get_shape()[0])
    rd.close()


def load_tifepel_checkpoint(model, path: str) -> dict:
    """Fill a ``TifepelModel`` from the design's safetensors layout: ``embed`` / ``bigram`` / ``pos`` /
    ``head`` / ``final.norm`` and per layer i ``l<i>.norm{1,2}``, ``l<i>.canon{1,2}``, ``l<i>.rg{1,2}``
    (+ ``.b``), ``l<i>.hc{1,2}.{in,out,mix}``, the mixer under ``l<i>.mix.`` (attention: q, k, v, rel, o;
    Mamba-2: in, conv, conv.b, dt_bias, A_log, D, norm, o) and the feed-forward under ``l<i>.mlp.``
    (router, correction, e<j>.{gate,up,down}, shared.{gate,up,down}).  q | k | v land in one fused
    weight, every expert's gate | up in one stacked tensor; norm weights, convolution taps, stream
    coefficients, the router and the scan's per-head constants stay fp32."""
    rd = CheckpointReader(path)
    n = 0

    def put(dst, name):
        nonlocal n
        src = rd.read(name)
        if src.dim() == dst.dim() and src.shape[0] < dst.shape[0] and src.shape[1:] == dst.shape[1:]:
            dst = dst[: src.shape[0]]        # a table the engine made longer than the checkpoint's
        _put(dst, src.reshape(dst.shape) if src.numel() == dst.numel() and src.dim() != dst.dim() else src)
        n += 1

    for i, L in enumerate(model.layers):
        p = f"l{i}."
        m, f = L.spec.mixer, L.spec.mlp
        for q in ("1", "2") if f is not None else ("1",):
            put(getattr(L, "norm" + q), p + "norm" + q)
            if getattr(L, "canon" + q) is not None:
                put(getattr(L, "canon" + q), p + "canon" + q)
            put(getattr(L, "rg" + q), p + "rg" + q)
            put(getattr(L, f"rg{q}_b"), f"{p}rg{q}.b")
            for k in ("in", "out", "mix"):
                put(getattr(L, f"hc{q}_{k}"), f"{p}hc{q}.{k}")
        if L.spec.type == "attention":
            r = 0
            for key, rows in (("q", m.q_size), ("k", m.k_size), ("v", m.v_size)):
                put(L.qkv[r:r + rows], p + "mix." + key)
                r += rows
            if L.rel is not None:
                put(L.rel, p + "mix.rel")
        else:
            for dst, key in ((L.in_proj, "in"), (L.conv, "conv"), (L.conv_b, "conv.b"), (L.dt_bias, "dt_bias"),
                             (L.a_log, "A_log"), (L.d_skip, "D"), (L.mnorm, "norm")):
                put(dst, p + "mix." + key)
        put(L.o, p + "mix.o")
        if f is not None:
            put(L.router, p + "mlp.router")
            put(L.correction, p + "mlp.correction")
            for e in range(f.experts):
                put(L.gate_up[e, : f.ff], f"{p}mlp.e{e}.gate")
                put(L.gate_up[e, f.ff:], f"{p}mlp.e{e}.up")
                put(L.down[e], f"{p}mlp.e{e}.down")
            if f.shared_ff:
                put(L.shared_gate_up[: f.shared_ff], p + "mlp.shared.gate")
                put(L.shared_gate_up[f.shared_ff:], p + "mlp.shared.up")
                put(L.shared_down, p + "mlp.shared.down")
    put(model.embed, "embed")
    if model.bigram is not None:
        put(model.bigram, "bigram")
    put(model.pos, "pos")
    put(model.head, "head")
    put(model.final_norm, "final.norm")
    out = {"tensors": n, "bytes": rd.bytes_read, "path": path}
    rd.close()
    return out


def load_depelix_checkpoint(model, path: str) -> dict:
    """Fill a ``DepelixModel`` from the design's safetensors layout: ``embed`` / ``bigram`` / ``side.embed`` /
    ``head`` / ``final.norm`` and per layer i ``l<i>.norm{1,2}``, the mixer under ``l<i>.mix.`` (dq, dq.norm, uq,
    dkv, dkv.norm — absent in a layer that reads another layer's latent — uk, uv, g, o), the feed-forward
    under ``l<i>.mlp.`` (dense: up, down; experts: router, e<j>.{gate,up,down}) and the token input
    ``l<i>.side.{gate,proj,norm}``.  dq | dkv | g land in one fused weight, every expert's gate | up in one
    stacked tensor, uk / uv as [heads, rows per head, kv_rank]; norm weights and the router stay fp32."""
    rd = CheckpointReader(path)
    n = 0

    def put(dst, name):
        nonlocal n
        src = rd.read(name)
        if tuple(src.shape) != tuple(dst.shape) and src.numel() != dst.numel():
            raise ValueError(f"{name}: checkpoint shape {tuple(src.shape)} does not fit {tuple(dst.shape)}")
        _put(dst, src.reshape(dst.shape))
        n += 1

    for i, L in enumerate(model.layers):
        p = f"l{i}."
        m, f = L.spec.mixer, L.spec.mlp
        put(L.norm1, p + "norm1")
        r = 0
        parts = [("dq", m.q_rank)] + ([("dkv", m.cache_dim)] if m.kv_from is None else []) + \
                ([("g", m.gate_rows)] if m.gate_rows else [])
        for key, rows in parts:
            put(L.in_proj[r:r + rows], p + "mix." + key)
            r += rows
        put(L.dq_norm, p + "mix.dq.norm")
        if m.kv_from is None:
            put(L.dkv_norm, p + "mix.dkv.norm")
        for dst, key in ((L.uq, "uq"), (L.uk, "uk"), (L.uv, "uv"), (L.o, "o")):
            put(dst, p + "mix." + key)
        if f is not None:
            put(L.norm2, p + "norm2")
            if f.kind == "dense":
                put(L.up, p + "mlp.up")
                put(L.down, p + "mlp.down")
            else:
                put(L.router, p + "mlp.router")
                for e in range(f.experts):
                    put(L.gate_up[e, : f.ff], f"{p}mlp.e{e}.gate")
                    put(L.gate_up[e, f.ff:], f"{p}mlp.e{e}.up")
                    put(L.down[e], f"{p}mlp.e{e}.down")
        if L.side_gate is not None:
            put(L.side_gate, p + "side.gate")
            put(L.side_proj, p + "side.proj")
            put(L.side_norm, p + "side.norm")
    put(model.embed, "embed")
    if model.bigram is not None:
        put(model.bigram, "bigram")
    if model.side_embed is not None:
        put(model.side_embed, "side.embed")
    put(model.head, "head")
    put(model.final_norm, "final.norm")
    out = {"tensors": n, "bytes": rd.bytes_read, "path": path}
    rd.close()
    return out


def lofuvik_checkpoint_shapes(cfg, path: str) -> None:
    """Sizes that only the checkpoint's tensor shapes give: the rank of every time-mixing layer's
    decay projection (rows of ``l<i>.mix.w1``)."""
    rd = CheckpointReader(path)
    for i, l in enumerate(cfg.layers):
        if l.type == "wkv":
            name = f"l{i}.mix.w1"
            l.mixer.decay_rank = int(rd._h(name).get_slice(name).get_shape()[0])
    rd.close()


def load_lofuvik_checkpoint(model, path: str) -> dict:
    """Fill a ``LofuvikModel`` from the design's safetensors layout: ``embed`` / ``head`` / ``final.norm`` and
    per layer i ``l<i>.norm1``, the feed-forward under ``l<i>.mlp.`` (router, router.b, e<j>.{gate,up,down})
    and the mixer under ``l<i>.mix.``: time mixing mu.{r,k,v,g,w}, r, k, v, g, w1, w2, w0, u, norm, o; delta
    rule q, k, v (each with ``.conv``), b, a, A_log, dt_bias, norm, g, o; the two-branch mixer left.{q, k, v,
    q.norm, k.norm, sink, g, o, out} and right.{q, k, v, g, o, norm, i, i.b, f, f.b, out}.  The router and
    the recurrence's gate projections land in one fp32 side projection (router | b | a, or router | i | f),
    a mixer's large projections in one fused weight, every expert's gate | up in one stacked tensor; norm
    weights, blends, taps, decay and gate parameters stay fp32."""
    rd = CheckpointReader(path)
    n = 0

    def put(dst, name):
        nonlocal n
        src = rd.read(name)
        if tuple(src.shape) != tuple(dst.shape) and src.numel() != dst.numel():
            raise ValueError(f"{name}: checkpoint shape {tuple(src.shape)} does not fit {tuple(dst.shape)}")
        _put(dst, src.reshape(dst.shape))
        n += 1

    def put_rows(dst, names):
        r = 0
        for name, rows in names:
            put(dst[r:r + rows], name)
            r += rows
        if r != dst.shape[0]:
            raise ValueError(f"{names[0][0]}...: {r} rows for a slot of {dst.shape[0]}")

    from dgi.models.lofuvik import SHIFT_BLENDS
    for i, L in enumerate(model.layers):
        p = f"l{i}."
        x = p + "mix."
        m, f = L.spec.mixer, L.spec.mlp
        put(L.norm1, p + "norm1")
        r0 = 0
        if f is not None:
            put(L.side[: f.routes], p + "mlp.router")
            put(L.side_b[: f.routes], p + "mlp.router.b")
            r0 = f.routes
            for e in range(f.experts):
                put(L.gate_up[e, : f.ff], f"{p}mlp.e{e}.gate")
                put(L.gate_up[e, f.ff:], f"{p}mlp.e{e}.up")
                put(L.down[e], f"{p}mlp.e{e}.down")
        if L.spec.type == "wkv":
            for j, s in enumerate(SHIFT_BLENDS):
                put(L.mu[j], x + "mu." + s)
            for j, s in enumerate(("r", "k", "v", "g")):
                put(L.rkvg[j], x + s)
            for dst, key in ((L.w1, "w1"), (L.w2, "w2"), (L.w0, "w0"), (L.bonus, "u"), (L.mnorm, "norm"), (L.o, "o")):
                put(dst, x + key)
        elif L.spec.type == "delta":
            H, qk = m.heads, m.qk_size
            put_rows(L.in_proj, [(x + "q", qk), (x + "k", qk), (x + "v", m.inner), (x + "g", m.inner)])
            put_rows(L.conv, [(x + "q.conv", qk), (x + "k.conv", qk), (x + "v.conv", m.inner)])
            put(L.side[r0: r0 + H], x + "b")
            put(L.side[r0 + H: r0 + 2 * H], x + "a")
            for dst, key in ((L.a_log, "A_log"), (L.dt_bias, "dt_bias"), (L.mnorm, "norm"), (L.o, "o")):
                put(dst, x + key)
        else:
            a, rr = m.left, m.right
            lf, rt = x + "left.", x + "right."
            put_rows(L.in_proj, [(lf + "q", a.q_size), (lf + "k", a.k_size), (lf + "v", a.v_size), (lf + "g", a.o_size),
                                 (rt + "q", rr.qk_size), (rt + "k", rr.qk_size), (rt + "v", rr.inner), (rt + "g", rr.inner)])
            H = rr.heads
            put(L.side[r0: r0 + H], rt + "i")
            put(L.side[r0 + H: r0 + 2 * H], rt + "f")
            put(L.side_b[r0: r0 + H], rt + "i.b")
            put(L.side_b[r0 + H: r0 + 2 * H], rt + "f.b")
            for dst, name in ((L.q_norm, lf + "q.norm"), (L.k_norm, lf + "k.norm"), (L.sink, lf + "sink"), (L.o, lf + "o"),
                              (L.out_left, lf + "out"), (L.o_right, rt + "o"), (L.rnorm, rt + "norm"),
                              (L.out_right, rt + "out")):
                put(dst, name)
    put(model.embed, "embed")
    put(model.head, "head")
    put(model.final_norm, "final.norm")
    out = {"tensors": n, "bytes": rd.bytes_read, "path": path}
    rd.close()
    return out
