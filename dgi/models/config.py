"""Model configurations (Llama-3 8B/70B, Qwen2.5 7B/0.5B, GLM-4-9B, OPT-125m, tiny test models).

Mirrors the fields the reference reads from HF ``AutoConfig``
(worker/distributed/model_shard.py:273-311 uses hidden_size,
num_attention_heads, num_key_value_heads, intermediate_size,
num_hidden_layers) so ``ShardedModelLoader`` and the native runtime share one
description.  No network: presets are built in; ``from_hf_dict`` accepts a
local ``config.json`` dictionary.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Optional


@dataclasses.dataclass
class ModelConfig:
    name: str
    arch: str = "llama"  # "llama" | "qwen2" | "opt"
    vocab_size: int = 128256
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    rope_theta: float = 500000.0
    rope_scaling: Optional[dict] = None
    rms_eps: float = 1e-5
    max_position: int = 8192
    tie_embeddings: bool = False
    qkv_bias: bool = False          # Qwen2 / GLM-4: biased q/k/v projections
    rotary_dim: Optional[int] = None  # rotated dims per head (GLM-4: head_dim / 2); None = head_dim
    rope_interleaved: bool = False  # GLM-4 / GPT-J pairing (2i, 2i+1) instead of NeoX (i, i+rd/2)
    bos_token_id: int = 128000
    eos_token_id: int = 128001

    @property
    def rope_dim(self) -> int:
        return self.rotary_dim or self.head_dim

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def qkv_size(self) -> int:
        return self.q_size + 2 * self.kv_size

    def param_count(self) -> int:
        H, I, V, L = self.hidden_size, self.intermediate_size, self.vocab_size, self.num_layers
        per_layer = H * self.qkv_size + self.q_size * H + 2 * H * I + I * H + 2 * H
        if self.qkv_bias:
            per_layer += self.qkv_size
        emb = V * H * (1 if self.tie_embeddings else 2)
        return L * per_layer + emb + H

    def kv_bytes_per_token(self, dtype_bytes: int = 2, layers: Optional[int] = None) -> int:
        L = self.num_layers if layers is None else layers
        return 2 * L * self.num_kv_heads * self.head_dim * dtype_bytes

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)

    @staticmethod
    def from_hf_dict(d: dict, name: str = "hf") -> "ModelConfig":
        mt = d.get("model_type", "llama")
        if mt == "opt":
            H = d["hidden_size"]
            nh = d["num_attention_heads"]
            return ModelConfig(name=name, arch="opt", vocab_size=d["vocab_size"], hidden_size=H,
                               intermediate_size=d.get("ffn_dim", 4 * H), num_layers=d["num_hidden_layers"],
                               num_heads=nh, num_kv_heads=nh, head_dim=H // nh,
                               max_position=d.get("max_position_embeddings", 2048),
                               tie_embeddings=True, bos_token_id=d.get("bos_token_id", 2),
                               eos_token_id=d.get("eos_token_id", 2), rms_eps=1e-5)
        H = d["hidden_size"]
        nh = d["num_attention_heads"]
        # transformers >= 5 nests RoPE settings under ``rope_parameters``
        rp = d.get("rope_parameters") or {}
        theta = d.get("rope_theta", rp.get("rope_theta", 10000.0))
        scaling = d.get("rope_scaling")
        if scaling is None and rp.get("rope_type", "default") != "default":
            scaling = dict(rp)
        eos = d.get("eos_token_id", 2)
        if isinstance(eos, list):
            eos = eos[0]
        arch = {"qwen2": "qwen2", "glm": "glm"}.get(mt, "llama")
        hd = d.get("head_dim") or H // nh
        prf = d.get("partial_rotary_factor", rp.get("partial_rotary_factor", 1.0))
        rot = int(hd * prf) if prf and prf < 1.0 else None
        return ModelConfig(name=name, arch=arch, vocab_size=d["vocab_size"], hidden_size=H,
                           intermediate_size=d["intermediate_size"], num_layers=d["num_hidden_layers"],
                           num_heads=nh, num_kv_heads=d.get("num_key_value_heads", nh),
                           head_dim=d.get("head_dim") or H // nh, rope_theta=float(theta),
                           rope_scaling=scaling, rms_eps=d.get("rms_norm_eps", 1e-5),
                           max_position=d.get("max_position_embeddings", 8192),
                           tie_embeddings=d.get("tie_word_embeddings", False),
                           qkv_bias=bool(d.get("attention_bias", mt == "qwen2")),
                           rotary_dim=rot, rope_interleaved=(mt == "glm"),
                           bos_token_id=d.get("bos_token_id", 1), eos_token_id=eos)

    @staticmethod
    def from_file(path: str):
        """The configuration a ``config.json`` describes: the class is chosen by the file
        (``architecture`` names a native design, else the HF ``model_type`` families)."""
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path) as f:
            d = json.load(f)
        name = os.path.basename(os.path.dirname(os.path.abspath(path)))
        arch = d.get("architecture")
        if isinstance(arch, str) and arch.lower() in NATIVE_CONFIGS:
            return NATIVE_CONFIGS[arch.lower()](d, name)
        return ModelConfig.from_hf_dict(d, name=name)


@dataclasses.dataclass
class RotarySpec:
    """Rotary position parameters of one attention mixer: the first ``dims`` dimensions of a
    head rotate in pairs at frequency base^(-2i/dims) — ``layout`` "interleaved" pairs (2i, 2i+1),
    "half" pairs (i, i + dims/2); ``scaling`` rescales the frequencies by wavelength, or None:
    (factor, low, high, original) the stepwise form, (factor, original, fast, slow) the ramp form
    that also stretches cos and sin (``dgi.ops.rope_cos_sin``)."""
    base: float
    dims: int
    scaling: Optional[dict] = None
    layout: str = "interleaved"


@dataclasses.dataclass
class AttentionSpec:
    """One softmax-attention mixer: H query heads over G key/value heads, query/key size
    ``dim`` and value size ``vdim``; ``mask_kind`` "chunk" limits a query to the keys of its
    own block of ``mask_size`` positions (counted from position 0), "causal" to all earlier."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[RotarySpec] = None
    mask_kind: str = "causal"
    mask_size: int = 0
    out_gate: bool = True        # sigmoid(W_g h) on the concatenated heads before the output projection
    qk_norm_weight: bool = True  # learned per-dim weight after the q / k unit-RMS norm
    # query temperature: q *= 1 + coef * ln(floor((p + 1) / every) + 1) at position p (every 0: none)
    q_temp_coef: float = 0.0
    q_temp_every: int = 0
    # learned distance bias added to the scaled scores: a table [bias_rows, heads] indexed by
    # ``distance_bucket(i - j, bias_rows, bias_max)`` (bias_rows 0: none)
    bias_rows: int = 0
    bias_max: float = 0.0
    # "head": q and k are RMS-normed per head with a weight of ``dim`` entries; "full": over the whole
    # projection (all heads at once) with a weight as long as the projection
    qk_norm: str = "head"
    softcap: float = 0.0         # scaled scores s become softcap * tanh(s / softcap) (0: none)
    sink: bool = False           # a learned per-head logit joins the softmax denominator (no key, no value)

    @property
    def q_size(self) -> int:
        return self.heads * self.dim

    @property
    def k_size(self) -> int:
        return self.kv_heads * self.dim

    @property
    def v_size(self) -> int:
        return self.kv_heads * self.vdim

    @property
    def o_size(self) -> int:
        return self.heads * self.vdim


@dataclasses.dataclass
class GluSpec:
    """Dense gated feed-forward: ``ff`` inner width, ``limit`` the clamp of gate and up."""
    ff: int
    limit: float
    kind: str = "dense"


def distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of a distance-bias table for distance ``n`` >= 0: the first ``rows // 2`` distances have
    a row each, the rest share rows on a logarithmic scale that reaches the last row at ``far``."""
    import math
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


@dataclasses.dataclass
class Mamba2Spec:
    """One Mamba-2 (state-space duality) mixer: ``heads`` heads of ``vdim`` channels share
    ``groups`` B / C projections of ``state`` dims; a causal convolution of ``conv`` taps over
    x | B | C; the gated output is RMS-normed in ``norm_groups`` equal parts."""
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int = 1

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state

    @property
    def in_size(self) -> int:
        """Rows of the input projection: z | x | B | C | dt."""
        return 2 * self.inner + 2 * self.groups * self.state + self.heads


@dataclasses.dataclass
class MoeSpec:
    """Mixture-of-experts feed-forward: ``experts`` gated-SiLU experts of width ``ff`` plus
    ``identity`` experts that return their input; a token takes the ``top`` experts with the
    largest softmax score + selection bias and weighs them by the plain scores (not
    renormalised).  ``shared_ff`` > 0: a shared expert of that width runs for every token.
    ``score`` "sigmoid": independent sigmoid scores instead of the softmax; "top_softmax": the
    ``top`` largest logits are taken and their weights are the softmax over those alone.
    ``router_bias``: the router has a bias that is part of the logits.  ``act`` "clamped":
    experts are clamped sigmoid-GLUs (``GluSpec`` with ``limit``) instead of gated SiLU.
    ``weigh`` "input": the route weight multiplies the expert's input, not its output."""
    experts: int
    identity: int
    top: int
    ff: int
    shared_ff: int = 0
    kind: str = "moe"
    score: str = "softmax"
    act: str = "silu"
    limit: float = 0.0
    weigh: str = "output"
    selection_bias: bool = True     # a learned per-route bias is added to the scores for the choice only
    router_bias: bool = False

    @property
    def routes(self) -> int:
        return self.experts + self.identity


@dataclasses.dataclass
class LatentAttentionSpec:
    """One latent-attention mixer: queries go through a normalised latent of ``q_rank`` dims, keys
    and values of all ``heads`` come from one normalised latent of ``kv_rank`` dims per token plus
    one rotated key part of ``rot_dim`` dims shared by the heads (the cache holds these two, not
    per-head keys and values).  A head's query/key has ``dim`` unrotated and ``rot_dim`` rotated
    dims, its value ``vdim``.  ``mask_kind`` "window": position i sees j with 0 <= i - j <
    ``mask_size``; "causal": every j <= i.  ``gate`` "head": one sigmoid gate per head, "elem": one
    per output element, "none".  ``kv_from`` = j: the layer has no latent projection of its own and
    reads layer j's cached latent and rotated key part."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: Optional[RotarySpec] = None
    mask_kind: str = "causal"
    mask_size: int = 0
    gate: str = "none"
    kv_from: Optional[int] = None

    @property
    def qk_dim(self) -> int:
        return self.dim + self.rot_dim

    @property
    def q_size(self) -> int:
        return self.heads * self.qk_dim

    @property
    def o_size(self) -> int:
        return self.heads * self.vdim

    @property
    def cache_dim(self) -> int:
        """Cached elements per token: latent | rotated key part."""
        return self.kv_rank + self.rot_dim

    @property
    def gate_rows(self) -> int:
        return {"head": self.heads, "elem": self.o_size, "none": 0}[self.gate]

    @property
    def window(self) -> int:
        return self.mask_size if self.mask_kind == "window" else 0


@dataclasses.dataclass
class DenseSpec:
    """Plain two-matrix feed-forward W_down act(W_up h); ``act`` "gelu_tanh"."""
    ff: int
    act: str = "gelu_tanh"
    kind: str = "dense"


@dataclasses.dataclass
class WkvSpec:
    """One RWKV-style time-mixing layer: ``heads`` heads whose receptance, key and value all have
    ``dim`` channels; every projection reads its own blend of the current and the previous input
    (static per-channel coefficients); the per-channel decay comes from a low-rank projection of
    ``decay_rank`` dims (0: read from the checkpoint's tensor shape); the current token gets a
    per-channel bonus instead of the decayed state."""
    heads: int
    dim: int
    decay_rank: int = 0

    @property
    def inner(self) -> int:
        return self.heads * self.dim


@dataclasses.dataclass
class DeltaSpec:
    """One gated delta-rule layer: ``kv_heads`` query/key heads of ``dim`` channels shared by
    ``heads`` value heads of ``vdim``; q, k and v pass a causal convolution of ``conv`` taps and
    SiLU; per head one decay and one write strength per token."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @property
    def qk_size(self) -> int:
        return self.kv_heads * self.dim

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return 2 * self.qk_size + self.inner


@dataclasses.dataclass
class MlstmSpec:
    """One matrix-memory (mLSTM) layer: ``heads`` heads with ``dim`` query/key and ``vdim`` value
    channels, exponential input gate and sigmoid forget gate in log space, both soft-capped at
    ``gate_cap``, with a running maximum as stabiliser and a normaliser vector."""
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @property
    def qk_size(self) -> int:
        return self.heads * self.dim

    @property
    def inner(self) -> int:
        return self.heads * self.vdim


@dataclasses.dataclass
class ParallelSpec:
    """Two mixers side by side on the same input: ``left`` softmax attention (``AttentionSpec``),
    ``right`` a matrix memory (``MlstmSpec``); the result is the mean of the two outputs, each
    RMS-normed over the model width with its own weight."""
    left: AttentionSpec
    right: MlstmSpec


@dataclasses.dataclass
class LayerSpec:
    type: str
    mixer: object                     # AttentionSpec | Mamba2Spec | LatentAttentionSpec | WkvSpec | DeltaSpec | ParallelSpec
    mlp: Optional[object] = None      # GluSpec | MoeSpec | DenseSpec


@dataclasses.dataclass
class BebovikConfig:
    """A Bebovik decoder: per-layer mixer geometry (every size may differ between layers),
    Dynamic-Tanh norms around both sublayers with layer scale, a scaled embedding with its own
    norm, and scaled + soft-capped logits.  Built from the design's ``config.json``
    (``from_dict``) or in code (tests, benchmarks)."""
    name: str
    vocab_size: int
    hidden_size: int
    layers: list
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    logit_softcap: float = 0.0
    norm_eps: float = 1e-6
    max_position: int = 8192
    bos_token_id: int = -1
    eos_token_id: int = -1
    arch: str = "bebovik"
    tie_embeddings: bool = False

    # the engine-facing view shared with ModelConfig
    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def num_heads(self) -> int:
        return max(l.mixer.heads for l in self.layers)

    @property
    def num_kv_heads(self) -> int:
        return max(l.mixer.kv_heads for l in self.layers)

    @property
    def head_dim(self) -> int:
        return max(max(l.mixer.dim, l.mixer.vdim) for l in self.layers)

    @property
    def rms_eps(self) -> float:
        return self.norm_eps

    def kv_layer_shapes(self, start: int = 0, end: Optional[int] = None) -> list:
        """(kv heads, key size, value size) of each layer's cache pages."""
        return [(l.mixer.kv_heads, l.mixer.dim, l.mixer.vdim) for l in self.layers[start:end]]

    def kv_bytes_per_token(self, dtype_bytes: int = 2, layers: Optional[int] = None) -> int:
        return sum(g * (dk + dv) for g, dk, dv in self.kv_layer_shapes(0, layers)) * dtype_bytes

    def param_count(self) -> int:
        W = self.hidden_size
        n = 2 * self.vocab_size * W
        for l in self.layers:
            m = l.mixer
            n += W * (m.q_size + m.k_size + m.v_size + m.o_size) + m.o_size * W
            if l.mlp is not None:
                n += 3 * W * l.mlp.ff
        return n

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)

    @staticmethod
    def from_dict(d: dict, name: str = "bebovik") -> "BebovikConfig":
        layers = []
        for e in d["layers"]:
            if e["type"] != "attention":
                raise ValueError(f"Bebovik: unknown mixer type {e['type']!r}")
            m = e["mixer"]
            rot = m.get("rot")
            mask = m.get("mask") or {}
            spec = AttentionSpec(
                heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                scale=float(m["scale"]),
                rot=None if not rot else RotarySpec(float(rot["base"]), int(rot["dims"]), rot.get("scaling") or None),
                mask_kind="chunk" if mask.get("size") else "causal", mask_size=int(mask.get("size") or 0))
            if spec.heads % spec.kv_heads:
                raise ValueError("Bebovik: heads must be a multiple of kv_heads")
            f = e.get("mlp")
            if f is not None and f.get("kind", "dense") != "dense":
                raise ValueError(f"Bebovik: unknown feed-forward kind {f.get('kind')!r}")
            layers.append(LayerSpec(e["type"], spec, None if f is None else GluSpec(int(f["ff"]), float(f["limit"]))))
        return BebovikConfig(name=name, vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), layers=layers,
                             embedding_scale=float(d.get("embedding", {}).get("scale", 1.0)),
                             logit_scale=float(d.get("logit_scale", 1.0)),
                             logit_softcap=float(d.get("logit_softcap") or 0.0),
                             norm_eps=float(d.get("norm", {}).get("eps", 1e-6)))


def bebovik_uniform(name: str, vocab: int, width: int, n_layers: int, heads: int, kv_heads: int, dim: int,
                    vdim: int, ff: int, chunk: int, rot_dims: Optional[int] = None, base: float = 10000.0,
                    scaling: Optional[dict] = None, limit: float = 7.0, **kw) -> BebovikConfig:
    """A Bebovik configuration whose layers all share one geometry (presets, benchmarks)."""
    def layer():
        return LayerSpec("attention", AttentionSpec(heads, kv_heads, dim, vdim, dim ** -0.5,
                                                    RotarySpec(base, rot_dims or dim, scaling),
                                                    "chunk" if chunk else "causal", chunk),
                         GluSpec(ff, limit) if ff else None)
    return BebovikConfig(name=name, vocab_size=vocab, hidden_size=width, layers=[layer() for _ in range(n_layers)], **kw)


@dataclasses.dataclass
class TifepelConfig:
    """A Tifepel decoder: token + hashed-bigram + learned-position embedding, ``streams``
    hyper-connected residual streams, per-layer attention (distance-biased, no rotation) or
    Mamba-2 mixers, mixture-of-experts feed-forwards, a causal input convolution and a sigmoid
    output gate around every sublayer, and a span of layers run several times with the same
    weights (``loop_start`` .. ``loop_stop`` - 1, ``loop_times`` times; every pass has its own
    cache and state)."""
    name: str
    vocab_size: int
    hidden_size: int
    layers: list
    streams: int = 1
    canon_taps: int = 0
    bigram_buckets: int = 0
    bigram_mul_prev: int = 0
    bigram_mul_cur: int = 0
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    norm_eps: float = 1e-6
    max_position: int = 2048
    bos_token_id: int = -1
    eos_token_id: int = -1
    arch: str = "tifepel"
    tie_embeddings: bool = False

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def layer_runs(self) -> list:
        """Layer index of every layer run, in execution order."""
        n = len(self.layers)
        if self.loop_times == 1 or self.loop_stop <= self.loop_start:
            return list(range(n))
        a, b = self.loop_start, self.loop_stop
        return list(range(a)) + list(range(a, b)) * self.loop_times + list(range(b, n))

    def _attn(self):
        return [l.mixer for l in self.layers if l.type == "attention"]

    @property
    def num_heads(self) -> int:
        return max([m.heads for m in self._attn()] or [1])

    @property
    def num_kv_heads(self) -> int:
        return max([m.kv_heads for m in self._attn()] or [1])

    @property
    def head_dim(self) -> int:
        return max([max(m.dim, m.vdim) for m in self._attn()] or [1])

    @property
    def rms_eps(self) -> float:
        return self.norm_eps

    def kv_layer_shapes(self, start: int = 0, end: Optional[int] = None) -> list:
        """(kv heads, key size, value size) of the cache pages of every attention layer RUN
        (a looped layer has pages per pass); Mamba-2 runs hold no pages."""
        out = []
        for li in self.layer_runs:
            l = self.layers[li]
            if l.type == "attention":
                out.append((l.mixer.kv_heads, l.mixer.dim, l.mixer.vdim))
        return out

    def kv_bytes_per_token(self, dtype_bytes: int = 2, layers: Optional[int] = None) -> int:
        return sum(g * (dk + dv) for g, dk, dv in self.kv_layer_shapes()) * dtype_bytes

    def param_count(self) -> int:
        W = self.hidden_size
        n = 2 * self.vocab_size * W + (self.bigram_buckets + 1) * W + self.max_position * W
        for l in self.layers:
            m = l.mixer
            if l.type == "attention":
                n += W * (m.q_size + m.k_size + m.v_size) + m.o_size * W
            else:
                n += W * m.in_size + m.inner * W
            n += 2 * W * W
            f = l.mlp
            if f is not None:
                n += 3 * W * f.ff * f.experts + 3 * W * f.shared_ff + W * f.routes
        return n

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)

    @staticmethod
    def from_dict(d: dict, name: str = "tifepel") -> "TifepelConfig":
        layers = []
        for e in d["layers"]:
            m = e["mixer"]
            if e["type"] == "attention":
                qt = m.get("q_temp") or {}
                spec = AttentionSpec(
                    heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                    scale=float(m["scale"]), rot=None, out_gate=False, qk_norm_weight=False,
                    q_temp_coef=float(qt.get("coef") or 0.0), q_temp_every=int(qt.get("every") or 0),
                    bias_rows=-1 if m.get("bias_max") else 0, bias_max=float(m.get("bias_max") or 0.0))
                if spec.heads % spec.kv_heads:
                    raise ValueError("Tifepel: heads must be a multiple of kv_heads")
            elif e["type"] == "mamba2":
                spec = Mamba2Spec(heads=int(m["heads"]), vdim=int(m["vdim"]), state=int(m["state"]),
                                  groups=int(m["groups"]), conv=int(m["conv"]),
                                  norm_groups=int(m.get("norm_groups") or 1))
                if spec.heads % spec.groups or spec.inner % spec.norm_groups:
                    raise ValueError("Tifepel: heads must divide into groups and the inner width into norm groups")
            else:
                raise ValueError(f"Tifepel: unknown mixer type {e['type']!r}")
            f = e.get("mlp")
            mlp = None
            if f is not None:
                if f.get("kind", "moe") != "moe":
                    raise ValueError(f"Tifepel: unknown feed-forward kind {f.get('kind')!r}")
                r = f["router"]
                mlp = MoeSpec(experts=int(r["experts"]), identity=int(r.get("identity") or 0), top=int(r["top"]),
                              ff=int(f["expert"]["ff"]), shared_ff=int((f.get("shared") or {}).get("ff") or 0))
            layers.append(LayerSpec(e["type"], spec, mlp))
        bg = (d.get("embedding") or {}).get("bigram") or {}
        lp = d.get("loop") or {}
        return TifepelConfig(
            name=name, vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), layers=layers,
            streams=int(d.get("streams") or 1), canon_taps=int((d.get("canon") or {}).get("taps") or 0),
            bigram_buckets=int(bg.get("buckets") or 0), bigram_mul_prev=int(bg.get("mul_prev") or 0),
            bigram_mul_cur=int(bg.get("mul_cur") or 0), loop_start=int(lp.get("start") or 0),
            loop_stop=int(lp.get("stop") or 0), loop_times=int(lp.get("times") or 1),
            norm_eps=float((d.get("norm") or {}).get("eps", 1e-6)), max_position=int(d.get("max_positions") or 2048))


def tifepel_uniform(name: str, vocab: int, width: int, pattern: str, heads: int, kv_heads: int, dim: int, vdim: int,
                    m_heads: int, m_vdim: int, state: int, groups: int, experts: int, identity: int, top: int, ff: int,
                    shared_ff: int, bias_rows: int = 32, bias_max: float = 128.0, norm_groups: int = 1, conv: int = 4,
                    **kw) -> TifepelConfig:
    """A Tifepel configuration from a layer pattern ('a' attention, 'm' Mamba-2), all layers of a
    kind sharing one geometry (presets, benchmarks)."""
    layers = []
    for ch in pattern:
        if ch == "a":
            mixer = AttentionSpec(heads, kv_heads, dim, vdim, dim ** -0.5, None, out_gate=False, qk_norm_weight=False,
                                  q_temp_coef=0.25, q_temp_every=128, bias_rows=bias_rows, bias_max=bias_max)
        else:
            mixer = Mamba2Spec(m_heads, m_vdim, state, groups, conv, norm_groups)
        layers.append(LayerSpec("attention" if ch == "a" else "mamba2", mixer,
                                MoeSpec(experts, identity, top, ff, shared_ff) if ff else None))
    return TifepelConfig(name=name, vocab_size=vocab, hidden_size=width, layers=layers, **kw)


@dataclasses.dataclass
class DepelixConfig:
    """A Depelix decoder: token + hashed-bigram embedding, pre-norm RMS layers on one fp32
    stream, latent-attention mixers of two kinds (sliding-window with half-split rotary and a
    per-head gate, possibly reading another layer's cached latent; causal with interleaved rotary
    and an element gate), dense GELU or sigmoid-routed mixture-of-experts feed-forwards (or
    none), and after every layer a small per-layer token input (``side_dim`` columns of one
    shared token table per layer, gated by the stream).  Every layer carries its own sizes."""
    name: str
    vocab_size: int
    hidden_size: int
    layers: list
    side_dim: int = 0
    bigram_buckets: int = 0
    bigram_mul_prev: int = 0
    bigram_mul_cur: int = 0
    norm_eps: float = 1e-6
    max_position: int = 8192
    bos_token_id: int = -1
    eos_token_id: int = -1
    arch: str = "depelix"
    tie_embeddings: bool = False

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def num_heads(self) -> int:
        return max(l.mixer.heads for l in self.layers)

    @property
    def num_kv_heads(self) -> int:
        return 1

    @property
    def head_dim(self) -> int:
        return max(l.mixer.cache_dim for l in self.layers)

    @property
    def rms_eps(self) -> float:
        return self.norm_eps

    def __post_init__(self):
        for i, l in enumerate(self.layers):
            m = l.mixer
            if m.kv_from is None:
                continue
            j = m.kv_from
            if not 0 <= j < i or self.layers[j].mixer.kv_from is not None:
                raise ValueError(f"Depelix: layer {i} reads the latent of layer {j}, which must be an earlier layer "
                                 "with a latent projection of its own")
            o = self.layers[j].mixer
            if (o.kv_rank, o.rot_dim) != (m.kv_rank, m.rot_dim):
                raise ValueError(f"Depelix: layers {i} and {j} share a latent but differ in its sizes")

    @property
    def kv_owners(self) -> list:
        """Layers that write cache pages (those with a latent projection of their own)."""
        return [i for i, l in enumerate(self.layers) if l.mixer.kv_from is None]

    def kv_layer_shapes(self, start: int = 0, end: Optional[int] = None) -> list:
        """(1, latent + rotated key part, 0) per layer that owns pages: one shared row per token
        serves as key and value of every head; layers that read another layer's latent own none."""
        return [(1, self.layers[i].mixer.cache_dim, 0) for i in self.kv_owners]

    def kv_bytes_per_token(self, dtype_bytes: int = 2, layers: Optional[int] = None) -> int:
        return sum(g * (dk + dv) for g, dk, dv in self.kv_layer_shapes()) * dtype_bytes

    def param_count(self) -> int:
        W = self.hidden_size
        n = 2 * self.vocab_size * W + (self.bigram_buckets + 1) * W * bool(self.bigram_buckets)
        n += self.vocab_size * self.side_dim * len(self.layers)
        for l in self.layers:
            m = l.mixer
            n += W * (m.q_rank + m.gate_rows) + m.q_rank * m.q_size + m.heads * (m.dim + m.vdim) * m.kv_rank + m.o_size * W
            if m.kv_from is None:
                n += W * m.cache_dim
            f = l.mlp
            if f is not None:
                n += 2 * W * f.ff if f.kind == "dense" else f.experts * (3 * W * f.ff + W)
            n += 2 * W * self.side_dim
        return n

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)

    @staticmethod
    def from_dict(d: dict, name: str = "depelix") -> "DepelixConfig":
        kinds = {"latent_attention": ("half", "head"), "latent_attention_2": ("interleaved", "elem")}
        layers = []
        for i, e in enumerate(d["layers"]):
            if e["type"] not in kinds:
                raise ValueError(f"Depelix: unknown mixer type {e['type']!r}")
            layout, gate = kinds[e["type"]]
            m = e["mixer"]
            rot = m.get("rot") or {}
            mask = m.get("mask") or {}
            rot_dim = int(m["rot_dim"])
            spec = LatentAttentionSpec(
                heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=rot_dim, vdim=int(m["vdim"]),
                kv_rank=int(m["kv_rank"]), q_rank=int(m["q_rank"]), scale=float(m["scale"]),
                rot=RotarySpec(float(rot.get("base", 10000.0)), int(rot.get("dims", rot_dim)), None, layout),
                mask_kind="window" if mask.get("size") else "causal", mask_size=int(mask.get("size") or 0),
                gate=gate, kv_from=None if m.get("kv_from") is None else int(m["kv_from"]))
            if spec.rot.dims > rot_dim or spec.rot.dims % 2:
                raise ValueError("Depelix: rot.dims must be even and at most rot_dim")
            f = e.get("mlp")
            mlp = None
            if f is not None:
                kind = f.get("kind", "dense")
                if kind == "dense":
                    mlp = DenseSpec(int(f["ff"]))
                elif kind == "moe":
                    r = f["router"]
                    mlp = MoeSpec(experts=int(r["experts"]), identity=0, top=int(r["top"]), ff=int(f["expert"]["ff"]),
                                  score="sigmoid", act="clamped", limit=float(f["expert"]["limit"]), weigh="input",
                                  selection_bias=False)
                    if not 1 <= mlp.top <= mlp.experts:
                        raise ValueError("Depelix: router.top must be between 1 and router.experts")
                else:
                    raise ValueError(f"Depelix: unknown feed-forward kind {kind!r}")
            layers.append(LayerSpec(e["type"], spec, mlp))
        bg = (d.get("embedding") or {}).get("bigram") or {}
        return DepelixConfig(
            name=name, vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), layers=layers,
            side_dim=int((d.get("token_side") or {}).get("dim") or 0),
            bigram_buckets=int(bg.get("buckets") or 0), bigram_mul_prev=int(bg.get("mul_prev") or 0),
            bigram_mul_cur=int(bg.get("mul_cur") or 0), norm_eps=float((d.get("norm") or {}).get("eps", 1e-6)))


def depelix_uniform(name: str, vocab: int, width: int, pattern: str, heads: int, dim: int, rot_dim: int, vdim: int,
                    kv_rank: int, q_rank: int, window: int, ff: int, experts: int = 0, top: int = 1, expert_ff: int = 0,
                    limit: float = 7.0, side_dim: int = 0, base: float = 10000.0, **kw) -> DepelixConfig:
    """A Depelix configuration from a layer pattern: 'w' windowed latent attention, 's' the same
    reading the latent of the nearest earlier 'w' layer, 'c' causal latent attention; upper case:
    the layer's feed-forward is a mixture of experts (else dense, ``ff`` 0: none).  All layers of
    a kind share one geometry (presets, benchmarks)."""
    layers = []
    owner = None
    for i, ch in enumerate(pattern):
        k = ch.lower()
        first = k in ("w", "s")
        if k == "w":
            owner = i
        if k == "s" and owner is None:
            raise ValueError("depelix_uniform: 's' needs an earlier 'w' layer")
        mixer = LatentAttentionSpec(heads, dim, rot_dim, vdim, kv_rank, q_rank, (dim + rot_dim) ** -0.5,
                                    RotarySpec(base, rot_dim, None, "half" if first else "interleaved"),
                                    "window" if first and window else "causal", window if first else 0,
                                    "head" if first else "elem", owner if k == "s" else None)
        if ch.isupper() and experts:
            mlp = MoeSpec(experts, 0, top, expert_ff, score="sigmoid", act="clamped", limit=limit, weigh="input",
                          selection_bias=False)
        else:
            mlp = DenseSpec(ff) if ff else None
        layers.append(LayerSpec("latent_attention" if first else "latent_attention_2", mixer, mlp))
    return DepelixConfig(name=name, vocab_size=vocab, hidden_size=width, layers=layers, side_dim=side_dim, **kw)


@dataclasses.dataclass
class LofuvikConfig:
    """A Lofuvik decoder: plain token embedding, one fp32 stream, layers of the parallel form
    ``x += Mix(h) + FF(h)`` with ``h = RMSnorm(x)``, where Mix is RWKV-style time mixing
    (``WkvSpec``), a gated delta rule (``DeltaSpec``) or softmax attention with a sink beside a
    matrix memory (``ParallelSpec``), and FF a mixture of experts chosen by the largest router
    logits (or none).  A span of layers (``loop_start`` .. ``loop_stop`` - 1) runs ``loop_times``
    times with the same weights; every pass has its own cache and state, and every pass but the
    first starts by adding the embedding output to the stream."""
    name: str
    vocab_size: int
    hidden_size: int
    layers: list
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    norm_eps: float = 1e-6
    max_position: int = 2048
    bos_token_id: int = -1
    eos_token_id: int = -1
    arch: str = "lofuvik"
    tie_embeddings: bool = False

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def layer_runs(self) -> list:
        """Layer index of every layer run, in execution order."""
        n = len(self.layers)
        if self.loop_times <= 1 or self.loop_stop <= self.loop_start:
            return list(range(n))
        a, b = self.loop_start, self.loop_stop
        return list(range(a)) + list(range(a, b)) * self.loop_times + list(range(b, n))

    @property
    def pass_starts(self) -> set:
        """Run indices at which a repeated pass begins (the embedding output is added there)."""
        if self.loop_times <= 1 or self.loop_stop <= self.loop_start:
            return set()
        a, b = self.loop_start, self.loop_stop
        return {a + k * (b - a) for k in range(1, self.loop_times)}

    def _attn(self):
        return [l.mixer.left for l in self.layers if l.type == "parallel"]

    @property
    def num_heads(self) -> int:
        return max([m.heads for m in self._attn()] or [1])

    @property
    def num_kv_heads(self) -> int:
        return max([m.kv_heads for m in self._attn()] or [1])

    @property
    def head_dim(self) -> int:
        return max([max(m.dim, m.vdim) for m in self._attn()] or [1])

    @property
    def rms_eps(self) -> float:
        return self.norm_eps

    def kv_layer_shapes(self, start: int = 0, end: Optional[int] = None) -> list:
        """(kv heads, key size, value size) of the cache pages of every attention RUN (a looped
        layer has pages per pass); the recurrent mixers hold no pages."""
        return [(self.layers[li].mixer.left.kv_heads, self.layers[li].mixer.left.dim, self.layers[li].mixer.left.vdim)
                for li in self.layer_runs if self.layers[li].type == "parallel"]

    def kv_bytes_per_token(self, dtype_bytes: int = 2, layers: Optional[int] = None) -> int:
        return sum(g * (dk + dv) for g, dk, dv in self.kv_layer_shapes()) * dtype_bytes

    def param_count(self) -> int:
        W = self.hidden_size
        n = 2 * self.vocab_size * W
        for l in self.layers:
            m = l.mixer
            if l.type == "wkv":
                n += 5 * W * m.inner + 2 * m.decay_rank * (W + m.inner) // 2
            elif l.type == "delta":
                n += W * (2 * m.qk_size + 3 * m.inner + 2 * m.heads)
            else:
                a, r = m.left, m.right
                n += W * (a.q_size + a.k_size + a.v_size + 2 * a.o_size) + W * (2 * r.qk_size + 3 * r.inner + 2 * r.heads)
            f = l.mlp
            if f is not None:
                n += 3 * W * f.ff * f.experts + W * f.routes
        return n

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)

    @staticmethod
    def from_dict(d: dict, name: str = "lofuvik") -> "LofuvikConfig":
        layers = []
        for e in d["layers"]:
            m, kind = e["mixer"], e["type"]
            if kind == "wkv":
                spec = WkvSpec(heads=int(m["heads"]), dim=int(m["dim"]), decay_rank=int(m.get("decay_rank") or 0))
            elif kind == "delta":
                spec = DeltaSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
                                 vdim=int(m["vdim"]), conv=int(m["conv"]))
                if spec.heads % spec.kv_heads:
                    raise ValueError("Lofuvik: heads must be a multiple of kv_heads")
            elif kind == "parallel":
                a, r = m["left"], m["right"]
                rot = a.get("rot")
                left = AttentionSpec(
                    heads=int(a["heads"]), kv_heads=int(a["kv_heads"]), dim=int(a["dim"]), vdim=int(a["vdim"]),
                    scale=float(a["scale"]),
                    rot=None if not rot or not int(rot.get("dims") or 0) else
                    RotarySpec(float(rot["base"]), int(rot["dims"]), rot.get("scaling") or None, "half"),
                    out_gate=True, qk_norm="full", softcap=float(a.get("softcap") or 0.0), sink=True)
                if left.heads % left.kv_heads:
                    raise ValueError("Lofuvik: heads must be a multiple of kv_heads")
                if left.rot is not None and (left.rot.dims > left.dim or left.rot.dims % 2):
                    raise ValueError("Lofuvik: rot.dims must be even and at most dim")
                spec = ParallelSpec(left, MlstmSpec(heads=int(r["heads"]), dim=int(r["dim"]), vdim=int(r["vdim"]),
                                                    gate_cap=float(r["gate_cap"])))
            else:
                raise ValueError(f"Lofuvik: unknown mixer type {kind!r}")
            f = e.get("mlp")
            mlp = None
            if f is not None:
                if f.get("kind", "moe") != "moe":
                    raise ValueError(f"Lofuvik: unknown feed-forward kind {f.get('kind')!r}")
                r = f["router"]
                mlp = MoeSpec(experts=int(r["experts"]), identity=0, top=int(r["top"]), ff=int(f["expert"]["ff"]),
                              score="top_softmax", selection_bias=False, router_bias=True)
                if not 1 <= mlp.top <= mlp.experts:
                    raise ValueError("Lofuvik: router.top must be between 1 and router.experts")
            layers.append(LayerSpec(kind, spec, mlp))
        lp = d.get("loop") or {}
        return LofuvikConfig(
            name=name, vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), layers=layers,
            loop_start=int(lp.get("start") or 0), loop_stop=int(lp.get("stop") or 0), loop_times=int(lp.get("times") or 1),
            norm_eps=float((d.get("norm") or {}).get("eps", 1e-6)), max_position=int(d.get("max_positions") or 2048))


def lofuvik_uniform(name: str, vocab: int, width: int, pattern: str, heads: int, kv_heads: int, dim: int, vdim: int,
                    r_heads: int, r_dim: int, r_vdim: int, experts: int, top: int, ff: int, conv: int = 4,
                    decay_rank: int = 32, rot_dims: Optional[int] = None, base: float = 10000.0,
                    scaling: Optional[dict] = None, softcap: float = 30.0, gate_cap: float = 15.0, **kw) -> LofuvikConfig:
    """A Lofuvik configuration from a layer pattern: 'd' gated delta rule, 'p' attention beside a
    matrix memory, 'w' RWKV-style time mixing; upper case: the layer has no feed-forward.
    ``heads`` / ``kv_heads`` / ``dim`` / ``vdim`` size the attention, ``r_*`` the recurrent mixers
    (the delta rule's q/k heads are ``r_heads // 2``, at least one); presets and benchmarks."""
    layers = []
    for ch in pattern:
        k = ch.lower()
        if k == "w":
            mixer, kind = WkvSpec(r_heads, r_dim, decay_rank), "wkv"
        elif k == "d":
            mixer, kind = DeltaSpec(r_heads, max(1, r_heads // 2), r_dim, r_vdim, conv), "delta"
        elif k == "p":
            rd = dim if rot_dims is None else rot_dims
            left = AttentionSpec(heads, kv_heads, dim, vdim, dim ** -0.5,
                                 RotarySpec(base, rd, scaling, "half") if rd else None, out_gate=True, qk_norm="full",
                                 softcap=softcap, sink=True)
            mixer, kind = ParallelSpec(left, MlstmSpec(r_heads, r_dim, r_vdim, gate_cap)), "parallel"
        else:
            raise ValueError(f"lofuvik_uniform: unknown layer kind {ch!r}")
        layers.append(LayerSpec(kind, mixer, MoeSpec(experts, 0, top, ff, score="top_softmax", selection_bias=False,
                                                     router_bias=True) if ff and ch.islower() else None))
    return LofuvikConfig(name=name, vocab_size=vocab, hidden_size=width, layers=layers, **kw)


NATIVE_CONFIGS = {"bebovik": BebovikConfig.from_dict, "tifepel": TifepelConfig.from_dict,
                  "depelix": DepelixConfig.from_dict, "lofuvik": LofuvikConfig.from_dict}


PRESETS: dict[str, ModelConfig] = {
    "llama3-8b": ModelConfig(name="llama3-8b"),
    "llama3-70b": ModelConfig(name="llama3-70b", hidden_size=8192, intermediate_size=28672, num_layers=80,
                              num_heads=64, num_kv_heads=8),
    # Small but shape-faithful (GQA 8:1, head_dim 128) Llama for tests / smoke.
    "llama-tiny": ModelConfig(name="llama-tiny", vocab_size=512, hidden_size=512, intermediate_size=1024,
                              num_layers=2, num_heads=8, num_kv_heads=1, head_dim=64, max_position=2048,
                              bos_token_id=1, eos_token_id=2),
    "llama-tiny-hd128": ModelConfig(name="llama-tiny-hd128", vocab_size=1024, hidden_size=1024,
                                    intermediate_size=2048, num_layers=4, num_heads=8, num_kv_heads=1,
                                    head_dim=128, max_position=4096, bos_token_id=1, eos_token_id=2),
    # GQA with 2 KV heads so tensor parallelism of degree 2 has a head per rank
    "llama-tiny-tp": ModelConfig(name="llama-tiny-tp", vocab_size=1024, hidden_size=1024, intermediate_size=2048,
                                 num_layers=2, num_heads=8, num_kv_heads=2, head_dim=128, max_position=4096,
                                 bos_token_id=1, eos_token_id=2),
    # Qwen2 / Qwen2.5 family (the reference's default LLM is Qwen2.5-7B-Instruct):
    # Llama block + biased QKV, GQA 7:1 (7B) / 7:1 (0.5B), theta 1e6
    "qwen2.5-7b": ModelConfig(name="qwen2.5-7b", arch="qwen2", vocab_size=152064, hidden_size=3584,
                              intermediate_size=18944, num_layers=28, num_heads=28, num_kv_heads=4, head_dim=128,
                              rope_theta=1000000.0, rms_eps=1e-6, max_position=32768, qkv_bias=True,
                              bos_token_id=151643, eos_token_id=151645),
    "qwen2.5-0.5b": ModelConfig(name="qwen2.5-0.5b", arch="qwen2", vocab_size=151936, hidden_size=896,
                                intermediate_size=4864, num_layers=24, num_heads=14, num_kv_heads=2, head_dim=64,
                                rope_theta=1000000.0, rms_eps=1e-6, max_position=32768, tie_embeddings=True,
                                qkv_bias=True, bos_token_id=151643, eos_token_id=151645),
    # shape-faithful tiny Qwen2 (biased QKV, GQA 7:1, tied embeddings) for tests
    "qwen-tiny": ModelConfig(name="qwen-tiny", arch="qwen2", vocab_size=1024, hidden_size=1024,
                             intermediate_size=1536, num_layers=2, num_heads=14, num_kv_heads=2, head_dim=128,
                             rope_theta=1000000.0, rms_eps=1e-6, max_position=4096, tie_embeddings=True,
                             qkv_bias=True, bos_token_id=1, eos_token_id=2),
    # GLM-4-9B (HF "glm"): Llama block + biased QKV, GQA 16:1, half-dim interleaved RoPE
    "glm-4-9b": ModelConfig(name="glm-4-9b", arch="glm", vocab_size=151552, hidden_size=4096,
                            intermediate_size=13696, num_layers=40, num_heads=32, num_kv_heads=2, head_dim=128,
                            rope_theta=10000.0, rms_eps=1.5625e-07, max_position=131072, qkv_bias=True,
                            rotary_dim=64, rope_interleaved=True, bos_token_id=151331, eos_token_id=151329),
    "glm-tiny": ModelConfig(name="glm-tiny", arch="glm", vocab_size=1024, hidden_size=1024, intermediate_size=1536,
                            num_layers=2, num_heads=8, num_kv_heads=2, head_dim=128, rope_theta=10000.0,
                            rms_eps=1.5625e-07, max_position=4096, qkv_bias=True, rotary_dim=64,
                            rope_interleaved=True, bos_token_id=1, eos_token_id=2),
    # Bebovik test / smoke sizes (random weights): chunk-masked GQA attention, half-rotary heads
    "bebovik-tiny": bebovik_uniform("bebovik-tiny", 1024, 256, 3, 4, 2, 64, 64, 512, 48, rot_dims=16,
                                    embedding_scale=4.0, logit_scale=0.5, logit_softcap=30.0, max_position=4096,
                                    bos_token_id=1, eos_token_id=2),
    # Tifepel test / smoke sizes (random weights): attention + Mamba-2 layers, the first two run twice
    "tifepel-tiny": tifepel_uniform("tifepel-tiny", 512, 128, "amma", 4, 2, 32, 32, 4, 32, 32, 2, 6, 2, 2, 64, 64,
                                    bias_rows=12, bias_max=40.0, norm_groups=2, streams=2, canon_taps=3,
                                    bigram_buckets=251, bigram_mul_prev=31, bigram_mul_cur=7, loop_start=0,
                                    loop_stop=2, loop_times=2, max_position=2048, bos_token_id=1, eos_token_id=2),
    # Depelix test / smoke sizes (random weights): windowed + shared-latent + causal latent attention,
    # dense and expert feed-forwards, per-layer token input
    "depelix-tiny": depelix_uniform("depelix-tiny", 512, 128, "wScW", 4, 16, 16, 24, 48, 64, 40, 256, experts=6, top=2,
                                    expert_ff=64, limit=2.0, side_dim=16, bigram_buckets=251, bigram_mul_prev=31,
                                    bigram_mul_cur=7, max_position=2048, bos_token_id=1, eos_token_id=2),
    # Lofuvik test / smoke sizes (random weights): delta rule, attention + matrix memory, time mixing; the
    # first two layers run twice
    "lofuvik-tiny": lofuvik_uniform("lofuvik-tiny", 512, 128, "dpwD", 4, 2, 32, 48, 4, 16, 32, 6, 2, 64, conv=3,
                                    decay_rank=8, rot_dims=16, base=10000.0,
                                    scaling={"factor": 2.0, "original": 64, "fast": 8.0, "slow": 1.0},
                                    loop_start=0, loop_stop=2, loop_times=2, max_position=2048,
                                    bos_token_id=1, eos_token_id=2),
    "opt-125m": ModelConfig(name="opt-125m", arch="opt", vocab_size=50272, hidden_size=768,
                            intermediate_size=3072, num_layers=12, num_heads=12, num_kv_heads=12, head_dim=64,
                            max_position=2048, tie_embeddings=True, bos_token_id=2, eos_token_id=2),
}

ALIASES = {
    "meta-llama/Meta-Llama-3-8B": "llama3-8b",
    "meta-llama/Meta-Llama-3-8B-Instruct": "llama3-8b",
    "meta-llama/Llama-3.1-8B-Instruct": "llama3-8b",
    "meta-llama/Meta-Llama-3-70B": "llama3-70b",
    "meta-llama/Meta-Llama-3-70B-Instruct": "llama3-70b",
    "facebook/opt-125m": "opt-125m",
    "Qwen/Qwen2.5-7B-Instruct": "qwen2.5-7b",
    "Qwen/Qwen2.5-7B": "qwen2.5-7b",
    "Qwen/Qwen2-7B-Instruct": "qwen2.5-7b",
    "Qwen/Qwen2.5-0.5B-Instruct": "qwen2.5-0.5b",
    "THUDM/glm-4-9b-chat-hf": "glm-4-9b",
    "THUDM/glm-4-9b-chat": "glm-4-9b",
    "THUDM/glm-4-9b-hf": "glm-4-9b",
}


def get_config(name_or_path: str) -> ModelConfig:
    """Preset, alias, HF config dir/file, or a family guess from the name.
    ``<model>@L<n>`` keeps the architecture and truncates it to ``n`` layers
    (multi-rank rehearsals of a big model's shapes on one GPU)."""
    if "@L" in name_or_path:
        base, n = name_or_path.rsplit("@L", 1)
        bc = get_config(base)
        if isinstance(bc, (BebovikConfig, TifepelConfig, DepelixConfig, LofuvikConfig)):
            return dataclasses.replace(bc, name=name_or_path, layers=bc.layers[: int(n)])
        return dataclasses.replace(bc, name=name_or_path, num_layers=int(n))
    key = ALIASES.get(name_or_path, name_or_path)
    if key in PRESETS:
        import copy
        return copy.deepcopy(PRESETS[key])
    if os.path.exists(name_or_path):
        return ModelConfig.from_file(name_or_path)
    lk = key.lower()
    if "glm-4" in lk or "glm4" in lk:
        return dataclasses.replace(PRESETS["glm-4-9b"], name=name_or_path)
    if "qwen" in lk:
        return dataclasses.replace(PRESETS["qwen2.5-0.5b" if "0.5b" in lk else "qwen2.5-7b"], name=name_or_path)
    if "70b" in lk:
        return dataclasses.replace(PRESETS["llama3-70b"], name=name_or_path)
    if "8b" in lk or "7b" in lk:
        return dataclasses.replace(PRESETS["llama3-8b"], name=name_or_path)
    raise KeyError(f"unknown model {name_or_path!r}; presets: {sorted(PRESETS)}")
