"""Model architecture registry (public config facts of the BASELINE.json model families).

SURVEY §2.4 op inventory lists the shapes; BASELINE.json configs name TinyLlama-1.1B,
Llama-3.2-1B, Llama-3-8B, Llama-3-70B, Mixtral-8x7B; the reference's own tiers ran
phi3-mini (Nano) and llama3-8B (Orin) under Ollama (src/devices/nano_api.py:16,
src/devices/orin_api.py:18).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, replace
from typing import Dict, Optional, Tuple, Union


@dataclass(frozen=True)
class ModelConfig:
    name: str
    hidden: int
    n_layers: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    intermediate: int
    vocab: int
    rope_theta: float = 10000.0
    rms_eps: float = 1e-5
    max_position: int = 8192
    tie_embeddings: bool = False
    n_experts: int = 0          # > 0: MoE MLP (Mixtral)
    experts_per_token: int = 2
    rope_scaling: Optional[Dict] = None
    bos_id: int = 1
    eos_id: int = 2

    @property
    def is_moe(self) -> bool:
        return self.n_experts > 0

    @property
    def q_size(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.n_kv_heads * self.head_dim

    def num_params(self) -> int:
        H, I, L, V = self.hidden, self.intermediate, self.n_layers, self.vocab
        attn = H * (self.q_size + 2 * self.kv_size) + self.q_size * H
        mlp = 3 * H * I * (self.n_experts if self.is_moe else 1) + (H * self.n_experts if self.is_moe else 0)
        emb = V * H * (1 if self.tie_embeddings else 2)
        return L * (attn + mlp + 2 * H) + emb + H


_LLAMA3_SCALING = {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                   "original_max_position_embeddings": 8192}

MODELS: Dict[str, ModelConfig] = {
    "tinyllama-1.1b": ModelConfig("tinyllama-1.1b", 2048, 22, 32, 4, 64, 5632, 32000, 10000.0, 1e-5, 16384),
    "llama-3.2-1b": ModelConfig("llama-3.2-1b", 2048, 16, 32, 8, 64, 8192, 128256, 500000.0, 1e-5, 131072,
                                tie_embeddings=True, rope_scaling=_LLAMA3_SCALING, bos_id=128000, eos_id=128001),
    "llama-3-8b": ModelConfig("llama-3-8b", 4096, 32, 32, 8, 128, 14336, 128256, 500000.0, 1e-5, 16384,
                              bos_id=128000, eos_id=128001),
    "llama-3-70b": ModelConfig("llama-3-70b", 8192, 80, 64, 8, 128, 28672, 128256, 500000.0, 1e-5, 16384,
                               bos_id=128000, eos_id=128001),
    "phi3-mini": ModelConfig("phi3-mini", 3072, 32, 32, 32, 96, 8192, 32064, 10000.0, 1e-5, 8192),
    "mixtral-8x7b": ModelConfig("mixtral-8x7b", 4096, 32, 32, 8, 128, 14336, 32000, 1e6, 1e-5, 32768,
                                n_experts=8, experts_per_token=2),
    # small shapes for CPU tests / smoke runs (same code paths)
    "tiny-llama-test": ModelConfig("tiny-llama-test", 128, 2, 4, 2, 32 * 2, 256, 512, 10000.0, 1e-5, 2048),
    "tiny-moe-test": ModelConfig("tiny-moe-test", 128, 2, 4, 2, 64, 128, 512, 10000.0, 1e-5, 2048,
                                 n_experts=4, experts_per_token=2),
}

ALIASES = {"tinyllama": "tinyllama-1.1b", "llama3-1b": "llama-3.2-1b", "llama3-8b": "llama-3-8b",
           "llama3": "llama-3-8b", "llama3-70b": "llama-3-70b", "phi3": "phi3-mini", "mixtral": "mixtral-8x7b"}


def get_model_config(name: str, **overrides) -> ModelConfig:
    key = ALIASES.get(name.lower(), name.lower())
    if key not in MODELS:
        raise KeyError(f"unknown model {name!r}; known: {sorted(MODELS)}")
    cfg = MODELS[key]
    return replace(cfg, **overrides) if overrides else cfg


# ----------------------------------------------------------------------------- layer-list designs
#
# A hybrid design is a list of layers, each with a token mixer (state-space scan, retention, latent
# attention, gated delta rule, grouped-query softmax attention, lightning attention, or two of
# them side by side) and an optional feed-forward; every size and constant comes from the model
# folder's config.json.  ``family`` picks the model class (models.registry).

@dataclass(frozen=True)
class RopeSpec:
    dims: int
    base: float


@dataclass(frozen=True)
class MixerSpec:
    """One token mixer.  ``kind``: ``mamba1`` (inner, state, dt_rank, conv), ``retention`` (heads,
    dim, vdim, decay per head, rot), ``latent_attention`` (heads, dim, rot_dim, vdim, kv_rank,
    q_rank, scale, rot), ``delta`` (gated delta rule: heads, kv_heads, dim, vdim, conv),
    ``softmax_attention`` (grouped-query, paged: heads, kv_heads, dim, vdim, scale, rot),
    ``lightning`` (heads, dim, vdim, decay per head), ``parallel`` (``left`` and ``right`` mixers
    over the same input), ``diff_attention`` (two softmax maps per head over shared values, combined
    as a1 - lambda a2: heads, kv_heads, dim, vdim, scale, rot, ``window`` keys seen (0: all),
    ``diff``, ``kv_from`` = the layer whose cached keys / values it reads instead of its own),
    ``mamba2`` (scalar decay per head: heads, vdim, state, groups of heads sharing B / C, conv,
    norm_groups of the gated output norm) or ``mlstm`` (matrix memory with exponential gates:
    heads, dim, vdim, gate_cap) or ``sink_attention`` (grouped-query softmax attention with an RMS norm
    over the whole q and k projections, rotary pairs (2i, 2i + 1), unit-RMS values, a learned number per
    head on the scores, a sliding ``window`` that also sees the first ``keep_first`` tokens, and one
    more term of score 0 and weight ``sink`` in the softmax denominator; ``kv_from`` as above)."""
    kind: str
    inner: int = 0
    state: int = 0
    dt_rank: int = 0
    conv: int = 0
    heads: int = 0
    dim: int = 0
    vdim: int = 0
    decay: Tuple[float, ...] = ()
    rot: Optional[RopeSpec] = None
    rot_dim: int = 0
    kv_rank: int = 0
    q_rank: int = 0
    scale: float = 1.0
    kv_heads: int = 0
    left: Optional["MixerSpec"] = None
    right: Optional["MixerSpec"] = None
    window: int = 0
    diff: float = 0.0
    kv_from: Optional[int] = None
    groups: int = 1
    norm_groups: int = 1
    gate_cap: float = 0.0
    keep_first: int = 0
    sink: float = 0.0

    @property
    def parts(self) -> Tuple["MixerSpec", ...]:
        return (self.left, self.right) if self.kind == "parallel" else (self,)

    @property
    def recurrent(self) -> bool:
        return any(p.kind in ("mamba1", "retention", "delta", "lightning", "mamba2", "mlstm") for p in self.parts)

    @property
    def paged(self) -> bool:
        return any(p.kind in ("latent_attention", "softmax_attention") or
                   (p.kind in ("diff_attention", "sink_attention") and p.kv_from is None) for p in self.parts)


@dataclass(frozen=True)
class MoESpec:
    """Routed experts (``ff`` wide, ``top`` of ``experts`` per token, weights times ``scale``) and an
    optional shared expert (``shared_ff`` > 0) that every token runs.  ``act``: ``relu2``
    (W_down relu(W_up x)^2) or ``swiglu`` (W_down (silu(W_gate x) * W_up x)).  ``score``:
    ``softmax`` (the chosen experts' weights renormalised) or ``sigmoid`` (weights = the chosen
    scores as they are); with ``group_count`` > 1 the experts form that many groups of neighbours,
    a group scores the sum of its two best experts and only the ``group_keep`` best groups' experts
    can be chosen.  ``group_score`` "max": a group scores its best expert instead.  ``renorm`` False
    with softmax scores: the chosen scores are the weights as they are.  ``correction``: a learned
    vector is added to the scores for the choice (groups and experts), not for the weights.
    ``identity`` > 0: the router has that many more outputs after the experts', standing for experts
    that return their input.  ``shared_gate``: the shared expert's output is multiplied by the
    sigmoid of one more projection of the token."""
    experts: int
    top: int
    scale: float
    ff: int
    shared_ff: int = 0
    act: str = "relu2"
    score: str = "softmax"
    group_count: int = 1
    group_keep: int = 1
    group_score: str = "top2"
    renorm: bool = True
    correction: bool = False
    identity: int = 0
    shared_gate: bool = False


@dataclass(frozen=True)
class DenseSpec:
    """One dense feed-forward ``W_down act(W_up x)``, ``ff`` wide; ``act``: ``gelu`` (the erf form) or
    ``polynorm`` (a N(z) + b N(z^2) + c N(z^3) + e with learned a, b, c, e and N the scaling of a
    token's ff values to unit RMS), or a gated one, ``W_down (g sigmoid(1.702 g) (u + 1))`` with
    g = min(W_gate x, limit) and u = clamp(W_up x, -limit, limit) (``clamped_glu``).  ``bias``: every
    projection has one."""
    ff: int
    act: str = "gelu"
    limit: float = 0.0
    bias: bool = False


@dataclass(frozen=True)
class LayerSpec:
    mixer: MixerSpec
    mlp: Optional[Union[MoESpec, DenseSpec]] = None


@dataclass(frozen=True)
class HybridConfig:
    name: str
    family: str
    hidden: int
    vocab: int
    layers: Tuple[LayerSpec, ...]
    rms_eps: float = 1e-6
    logit_scale: float = 1.0
    max_position: int = 1 << 20       # the design has no position limit; the engine's max_model_len bounds it
    bos_id: int = 1
    eos_id: int = 2
    # layer form.  False: x += norm(sublayer(x)).  True: x += norm_b(sublayer(norm(x))), a norm on
    # both sides of every sublayer.
    pre_norm: bool = False
    # what a layer hands on is a learned weighted sum of the embedding output and every layer result so far
    depth_average: bool = False
    # the model's norms (after each sublayer, before the head) split the vector into this many equal
    # consecutive parts, each divided by its own root mean square
    norm_groups: int = 1
    # logits <- cap * tanh(logits / cap) (0: none)
    logit_softcap: float = 0.0
    # with pre_norm: False leaves out the norm after a sublayer, x += sublayer(norm(x))
    post_norm: bool = True
    # "rms" (weight) or "layer" (mean and variance, weight and bias) for the model's norms
    norm_kind: str = "rms"
    # a sublayer's output is multiplied by a learned vector before it is added to the stream
    layer_scale: bool = False
    # taps of a causal convolution over time on every channel of the mixer's input, h <- h + conv(h)
    # (0: none); the last taps - 1 inputs of every layer are part of a sequence's state
    input_conv: int = 0
    # the embedding output is multiplied by this number
    embed_scale: float = 1.0
    # the output projection is the embedding table
    tied_head: bool = False

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return any(isinstance(L.mlp, MoESpec) for L in self.layers)

    def num_params(self) -> int:
        H, n = self.hidden, (1 if self.tied_head else 2) * self.vocab * self.hidden + self.hidden
        nb = 2 if self.norm_kind == "layer" else 1
        n += (nb - 1) * H
        for L in self.layers:
            n += H * (self.input_conv + (nb - 1) + (1 if self.layer_scale else 0))
            if L.mlp is not None:
                n += H * ((nb - 1) + (1 if self.layer_scale else 0))
            m = L.mixer
            if m.kind == "mamba1":
                n += 2 * m.inner * H + m.inner * (m.conv + 1) + (m.dt_rank + 2 * m.state) * m.inner
                n += m.inner * (m.dt_rank + 1) + m.inner * m.state + m.inner + H * m.inner
            if m.kind == "parallel":
                n += 2 * H      # each side's output norm
            for m in L.mixer.parts:
                if m.kind in ("retention", "lightning"):
                    n += 2 * m.heads * m.dim * H + 2 * m.heads * m.vdim * H + H * m.heads * m.vdim
                    n += m.heads * m.vdim if m.kind == "lightning" else 0
                elif m.kind == "latent_attention":
                    n += m.q_rank * (H + 1) + m.heads * (m.dim + m.rot_dim) * m.q_rank + (m.kv_rank + m.rot_dim) * H
                    n += m.kv_rank + m.heads * (m.dim + m.vdim) * m.kv_rank + H * m.heads * m.vdim
                elif m.kind == "softmax_attention":
                    n += (m.heads + m.kv_heads) * m.dim * H + m.kv_heads * m.vdim * H + 2 * m.heads * m.vdim * H + m.heads
                elif m.kind == "delta":
                    c = 2 * m.kv_heads * m.dim + m.heads * m.vdim
                    n += c * (H + m.conv) + 2 * m.heads * (H + 1) + m.vdim + 2 * m.heads * m.vdim * H
                elif m.kind == "diff_attention":
                    n += 2 * m.heads * m.dim * (H + 1) + 5 * m.dim + m.heads * m.vdim * H + H
                    if m.kv_from is None:
                        n += (2 * m.kv_heads * m.dim + m.kv_heads * m.vdim) * (H + 1) + m.dim
                elif m.kind == "mamba2":
                    inner, bc = m.heads * m.vdim, 2 * m.groups * m.state
                    n += (2 * inner + bc + m.heads) * H + (inner + bc) * (m.conv + 1) + 3 * m.heads + inner + H * inner
                elif m.kind == "mlstm":
                    n += 2 * m.heads * m.dim * H + 3 * m.heads * m.vdim * H + m.heads * m.vdim + 2 * m.heads * (H + 1)
                elif m.kind == "sink_attention":
                    n += m.heads * m.dim * (H + 1) + m.heads + m.heads * m.vdim * H
                    if m.kv_from is None:
                        n += m.kv_heads * m.dim * (H + 1) + m.kv_heads * m.vdim * H
            sides = 2 if self.pre_norm and self.post_norm else 1
            n += H * sides
            if isinstance(L.mlp, MoESpec):
                f = L.mlp
                mats = 3 if f.act == "swiglu" else 2
                n += H + f.experts * (H + mats * f.ff * H) + mats * f.shared_ff * H
                n += f.identity * H + (f.experts + f.identity if f.correction else 0) + (H if f.shared_gate else 0)
            elif isinstance(L.mlp, DenseSpec):
                f = L.mlp
                mats = 3 if f.act == "clamped_glu" else 2
                n += sides * H + mats * f.ff * H + (4 if f.act == "polynorm" else 0)
                n += (2 * f.ff + H if f.bias else 0)
        if self.depth_average:
            n += sum(i + 2 for i in range(len(self.layers)))
        return n


def _rope(d: Optional[dict]) -> Optional[RopeSpec]:
    return RopeSpec(int(d["dims"]), float(d["base"])) if d else None


def filevik_config(raw: dict, name: str = "filevik") -> HybridConfig:
    """A Filevik config.json: ``layers`` (type, mixer sizes, mlp or null), ``norm.eps``,
    ``logit_scale``, ``vocab``, ``width``."""
    layers = []
    for L in raw["layers"]:
        m, kind = L["mixer"], L["type"]
        if kind == "mamba1":
            mix = MixerSpec(kind, inner=int(m["inner"]), state=int(m["state"]), dt_rank=int(m["dt_rank"]),
                            conv=int(m["conv"]))
        elif kind == "retention":
            mix = MixerSpec(kind, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                            decay=tuple(float(x) for x in m["decay"]), rot=_rope(m.get("rot")))
        elif kind == "latent_attention":
            mix = MixerSpec(kind, heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]),
                            vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]), q_rank=int(m["q_rank"]),
                            scale=float(m["scale"]), rot=_rope(m.get("rot")))
        else:
            raise ValueError(f"unknown mixer type {kind!r}")
        f = L.get("mlp")
        mlp = None
        if f:
            if f.get("kind", "moe") != "moe":
                raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
            sh = f.get("shared")
            mlp = MoESpec(int(f["router"]["experts"]), int(f["router"]["top"]), float(f["router"].get("scale", 1.0)),
                          int(f["expert"]["ff"]), int(sh["ff"]) if sh else 0)
        layers.append(LayerSpec(mix, mlp))
    return HybridConfig(name, "filevik", int(raw["width"]), int(raw["vocab"]), tuple(layers),
                        rms_eps=float(raw["norm"]["eps"]), logit_scale=float(raw.get("logit_scale", 1.0)))


def sedopel_config(raw: dict, name: str = "sedopel") -> HybridConfig:
    """A Sedopel config.json: ``layers`` (type ``delta`` or ``parallel``, mixer sizes, mlp or null),
    ``norm.eps``, ``vocab``, ``width``.  Every sublayer has a norm on both sides and every layer
    ends in a weighted sum over depth."""
    def attention(m: dict) -> MixerSpec:
        return MixerSpec("softmax_attention", heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
                         dim=int(m["dim"]), vdim=int(m["vdim"]), scale=float(m["scale"]), rot=_rope(m.get("rot")))

    def lightning(m: dict) -> MixerSpec:
        return MixerSpec("lightning", heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                         decay=tuple(float(x) for x in m["decay"]))

    layers = []
    for L in raw["layers"]:
        m, kind = L["mixer"], L["type"]
        if kind == "delta":
            mix = MixerSpec(kind, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                            vdim=int(m["vdim"]), conv=int(m["conv"]))
        elif kind == "parallel":
            mix = MixerSpec(kind, left=attention(m["left"]), right=lightning(m["right"]))
        else:
            raise ValueError(f"unknown mixer type {kind!r}")
        for p in mix.parts:
            if p.kv_heads and p.heads % p.kv_heads:
                raise ValueError("heads must be a multiple of kv_heads")
            if p.kind == "lightning" and len(p.decay) != p.heads:
                raise ValueError("one decay per head")
        f = L.get("mlp")
        mlp = None
        if f:
            if f.get("kind", "dense") != "dense":
                raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
            mlp = DenseSpec(int(f["ff"]))
        layers.append(LayerSpec(mix, mlp))
    return HybridConfig(name, "sedopel", int(raw["width"]), int(raw["vocab"]), tuple(layers),
                        rms_eps=float(raw["norm"]["eps"]), pre_norm=True, depth_average=True)


def pebodra_config(raw: dict, name: str = "pebodra") -> HybridConfig:
    """A Pebodra config.json: ``layers`` (type ``attention``, ``mamba2`` or ``mlstm``, mixer sizes,
    mlp ``dense`` / ``moe`` or null), ``norm.eps``, ``norm.groups``, ``logit_softcap``, ``vocab``,
    ``width``.  An attention mixer with ``kv_from`` reads that layer's cached keys and values."""
    W = int(raw["width"])
    layers = []
    for i, L in enumerate(raw["layers"]):
        m, kind = L["mixer"], L["type"]
        if kind == "attention":
            mask = m.get("mask") or {}
            src = m.get("kv_from")
            mix = MixerSpec("diff_attention", heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
                            dim=int(m["dim"]), vdim=int(m["vdim"]), scale=float(m["scale"]), rot=_rope(m.get("rot")),
                            window=int(mask.get("size", 0)), diff=float(m["diff"]),
                            kv_from=None if src is None else int(src))
            if mix.heads % mix.kv_heads:
                raise ValueError("heads must be a multiple of kv_heads")
            if mix.kv_from is not None:
                if not 0 <= mix.kv_from < i or layers[mix.kv_from].mixer.kind != "diff_attention" \
                        or layers[mix.kv_from].mixer.kv_from is not None:
                    raise ValueError(f"layer {i}: kv_from must name an earlier attention layer with keys of its own")
                src_m = layers[mix.kv_from].mixer
                if (src_m.kv_heads, src_m.dim, src_m.vdim) != (mix.kv_heads, mix.dim, mix.vdim):
                    raise ValueError(f"layer {i}: the layer it takes keys and values from has other head sizes")
        elif kind == "mamba2":
            mix = MixerSpec(kind, heads=int(m["heads"]), vdim=int(m["vdim"]), state=int(m["state"]),
                            groups=int(m.get("groups", 1)), conv=int(m["conv"]), norm_groups=int(m.get("norm_groups", 1)))
            if mix.heads % mix.groups or (mix.heads * mix.vdim) % mix.norm_groups:
                raise ValueError("heads must be a multiple of groups, heads * vdim of norm_groups")
        elif kind == "mlstm":
            mix = MixerSpec(kind, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                            gate_cap=float(m["gate_cap"]))
        else:
            raise ValueError(f"unknown mixer type {kind!r}")
        f = L.get("mlp")
        mlp = None
        if f:
            if f["kind"] == "dense":
                mlp = DenseSpec(int(f["ff"]), act="polynorm")
            elif f["kind"] == "moe":
                r = f["router"]
                g = r.get("groups") or {}
                mlp = MoESpec(int(r["experts"]), int(r["top"]), 1.0, int(f["expert"]["ff"]), act="swiglu", score="sigmoid",
                              group_count=int(g.get("count", 1)), group_keep=int(g.get("keep", g.get("count", 1))))
                if mlp.experts % mlp.group_count or not 1 <= mlp.group_keep <= mlp.group_count \
                        or mlp.top > mlp.group_keep * (mlp.experts // mlp.group_count):
                    raise ValueError("router: experts / groups / top do not fit")
            else:
                raise ValueError(f"unknown feed-forward kind {f['kind']!r}")
        layers.append(LayerSpec(mix, mlp))
    groups = int(raw["norm"].get("groups", 1))
    if W % groups:
        raise ValueError("width must be a multiple of norm.groups")
    return HybridConfig(name, "pebodra", W, int(raw["vocab"]), tuple(layers), rms_eps=float(raw["norm"]["eps"]),
                        norm_groups=groups, logit_softcap=float(raw.get("logit_softcap") or 0.0))


def dogilorn_config(raw: dict, name: str = "dogilorn") -> HybridConfig:
    """A Dogilorn config.json: ``layers`` (type ``attention``, mixer sizes with ``mask.size`` /
    ``mask.keep_first``, ``rot``, ``scale``, optional ``kv_from``; mlp ``dense`` with ``ff`` and
    ``limit``, ``moe`` with ``expert.ff``, ``router`` (experts, identity, top, groups) and an optional
    ``shared`` expert, or null), ``canon.taps``, ``embedding.scale``, ``norm.eps``, ``vocab``,
    ``width``.  Layer norms with bias ahead of every sublayer, none after it, a learned scale on
    every sublayer's output, the head tied to the embedding."""
    layers = []
    for i, L in enumerate(raw["layers"]):
        m, kind = L["mixer"], L["type"]
        if kind != "attention":
            raise ValueError(f"unknown mixer type {kind!r}")
        mask = m.get("mask") or {}
        src = m.get("kv_from")
        o = None
        if src is not None:      # sizes of the keys and values it reads default to their owner's
            if not 0 <= int(src) < i or layers[int(src)].mixer.kv_from is not None:
                raise ValueError(f"layer {i}: kv_from must name an earlier attention layer with keys of its own")
            o = layers[int(src)].mixer
        mix = MixerSpec("sink_attention", heads=int(m["heads"]),
                        kv_heads=int(m.get("kv_heads", o.kv_heads if o else m["heads"])),
                        dim=int(m["dim"]), vdim=int(m.get("vdim", o.vdim if o else m["dim"])), scale=float(m["scale"]),
                        rot=_rope(m["rot"]) if "rot" in m else (o.rot if o else None),
                        window=int(mask.get("size", 0)), keep_first=int(mask.get("keep_first", 0)), sink=1.0,
                        kv_from=None if src is None else int(src))
        if mix.heads % mix.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        if mix.rot is not None and (mix.rot.dims % 2 or mix.rot.dims > mix.dim):
            raise ValueError("rot.dims must be even and at most dim")
        if o is not None:
            if (o.kv_heads, o.dim, o.vdim, o.rot) != (mix.kv_heads, mix.dim, mix.vdim, mix.rot):
                raise ValueError(f"layer {i}: the layer it takes keys and values from has other head sizes or rotation")
        f = L.get("mlp")
        mlp = None
        if f:
            if f["kind"] == "dense":
                mlp = DenseSpec(int(f["ff"]), act="clamped_glu", limit=float(f["limit"]), bias=True)
            elif f["kind"] == "moe":
                r = f["router"]
                g = r.get("groups") or {}
                sh = f.get("shared")
                mlp = MoESpec(int(r["experts"]), int(r["top"]), 1.0, int(f["expert"]["ff"]), int(sh["ff"]) if sh else 0,
                              act="swiglu", score="softmax", group_count=int(g.get("count", 1)),
                              group_keep=int(g.get("keep", g.get("count", 1))), group_score="max", renorm=False,
                              correction=True, identity=int(r.get("identity", 0)), shared_gate=bool(sh))
                outs = mlp.experts + mlp.identity
                if outs % mlp.group_count or not 1 <= mlp.group_keep <= mlp.group_count \
                        or mlp.top > mlp.group_keep * (outs // mlp.group_count):
                    raise ValueError("router: experts / groups / top do not fit")
            else:
                raise ValueError(f"unknown feed-forward kind {f['kind']!r}")
        layers.append(LayerSpec(mix, mlp))
    return HybridConfig(name, "dogilorn", int(raw["width"]), int(raw["vocab"]), tuple(layers),
                        rms_eps=float(raw["norm"]["eps"]), pre_norm=True, post_norm=False, norm_kind="layer",
                        layer_scale=True, input_conv=int((raw.get("canon") or {}).get("taps", 0)),
                        embed_scale=float((raw.get("embedding") or {}).get("scale", 1.0)), tied_head=True)


# config.json "architecture" -> parser of that design's keys
ARCHITECTURES = {"Filevik": filevik_config, "Sedopel": sedopel_config, "Pebodra": pebodra_config,
                 "Dogilorn": dogilorn_config}

AnyConfig = Union[ModelConfig, HybridConfig]


def config_from_dir(path: str) -> AnyConfig:
    """The configuration of a model folder (config.json + model.safetensors): the parser is chosen
    by the file's ``architecture``."""
    with open(os.path.join(path, "config.json")) as f:
        raw = json.load(f)
    arch = raw.get("architecture")
    if arch not in ARCHITECTURES:
        raise KeyError(f"unknown architecture {arch!r}; known: {sorted(ARCHITECTURES)}")
    return ARCHITECTURES[arch](raw, name=os.path.basename(os.path.normpath(path)) or arch.lower())


def resolve_config(model: Union[str, AnyConfig]) -> AnyConfig:
    """A registry name, a model folder, or a config object -> config."""
    if not isinstance(model, str):
        return model
    if os.path.isdir(model) and os.path.exists(os.path.join(model, "config.json")):
        return config_from_dir(model)
    return get_model_config(model)
