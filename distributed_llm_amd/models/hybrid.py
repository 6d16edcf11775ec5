"""Layer-list decoders (Filevik, Sedopel, Pebodra): every layer has a token mixer (Mamba-1 selective
scan, retention, latent attention, gated delta rule, grouped-query softmax attention beside lightning
attention, differential sliding-window attention, Mamba-2, mLSTM) and an optional feed-forward
(mixture of experts or dense), in the order config.json gives.

The residual stream lives in f32; each sublayer reads its rounding to the model dtype and adds
``rmsnorm(sublayer(x)) * w`` (ops.seqmix.norm_resadd: the f32 add, the norm and the rounded copy in
one launch).  Projections run on the framework's GEMMs (ops.linear; the vendor GEMM for shapes
they do not take and for f32 models), everything between them on the HIP kernels of ops.seqmix:

  mamba1     in-proj -> causal conv + SiLU (reads the slot's last inputs) -> x-proj -> dt-proj ->
             selective scan (f32 state per slot, softplus / decay / gate in f32; refills the
             convolution state) -> out-proj
  retention  one fused q|k|v|gate projection -> decayed linear attention (rotate-half positions,
             f32 state per slot, unit-RMS heads, SiLU gate in the kernel) -> out-proj
  latent     one fused down projection (query latent | key/value latent | shared rotated key) ->
             query up-projection -> the key up-projection is absorbed into the query (per-head
             batched GEMM), so attention runs over the cached latent alone (paged, written by a
             kernel that norms the latent and rotates the shared key) -> value up-projection per
             head -> out-proj
  experts    fused router (f32 softmax top-k, renormalised) -> grouped squared-ReLU expert GEMMs, or
             the dense form (all experts' columns, unused ones gated to zero) for f32 models and
             unaligned widths -> plus the shared expert
  delta      one fused projection (q | k | v | gate | beta | decay logits) -> causal conv + SiLU ->
             gated delta rule (unit q / k, decay, beta, f32 state per slot, per-head norm and SiLU
             gate in the kernel) -> out-proj
  parallel   one fused projection for both sides.  Left: rotation + unit-RMS q / k, k and v written
             to their pages, causal softmax attention over the pages with the sigmoid gate ->
             out-proj.  Right: lightning attention (the retention kernels on SiLU'd inputs, heads
             normed together, sigmoid gate) -> out-proj.  The two outputs are normed and averaged
             in the launch that also adds the sublayer to the stream.
  dense      up-proj -> erf GELU or PolyNorm -> down-proj
  diff_attn  one fused q | k | v projection -> biases, weighted RMS norm of every q / k map, rotation,
             k and v to their pages (a layer with ``kv_from`` projects q alone and reads that layer's
             pages) -> windowed causal softmax attention with the two maps of a head as two query
             rows over the shared values (f32 out) -> a1 - lambda a2, unit RMS per head -> out-proj
  mamba2     one fused projection (z | x | B | C | dt) -> causal conv + SiLU over x | B | C ->
             recurrence with a scalar decay per head (f32 state per slot) -> y silu(z), RMS norm in
             groups -> out-proj
  mlstm      one fused projection (q | k | v | gate | input gate | forget gate) -> matrix memory with
             a running maximum and a normaliser (f32 state per slot; unit-RMS heads, weight and
             sigmoid gate in the kernel) -> out-proj
  experts    (sigmoid scores) f32 router logits -> group-limited top-k, weights = scores -> grouped
             SwiGLU expert GEMMs or their dense form
  sink_attn  (input: h + a short causal convolution of h, its last inputs kept in the slot) one fused
             q | k | v projection -> RMS norm over the whole q and k projections, rotary pairs
             (2i, 2i + 1), unit-RMS values, k and v to their pages (a layer with ``kv_from`` projects q
             alone) -> attention inside a sliding window that also keeps the first tokens, with one
             more term of score 0 in the softmax denominator -> out-proj
  clamped    one fused gate | up projection -> biases, clamps, g sigmoid(1.702 g) (u + 1) -> down-proj
  experts    (softmax scores + a correction for the choice, identity experts) one f32 GEMM for the
             router logits and the shared expert's gate logit -> group-limited top-k -> SwiGLU experts;
             identity experts, the gated shared expert and the layer scale ride in the residual launch

Layer forms: ``x += norm(sublayer(x))`` (Filevik) or, with ``cfg.pre_norm``, a norm on both sides,
``x += norm_b(sublayer(norm(x)))``, or without ``cfg.post_norm`` ``x += ls * sublayer(layernorm(x))``
(layer norms with bias, a learned scale per channel); with ``cfg.depth_average`` a layer hands on a
learned weighted sum of the embedding output and all layer results so far (kept as an f32 stack for
the step).

Per-sequence state lives in slots owned by the engine (its batch rows); paged latents use the
engine's block tables.  No tensor parallelism.
"""
from __future__ import annotations

import math
import os
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn.functional as F

from .. import ops
from ..ops import seqmix
from ..parallel.comm import SINGLE, ParallelContext
from .configs import DenseSpec, HybridConfig, LayerSpec, MixerSpec, MoESpec


def _mm(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x @ w.T: the framework's tuned GEMM where it takes the shape, else the vendor GEMM."""
    if (x.is_cuda and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2 and x.stride(1) == 1
            and x.shape[1] % 64 == 0 and w.shape[0] % 64 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
            and w.is_contiguous()):
        return ops.linear(x, w)
    return F.linear(x, w)


class HybridModel:
    fused = False                      # no folded-norm GEMM epilogues (engine autotune hook)
    has_recurrent_state = True
    attn_geometry = None               # no softmax-attention split-K workspace

    def __init__(self, cfg: HybridConfig, device="cuda", dtype=torch.bfloat16, par: ParallelContext = SINGLE,
                 seed: int = 0, weights: Optional[str] = None, init_std: float = 0.02):
        if par.tp_size > 1:
            raise ValueError(f"{cfg.name}: layer-list models run on one GPU (no tensor parallelism)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("dtype must be bfloat16 or float32")
        self.cfg, self.device, self.dtype, self.par = cfg, torch.device(device), dtype, par
        if cfg.pre_norm and not cfg.post_norm and (cfg.norm_kind != "layer" or cfg.depth_average):
            raise ValueError(f"{cfg.name}: layers without a norm after the sublayer use layer norms and no depth average")
        if cfg.norm_kind == "layer" and (not cfg.pre_norm or cfg.post_norm):
            raise ValueError(f"{cfg.name}: layer norms are built for the pre-norm layer form only")
        # the input convolution's last inputs are per-sequence state like a recurrence's
        self.has_recurrent_state = any(L.mixer.recurrent for L in cfg.layers) or cfg.input_conv > 1
        self.layers: List[Dict[str, torch.Tensor]] = []
        self.tap: Optional[list] = None      # debugging: residual stream after every layer
        self._rot: Dict[Tuple[int, float], torch.Tensor] = {}
        self._max_pos = 0
        raw = self._load(weights) if weights else self._random(seed, init_std)
        self._place(raw)
        self.ensure_positions(2048)

    # ------------------------------------------------------------------ weights
    def _random(self, seed: int, std: float) -> Dict[str, torch.Tensor]:
        """Seeded random tensors under the checkpoint's names (benchmarks, tests)."""
        g = torch.Generator().manual_seed(seed)
        cfg, W = self.cfg, self.cfg.hidden
        t: Dict[str, torch.Tensor] = {}

        def rnd(*shape, s=std):
            return torch.randn(*shape, generator=g) * s

        def lin(n_out, n_in):
            return rnd(n_out, n_in, s=1.0 / math.sqrt(n_in))

        t["embed"] = rnd(cfg.vocab, W, s=1.0)
        if not cfg.tied_head:
            t["head"] = lin(cfg.vocab, W)
        t["final.norm"] = torch.ones(W)
        lnb = cfg.norm_kind == "layer"
        if lnb:
            t["final.norm.b"] = rnd(W, s=0.1)
        for i, L in enumerate(cfg.layers):
            p, m = f"l{i}.", L.mixer
            t[p + "norm1"] = torch.ones(W)
            if lnb:
                t[p + "norm1.b"] = rnd(W, s=0.1)
            if cfg.layer_scale:
                t[p + "ls1"] = torch.full((W,), 0.5)
            if cfg.input_conv:
                t[p + "canon1"] = rnd(W, cfg.input_conv, s=0.3)
            if cfg.pre_norm and cfg.post_norm:
                t[p + "norm1b"] = torch.ones(W)
            if cfg.depth_average:
                t[p + "dwa"] = torch.cat([rnd(i + 1, s=0.05), torch.ones(1)])
            if m.kind == "delta":
                gd, hv = m.kv_heads * m.dim, m.heads * m.vdim
                for n_, c in (("q", gd), ("k", gd), ("v", hv)):
                    t[p + "mix." + n_] = lin(c, W)
                    t[p + f"mix.{n_}.conv"] = rnd(c, m.conv, s=1.0 / math.sqrt(m.conv))
                t[p + "mix.g"], t[p + "mix.o"] = lin(hv, W), lin(W, hv)
                t[p + "mix.b"], t[p + "mix.a"] = lin(m.heads, W), lin(m.heads, W)
                t[p + "mix.A_log"] = torch.log(torch.rand(m.heads, generator=g) * 15 + 1)
                dt = torch.exp(torch.rand(m.heads, generator=g) * (math.log(0.1) - math.log(0.001)) + math.log(0.001))
                t[p + "mix.dt_bias"] = dt + torch.log(-torch.expm1(-dt))
                t[p + "mix.norm"] = torch.ones(m.vdim)
            elif m.kind == "parallel":
                a, b = m.left, m.right
                t[p + "mix.left.q"], t[p + "mix.left.k"] = lin(a.heads * a.dim, W), lin(a.kv_heads * a.dim, W)
                t[p + "mix.left.v"], t[p + "mix.left.g"] = lin(a.kv_heads * a.vdim, W), lin(a.heads * a.vdim, W)
                t[p + "mix.left.o"], t[p + "mix.left.temp"] = lin(W, a.heads * a.vdim), torch.ones(a.heads)
                t[p + "mix.right.q"], t[p + "mix.right.k"] = lin(b.heads * b.dim, W), lin(b.heads * b.dim, W)
                t[p + "mix.right.v"], t[p + "mix.right.g"] = lin(b.heads * b.vdim, W), lin(b.heads * b.vdim, W)
                t[p + "mix.right.o"], t[p + "mix.right.norm"] = lin(W, b.heads * b.vdim), torch.ones(b.heads * b.vdim)
                t[p + "mix.left.out"], t[p + "mix.right.out"] = torch.ones(W), torch.ones(W)
            elif m.kind == "diff_attention":
                nq, nk = m.heads * 2 * m.dim, m.kv_heads * 2 * m.dim
                t[p + "mix.q"], t[p + "mix.q.b"], t[p + "mix.q.norm"] = lin(nq, W), rnd(nq, s=0.1), torch.ones(m.dim)
                if m.kv_from is None:
                    t[p + "mix.k"], t[p + "mix.k.b"], t[p + "mix.k.norm"] = lin(nk, W), rnd(nk, s=0.1), torch.ones(m.dim)
                    t[p + "mix.v"], t[p + "mix.v.b"] = lin(m.kv_heads * m.vdim, W), rnd(m.kv_heads * m.vdim, s=0.1)
                for n_ in ("lq1", "lk1", "lq2", "lk2"):
                    t[p + "mix." + n_] = rnd(m.dim, s=0.1)
                t[p + "mix.o"], t[p + "mix.o.b"] = lin(W, m.heads * m.vdim), rnd(W, s=0.1)
            elif m.kind == "mamba2":
                inner, bc = m.heads * m.vdim, 2 * m.groups * m.state
                t[p + "mix.in"] = lin(2 * inner + bc + m.heads, W)
                t[p + "mix.conv"] = rnd(inner + bc, m.conv, s=1.0 / math.sqrt(m.conv))
                t[p + "mix.conv.b"] = rnd(inner + bc, s=0.1)
                dt = torch.exp(torch.rand(m.heads, generator=g) * (math.log(0.1) - math.log(0.001)) + math.log(0.001))
                t[p + "mix.dt_bias"] = dt + torch.log(-torch.expm1(-dt))
                t[p + "mix.A_log"] = torch.log(torch.rand(m.heads, generator=g) * 15 + 1)
                t[p + "mix.D"], t[p + "mix.norm"] = torch.ones(m.heads), torch.ones(inner)
                t[p + "mix.o"] = lin(W, inner)
            elif m.kind == "mlstm":
                hd, hv = m.heads * m.dim, m.heads * m.vdim
                t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"] = lin(hd, W), lin(hd, W), lin(hv, W)
                t[p + "mix.g"], t[p + "mix.o"], t[p + "mix.norm"] = lin(hv, W), lin(W, hv), torch.ones(hv)
                t[p + "mix.i"], t[p + "mix.f"] = lin(m.heads, W), lin(m.heads, W)
                t[p + "mix.i.b"] = rnd(m.heads, s=0.1)
                t[p + "mix.f.b"] = torch.linspace(3.0, 6.0, m.heads)
            elif m.kind == "sink_attention":
                t[p + "mix.q"], t[p + "mix.q.norm"] = lin(m.heads * m.dim, W), torch.ones(m.heads * m.dim)
                t[p + "mix.temp"], t[p + "mix.o"] = torch.ones(m.heads), lin(W, m.heads * m.vdim)
                if m.kv_from is None:
                    t[p + "mix.k"], t[p + "mix.k.norm"] = lin(m.kv_heads * m.dim, W), torch.ones(m.kv_heads * m.dim)
                    t[p + "mix.v"] = lin(m.kv_heads * m.vdim, W)
            elif m.kind == "mamba1":
                t[p + "mix.in"] = lin(2 * m.inner, W)
                t[p + "mix.conv"] = rnd(m.inner, m.conv, s=1.0 / math.sqrt(m.conv))
                t[p + "mix.conv.b"] = rnd(m.inner, s=0.1)
                t[p + "mix.x"] = lin(m.dt_rank + 2 * m.state, m.inner)
                t[p + "mix.dt"] = lin(m.inner, m.dt_rank)
                dt = torch.exp(torch.rand(m.inner, generator=g) * (math.log(0.1) - math.log(0.001)) + math.log(0.001))
                t[p + "mix.dt.b"] = dt + torch.log(-torch.expm1(-dt))
                t[p + "mix.A_log"] = torch.log(torch.arange(1, m.state + 1, dtype=torch.float32))[None, :].repeat(m.inner, 1)
                t[p + "mix.D"] = torch.ones(m.inner)
                t[p + "mix.o"] = lin(W, m.inner)
            elif m.kind == "retention":
                t[p + "mix.q"], t[p + "mix.k"] = lin(m.heads * m.dim, W), lin(m.heads * m.dim, W)
                t[p + "mix.v"], t[p + "mix.g"] = lin(m.heads * m.vdim, W), lin(m.heads * m.vdim, W)
                t[p + "mix.o"] = lin(W, m.heads * m.vdim)
            else:
                t[p + "mix.dq"], t[p + "mix.dq.norm"] = lin(m.q_rank, W), torch.ones(m.q_rank)
                t[p + "mix.uq"] = lin(m.heads * (m.dim + m.rot_dim), m.q_rank)
                t[p + "mix.dkv"], t[p + "mix.dkv.norm"] = lin(m.kv_rank + m.rot_dim, W), torch.ones(m.kv_rank)
                t[p + "mix.uk"], t[p + "mix.uv"] = lin(m.heads * m.dim, m.kv_rank), lin(m.heads * m.vdim, m.kv_rank)
                t[p + "mix.o"] = lin(W, m.heads * m.vdim)
            f = L.mlp
            if f is not None:
                t[p + "norm2"] = torch.ones(W)
                if lnb:
                    t[p + "norm2.b"] = rnd(W, s=0.1)
                if cfg.layer_scale:
                    t[p + "ls2"] = torch.full((W,), 0.5)
            if isinstance(f, DenseSpec):
                if cfg.pre_norm and cfg.post_norm:
                    t[p + "norm2b"] = torch.ones(W)
                t[p + "mlp.up"], t[p + "mlp.down"] = lin(f.ff, W), lin(W, f.ff)
                if f.act == "polynorm":
                    t[p + "mlp.act"] = torch.tensor([1.0, 0.5, 0.25, 0.0])
                if f.act == "clamped_glu":
                    t[p + "mlp.gate"] = lin(f.ff, W)
                if f.bias:
                    for n_, c in (("gate", f.ff), ("up", f.ff), ("down", W)):
                        t[p + f"mlp.{n_}.b"] = rnd(c, s=0.1)
            elif f is not None:
                t[p + "mlp.router"] = lin(f.experts + f.identity, W)
                if f.correction:
                    t[p + "mlp.correction"] = rnd(f.experts + f.identity, s=0.01)
                for e in range(f.experts):
                    t[p + f"mlp.e{e}.up"], t[p + f"mlp.e{e}.down"] = lin(f.ff, W), lin(W, f.ff)
                    if f.act == "swiglu":
                        t[p + f"mlp.e{e}.gate"] = lin(f.ff, W)
                if f.shared_ff:
                    t[p + "mlp.shared.up"], t[p + "mlp.shared.down"] = lin(f.shared_ff, W), lin(W, f.shared_ff)
                    if f.act == "swiglu":
                        t[p + "mlp.shared.gate"] = lin(f.shared_ff, W)
                    if f.shared_gate:
                        t[p + "mlp.shared.sg"] = lin(1, W)
        return t

    @staticmethod
    def _load(path: str) -> Dict[str, torch.Tensor]:
        from safetensors import safe_open
        files = [path] if os.path.isfile(path) else sorted(
            os.path.join(path, f) for f in os.listdir(path) if f.endswith(".safetensors"))
        out: Dict[str, torch.Tensor] = {}
        for f in files:
            with safe_open(f, framework="pt", device="cpu") as fh:
                for k in fh.keys():
                    out[k] = fh.get_tensor(k)
        return out

    def _place(self, t: Dict[str, torch.Tensor]) -> None:
        """Checkpoint tensors -> device layouts (fused projections, per-head batched matrices,
        f32 copies of what the recurrences read)."""
        cfg, dev, dt = self.cfg, self.device, self.dtype
        put = lambda x: x.to(dev, dt).contiguous()
        f32 = lambda x: x.to(dev, torch.float32).contiguous()
        W = cfg.hidden
        self.embed, self.final_norm = put(t["embed"]), f32(t["final.norm"])
        self.lm_head = self.embed if cfg.tied_head else put(t["head"])      # tied: the table itself, unscaled
        lnb = cfg.norm_kind == "layer"
        self.final_norm_b = f32(t["final.norm.b"]) if lnb else None
        if tuple(self.embed.shape) != (cfg.vocab, W) or tuple(self.lm_head.shape) != (cfg.vocab, W):
            raise ValueError("embed / head do not fit config vocab x width")
        for i, L in enumerate(cfg.layers):
            p, m = f"l{i}.", L.mixer
            D: Dict[str, torch.Tensor] = {"norm1": f32(t[p + "norm1"])}
            if cfg.pre_norm and cfg.post_norm:
                D["norm1b"] = f32(t[p + "norm1b"])
            if lnb:
                D["norm1.b"] = f32(t[p + "norm1.b"])
            if cfg.layer_scale:
                D["ls1"] = f32(t[p + "ls1"])
                assert D["ls1"].numel() == W
            if cfg.input_conv:
                D["canon"] = f32(t[p + "canon1"])
                D["canon_b"] = torch.zeros(W, dtype=torch.float32, device=dev)
                assert tuple(D["canon"].shape) == (W, cfg.input_conv)
            if cfg.depth_average:
                D["dwa"] = f32(t[p + "dwa"])
                assert D["dwa"].numel() == i + 2
            if m.kind == "delta":
                # one projection: q | k | v (the convolved channels) | gate | beta | decay logits
                D["proj"] = put(torch.cat([t[p + "mix." + n] for n in ("q", "k", "v", "g", "b", "a")], 0))
                D["conv"] = f32(torch.cat([t[p + f"mix.{n}.conv"] for n in "qkv"], 0))
                D["conv_b"] = torch.zeros(D["conv"].shape[0], dtype=torch.float32, device=dev)
                D["neg_a"], D["dt_b"] = -torch.exp(f32(t[p + "mix.A_log"])), f32(t[p + "mix.dt_bias"])
                D["hnorm"], D["o"] = f32(t[p + "mix.norm"]), put(t[p + "mix.o"])
                assert tuple(D["conv"].shape) == (2 * m.kv_heads * m.dim + m.heads * m.vdim, m.conv)
                assert D["neg_a"].numel() == m.heads and D["hnorm"].numel() == m.vdim
            elif m.kind == "parallel":
                a, b = m.left, m.right
                names = [f"mix.left.{n}" for n in "qkvg"] + [f"mix.right.{n}" for n in "qkvg"]
                D["proj"] = put(torch.cat([t[p + n] for n in names], 0))
                D["lo"], D["ro"] = put(t[p + "mix.left.o"]), put(t[p + "mix.right.o"])
                D["qscale"] = f32(t[p + "mix.left.temp"]) * a.scale
                D["decay"] = torch.tensor(b.decay, dtype=torch.float32, device=dev)
                D["rnorm"] = f32(t[p + "mix.right.norm"])
                D["lout"], D["rout"] = f32(t[p + "mix.left.out"]), f32(t[p + "mix.right.out"])
                assert D["qscale"].numel() == a.heads and D["rnorm"].numel() == b.heads * b.vdim
                assert D["proj"].shape[0] == self._left_cols(a) + 2 * b.heads * (b.dim + b.vdim)
            elif m.kind == "diff_attention":
                own = m.kv_from is None
                names = ("q", "k", "v") if own else ("q",)
                D["proj"] = put(torch.cat([t[p + "mix." + n] for n in names], 0))
                D["bias"] = f32(torch.cat([t[p + f"mix.{n}.b"] for n in names], 0))
                D["qnorm"] = f32(t[p + "mix.q.norm"])
                D["knorm"] = f32(t[p + "mix.k.norm"]) if own else D["qnorm"]
                l1 = (f32(t[p + "mix.lq1"]) * f32(t[p + "mix.lk1"])).sum()
                l2 = (f32(t[p + "mix.lq2"]) * f32(t[p + "mix.lk2"])).sum()
                D["lam"] = float(torch.exp(l1) - torch.exp(l2)) + m.diff       # one number for the layer
                D["o"], D["ob"] = put(t[p + "mix.o"]), f32(t[p + "mix.o.b"])
                cols = 2 * m.heads * m.dim + ((2 * m.kv_heads * m.dim + m.kv_heads * m.vdim) if own else 0)
                assert D["proj"].shape[0] == cols == D["bias"].numel() and D["qnorm"].numel() == m.dim
                assert tuple(D["o"].shape) == (W, m.heads * m.vdim)
            elif m.kind == "sink_attention":
                own = m.kv_from is None
                D["proj"] = put(torch.cat([t[p + "mix." + n] for n in (("q", "k", "v") if own else ("q",))], 0))
                D["qnorm"] = f32(t[p + "mix.q.norm"])
                D["knorm"] = f32(t[p + "mix.k.norm"]) if own else D["qnorm"]
                D["qscale"] = f32(t[p + "mix.temp"]) * m.scale         # score scale times the head's number
                D["o"] = put(t[p + "mix.o"])
                cols = m.heads * m.dim + (m.kv_heads * (m.dim + m.vdim) if own else 0)
                assert D["proj"].shape[0] == cols and D["qnorm"].numel() == m.heads * m.dim and D["qscale"].numel() == m.heads
                assert not own or D["knorm"].numel() == m.kv_heads * m.dim
                assert tuple(D["o"].shape) == (W, m.heads * m.vdim)
            elif m.kind == "mamba2":
                inner, bc = m.heads * m.vdim, 2 * m.groups * m.state
                D["in"], D["o"] = put(t[p + "mix.in"]), put(t[p + "mix.o"])
                D["conv"], D["conv_b"] = f32(t[p + "mix.conv"]), f32(t[p + "mix.conv.b"])
                D["dt_b"], D["D"] = f32(t[p + "mix.dt_bias"]), f32(t[p + "mix.D"])
                D["neg_a"], D["gnorm"] = -torch.exp(f32(t[p + "mix.A_log"])), f32(t[p + "mix.norm"])
                assert D["in"].shape[0] == 2 * inner + bc + m.heads and tuple(D["conv"].shape) == (inner + bc, m.conv)
                assert D["neg_a"].numel() == m.heads and D["gnorm"].numel() == inner
            elif m.kind == "mlstm":
                D["proj"] = put(torch.cat([t[p + "mix." + n] for n in ("q", "k", "v", "g", "i", "f")], 0))
                D["gate_b"] = f32(torch.cat([t[p + "mix.i.b"], t[p + "mix.f.b"]], 0))
                D["hnorm"], D["o"] = f32(t[p + "mix.norm"]), put(t[p + "mix.o"])
                assert D["proj"].shape[0] == 2 * m.heads * (m.dim + m.vdim + 1) and D["hnorm"].numel() == m.heads * m.vdim
            elif m.kind == "mamba1":
                D["in"], D["x"], D["dt"], D["o"] = (put(t[p + "mix." + n]) for n in ("in", "x", "dt", "o"))
                D["conv"], D["conv_b"] = f32(t[p + "mix.conv"]), f32(t[p + "mix.conv.b"])
                D["dt_b"], D["D"] = f32(t[p + "mix.dt.b"]), f32(t[p + "mix.D"])
                D["A"] = -torch.exp(f32(t[p + "mix.A_log"]))
                assert tuple(D["A"].shape) == (m.inner, m.state) and tuple(D["conv"].shape) == (m.inner, m.conv)
            elif m.kind == "retention":
                D["qkvg"] = put(torch.cat([t[p + "mix." + n] for n in "qkvg"], 0))
                D["o"] = put(t[p + "mix.o"])
                D["decay"] = torch.tensor(m.decay, dtype=torch.float32, device=dev)
                assert D["decay"].numel() == m.heads
            else:
                D["dqkv"] = put(torch.cat([t[p + "mix.dq"], t[p + "mix.dkv"]], 0))
                D["dq_norm"], D["dkv_norm"] = f32(t[p + "mix.dq.norm"]), f32(t[p + "mix.dkv.norm"])
                D["uq"], D["o"] = put(t[p + "mix.uq"]), put(t[p + "mix.o"])
                D["uk"] = put(t[p + "mix.uk"].view(m.heads, m.dim, m.kv_rank))                       # [H, d, r]
                D["uvT"] = put(t[p + "mix.uv"].view(m.heads, m.vdim, m.kv_rank).transpose(1, 2))    # [H, r, dv]
            f = L.mlp
            if f is not None:
                if lnb:
                    D["norm2.b"] = f32(t[p + "norm2.b"])
                if cfg.layer_scale:
                    D["ls2"] = f32(t[p + "ls2"])
            if isinstance(f, DenseSpec):
                D["norm2"], D["down"] = f32(t[p + "norm2"]), put(t[p + "mlp.down"])
                if f.act == "clamped_glu":     # one projection: gate rows, then up rows
                    D["up"] = put(torch.cat([t[p + "mlp.gate"], t[p + "mlp.up"]], 0))
                    assert tuple(D["up"].shape) == (2 * f.ff, W)
                else:
                    D["up"] = put(t[p + "mlp.up"])
                    assert tuple(D["up"].shape) == (f.ff, W)
                if f.bias:
                    names = ("gate", "up") if f.act == "clamped_glu" else ("up",)
                    D["up_b"] = f32(torch.cat([t[p + f"mlp.{n}.b"] for n in names], 0))
                    D["down_b"] = f32(t[p + "mlp.down.b"])
                    assert D["up_b"].numel() == D["up"].shape[0] and D["down_b"].numel() == W
                if cfg.pre_norm and cfg.post_norm:
                    D["norm2b"] = f32(t[p + "norm2b"])
                if f.act == "polynorm":
                    D["act"] = f32(t[p + "mlp.act"])
                    assert D["act"].numel() == 4
            elif f is not None:
                D["norm2"] = f32(t[p + "norm2"])
                D["router"] = put(t[p + "mlp.router"])
                if f.score == "sigmoid" or not f.renorm:
                    D["router"] = f32(t[p + "mlp.router"])     # the router runs in f32
                    assert tuple(D["router"].shape) == (f.experts + f.identity, W)
                if f.shared_gate:     # the shared expert's gate logit is one more row of the router's GEMM
                    D["router"] = torch.cat([D["router"], f32(t[p + "mlp.shared.sg"]).view(1, W)], 0).contiguous()
                if f.correction:
                    D["corr"] = f32(t[p + "mlp.correction"])
                    assert D["corr"].numel() == f.experts + f.identity
                if f.act == "swiglu":      # per expert: gate rows, then up rows
                    w1 = torch.stack([torch.cat([t[p + f"mlp.e{e}.gate"], t[p + f"mlp.e{e}.up"]], 0)
                                      for e in range(f.experts)])                         # [E, 2 ff, W]
                else:
                    w1 = torch.stack([t[p + f"mlp.e{e}.up"] for e in range(f.experts)])   # [E, ff, W]
                w2 = torch.stack([t[p + f"mlp.e{e}.down"] for e in range(f.experts)])     # [E, W, ff]
                grouped = (dt == torch.bfloat16 and dev.type == "cuda" and W % 32 == 0 and f.ff % 32 == 0
                           and f.experts <= 64)
                if f.act == "swiglu" and grouped and W % 64 == 0 and f.ff % 64 == 0:
                    # the LDS-tiled grouped GEMM pairs gate and up rows in its epilogue: rows interleaved
                    from .llama import gate_up_order
                    w1 = w1.index_select(1, gate_up_order(f.ff))
                    D["tg"] = True
                D["w1"] = put(w1)
                if grouped or dev.type != "cuda":
                    D["w2"] = put(w2)
                else:   # dense form: one down projection over every expert's columns
                    D["w2d"] = put(w2.permute(1, 0, 2).reshape(W, f.experts * f.ff))
                if f.shared_ff:
                    D["sh_up"], D["sh_down"] = put(t[p + "mlp.shared.up"]), put(t[p + "mlp.shared.down"])
                    if f.act == "swiglu":     # gate rows, then up rows
                        D["sh_up"] = put(torch.cat([t[p + "mlp.shared.gate"], t[p + "mlp.shared.up"]], 0))
                    assert D["sh_down"].shape[1] == f.shared_ff
            self.layers.append(D)

    def weight_bytes(self) -> int:
        n = sum(x.numel() * x.element_size() for x in (self.embed, self.final_norm))
        n += 0 if self.cfg.tied_head else self.lm_head.numel() * self.lm_head.element_size()
        return n + sum(x.numel() * x.element_size() for L in self.layers for x in L.values() if torch.is_tensor(x))

    def decode_read_bytes(self, top_only: bool = True) -> int:
        """Weight bytes one decode token reads (routed experts: ``top`` of them)."""
        n = self.lm_head.numel() * self.lm_head.element_size()
        for L, S in zip(self.layers, self.cfg.layers):
            for k, x in L.items():
                if not torch.is_tensor(x):
                    continue
                b = x.numel() * x.element_size()
                if k in ("w1", "w2", "w2d") and top_only and isinstance(S.mlp, MoESpec):
                    b = b * S.mlp.top // S.mlp.experts
                n += b
        return n

    # ------------------------------------------------------------------ positions, caches
    def ensure_positions(self, n: int) -> None:
        """cos | sin tables (f64 on the host, stored f32) for positions < n of every rotation used."""
        if n <= self._max_pos:
            return
        self._max_pos = n
        for L in self.cfg.layers:
            for m in L.mixer.parts:
                r = m.rot
                if r is not None and r.dims > 0:
                    self._rot[(r.dims, r.base)] = ops.rope_cos_sin(n, r.dims, r.base, self.device)

    def _table(self, m: MixerSpec) -> torch.Tensor:
        return self._rot[(m.rot.dims, m.rot.base)]

    def block_bytes(self, block_size: int) -> int:
        """Bytes of one paged block over all layers (latent attention layers only)."""
        it = torch.empty((), dtype=self.dtype).element_size()
        n = 0
        for L in self.cfg.layers:
            for m in L.mixer.parts:
                if m.kind == "latent_attention":
                    n += block_size * (m.kv_rank + m.rot_dim) * it
                elif m.kind == "softmax_attention":
                    n += block_size * m.kv_heads * (m.dim + m.vdim) * it
                elif m.kind == "diff_attention" and m.kv_from is None:
                    n += block_size * m.kv_heads * (2 * m.dim + m.vdim) * it
                elif m.kind == "sink_attention" and m.kv_from is None:
                    n += block_size * m.kv_heads * (m.dim + m.vdim) * it
        return n

    def alloc_caches(self, num_blocks: int, block_size: int, slots: int) -> List[tuple]:
        """Per layer: (paged latent [blocks, block, rank + rot],) or the recurrent state of ``slots``
        sequences: (conv inputs [slots, taps - 1, inner], scan state [slots, inner, state] f32) /
        (retention state [slots, heads, dim, vdim] f32,) / delta: (conv inputs [slots, taps - 1,
        q | k | v channels], state [slots, heads, vdim, dim] f32) / parallel: (paged keys [blocks,
        kv_heads, block, dim], paged values [blocks, kv_heads, vdim, block], lightning state [slots,
        heads, dim, vdim] f32) / diff_attention: (paged keys [blocks, 2 kv_heads, block, dim], paged
        values [blocks, kv_heads, vdim, block]), for a layer with ``kv_from`` the tensors of that
        layer / mamba2: (conv inputs [slots, taps - 1, x | B | C channels], state [slots, heads, N,
        vdim] f32) / mlstm: (memory [slots, heads, dim, vdim] f32, normaliser and maximum [slots,
        heads, column blocks, dim + 1] f32) / sink_attention: (paged keys [blocks, kv_heads, block,
        dim], paged values [blocks, kv_heads, vdim, block]), of the layer ``kv_from`` names if any.
        With an input convolution every layer's tuple ends with its own last inputs [slots, taps - 1,
        width]."""
        dev, out = self.device, []
        for L in self.cfg.layers:
            m = L.mixer
            if m.kind == "sink_attention":
                if m.kv_from is not None:
                    out.append(out[m.kv_from][:2])
                else:
                    out.append((torch.zeros((num_blocks, m.kv_heads, block_size, m.dim), dtype=self.dtype, device=dev),
                                torch.zeros((num_blocks, m.kv_heads, m.vdim, block_size), dtype=self.dtype, device=dev)))
            elif m.kind == "diff_attention":
                if m.kv_from is not None:
                    out.append(out[m.kv_from])
                else:
                    out.append((torch.zeros((num_blocks, 2 * m.kv_heads, block_size, m.dim), dtype=self.dtype, device=dev),
                                torch.zeros((num_blocks, m.kv_heads, m.vdim, block_size), dtype=self.dtype, device=dev)))
            elif m.kind == "mamba2":
                c = m.heads * m.vdim + 2 * m.groups * m.state
                out.append((torch.zeros((slots, max(m.conv - 1, 0), c), dtype=self.dtype, device=dev),
                            torch.zeros((slots, m.heads, m.state, m.vdim), dtype=torch.float32, device=dev)))
            elif m.kind == "mlstm":
                out.append((torch.zeros((slots, m.heads, m.dim, m.vdim), dtype=torch.float32, device=dev),
                            torch.zeros((slots, m.heads, seqmix.scan_col_blocks(m.vdim), m.dim + 1), dtype=torch.float32,
                                        device=dev)))
            elif m.kind == "delta":
                c = 2 * m.kv_heads * m.dim + m.heads * m.vdim
                out.append((torch.zeros((slots, max(m.conv - 1, 0), c), dtype=self.dtype, device=dev),
                            torch.zeros((slots, m.heads, m.vdim, m.dim), dtype=torch.float32, device=dev)))
            elif m.kind == "parallel":
                a, b = m.left, m.right
                out.append((torch.zeros((num_blocks, a.kv_heads, block_size, a.dim), dtype=self.dtype, device=dev),
                            torch.zeros((num_blocks, a.kv_heads, a.vdim, block_size), dtype=self.dtype, device=dev),
                            torch.zeros((slots, b.heads, b.dim, b.vdim), dtype=torch.float32, device=dev)))
            elif m.kind == "mamba1":
                out.append((torch.zeros((slots, max(m.conv - 1, 0), m.inner), dtype=self.dtype, device=dev),
                            torch.zeros((slots, m.inner, m.state), dtype=torch.float32, device=dev)))
            elif m.kind == "retention":
                out.append((torch.zeros((slots, m.heads, m.dim, m.vdim), dtype=torch.float32, device=dev),))
            else:
                out.append((torch.zeros((num_blocks, block_size, m.kv_rank + m.rot_dim), dtype=self.dtype, device=dev),))
            if self.cfg.input_conv:
                out[-1] = out[-1] + (torch.zeros((slots, max(self.cfg.input_conv - 1, 0), self.cfg.hidden),
                                                 dtype=self.dtype, device=dev),)
        return out

    # ------------------------------------------------------------------ mixers
    def _mamba(self, L, m: MixerSpec, x, meta, cache):
        conv_state, ssm_state = cache
        rows = meta.state_rows
        xz = _mm(x, L["in"])
        xc = seqmix.causal_conv_silu(xz, L["conv"], L["conv_b"], conv_state, meta.qstart, meta.qlen, meta.ctx, rows)
        dbc = _mm(xc, L["x"])
        dt_raw = _mm(dbc[:, :m.dt_rank], L["dt"])
        y = seqmix.selective_scan(xc, dt_raw, L["dt_b"], L["A"], dbc, m.dt_rank, L["D"], xz, ssm_state, conv_state,
                                  meta.qstart, meta.qlen, meta.ctx, rows)
        return _mm(y, L["o"])

    def _retention(self, L, m: MixerSpec, x, positions, meta, cache):
        qkvg = _mm(x, L["qkvg"])
        rot = m.rot.dims if m.rot is not None else 0
        table = self._table(m) if rot else self._any_table()
        o = seqmix.retention(qkvg, m.heads, m.dim, m.vdim, table, rot, L["decay"], cache[0], self.cfg.rms_eps,
                             positions, meta.qstart, meta.qlen, meta.ctx, meta.state_rows)
        return _mm(o, L["o"])

    def _any_table(self) -> torch.Tensor:
        if not self._rot:
            self._rot[(2, 1.0)] = ops.rope_cos_sin(self._max_pos, 2, 1.0, self.device)
        return next(iter(self._rot.values()))

    def _latent(self, L, m: MixerSpec, x, positions, meta, cache):
        T, H, eps = x.shape[0], m.heads, self.cfg.rms_eps
        down = _mm(x, L["dqkv"])
        cq = seqmix.rms_rows(down[:, :m.q_rank], L["dq_norm"], eps)
        q = _mm(cq, L["uq"])                                            # [T, H (dim + rot)]
        table = self._table(m)
        seqmix.latent_kv_write(down[:, m.q_rank:], m.kv_rank, L["dkv_norm"], eps, positions, table, meta.slots,
                               cache[0])
        qn = q.view(T, H, m.dim + m.rot_dim)[:, :, :m.dim].transpose(0, 1)
        qa = torch.bmm(qn, L["uk"])                                     # key up-projection absorbed: [H, T, rank]
        rows = (seqmix.LAT_ROWS if meta.host_qlen is None else
                seqmix.latent_rows(x, m.kv_rank, m.rot_dim, T, len(meta.host_qlen)))
        ts, tr = meta.latent_tiles(H, self.device, rows)
        lat = seqmix.latent_attention(qa, q, m.dim, m.rot_dim, positions, table, cache[0], meta.block_tables,
                                      meta.qstart, meta.qlen, meta.ctx, ts, tr, m.scale, rows=rows)
        o = torch.bmm(lat, L["uvT"])                                    # [H, T, vdim]
        return _mm(o.transpose(0, 1).reshape(T, H * m.vdim), L["o"])

    @staticmethod
    def _left_cols(a: MixerSpec) -> int:
        """Columns of the softmax side in the fused projection: q | k | v | gate."""
        return (a.heads + a.kv_heads) * a.dim + a.kv_heads * a.vdim + a.heads * a.vdim

    def _delta(self, L, m: MixerSpec, x, meta, cache):
        conv_state, state = cache
        rows = meta.state_rows
        c = 2 * m.kv_heads * m.dim + m.heads * m.vdim
        proj = _mm(x, L["proj"])                                        # q | k | v | gate | beta | decay logits
        single = meta.host_qlen is None      # a decode step: the convolution refills its slots itself
        qkv = seqmix.causal_conv_silu(proj, L["conv"], L["conv_b"], conv_state, meta.qstart, meta.qlen, meta.ctx, rows,
                                      refill=single)
        if not single:
            seqmix.conv_state_refill(proj, conv_state, meta.qstart, meta.qlen, meta.ctx, rows)
        o = seqmix.delta_rule(qkv, proj[:, c:], m.heads, m.kv_heads, m.dim, m.vdim, L["neg_a"], L["dt_b"], L["hnorm"],
                              self.cfg.rms_eps, state, meta.qstart, meta.qlen, meta.ctx, rows)
        return _mm(o, L["o"])

    def _parallel(self, L, m: MixerSpec, x, positions, meta, cache):
        """Both sides' outputs, un-normed: the caller's residual launch norms and averages them."""
        a, b, eps = m.left, m.right, self.cfg.rms_eps
        k_cache, v_cache, state = cache
        proj = _mm(x, L["proj"])
        nl = self._left_cols(a)
        rot = a.rot.dims if a.rot is not None else 0
        table = self._table(a) if rot else self._any_table()
        q = seqmix.attn_prep(proj, a.heads, a.kv_heads, a.dim, a.vdim, table, rot, eps, L["qscale"], positions,
                             meta.slots, k_cache, v_cache)
        mfma = seqmix.gqa_use_mfma(q, a.heads, a.kv_heads, a.dim, a.vdim, k_cache.shape[2])
        ts, tt = meta.latent_tiles(1, self.device, seqmix.gqa_tokens_per_tile(a.heads, a.kv_heads, mfma))
        gate = proj[:, nl - a.heads * a.vdim:nl]
        splits = seqmix.gqa_splits(int(ts.numel()), a.kv_heads, meta.max_ctx) if mfma else 1
        lo = seqmix.paged_gqa_attention(q, k_cache, v_cache, meta.block_tables, meta.qstart, meta.qlen, meta.ctx, ts, tt,
                                        gate, mfma, splits)
        ro = seqmix.lightning_attention(proj[:, nl:], b.heads, b.dim, b.vdim, L["decay"], state, eps, L["rnorm"],
                                        meta.qstart, meta.qlen, meta.ctx, meta.state_rows)
        return _mm(lo, L["lo"]), _mm(ro, L["ro"])

    def _diff_attention(self, L, m: MixerSpec, x, positions, meta, cache):
        """Both maps of every head run as rows of one grouped-query attention over 2 kv_heads key
        heads and kv_heads shared value heads; the maps are combined afterwards."""
        k_cache, v_cache = cache
        own = m.kv_from is None
        proj = _mm(x, L["proj"])
        rot = m.rot.dims if m.rot is not None else 0
        table = self._table(m) if rot else self._any_table()
        q = seqmix.qk_norm_prep(proj, L["bias"], m.heads, m.kv_heads, 2, m.dim, m.vdim, L["qnorm"], L["knorm"], table, rot,
                                self.cfg.rms_eps, m.scale, positions, meta.slots, k_cache if own else None,
                                v_cache if own else None)
        H2, G2 = 2 * m.heads, 2 * m.kv_heads
        mfma = seqmix.gqa_use_mfma(q, H2, G2, m.dim, m.vdim, k_cache.shape[2])
        ts, tt = meta.latent_tiles(1, self.device, seqmix.gqa_tokens_per_tile(H2, G2, mfma))
        splits = seqmix.gqa_splits(int(ts.numel()), G2, meta.max_ctx, m.window) if mfma else 1
        a = seqmix.paged_gqa_attention(q, k_cache, v_cache, meta.block_tables, meta.qstart, meta.qlen, meta.ctx, ts, tt,
                                       None, mfma, splits, window=m.window, out_f32=True)
        o = seqmix.diff_combine(a, m.heads, m.kv_heads, m.vdim, L["lam"], self.cfg.rms_eps, 1.0 - m.diff, self.dtype)
        return _mm(o, L["o"])

    def _input_conv(self, L, h, meta, state):
        """h + a short causal convolution of h over time (per channel, no activation); the slot keeps
        the sequence's last inputs."""
        single = meta.host_qlen is None      # a decode step: the convolution refills its slots itself
        y = seqmix.causal_conv_silu(h, L["canon"], L["canon_b"], state, meta.qstart, meta.qlen, meta.ctx,
                                    meta.state_rows, refill=single, act="residual", all_rows=self._all_rows(h, meta),
                                    inplace=single)
        if not single:
            seqmix.conv_state_refill(h, state, meta.qstart, meta.qlen, meta.ctx, meta.state_rows)
        return y

    def _sink_attention(self, L, m: MixerSpec, x, positions, meta, cache):
        k_cache, v_cache = cache[0], cache[1]
        own = m.kv_from is None
        proj = _mm(x, L["proj"])                                        # q | k | v, or q alone
        rot = m.rot.dims if m.rot is not None else 0
        table = self._table(m) if rot else self._any_table()
        # a step with padding rows (decode graphs): the prep launch clears the attention output's rows
        out = None if self._all_rows(x, meta) else torch.empty((x.shape[0], m.heads * m.vdim), dtype=x.dtype, device=x.device)
        q = seqmix.proj_norm_prep(proj, m.heads, m.kv_heads, m.dim, m.vdim, L["qnorm"], L["knorm"], table, rot, True,
                                  self.cfg.rms_eps, L["qscale"], True, positions, meta.slots, k_cache if own else None,
                                  v_cache if own else None, zero_rows=out)
        mfma = seqmix.gqa_use_mfma(q, m.heads, m.kv_heads, m.dim, m.vdim, k_cache.shape[2])
        ts, tt = meta.latent_tiles(1, self.device, seqmix.gqa_tokens_per_tile(m.heads, m.kv_heads, mfma))
        splits = seqmix.gqa_splits(int(ts.numel()), m.kv_heads, meta.max_ctx, m.window, m.keep_first) if mfma else 1
        o = seqmix.paged_gqa_attention(q, k_cache, v_cache, meta.block_tables, meta.qstart, meta.qlen, meta.ctx, ts, tt,
                                       None, mfma, splits, window=m.window, keep_first=m.keep_first, sink=m.sink,
                                       all_rows=self._all_rows(x, meta), out=out)
        return _mm(o, L["o"])

    @staticmethod
    def _all_rows(x, meta) -> bool:
        """A step of prompt portions whose sequences cover every packed row (no padding rows)."""
        return meta.host_qlen is not None and sum(int(n) for n in meta.host_qlen) == x.shape[0]

    def _mamba2(self, L, m: MixerSpec, x, meta, cache):
        conv_state, state = cache
        rows = meta.state_rows
        inner = m.heads * m.vdim
        proj = _mm(x, L["in"])                                          # z | x | B | C | dt
        xbc_in = proj[:, inner:]
        single = meta.host_qlen is None      # a decode step: the convolution refills its slots itself
        xbc = seqmix.causal_conv_silu(xbc_in, L["conv"], L["conv_b"], conv_state, meta.qstart, meta.qlen, meta.ctx, rows,
                                      refill=single)
        if not single:
            seqmix.conv_state_refill(xbc_in, conv_state, meta.qstart, meta.qlen, meta.ctx, rows)
        y = seqmix.ssd_scan(xbc, proj, 2 * inner + 2 * m.groups * m.state, m.heads, m.vdim, m.state, m.groups, L["dt_b"],
                            L["neg_a"], L["D"], state, meta.qstart, meta.qlen, meta.ctx, rows)
        return _mm(seqmix.gated_group_norm(y, proj, L["gnorm"], m.norm_groups, self.cfg.rms_eps, self.dtype), L["o"])

    def _mlstm(self, L, m: MixerSpec, x, meta, cache):
        state, nm = cache
        proj = _mm(x, L["proj"])                                        # q | k | v | gate | input gate | forget gate
        o = seqmix.mlstm(proj, m.heads, m.dim, m.vdim, L["gate_b"], m.gate_cap, state, nm, self.cfg.rms_eps, L["hnorm"],
                         meta.qstart, meta.qlen, meta.ctx, meta.state_rows)
        return _mm(o, L["o"])

    def _dense(self, L, f: DenseSpec, x):
        z = _mm(x, L["up"])
        if f.act == "clamped_glu":      # the down projection's bias rides in the residual launch
            a = seqmix.glu_act(z, L.get("up_b"), "clamped", f.limit, 1.702)
        else:
            a = seqmix.polynorm(z, L["act"], self.cfg.rms_eps) if f.act == "polynorm" else seqmix.gelu_erf(z)
        return _mm(a, L["down"])

    def _experts_swiglu(self, L, f: MoESpec, x):
        """Sigmoid router in f32 with group-limited top-k, weights = the chosen scores; SwiGLU experts
        on the grouped MFMA kernels, or in the dense form (all experts' columns in two GEMMs, unused
        experts gated to zero) for f32 models and widths the grouped kernels do not take."""
        logits = F.linear(x.float(), L["router"])
        ids, w = seqmix.group_router(logits, f.top, f.group_count, f.group_keep)
        if f.scale != 1.0:
            w = w * f.scale
        return self._swiglu_experts(L, f, x, ids, w)

    def _experts_terms(self, L, f: MoESpec, x) -> dict:
        """Softmax router in f32 whose choice (not its weights) sees a learned correction, group-limited
        top-k over experts and identity experts together, weights = the chosen scores; returns the
        terms of the residual launch (ops.seqmix.ls_resadd_ln): the routed experts' sum, the input
        times the identity experts' weights, the shared expert and its gate logit."""
        logits = F.linear(x.float(), L["router"])      # [T, experts + identity (+ 1: the shared expert's gate)]
        R = f.experts + f.identity
        ids, w, idw = seqmix.route_topk(logits, R, f.top, f.group_count, f.group_keep, f.score, f.group_score,
                                        L.get("corr"), f.experts)
        if f.scale != 1.0:
            w, idw = w * f.scale, idw * f.scale
        out = dict(y=self._swiglu_experts(L, f, x, ids, w))
        if f.identity:
            out.update(h=x, hw=idw)
        if f.shared_ff:
            out.update(y2=_mm(seqmix.glu_act(_mm(x, L["sh_up"])), L["sh_down"]), g2=logits[:, R] if f.shared_gate else None)
        return out

    def _swiglu_experts(self, L, f: MoESpec, x, ids, w):
        """sum_j w[t, j] expert_(ids[t, j])(x_t); ids beyond the experts (identity experts, whose weight
        here is 0) add nothing."""
        if L.get("tg"):
            return ops.moe_ffn_tg(x if x.stride(1) == 1 else x.contiguous(), ids, w, L["w1"], L["w2"])
        if "w2" in L and (not x.is_cuda or seqmix.moe_ffn_relu2_ok(x, L["w1"])):
            return ops.moe_ffn(x, ids, w, L["w1"], L["w2"])
        if "w2d" not in L:
            L["w2d"] = L["w2"].permute(1, 0, 2).reshape(x.shape[1], -1).contiguous()
        g = seqmix.dense_gate(ids, w, f.experts)
        a = seqmix.swiglu_scale(_mm(x, L["w1"].view(f.experts * 2 * f.ff, -1)), g, f.ff)
        return _mm(a, L["w2d"])

    def _experts(self, L, f: MoESpec, x):
        if f.act == "swiglu":
            return self._experts_swiglu(L, f, x)
        if f.experts > 64 or f.top > 8:      # beyond the router kernels' register budget: library top-k
            val, ids = torch.topk(torch.softmax(F.linear(x.float(), L["router"].float()), -1), f.top, -1)
            ids, w = ids.to(torch.int32), val / (val.sum(-1, keepdim=True) + 1e-20)
        elif x.is_cuda and x.dtype == torch.bfloat16:
            ids, w = ops.moe_router(x, L["router"], f.top)      # f32 logits, softmax over the chosen = s / sum s
        else:
            ids, w = ops.moe_gate(F.linear(x.float(), L["router"].float()), f.top)
        w = w * f.scale
        if "w2" in L and (not x.is_cuda or seqmix.moe_ffn_relu2_ok(x, L["w1"])):
            y = seqmix.moe_ffn_relu2(x, ids, w, L["w1"], L["w2"])
        else:
            if "w2d" not in L:
                L["w2d"] = L["w2"].permute(1, 0, 2).reshape(x.shape[1], -1).contiguous()
            g = seqmix.dense_gate(ids, w, f.experts)
            a = seqmix.relu2_scale(_mm(x, L["w1"].view(f.experts * f.ff, -1)), g, f.ff)
            y = _mm(a, L["w2d"])
        if f.shared_ff:
            y = y + _mm(seqmix.relu2_scale(_mm(x, L["sh_up"])), L["sh_down"])
        return y

    # ------------------------------------------------------------------ forward
    def hidden_states(self, input_ids: torch.Tensor, positions: torch.Tensor, meta, kv_caches: List[tuple],
                      scatter: Optional[Tuple[torch.Tensor, torch.Tensor]] = None) -> torch.Tensor:
        """Final-normed hidden states of the packed rows ``meta.last_idx`` (every row when
        ``meta.all_last``): [S, width] in the model dtype."""
        cfg, eps = self.cfg, self.cfg.rms_eps
        if scatter is not None:
            ops.scatter_pairs(*scatter)
        if self.dtype == torch.bfloat16:
            if cfg.hidden % 8 == 0:
                xl = ops.embedding(input_ids, self.embed)
            else:      # the gather kernel moves 16-byte vectors
                xl = self.embed.index_select(0, input_ids.long())
            x = xl.float()
        else:
            x = self.embed.index_select(0, input_ids.long())
            xl = None
        if cfg.embed_scale != 1.0:
            x = x * cfg.embed_scale      # f32; the pre-norm layers read their own normed copy
            xl = None if xl is None else x.to(self.dtype)
        T, W, nL = x.shape[0], cfg.hidden, len(self.layers)
        X = None
        if cfg.depth_average:
            # f32 stack of the embedding output and every layer's result; layer i works in place on
            # slot i + 1, which the previous layer's weighted sum has filled with its input
            X = torch.empty((nL + 2, T, W), dtype=torch.float32, device=x.device)
            X[0].copy_(x)
            X[1].copy_(x)
            x = X[1]
        h = None
        ln = cfg.norm_kind == "layer"
        if ln:
            h = seqmix.ls_resadd_ln(x, self.layers[0]["norm1"], self.layers[0]["norm1.b"], eps, self.dtype)
        elif cfg.pre_norm:
            h = seqmix.rms_rows(x, self.layers[0]["norm1"], eps, out_dtype=self.dtype)
        for i, (L, S, cache) in enumerate(zip(self.layers, cfg.layers, kv_caches)):
            m = S.mixer
            if not cfg.pre_norm:
                h = x if xl is None else xl
            if cfg.input_conv:
                h = self._input_conv(L, h, meta, cache[-1])
            if m.kind == "mamba1":
                y = self._mamba(L, m, h, meta, cache)
            elif m.kind == "retention":
                y = self._retention(L, m, h, positions, meta, cache)
            elif m.kind == "delta":
                y = self._delta(L, m, h, meta, cache)
            elif m.kind == "parallel":
                y = self._parallel(L, m, h, positions, meta, cache)
            elif m.kind == "diff_attention":
                y = self._diff_attention(L, m, h, positions, meta, cache)
            elif m.kind == "mamba2":
                y = self._mamba2(L, m, h, meta, cache)
            elif m.kind == "mlstm":
                y = self._mlstm(L, m, h, meta, cache)
            elif m.kind == "sink_attention":
                y = self._sink_attention(L, m, h, positions, meta, cache)
            else:
                y = self._latent(L, m, h, positions, meta, cache)
            if ln:
                # x += ls * sublayer, and the layer norm ahead of the next sublayer, in one launch
                nw, nb = (self.layers[i + 1]["norm1"], self.layers[i + 1]["norm1.b"]) if i + 1 < nL else \
                    (self.final_norm, self.final_norm_b)
                if S.mlp is not None:
                    h = seqmix.ls_resadd_ln(x, L["norm2"], L["norm2.b"], eps, self.dtype, y=y, ls=L.get("ls1"))
                    terms = dict(y=self._dense(L, S.mlp, h), bias=L.get("down_b")) if isinstance(S.mlp, DenseSpec) else \
                        self._experts_terms(L, S.mlp, h)
                    h = seqmix.ls_resadd_ln(x, nw, nb, eps, self.dtype, ls=L.get("ls2"), **terms)
                else:
                    h = seqmix.ls_resadd_ln(x, nw, nb, eps, self.dtype, y=y, ls=L.get("ls1"))
            elif cfg.pre_norm:
                # the sublayer's tail and the next sublayer's input norm in one launch
                nxt = self.layers[i + 1]["norm1"] if i + 1 < nL else self.final_norm
                pair = dict(b=y[1], wa=L["lout"], wb=L["rout"]) if isinstance(y, tuple) else {}
                a = y[0] if isinstance(y, tuple) else y
                if S.mlp is not None:
                    h = torch.empty((T, W), dtype=self.dtype, device=x.device)
                    seqmix.resadd_norm(a, L["norm1b"], eps, x, L["norm2"], h, **pair)
                    y = self._dense(L, S.mlp, h) if isinstance(S.mlp, DenseSpec) else self._experts(L, S.mlp, h)
                    a, pair, post = y, {}, L["norm2b"]
                else:
                    post = L["norm1b"]
                if X is not None:     # ... and the layer's weighted sum over depth
                    h = torch.empty((T, W), dtype=self.dtype, device=x.device)
                    x = seqmix.resadd_norm(a, post, eps, x, nxt, h, depth=(X, L["dwa"], i + 2), **pair)
                else:
                    h = torch.empty((T, W), dtype=self.dtype, device=x.device)
                    seqmix.resadd_norm(a, post, eps, x, nxt, h, **pair)
            else:
                ng = cfg.norm_groups
                seqmix.norm_resadd(y, L["norm1"], eps, x, xl, groups=ng, bias=L.get("ob"))
                if S.mlp is not None:
                    hin = x if xl is None else xl
                    y = self._dense(L, S.mlp, hin) if isinstance(S.mlp, DenseSpec) else self._experts(L, S.mlp, hin)
                    seqmix.norm_resadd(y, L["norm2"], eps, x, xl, groups=ng)
                if X is not None:
                    x = seqmix.depth_mix(X, L["dwa"], i + 2)
                    if xl is not None:
                        xl.copy_(x)
            if self.tap is not None:
                self.tap.append(x.clone())
        if cfg.pre_norm:     # h is the final-normed stream of every row
            return h if meta.all_last else h.index_select(0, meta.last_idx)
        sel = x if meta.all_last else x.index_select(0, meta.last_idx)
        return seqmix.rms_rows(sel, self.final_norm, eps, out_dtype=self.dtype, groups=cfg.norm_groups)

    def logits(self, hidden: torch.Tensor) -> torch.Tensor:
        lg = _mm(hidden, self.lm_head)
        if self.cfg.logit_softcap > 0:
            return seqmix.softcap(lg, self.cfg.logit_softcap).to(lg.dtype)
        return lg if self.cfg.logit_scale == 1.0 else lg * self.cfg.logit_scale

    def logits_f32(self, hidden: torch.Tensor) -> torch.Tensor:
        lg = _mm(hidden, self.lm_head)
        if self.cfg.logit_softcap > 0:
            return seqmix.softcap(lg, self.cfg.logit_softcap)
        return lg.float() * self.cfg.logit_scale

    def _sampler_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """bf16 logits [S, vocab] whose rows start 16-byte aligned (the sampler kernels read vectors)."""
        lg = self.logits(hidden)
        V = lg.shape[1]
        if V % 8 == 0 or not lg.is_cuda:
            return lg.to(torch.bfloat16)
        buf = torch.zeros((lg.shape[0], (V + 7) // 8 * 8), dtype=torch.bfloat16, device=lg.device)
        buf[:, :V].copy_(lg)
        return buf[:, :V]

    def greedy(self, hidden: torch.Tensor) -> torch.Tensor:
        return ops.argmax(self._sampler_logits(hidden))

    def sample(self, hidden, temperature, top_p, top_k, seed, out):
        return ops.sample_rows(self._sampler_logits(hidden), temperature, top_p, top_k, seed, out=out)

    def topk_candidates(self, hidden: torch.Tensor, k: int):
        v, i = torch.topk(self.logits(hidden).float(), min(k, self.cfg.vocab), dim=-1)
        return v.contiguous(), i.contiguous()
