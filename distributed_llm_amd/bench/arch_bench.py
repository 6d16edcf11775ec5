"""Layer-list (Filevik, Sedopel, Pebodra, Dogilorn) models beside the closest Llama-family model at equal size:
prefill and decode throughput through the engine, and the time of each mixer kernel against its roofline.

``python bench.py --arch-bench [--arch-design filevik|sedopel|pebodra|dogilorn] [--arch-size s|m]`` (random
weights, synthetic tokens).  The default bench workload and its JSON line are untouched; this prints one
JSON object of its own.

The Dogilorn stack is attention only (grouped-query, an RMS norm over the whole q and k projections,
a sliding window that also keeps the first tokens, a sink term in the softmax; every third layer reads
the keys and values of the layer before it), behind an input convolution and layer norms; its
feed-forwards alternate between a dense clamped GLU and routed SwiGLU experts with identity experts
and a gated shared expert.  Its comparison model is the Mixtral-style Llama of the same width, depth
and experts, and kernel by kernel: attention against the Pebodra and Sedopel attention (the same
kernels with other options) and the Llama kernels at the same heads, its prep, convolution, residual
and router launches against the like launches of the other designs.

The Sedopel stack alternates parallel layers (grouped-query softmax attention beside lightning
attention, dense GELU feed-forward) and gated-delta-rule layers without a feed-forward; its
comparison model is a dense Llama (grouped-query attention + SwiGLU of equal parameter count) of
the same width and depth, and kernel by kernel: paged attention against the Llama attention kernels
at the same head counts, lightning attention against retention, the delta rule against the
selective scan.

The Pebodra stack cycles differential sliding-window attention -> mLSTM -> attention on the first
layer's keys and values -> Mamba-2, the first layer with a dense PolyNorm feed-forward and the
others with group-routed SwiGLU experts; its comparison model is the Mixtral-style Llama of the same
width, depth and experts, and kernel by kernel: windowed attention with two maps a head against the
Sedopel attention kernel (the same kernel without a window) and the Llama kernels at the same
number of score rows, Mamba-2 against the selective scan and the delta rule, mLSTM against retention.

Sizes: width / layers of a small and a mid-size decoder.  The Filevik stack cycles mamba1 ->
retention -> latent attention, each with routed squared-ReLU experts and a shared expert; the
comparison model is a Mixtral-style Llama (grouped-query attention + SwiGLU experts) with the same
width, layer count, expert count / top-k and per-token expert width.
"""
from __future__ import annotations

import json
import time
from typing import Dict, List

import torch

PEAK_BW = 8.0e12          # HBM3E bytes/s
PEAK_BF16 = 2.5e15        # dense bf16 MFMA flop/s
PEAK_F32 = 157e12         # f32 vector flop/s

SIZES = {
    "s": dict(width=1024, layers=6, inner=2048, state=16, dt_rank=64, conv=4, heads=8, dim=64, vdim=128, rot=64,
              lat_heads=16, lat_dim=64, lat_rot=32, lat_v=64, kv_rank=256, q_rank=768, experts=8, top=2, ff=1024,
              shared=1024, vocab=32000),
    "m": dict(width=2048, layers=12, inner=4096, state=16, dt_rank=128, conv=4, heads=16, dim=128, vdim=128, rot=64,
              lat_heads=16, lat_dim=128, lat_rot=64, lat_v=128, kv_rank=512, q_rank=1536, experts=8, top=2, ff=2048,
              shared=2048, vocab=32000),
}


SEDOPEL_SIZES = {
    "s": dict(width=1024, layers=6, heads=16, kv_heads=4, dim=64, vdim=64, rot=32, l_heads=8, l_dim=64, l_vdim=128,
              d_heads=8, d_kv_heads=4, d_dim=128, d_vdim=128, conv=4, ff=4096, vocab=32000),
    "m": dict(width=2048, layers=12, heads=32, kv_heads=8, dim=64, vdim=64, rot=32, l_heads=16, l_dim=128, l_vdim=128,
              d_heads=16, d_kv_heads=8, d_dim=128, d_vdim=128, conv=4, ff=8192, vocab=32000),
}


PEBODRA_SIZES = {
    "s": dict(width=1024, layers=6, heads=8, kv_heads=2, dim=64, vdim=128, rot=64, window=1024, m_heads=32, m_vdim=64,
              state=128, groups=4, conv=4, norm_groups=8, x_heads=8, x_dim=64, x_vdim=128, experts=8, top=2, ff=1024,
              dense_ff=4096, vocab=32000),
    "m": dict(width=2048, layers=12, heads=16, kv_heads=4, dim=64, vdim=128, rot=64, window=1024, m_heads=64, m_vdim=64,
              state=128, groups=8, conv=4, norm_groups=8, x_heads=16, x_dim=128, x_vdim=128, experts=8, top=2, ff=2048,
              dense_ff=8192, vocab=32000),
}


DOGILORN_SIZES = {
    "s": dict(width=1024, layers=6, heads=16, kv_heads=4, dim=64, vdim=64, rot=32, window=1024, keep_first=64, taps=4,
              experts=8, identity=2, top=2, ff=1024, shared=1024, dense_ff=4096, vocab=32000),
    "m": dict(width=2048, layers=12, heads=16, kv_heads=4, dim=128, vdim=128, rot=64, window=1024, keep_first=128, taps=4,
              experts=8, identity=2, top=2, ff=2048, shared=2048, dense_ff=8192, vocab=32000),
}


def dogilorn_raw(z: dict) -> dict:
    moe = {"kind": "moe", "expert": {"ff": z["ff"]}, "shared": {"ff": z["shared"]},
           "router": {"experts": z["experts"], "identity": z["identity"], "top": z["top"], "groups": {"count": 2, "keep": 1}}}
    att = {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["vdim"], "scale": z["dim"] ** -0.5 * 4.0,
           "mask": {"size": z["window"], "keep_first": z["keep_first"]}, "rot": {"dims": z["rot"], "base": 10000.0}}
    layers = []
    for i in range(z["layers"]):
        L = {"type": "attention", "mixer": dict(att, kv_from=i - 1) if i % 3 == 2 else dict(att)}
        L["mlp"] = {"kind": "dense", "ff": z["dense_ff"], "limit": 7.0} if i % 2 == 0 else moe
        layers.append(L)
    return {"architecture": "Dogilorn", "width": z["width"], "vocab": z["vocab"], "norm": {"eps": 1e-5},
            "canon": {"taps": z["taps"]}, "embedding": {"scale": 1.0}, "layers": layers}


def dogilorn_kernel_rooflines(z: dict, T: int = 4096, B: int = 64, ctx: int = 2048) -> Dict[str, dict]:
    """Each Dogilorn kernel alone (bf16): prefill of one T-token sequence, decode of B sequences at
    ``ctx``; time, the bound resource's minimum time, and their ratio."""
    from .. import ops
    from ..models.llama import AttnMeta
    from ..ops import seqmix
    dev, bf = "cuda", torch.bfloat16
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    res: Dict[str, dict] = {}

    def rec(name, sec, bytes_, flops, peak_flops):
        floor = max(bytes_ / PEAK_BW, flops / peak_flops)
        res[name] = {"us": round(sec * 1e6, 1), "roofline_us": round(floor * 1e6, 2), "x_roofline": round(sec / floor, 1),
                     "bound": "memory" if bytes_ / PEAK_BW >= flops / peak_flops else "compute"}

    W = z["width"]
    for tag, qlens, starts in (("prefill", [T], [0]), ("decode", [1] * B, [ctx] * B)):
        n, S = sum(qlens), len(qlens)
        qstart = i32([sum(qlens[:i]) for i in range(S)])
        cxl = [a + b for a, b in zip(starts, qlens)]
        qlen, cx, rows = i32(qlens), i32(cxl), i32(list(range(S)))
        pos = i32([p for a, m in zip(starts, qlens) for p in range(a, a + m)])
        H, G, d, dv, Wn, Kf = z["heads"], z["kv_heads"], z["dim"], z["vdim"], z["window"], z["keep_first"]
        see = lambda p: min(p + 1, Wn) + max(0, min(Kf, p + 1 - Wn))       # keys position p sees
        pairs = sum(see(p) for a, m in zip(starts, qlens) for p in range(a, a + m))
        seen = sum(min(c, Wn + m - 1 + Kf) for c, m in zip(cxl, qlens))    # keys any row of a sequence sees
        nb = (max(cxl) + 15) // 16
        bt = torch.arange(S * nb, dtype=torch.int32, device=dev).view(S, nb)
        kc = (torch.randn(S * nb, G, 16, d, device=dev) * 0.3).to(bf)
        vc = (torch.randn(S * nb, G, dv, 16, device=dev) * 0.3).to(bf)
        cols = H * d + G * (d + dv)
        proj = torch.randn(n, cols, device=dev).to(bf)
        table = ops.rope_cos_sin(ctx + T + 8, z["rot"], 10000.0, dev)
        slots = i32([int(bt[i, p // 16]) * 16 + p % 16 for i, (a, m) in enumerate(zip(starts, qlens)) for p in range(a, a + m)])
        qw, kw, qs = torch.ones(H * d, device=dev), torch.ones(G * d, device=dev), torch.full((H,), d ** -0.5, device=dev)
        prep = lambda: seqmix.proj_norm_prep(proj, H, G, d, dv, qw, kw, table, z["rot"], True, 1e-5, qs, True, pos, slots, kc, vc)
        q = prep()
        rec(f"proj_norm_prep_{tag}", _timed(prep), n * cols * 4, n * cols * 10, PEAK_F32)
        meta = AttnMeta(slots=None, block_tables=bt, qstart=qstart, qlen=qlen, ctx=cx, tile_seq=None, tile_tok0=None,
                        last_idx=None, host_qlen=qlens)
        mfma = seqmix.gqa_use_mfma(q, H, G, d, dv, 16)
        ts, tt = meta.latent_tiles(1, dev, seqmix.gqa_tokens_per_tile(H, G, mfma))
        sp = seqmix.gqa_splits(int(ts.numel()), G, max(cxl), Wn, Kf) if mfma else 1
        att = lambda: seqmix.paged_gqa_attention(q, kc, vc, bt, qstart, qlen, cx, ts, tt, None, mfma, sp, window=Wn,
                                                 keep_first=Kf, sink=1.0)
        att()
        rec(f"attention_{tag}", _timed(att, 3), seen * G * (d + dv) * 2 + n * H * (d + dv) * 2, pairs * H * 2 * (d + dv), PEAK_BF16)
        # input convolution (h + conv(h)) and its slot
        K = z["taps"]
        h = torch.randn(n, W, device=dev).to(bf)
        cw, cb, cs_ = torch.randn(W, K, device=dev) * 0.3, torch.zeros(W, device=dev), torch.zeros(S, K - 1, W, device=dev, dtype=bf)
        single = tag == "decode"
        rec(f"input_conv_{tag}",
            _timed(lambda: seqmix.causal_conv_silu(h, cw, cb, cs_, qstart, qlen, cx, rows, refill=single, act="residual")),
            n * W * 4 + (S * (K - 1) * W * 4 if single else 0), n * W * 2 * K, PEAK_F32)
        # sublayer tail + layer norm (with the expert terms), gated activation, router
        x = torch.randn(n, W, device=dev)
        y, y2 = torch.randn(n, W, device=dev).to(bf), torch.randn(n, W, device=dev).to(bf)
        lw, lb, ls = torch.ones(W, device=dev), torch.zeros(W, device=dev), torch.full((W,), 0.5, device=dev)
        R = z["experts"] + z["identity"]
        logits = torch.randn(n, R + 1, device=dev)
        hw = torch.rand(n, device=dev)
        rec(f"ls_resadd_ln_{tag}", _timed(lambda: seqmix.ls_resadd_ln(x, lw, lb, 1e-5, bf, y=y, ls=ls)),
            n * W * (8 + 2 + 2), n * W * 10, PEAK_F32)
        rec(f"ls_resadd_ln_experts_{tag}",
            _timed(lambda: seqmix.ls_resadd_ln(x, lw, lb, 1e-5, bf, y=y, ls=ls, y2=y2, g2=logits[:, R], h=h, hw=hw)),
            n * W * (8 + 2 + 2 + 4), n * W * 14, PEAK_F32)
        gu, gb = torch.randn(n, 2 * z["dense_ff"], device=dev).to(bf), torch.zeros(2 * z["dense_ff"], device=dev)
        rec(f"glu_act_{tag}", _timed(lambda: seqmix.glu_act(gu, gb, "clamped", 7.0, 1.702)),
            n * z["dense_ff"] * 6, n * z["dense_ff"] * 12, PEAK_F32)
        corr = torch.zeros(R, device=dev)
        rec(f"route_topk_{tag}", _timed(lambda: seqmix.route_topk(logits, R, z["top"], 2, 1, "softmax", "max", corr, z["experts"])),
            n * (R + 1) * 4 + n * z["top"] * 8, n * R * 20, PEAK_F32)
    return res


def pebodra_raw(z: dict) -> dict:
    moe = {"kind": "moe", "expert": {"ff": z["ff"]},
           "router": {"experts": z["experts"], "top": z["top"], "groups": {"count": 2, "keep": 1}}}
    att = {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["vdim"], "diff": 0.2,
           "scale": z["dim"] ** -0.5, "mask": {"size": z["window"]}, "rot": {"dims": z["rot"], "base": 10000.0}}
    layers = []
    for i in range(z["layers"]):
        k = i % 4
        if k == 0:
            L = {"type": "attention", "mixer": dict(att)}
        elif k == 2:
            L = {"type": "attention", "mixer": dict(att, kv_from=i - 2)}
        elif k == 1:
            L = {"type": "mlstm", "mixer": {"heads": z["x_heads"], "dim": z["x_dim"], "vdim": z["x_vdim"], "gate_cap": 10.0}}
        else:
            L = {"type": "mamba2", "mixer": {"heads": z["m_heads"], "vdim": z["m_vdim"], "state": z["state"],
                                             "groups": z["groups"], "conv": z["conv"], "norm_groups": z["norm_groups"]}}
        L["mlp"] = {"kind": "dense", "ff": z["dense_ff"]} if i == 0 else moe
        layers.append(L)
    return {"architecture": "Pebodra", "width": z["width"], "vocab": z["vocab"], "norm": {"eps": 1e-6, "groups": 4},
            "logit_softcap": 50.0, "layers": layers}


def pebodra_twin(z: dict):
    """Mixtral-style Llama of the same width, depth, vocabulary, expert count / top-k and expert width
    (both run SwiGLU experts)."""
    from ..models.configs import ModelConfig
    return ModelConfig(f"moe-llama-{z['width']}", z["width"], z["layers"], z["width"] // 64, max(1, z["width"] // 256), 64,
                       z["ff"], z["vocab"], 10000.0, 1e-6, 16384, n_experts=z["experts"], experts_per_token=z["top"])


def pebodra_kernel_rooflines(z: dict, T: int = 4096, B: int = 64, ctx: int = 2048) -> Dict[str, dict]:
    """Each Pebodra mixer kernel alone (bf16): prefill of one T-token sequence, decode of B sequences
    at ``ctx``; time, the bound resource's minimum time, and their ratio."""
    from .. import ops
    from ..models.llama import AttnMeta
    from ..ops import seqmix
    dev, bf = "cuda", torch.bfloat16
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    res: Dict[str, dict] = {}

    def rec(name, sec, bytes_, flops, peak_flops):
        floor = max(bytes_ / PEAK_BW, flops / peak_flops)
        res[name] = {"us": round(sec * 1e6, 1), "roofline_us": round(floor * 1e6, 2), "x_roofline": round(sec / floor, 1),
                     "bound": "memory" if bytes_ / PEAK_BW >= flops / peak_flops else "compute"}

    for tag, qlens, starts in (("prefill", [T], [0]), ("decode", [1] * B, [ctx] * B)):
        n, S = sum(qlens), len(qlens)
        qstart = i32([sum(qlens[:i]) for i in range(S)])
        cxl = [a + b for a, b in zip(starts, qlens)]
        qlen, cx, rows = i32(qlens), i32(cxl), i32(list(range(S)))
        pos = i32([p for a, m in zip(starts, qlens) for p in range(a, a + m)])
        # differential attention: prep, windowed attention over both maps, combination
        H, G, d, dv, Wn = z["heads"], z["kv_heads"], z["dim"], z["vdim"], z["window"]
        pairs = sum(min(p + 1, Wn) for a, m in zip(starts, qlens) for p in range(a, a + m))   # (query, visible key) pairs
        seen = sum(min(c, Wn + m - 1) for c, m in zip(cxl, qlens))                            # keys any row of a sequence sees
        nb = (max(cxl) + 15) // 16
        bt = torch.arange(S * nb, dtype=torch.int32, device=dev).view(S, nb)
        kc = (torch.randn(S * nb, 2 * G, 16, d, device=dev) * 0.3).to(bf)
        vc = (torch.randn(S * nb, G, dv, 16, device=dev) * 0.3).to(bf)
        cols = 2 * H * d + 2 * G * d + G * dv
        proj, bias = torch.randn(n, cols, device=dev).to(bf), torch.zeros(cols, device=dev)
        table = ops.rope_cos_sin(ctx + T + 8, z["rot"], 10000.0, dev)
        slots = i32([int(bt[i, p // 16]) * 16 + p % 16 for i, (a, m) in enumerate(zip(starts, qlens)) for p in range(a, a + m)])
        nw = torch.ones(d, device=dev)
        prep = lambda: seqmix.qk_norm_prep(proj, bias, H, G, 2, d, dv, nw, nw, table, z["rot"], 1e-6, d ** -0.5, pos, slots, kc, vc)
        q = prep()
        rec(f"qk_prep_{tag}", _timed(prep), n * cols * 4 + n * 2 * H * d * 2, n * 2 * (H + G) * d * 10, PEAK_F32)
        meta = AttnMeta(slots=None, block_tables=bt, qstart=qstart, qlen=qlen, ctx=cx, tile_seq=None, tile_tok0=None,
                        last_idx=None, host_qlen=qlens)
        mfma = seqmix.gqa_use_mfma(q, 2 * H, 2 * G, d, dv, 16)
        ts, tt = meta.latent_tiles(1, dev, seqmix.gqa_tokens_per_tile(2 * H, 2 * G, mfma))
        sp = seqmix.gqa_splits(int(ts.numel()), 2 * G, max(cxl), Wn) if mfma else 1
        att = lambda: seqmix.paged_gqa_attention(q, kc, vc, bt, qstart, qlen, cx, ts, tt, None, mfma, sp, window=Wn, out_f32=True)
        a = att()
        rec(f"attention_{tag}", _timed(att, 3), seen * G * (2 * d + dv) * 2 + n * 2 * H * (d * 2 + dv * 4),
            pairs * 2 * H * 2 * (d + dv), PEAK_BF16)
        rec(f"diff_combine_{tag}", _timed(lambda: seqmix.diff_combine(a, H, G, dv, 0.2, 1e-6, 0.8, bf)),
            n * H * dv * (8 + 2), n * H * dv * 6, PEAK_F32)
        # Mamba-2: convolution, recurrence, gated norm
        Hm, dvm, N, Gm, K = z["m_heads"], z["m_vdim"], z["state"], z["groups"], z["conv"]
        inner, C = Hm * dvm, Hm * dvm + 2 * Gm * N
        pr = torch.randn(n, 2 * inner + 2 * Gm * N + Hm, device=dev).to(bf)
        conv_s, st = torch.zeros(S, K - 1, C, device=dev, dtype=bf), torch.zeros(S, Hm, N, dvm, device=dev)
        w, b_ = torch.randn(C, K, device=dev) * 0.5, torch.zeros(C, device=dev)
        xin = pr[:, inner:]
        xbc = seqmix.causal_conv_silu(xin, w, b_, conv_s, qstart, qlen, cx, rows)
        dtb, na, D = torch.zeros(Hm, device=dev), -torch.rand(Hm, device=dev), torch.ones(Hm, device=dev)
        rec(f"ssd_conv_{tag}", _timed(lambda: seqmix.causal_conv_silu(xin, w, b_, conv_s, qstart, qlen, cx, rows)),
            n * C * 4 + (S * (K - 1) * C * 2 if tag == "decode" else 0), n * C * 2 * K, PEAK_F32)
        scan = lambda: seqmix.ssd_scan(xbc, pr, 2 * inner + 2 * Gm * N, Hm, dvm, N, Gm, dtb, na, D, st, qstart, qlen, cx, rows)
        y = scan()
        rec(f"ssd_scan_{tag}", _timed(scan), n * (C * 2 + inner * 4) + (S * Hm * N * dvm * 8 if tag == "decode" else 0),
            n * Hm * N * dvm * 4, PEAK_F32)
        gw = torch.ones(inner, device=dev)
        rec(f"gated_norm_{tag}", _timed(lambda: seqmix.gated_group_norm(y, pr, gw, z["norm_groups"], 1e-6, bf)),
            n * inner * (4 + 2 + 2), n * inner * 8, PEAK_F32)
        # mLSTM
        Hx, dx, dvx = z["x_heads"], z["x_dim"], z["x_vdim"]
        px = torch.randn(n, 2 * Hx * (dx + dvx + 1), device=dev).to(bf)
        sx = torch.zeros(S, Hx, dx, dvx, device=dev)
        nm = torch.zeros(S, Hx, seqmix.scan_col_blocks(dvx), dx + 1, device=dev)
        gb, hw = torch.zeros(2 * Hx, device=dev), torch.ones(Hx * dvx, device=dev)
        rec(f"mlstm_{tag}", _timed(lambda: seqmix.mlstm(px, Hx, dx, dvx, gb, 10.0, sx, nm, 1e-6, hw, qstart, qlen, cx, rows)),
            n * (2 * Hx * dx + 3 * Hx * dvx) * 2 + (S * Hx * dx * dvx * 8 if tag == "decode" else 0),
            n * Hx * dx * (dvx + 1) * 4, PEAK_F32)
    return res


def sedopel_raw(z: dict) -> dict:
    par = {"type": "parallel",
           "mixer": {"left": {"heads": z["heads"], "kv_heads": z["kv_heads"], "dim": z["dim"], "vdim": z["vdim"],
                              "scale": z["dim"] ** -0.5 * 4.0, "rot": {"dims": z["rot"], "base": 10000.0}},
                     "right": {"heads": z["l_heads"], "dim": z["l_dim"], "vdim": z["l_vdim"],
                               "decay": [1.0 - 2.0 ** (-5 - i % 4) for i in range(z["l_heads"])]}},
           "mlp": {"kind": "dense", "ff": z["ff"]}}
    dlt = {"type": "delta", "mixer": {"heads": z["d_heads"], "kv_heads": z["d_kv_heads"], "dim": z["d_dim"],
                                      "vdim": z["d_vdim"], "conv": z["conv"]}, "mlp": None}
    return {"architecture": "Sedopel", "width": z["width"], "vocab": z["vocab"], "norm": {"eps": 1e-6},
            "layers": [par if i % 2 == 0 else dlt for i in range(z["layers"])]}


def dense_llama_twin(z: dict):
    """Dense Llama of the same width, depth, vocabulary and attention heads, its SwiGLU width chosen
    so that the parameter counts are equal."""
    from ..models.configs import ModelConfig, sedopel_config
    mk = lambda inter: ModelConfig(f"llama-{z['width']}", z["width"], z["layers"], z["heads"], z["kv_heads"], z["dim"],
                                   inter, z["vocab"], 10000.0, 1e-6, 16384)
    target = sedopel_config(sedopel_raw(z)).num_params()
    inter = (target - mk(0).num_params()) // (3 * z["width"] * z["layers"])
    return mk(max(64, inter // 64 * 64))


def sedopel_kernel_rooflines(z: dict, T: int = 4096, B: int = 64, ctx: int = 2048) -> Dict[str, dict]:
    """Each Sedopel mixer kernel alone (bf16): prefill of one T-token sequence, decode of B sequences
    at ``ctx``; time, the bound resource's minimum time, and their ratio."""
    from .. import ops
    from ..models.llama import AttnMeta
    from ..ops import seqmix
    dev, bf = "cuda", torch.bfloat16
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    res: Dict[str, dict] = {}

    def rec(name, sec, bytes_, flops, peak_flops):
        floor = max(bytes_ / PEAK_BW, flops / peak_flops)
        res[name] = {"us": round(sec * 1e6, 1), "roofline_us": round(floor * 1e6, 2), "x_roofline": round(sec / floor, 1),
                     "bound": "memory" if bytes_ / PEAK_BW >= flops / peak_flops else "compute"}

    for tag, qlens, starts in (("prefill", [T], [0]), ("decode", [1] * B, [ctx] * B)):
        n, S = sum(qlens), len(qlens)
        qstart = i32([sum(qlens[:i]) for i in range(S)])
        cxl = [a + b for a, b in zip(starts, qlens)]
        qlen, cx, rows = i32(qlens), i32(cxl), i32(list(range(S)))
        pos = i32([p for a, m in zip(starts, qlens) for p in range(a, a + m)])
        keys = sum((a + (m + 1) / 2) * m for a, m in zip(starts, qlens))     # causal (query, key) pairs
        # softmax attention over pages
        H, G, d, dv = z["heads"], z["kv_heads"], z["dim"], z["vdim"]
        nb = (max(cxl) + 15) // 16
        bt = torch.arange(S * nb, dtype=torch.int32, device=dev).view(S, nb)
        kc = (torch.randn(S * nb, G, 16, d, device=dev) * 0.3).to(bf)
        vc = (torch.randn(S * nb, G, dv, 16, device=dev) * 0.3).to(bf)
        proj = torch.randn(n, (H + G) * d + G * dv + H * dv, device=dev).to(bf)
        table = ops.rope_cos_sin(ctx + T + 8, z["rot"], 10000.0, dev)
        slots = i32([int(bt[i, p // 16]) * 16 + p % 16 for i, (a, m) in enumerate(zip(starts, qlens)) for p in range(a, a + m)])
        qs = torch.full((H,), d ** -0.5, device=dev)
        q = seqmix.attn_prep(proj, H, G, d, dv, table, z["rot"], 1e-6, qs, pos, slots, kc, vc)
        rec(f"attn_prep_{tag}", _timed(lambda: seqmix.attn_prep(proj, H, G, d, dv, table, z["rot"], 1e-6, qs, pos, slots, kc, vc)),
            n * ((H + G) * d + G * dv) * 4 + n * H * d * 2, n * (H + G) * d * 8, PEAK_F32)
        meta = AttnMeta(slots=None, block_tables=bt, qstart=qstart, qlen=qlen, ctx=cx, tile_seq=None, tile_tok0=None,
                        last_idx=None, host_qlen=qlens)
        mfma = seqmix.gqa_use_mfma(q, H, G, d, dv, 16)
        ts, tt = meta.latent_tiles(1, dev, seqmix.gqa_tokens_per_tile(H, G, mfma))
        gate = proj[:, (H + G) * d + G * dv:]
        rec(f"attention_{tag}",
            _timed(lambda: seqmix.paged_gqa_attention(q, kc, vc, bt, qstart, qlen, cx, ts, tt, gate, mfma,
                                                      seqmix.gqa_splits(int(ts.numel()), G, max(cxl)) if mfma else 1), 3),
            sum(cxl) * G * (d + dv) * 2 + n * H * (d + 2 * dv) * 2, keys * H * 2 * (d + dv), PEAK_BF16)
        # lightning attention
        Hl, dl, dvl = z["l_heads"], z["l_dim"], z["l_vdim"]
        qkvg = torch.randn(n, 2 * Hl * dl + 2 * Hl * dvl, device=dev).to(bf)
        dec, st = torch.full((Hl,), 0.98, device=dev), torch.zeros(S, Hl, dl, dvl, device=dev)
        nw = torch.ones(Hl * dvl, device=dev)
        rec(f"lightning_{tag}",
            _timed(lambda: seqmix.lightning_attention(qkvg, Hl, dl, dvl, dec, st, 1e-6, nw, qstart, qlen, cx, rows)),
            n * (2 * Hl * dl + 3 * Hl * dvl) * 2 + (S * Hl * dl * dvl * 8 if tag == "decode" else 0),
            n * Hl * dl * dvl * 4 if tag == "decode" else n * Hl * (4 * dl * dvl + 2 * 64 * (dl + dvl)), PEAK_F32)
        # gated delta rule (+ its convolution)
        Hd, Gd, dd, dvd, K = z["d_heads"], z["d_kv_heads"], z["d_dim"], z["d_vdim"], z["conv"]
        C = 2 * Gd * dd + Hd * dvd
        pr = torch.randn(n, C + Hd * dvd + 2 * Hd, device=dev).to(bf)
        conv_s, sd = torch.zeros(S, K - 1, C, device=dev, dtype=bf), torch.zeros(S, Hd, dvd, dd, device=dev)
        w, b_ = torch.randn(C, K, device=dev) * 0.5, torch.zeros(C, device=dev)
        qkv = seqmix.causal_conv_silu(pr, w, b_, conv_s, qstart, qlen, cx, rows)
        na, dtb, hn = -torch.rand(Hd, device=dev), torch.zeros(Hd, device=dev), torch.ones(dvd, device=dev)
        rec(f"delta_conv_{tag}", _timed(lambda: seqmix.causal_conv_silu(pr, w, b_, conv_s, qstart, qlen, cx, rows)),
            n * C * 4 + (S * (K - 1) * C * 2 if tag == "decode" else 0), n * C * 2 * K, PEAK_F32)
        rec(f"delta_rule_{tag}",
            _timed(lambda: seqmix.delta_rule(qkv, pr[:, C:], Hd, Gd, dd, dvd, na, dtb, hn, 1e-6, sd, qstart, qlen, cx, rows)),
            n * (C + 2 * Hd * dvd) * 2 + (S * Hd * dd * dvd * 8 if tag == "decode" else 0), n * Hd * dd * dvd * 6, PEAK_F32)
    return res


def filevik_raw(z: dict) -> dict:
    mlp = {"kind": "moe", "router": {"experts": z["experts"], "top": z["top"], "scale": 1.0}, "expert": {"ff": z["ff"]},
           "shared": {"ff": z["shared"]}}
    kinds = [
        {"type": "mamba1", "mixer": {"inner": z["inner"], "state": z["state"], "dt_rank": z["dt_rank"], "conv": z["conv"]}},
        {"type": "retention", "mixer": {"heads": z["heads"], "dim": z["dim"], "vdim": z["vdim"],
                                        "decay": [1.0 - 2.0 ** (-5 - i % 4) for i in range(z["heads"])],
                                        "rot": {"dims": z["rot"], "base": 10000.0}}},
        {"type": "latent_attention", "mixer": {"heads": z["lat_heads"], "dim": z["lat_dim"], "rot_dim": z["lat_rot"],
                                               "vdim": z["lat_v"], "kv_rank": z["kv_rank"], "q_rank": z["q_rank"],
                                               "scale": (z["lat_dim"] + z["lat_rot"]) ** -0.5,
                                               "rot": {"dims": z["lat_rot"], "base": 10000.0}}},
    ]
    return {"architecture": "Filevik", "width": z["width"], "vocab": z["vocab"], "norm": {"eps": 1e-6}, "logit_scale": 1.0,
            "layers": [dict(kinds[i % 3], mlp=mlp) for i in range(z["layers"])]}


def llama_twin(z: dict):
    from ..models.configs import ModelConfig
    return ModelConfig(f"moe-llama-{z['width']}", z["width"], z["layers"], z["width"] // 64, max(1, z["width"] // 256), 64,
                       z["ff"] * 3 // 2 // 64 * 64, z["vocab"], 10000.0, 1e-6, 16384, n_experts=z["experts"],
                       experts_per_token=z["top"])


def _timed(fn, iters: int = 5) -> float:
    fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters * 1e-3


def engine_throughput(model, prompts: List[int], batches: List[int], ctx: int, new: int, rows: int) -> Dict[str, float]:
    from ..engine.llm_engine import LLMEngine
    from ..engine.sampling import SamplingParams
    eng = LLMEngine(model, device="cuda", kv_cache_gb=8.0, max_num_seqs=rows, max_model_len=max(max(prompts), ctx) + new + 64,
                    prefix_cache=False)
    out: Dict[str, float] = {}
    g = torch.Generator().manual_seed(0)
    V = eng.cfg.vocab
    mk = lambda n, L: [torch.randint(3, V, (L,), generator=g).tolist() for _ in range(n)]
    one = SamplingParams(max_new_tokens=1, temperature=0.0, ignore_eos=True)
    for L in prompts:                      # prefill: whole prompts, one generated token each
        n = max(1, min(rows, 16384 // L))
        eng.generate(mk(n, L), one)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.generate(mk(n, L), one)
        torch.cuda.synchronize()
        out[f"prefill_tok_s_L{L}"] = round(n * L / (time.perf_counter() - t0), 1)
    for B in batches:                      # decode: B sequences of ctx tokens, `new` tokens each
        sp = SamplingParams(max_new_tokens=new, temperature=0.0, ignore_eos=True)
        eng.generate(mk(B, ctx), SamplingParams(max_new_tokens=4, temperature=0.0, ignore_eos=True))
        st0 = dict(eng.timers)
        s0 = dict(eng.steps)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.generate(mk(B, ctx), sp)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0 - (eng.timers["prefill"] - st0["prefill"])
        steps = eng.steps["decode"] - s0["decode"]
        out[f"decode_tok_s_B{B}"] = round(B * new / dt, 1)
        out[f"decode_ms_step_B{B}"] = round(dt / max(1, steps) * 1e3, 3)
    del eng
    torch.cuda.empty_cache()
    return out


def kernel_rooflines(z: dict, T: int = 4096, B: int = 64, ctx: int = 2048) -> Dict[str, dict]:
    """Each mixer kernel alone (bf16): prefill of one T-token sequence, decode of B sequences at
    ``ctx``; time, the bound resource's minimum time, and their ratio."""
    from .. import ops
    from ..ops import seqmix
    dev, bf = "cuda", torch.bfloat16
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    res: Dict[str, dict] = {}

    def rec(name, sec, bytes_, flops, peak_flops):
        floor = max(bytes_ / PEAK_BW, flops / peak_flops)
        res[name] = {"us": round(sec * 1e6, 1), "roofline_us": round(floor * 1e6, 2), "x_roofline": round(sec / floor, 1),
                     "bound": "memory" if bytes_ / PEAK_BW >= flops / peak_flops else "compute"}

    for tag, qlens, starts in (("prefill", [T], [0]), ("decode", [1] * B, [ctx] * B)):
        n = sum(qlens)
        S = len(qlens)
        qstart = i32([sum(qlens[:i]) for i in range(S)])
        qlen, cx, rows = i32(qlens), i32([a + b for a, b in zip(starts, qlens)]), i32(list(range(S)))
        pos = i32([p for a, m in zip(starts, qlens) for p in range(a, a + m)])
        # selective scan (+ conv)
        C, N, R, K = z["inner"], z["state"], z["dt_rank"], z["conv"]
        xz = torch.randn(n, 2 * C, device=dev).to(bf)
        conv_s, ssm = torch.zeros(S, K - 1, C, device=dev, dtype=bf), torch.zeros(S, C, N, device=dev)
        w, b_ = torch.randn(C, K, device=dev), torch.zeros(C, device=dev)
        xc = seqmix.causal_conv_silu(xz, w, b_, conv_s, qstart, qlen, cx, rows)
        dbc = torch.randn(n, R + 2 * N, device=dev).to(bf)
        dtr, dtb = torch.randn(n, C, device=dev).to(bf), torch.zeros(C, device=dev)
        A, D = -torch.rand(C, N, device=dev), torch.ones(C, device=dev)
        rec(f"conv_{tag}", _timed(lambda: seqmix.causal_conv_silu(xz, w, b_, conv_s, qstart, qlen, cx, rows)),
            n * C * 4 + (S * (K - 1) * C * 2 if tag == "decode" else 0), n * C * 2 * K, PEAK_F32)
        rec(f"scan_{tag}", _timed(lambda: seqmix.selective_scan(xc, dtr, dtb, A, dbc, R, D, xz, ssm, conv_s, qstart, qlen, cx, rows)),
            n * C * 8 + (S * C * N * 8 if tag == "decode" else 0), n * C * N * 12, PEAK_F32)
        # retention
        H, d, dv = z["heads"], z["dim"], z["vdim"]
        qkvg = torch.randn(n, 2 * H * d + 2 * H * dv, device=dev).to(bf)
        table = ops.rope_cos_sin(ctx + T + 8, z["rot"], 10000.0, dev)
        dec, st = torch.full((H,), 0.98, device=dev), torch.zeros(S, H, d, dv, device=dev)
        rec(f"retention_{tag}", _timed(lambda: seqmix.retention(qkvg, H, d, dv, table, z["rot"], dec, st, 1e-6, pos, qstart, qlen, cx, rows)),
            n * (2 * H * d + 3 * H * dv) * 2 + (S * H * d * dv * 8 if tag == "decode" else 0),
            n * H * d * dv * 4 if tag == "decode" else n * H * (4 * d * dv + 2 * 64 * (d + dv)), PEAK_F32)
        # latent attention
        Hl, r, dr, dl = z["lat_heads"], z["kv_rank"], z["lat_rot"], z["lat_dim"]
        nb = (max(cx.tolist()) + 15) // 16
        bt = torch.arange(S * nb, dtype=torch.int32, device=dev).view(S, nb)
        cache = (torch.randn(S * nb, 16, r + dr, device=dev) * 0.3).to(bf)
        qa, q = (torch.randn(Hl, n, r, device=dev) * 0.3).to(bf), torch.randn(n, Hl * (dl + dr), device=dev).to(bf)
        tab2 = ops.rope_cos_sin(ctx + T + 8, dr, 10000.0, dev)
        from ..models.llama import AttnMeta
        meta = AttnMeta(slots=None, block_tables=bt, qstart=qstart, qlen=qlen, ctx=cx, tile_seq=None, tile_tok0=None,
                        last_idx=None, host_qlen=qlens)
        lrows = seqmix.latent_rows(qa, r, dr, n, S)
        ts, tt = meta.latent_tiles(Hl, dev, lrows)
        keys = sum((a + (m + 1) / 2) * m for a, m in zip(starts, qlens))     # causal (query, key) pairs
        rec(f"latent_attention_{tag}",
            _timed(lambda: seqmix.latent_attention(qa, q, dl, dr, pos, tab2, cache, bt, qstart, qlen, cx, ts, tt, 0.1, rows=lrows), 3),
            (sum(a + m for a, m in zip(starts, qlens)) * (r + dr) * 2 + n * Hl * r * 4),
            keys * Hl * (2 * (r + dr) + 2 * r), PEAK_BF16)
    return res


def llama_kernel_rooflines(T: int = 4096, B: int = 64, ctx: int = 2048, nq: int = 32, nkv: int = 8, d: int = 64) -> Dict[str, dict]:
    """The comparison model's attention kernels at the same token counts."""
    from .. import ops
    dev, bf = "cuda", torch.bfloat16
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    res = {}
    for tag, qlens, starts in (("prefill", [T], [0]), ("decode", [1] * B, [ctx] * B)):
        n, S = sum(qlens), len(qlens)
        cx = [a + m for a, m in zip(starts, qlens)]
        nb = (max(cx) + 15) // 16
        bt = torch.arange(S * nb, dtype=torch.int32, device=dev).view(S, nb)
        kc = (torch.randn(S * nb, nkv, 16, d, device=dev) * 0.3).to(bf)
        vc = (torch.randn(S * nb, nkv, d, 16, device=dev) * 0.3).to(bf)
        q = torch.randn(n, nq, d, device=dev).to(bf)
        qstart = i32([sum(qlens[:i]) for i in range(S)])
        G = nq // nkv
        if tag == "prefill" and ops.flash_supported(d, G, nb):
            ts, tt = ops.flash_tiles(qlens, G)
            fn = lambda: ops.flash_attention(q, kc, vc, bt, qstart, i32(qlens), i32(cx), i32(ts), i32(tt), max_ctx=max(cx))
        else:
            ts, tt = ops.build_tiles(qlens, G)
            fn = lambda: ops.paged_attention(q, kc, vc, bt, qstart, i32(qlens), i32(cx), i32(ts), i32(tt))
        sec = _timed(fn)
        keys = sum((a + (m + 1) / 2) * m for a, m in zip(starts, qlens))
        bytes_, flops = sum(cx) * nkv * d * 4 + n * nq * d * 4, keys * nq * d * 4
        floor = max(bytes_ / PEAK_BW, flops / PEAK_BF16)
        res[f"attention_{tag}"] = {"us": round(sec * 1e6, 1), "roofline_us": round(floor * 1e6, 2),
                                   "x_roofline": round(sec / floor, 1),
                                   "bound": "memory" if bytes_ / PEAK_BW >= flops / PEAK_BF16 else "compute"}
    return res


def run(size: str = "s", kernels_only: bool = False, design: str = "filevik") -> dict:
    from ..models.configs import dogilorn_config, filevik_config, pebodra_config, sedopel_config
    if design == "dogilorn":
        z = DOGILORN_SIZES[size]
        out = {"bench": "arch", "design": design, "size": size, "dtype": "bf16", "data": "synthetic", "sizes": z}
        out["dogilorn_kernels"] = dogilorn_kernel_rooflines(z)
        # the like kernels at like sizes: windowed attention with two maps (Pebodra) and plain grouped-query
        # attention (Sedopel) at the same score rows and head widths, the Llama attention kernels at the
        # same heads, and the other designs' prep, convolution and residual launches
        pz = dict(PEBODRA_SIZES[size], heads=z["heads"] // 2, kv_heads=max(1, z["kv_heads"] // 2), dim=z["dim"], vdim=z["vdim"],
                  window=z["window"])
        out["pebodra_kernels"] = pebodra_kernel_rooflines(pz)
        out["sedopel_kernels"] = sedopel_kernel_rooflines(dict(SEDOPEL_SIZES[size], heads=z["heads"], kv_heads=z["kv_heads"],
                                                               dim=z["dim"], vdim=z["vdim"]))
        out["llama_kernels"] = llama_kernel_rooflines(nq=z["heads"], nkv=z["kv_heads"], d=z["dim"])
        if not kernels_only:
            prompts, batches = [512, 2048], [1, 16, 64]
            out["dogilorn"] = engine_throughput(dogilorn_config(dogilorn_raw(z), name=f"dogilorn-{size}"), prompts, batches,
                                                ctx=1024, new=32, rows=64)
            out["moe_llama"] = engine_throughput(pebodra_twin(z), prompts, batches, ctx=1024, new=32, rows=64)
        print(json.dumps(out))
        return out
    if design == "pebodra":
        z = PEBODRA_SIZES[size]
        out = {"bench": "arch", "design": design, "size": size, "dtype": "bf16", "data": "synthetic", "sizes": z}
        out["pebodra_kernels"] = pebodra_kernel_rooflines(z)
        # the like kernels at like sizes: the attention kernel without window and maps at the same
        # number of score rows, the delta rule, lightning / retention, the selective scan
        out["sedopel_kernels"] = sedopel_kernel_rooflines(dict(SEDOPEL_SIZES[size], heads=2 * z["heads"],
                                                               kv_heads=2 * z["kv_heads"], dim=z["dim"], vdim=z["vdim"]))
        out["filevik_kernels"] = kernel_rooflines(SIZES[size])
        out["llama_kernels"] = llama_kernel_rooflines(nq=2 * z["heads"], nkv=2 * z["kv_heads"], d=z["dim"])
        if not kernels_only:
            prompts, batches = [512, 2048], [1, 16, 64]
            out["pebodra"] = engine_throughput(pebodra_config(pebodra_raw(z), name=f"pebodra-{size}"), prompts, batches,
                                               ctx=1024, new=32, rows=64)
            out["moe_llama"] = engine_throughput(pebodra_twin(z), prompts, batches, ctx=1024, new=32, rows=64)
        print(json.dumps(out))
        return out
    if design == "sedopel":
        z = SEDOPEL_SIZES[size]
        out = {"bench": "arch", "design": design, "size": size, "dtype": "bf16", "data": "synthetic", "sizes": z}
        out["sedopel_kernels"] = sedopel_kernel_rooflines(z)
        out["filevik_kernels"] = kernel_rooflines(SIZES[size])
        out["llama_kernels"] = llama_kernel_rooflines(nq=z["heads"], nkv=z["kv_heads"], d=z["dim"])
        if not kernels_only:
            prompts, batches = [512, 2048], [1, 16, 64]
            out["sedopel"] = engine_throughput(sedopel_config(sedopel_raw(z), name=f"sedopel-{size}"), prompts, batches,
                                               ctx=1024, new=32, rows=64)
            out["llama"] = engine_throughput(dense_llama_twin(z), prompts, batches, ctx=1024, new=32, rows=64)
        print(json.dumps(out))
        return out
    z = SIZES[size]
    out = {"bench": "arch", "size": size, "dtype": "bf16", "data": "synthetic", "sizes": z}
    out["filevik_kernels"] = kernel_rooflines(z)
    out["llama_kernels"] = llama_kernel_rooflines()
    if not kernels_only:
        fcfg = filevik_config(filevik_raw(z), name=f"filevik-{size}")
        prompts, batches = [512, 2048], [1, 16, 64]
        out["filevik"] = engine_throughput(fcfg, prompts, batches, ctx=1024, new=32, rows=64)
        out["moe_llama"] = engine_throughput(llama_twin(z), prompts, batches, ctx=1024, new=32, rows=64)
    print(json.dumps(out))
    return out
