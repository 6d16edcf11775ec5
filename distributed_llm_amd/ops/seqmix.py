"""Sequence-mixer ops beside softmax attention: short causal convolution, selective scan, decayed
linear attention (retention), latent attention over a shared compressed key/value, the f32
residual update, squared-ReLU experts (csrc/kernels/seqmix.hip, latent.hip, moe.hip); grouped-query
attention over pages with an optional window and shared value heads, its input kernels (unit-RMS or
weighted q/k norms, one or two score maps a head) and the gated delta rule (gqa.hip, delta.hip); the
Mamba-2 and mLSTM recurrences (outer_scan.hip); PolyNorm, the group-limited sigmoid router, the
dense form of SwiGLU experts and the logit soft cap; for pre-norm layer-norm models the sublayer
tail with layer scale and the next layer norm in one launch, an input convolution without activation,
attention inputs normed over the whole q / k projection, kept first keys and a softmax sink in the
paged attention, gated activations with clamps, and top-k routing with softmax scores, a correction
on the choice and identity experts.

Same dispatch rule as the rest of the op library: GPU tensors run the HIP kernel (or raise when the
extension is missing), CPU tensors the torch reference.  Every kernel takes bf16 or f32 activations
(the model's dtype) and computes scores, states, norms and gates in f32.

A step is a packed batch of S sequences: sequence s brings tokens [qstart[s], qstart[s] + qlen[s])
at positions [ctx[s] - qlen[s], ctx[s]) and keeps its recurrent state in slot ``rows[s]``.  A
sequence whose first new position is 0 starts from a zero state, so a re-used slot needs no reset.
"""
from __future__ import annotations

import os
from typing import Optional, Tuple

import torch

from . import _native, reference as ref

LAT_ROWS = 16      # (token, head) rows per workgroup of the latent attention kernel; a tile entry
                   # (sequence, first token) covers max(1, 16 // heads) tokens (AttnMeta.latent_tiles)


def rms_rows(x: torch.Tensor, w: Optional[torch.Tensor], eps: float, out_dtype=None, groups: int = 1) -> torch.Tensor:
    """Row-wise x / sqrt(mean(x^2) + eps) (* w) for any row length; x may be a column slice.
    ``groups`` > 1: each of that many equal consecutive parts of a row by its own root mean square."""
    ext = _native(x)
    if ext is None:
        return ref.rms_rows(x, w, eps, out_dtype, groups)
    y = torch.empty(x.shape, dtype=out_dtype or x.dtype, device=x.device)
    ext.rms_rows(x, w, y, float(eps), int(groups))
    return y


def norm_resadd(y: torch.Tensor, w: torch.Tensor, eps: float, x: torch.Tensor,
                x_lp: Optional[torch.Tensor] = None, groups: int = 1, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Residual update in f32: ``x += rmsnorm(y) * w`` in place (x f32 [T, H]); ``x_lp`` (the model
    dtype) receives the rounded stream for the next projections, in the same launch.  ``groups`` as
    in ``rms_rows``; ``bias`` (the sublayer's output bias) is added to y before the norm."""
    ext = _native(y)
    if ext is None:
        return ref.norm_resadd(y, w, eps, x, x_lp, groups, bias)
    ext.norm_resadd(y, w, float(eps), x, x_lp, int(groups), bias)
    return x


def causal_conv_silu(x, w, b, conv_state, qstart, qlen, ctx, rows, refill: bool = False,
                     act: str = "silu", all_rows: bool = False, inplace: bool = False) -> torch.Tensor:
    """``refill``: the step brings at most one token per sequence (a decode step) and the kernel also
    moves each token's input into its slot; otherwise the slot is left to ``conv_state_refill`` or
    to the scan.  ``act`` "residual": no activation, y = x + the convolution (an input convolution
    ahead of a mixer).  ``all_rows``: every row of x belongs to a sequence (a step of prompt portions
    without padding), so the output needs no zero fill.  ``inplace`` (with ``refill``, x [T, C]
    contiguous): the output overwrites x; rows of no sequence keep their input."""
    ext = _native(x)
    if ext is None:
        y = ref.causal_conv_silu(x, w, b, conv_state, qstart, qlen, ctx, rows, act)
        if refill:
            ref.conv_state_refill(x, conv_state, qstart, qlen, ctx, rows)
        return y
    if inplace and refill and x.is_contiguous() and x.shape[1] == w.shape[0]:
        ext.causal_conv_silu(x, w, b, conv_state, qstart, qlen, ctx, rows, x, True, 0 if act == "silu" else 1)
        return x
    # rows of no sequence (graph padding) stay zero, never stale memory
    y = (torch.empty if all_rows else torch.zeros)((x.shape[0], w.shape[0]), dtype=x.dtype, device=x.device)
    ext.causal_conv_silu(x, w, b, conv_state, qstart, qlen, ctx, rows, y, bool(refill), 0 if act == "silu" else 1)
    return y


def selective_scan(xc, dt_raw, dt_bias, A, dbc, dt_rank, D, xz, ssm_state, conv_state, qstart, qlen, ctx,
                   rows) -> torch.Tensor:
    ext = _native(xc)
    if ext is None:
        return ref.selective_scan(xc, dt_raw, dt_bias, A, dbc, dt_rank, D, xz, ssm_state, conv_state, qstart, qlen,
                                  ctx, rows)
    out = torch.zeros_like(xc)
    ext.selective_scan(xc, dt_raw, dt_bias, A, dbc, int(dt_rank), D, xz, ssm_state, conv_state, qstart, qlen, ctx,
                       rows, out)
    return out


def retention_step_lds(dim: int, vdim: int) -> int:
    """LDS bytes of the token-by-token retention kernel (csrc/kernels/seqmix.hip dllm_retention_lds)."""
    lj = 1
    while lj < vdim and lj < 64:
        lj <<= 1
    return 4 * (dim * vdim + 8 * (2 * dim + 2 * vdim) + 2 * (256 // lj) * vdim)


RETENTION_CHUNK_MIN = 4    # average new tokens per sequence from which the chunked kernel runs


def retention(qkvg, heads, dim, vdim, cos_sin, rot_dims, decay, state, eps, positions, qstart, qlen, ctx,
              rows, chunked: Optional[bool] = None) -> torch.Tensor:
    """``chunked`` (GPU): the chunk-parallel kernel (prompt portions) or the token-by-token one
    (decode steps); default by the step's tokens per sequence.  Same results either way."""
    ext = _native(qkvg)
    if ext is None:
        return ref.retention(qkvg, heads, dim, vdim, cos_sin, rot_dims, decay, state, eps, positions, qstart, qlen,
                             ctx, rows)
    out = torch.zeros((qkvg.shape[0], heads * vdim), dtype=qkvg.dtype, device=qkvg.device)
    if chunked is None:
        chunked = qkvg.shape[0] >= RETENTION_CHUNK_MIN * qstart.numel()
    if not chunked and retention_step_lds(dim, vdim) > 150 * 1024:
        chunked = True      # the token-by-token kernel keeps the whole [dim, vdim] state in LDS
    raw = torch.empty((qkvg.shape[0], heads, vdim), dtype=torch.float32, device=qkvg.device) if chunked else None
    ext.retention(qkvg, int(heads), int(dim), int(vdim), cos_sin, int(rot_dims), decay, state, float(eps), positions,
                  qstart, qlen, ctx, rows, out, raw)
    return out


def latent_kv_write(ckv, rank, norm_w, eps, positions, cos_sin, slots, cache) -> None:
    ext = _native(ckv)
    if ext is None:
        return ref.latent_kv_write(ckv, rank, norm_w, eps, positions, cos_sin, slots, cache)
    ext.latent_kv_write(ckv, int(rank), norm_w, float(eps), positions, cos_sin, slots, cache)


LAT_SPLIT_TARGET = 512     # workgroups a small latent-attention grid is split up to (over keys)
LAT_SPLIT_MAX = 16


def latent_splits(n_entries: int, heads: int, rows: int = LAT_ROWS) -> int:
    """Key splits of a latent attention launch: grids with fewer than ``LAT_SPLIT_TARGET`` workgroups
    (decode steps, short portions) split every row's keys over up to ``LAT_SPLIT_MAX`` workgroups."""
    gx = ((1 if heads >= rows else rows // heads) * heads + rows - 1) // rows
    return max(1, min(LAT_SPLIT_MAX, LAT_SPLIT_TARGET // max(1, n_entries * gx)))


def latent_rows(x: torch.Tensor, rank: int, rot_dim: int, tokens: int, seqs: int) -> int:
    """(token, head) rows per workgroup of a latent attention launch: 32 for prompt portions of bf16
    models on the GPU where the matrix-core kernel's 32-row form fits the LDS, else 16.  The step's
    tile table (AttnMeta.latent_tiles) must be built for the same number."""
    if not x.is_cuda or x.dtype != torch.bfloat16 or tokens < 8 * max(1, seqs):
        return LAT_ROWS
    if os.environ.get("DLLM_LATENT_MFMA", "1") != "1" or os.environ.get("DLLM_LATENT_ROWS", "32") != "32":
        return LAT_ROWS
    ext = _native(x)
    return 32 if ext is not None and ext.latent_mfma_ok(int(rank), int(rot_dim), 32) else LAT_ROWS


def latent_attention(qa, q, dim, rot_dim, positions, cos_sin, cache, block_tables, qstart, qlen, ctx, tile_seq,
                     tile_tok0, scale, splits: Optional[int] = None, mfma: Optional[bool] = None,
                     rows: int = LAT_ROWS) -> torch.Tensor:
    """``mfma`` (GPU, bf16): the matrix-core kernel (default where the shape fits it;
    ``DLLM_LATENT_MFMA=0`` or ``mfma=False`` keeps the vector-ALU kernel that f32 models run)."""
    ext = _native(qa)
    if ext is None:
        return ref.latent_attention(qa, q, dim, rot_dim, positions, cos_sin, cache, block_tables, qstart, qlen, ctx,
                                    scale)
    out = torch.zeros_like(qa)
    H, n_entries = qa.shape[0], int(tile_seq.numel())
    sp = latent_splits(n_entries, H, rows) if splits is None else int(splits)
    po = pml = None
    if sp > 1:
        gx = ((1 if H >= rows else rows // H) * H + rows - 1) // rows
        prow = n_entries * gx * rows * sp
        po = torch.empty(prow * qa.shape[2], dtype=torch.float32, device=qa.device)
        pml = torch.empty(prow * 2, dtype=torch.float32, device=qa.device)
    if mfma is None:
        mfma = os.environ.get("DLLM_LATENT_MFMA", "1") == "1"
    ext.latent_attention(qa, q, int(dim), int(rot_dim), positions, cos_sin, cache, block_tables, qstart, qlen, ctx,
                         tile_seq, tile_tok0, float(scale), out, sp, po, pml, bool(mfma), int(rows))
    return out


def relu2_scale(x: torch.Tensor, gate: Optional[torch.Tensor] = None, ff: int = 0) -> torch.Tensor:
    ext = _native(x)
    if ext is None:
        return ref.relu2_scale(x, gate, ff)
    y = torch.empty_like(x)
    ext.relu2_scale(x, gate, int(ff), y)
    return y


def moe_ffn_relu2(x, ids, wts, w1, w2) -> torch.Tensor:
    """Top-k experts with a squared-ReLU activation and no gate projection on the grouped MFMA
    kernels of the SwiGLU experts (csrc/kernels/moe.hip, activation mode 1)."""
    ext = _native(x)
    if ext is None:
        return ref.moe_ffn_relu2(x, ids, wts, w1, w2)
    out = torch.empty((x.shape[0], x.shape[1]), dtype=x.dtype, device=x.device)
    ext.moe_ffn(x, ids.to(torch.int32).contiguous(), wts.float().contiguous(), w1, w2, out, 1)
    return out


def moe_ffn_relu2_ok(x: torch.Tensor, w1: torch.Tensor) -> bool:
    """The grouped kernels need bf16 and 32-aligned widths; other shapes run the dense form."""
    return (x.dtype == torch.bfloat16 and x.shape[1] % 32 == 0 and w1.shape[1] % 32 == 0 and w1.shape[0] <= 64
            and x.stride(1) == 1 and x.stride(0) % 8 == 0)


def dense_gate(ids, wts, E) -> torch.Tensor:
    ext = _native(ids)
    if ext is None:
        return ref.dense_gate(ids, wts, E)
    g = torch.zeros((ids.shape[0], E), dtype=torch.float32, device=ids.device)   # fill kernel (graph-safe)
    ext.dense_gate(ids.to(torch.int32).contiguous(), wts.float().contiguous(), g)
    return g


# ----------------------------------------------------------------------------- layers with a norm on both sides, depth average

def resadd_norm(a: torch.Tensor, w_post: torch.Tensor, eps: float, x: torch.Tensor,
                w_next: Optional[torch.Tensor] = None, x_next: Optional[torch.Tensor] = None,
                b: Optional[torch.Tensor] = None, wa: Optional[torch.Tensor] = None,
                wb: Optional[torch.Tensor] = None, depth: Optional[Tuple[torch.Tensor, torch.Tensor, int]] = None
                ) -> torch.Tensor:
    """The tail of a sublayer in one launch: ``x += rmsnorm(y) * w_post`` on the f32 stream, where y
    is the sublayer's output ``a`` or, for two mixers side by side, ``(rmsnorm(a) wa + rmsnorm(b) wb) / 2``;
    ``x_next`` (the model dtype) receives ``rmsnorm(x) * w_next``, the next sublayer's input.
    ``depth`` = (X, w, n) ends a layer of a depth-averaged model in the same launch: x is slot n - 1 of
    the f32 stack X, slot n receives ``sum_{j<n} w[j] X[j]`` (as ``depth_mix``) and ``x_next`` is
    normed from that; returns the slot handed on."""
    ext = _native(a)
    if ext is None:
        ref.resadd_norm(a, w_post, eps, x, None if depth else w_next, None if depth else x_next, b, wa, wb)
        return ref.depth_mix(depth[0], depth[1], depth[2], w_next, eps, x_next) if depth else x
    if depth is None:
        ext.resadd_norm(a, b, wa, wb, w_post, float(eps), x, w_next, x_next)
        return x
    X, w, n = depth
    ext.resadd_norm(a, b, wa, wb, w_post, float(eps), x, w_next, x_next, X, w, int(n))
    return X[n]


def depth_mix(X: torch.Tensor, w: torch.Tensor, n: int, w_next: Optional[torch.Tensor] = None, eps: float = 0.0,
              out_next: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Weighted sum over depth: ``X[n] = sum_{j<n} w[j] X[j]`` (X [slots, T, width] f32, w f32), plus
    ``out_next = rmsnorm(X[n]) * w_next`` in the same launch."""
    ext = _native(X)
    if ext is None:
        return ref.depth_mix(X, w, n, w_next, eps, out_next)
    ext.depth_mix(X, w, int(n), w_next, float(eps), out_next)
    return X[n]


def gelu_erf(x: torch.Tensor) -> torch.Tensor:
    """0.5 x (1 + erf(x / sqrt 2)) on bf16 or f32 activations."""
    ext = _native(x)
    if ext is None:
        return ref.gelu_erf(x)
    y = torch.empty_like(x)
    ext.gelu_erf(x, y)
    return y


# ----------------------------------------------------------------------------- grouped-query attention over pages

GQA_ROWS = 16          # (token, query head) rows per workgroup of the vector-ALU paged attention kernel
GQA_ROWS_MFMA = 64     # ... of the matrix-core kernel (bf16)


def gqa_use_mfma(q_like: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int, block: int) -> bool:
    """The matrix-core attention kernel runs bf16 models on the GPU whose shapes it takes
    (``DLLM_GQA_MFMA=0`` keeps the vector-ALU kernel that f32 models run)."""
    if not q_like.is_cuda or q_like.dtype != torch.bfloat16 or os.environ.get("DLLM_GQA_MFMA", "1") != "1":
        return False
    ext = _native(q_like)
    return ext is not None and bool(ext.gqa_mfma_ok(False, int(heads), int(kv_heads), int(dim), int(vdim), int(block)))


def gqa_tokens_per_tile(heads: int, kv_heads: int, mfma: bool = False) -> int:
    """New tokens one attention workgroup covers (its rows are these tokens x the query heads of
    one key/value head); the step's tile table (AttnMeta.latent_tiles) is built for this number."""
    return max(1, (GQA_ROWS_MFMA if mfma else GQA_ROWS) // max(1, heads // kv_heads))


def attn_prep(proj, heads, kv_heads, dim, vdim, cos_sin, rot_dims, eps, qscale, positions, slots, k_cache,
              v_cache) -> torch.Tensor:
    """Rotate q and k (rotate-half, first ``rot_dims`` dims), bring every head to unit RMS, scale q
    per head, write k and v to their page slots (k_cache [blocks, kv_heads, block, dim], v_cache
    [blocks, kv_heads, vdim, block]); returns q [T, heads, dim]."""
    ext = _native(proj)
    if ext is None:
        return ref.attn_prep(proj, heads, kv_heads, dim, vdim, cos_sin, rot_dims, eps, qscale, positions, slots,
                             k_cache, v_cache)
    q = torch.empty((proj.shape[0], heads, dim), dtype=proj.dtype, device=proj.device)     # every row is written
    ext.attn_prep(proj, int(heads), int(kv_heads), int(dim), int(vdim), cos_sin, int(rot_dims), float(eps), qscale,
                  positions, slots, k_cache, v_cache, q)
    return q


GQA_SPLIT_TARGET = 512     # workgroups a small matrix-core attention grid is split up to (over keys)
GQA_SPLIT_MAX = 16


def gqa_splits(n_tiles: int, kv_heads: int, max_ctx: int, window: int = 0, keep_first: int = 0) -> int:
    """Key splits of a matrix-core attention launch: grids with few workgroups (decode steps at small
    batch, short portions) split every row's 64-key tiles over up to ``GQA_SPLIT_MAX`` workgroups."""
    tiles = (int(max_ctx) + 63) // 64 if max_ctx > 0 else GQA_SPLIT_MAX     # decode graphs: any context
    if window > 0:
        tiles = min(tiles, (int(window) + 62) // 64 + 1 + (int(keep_first) + 63) // 64)
    return max(1, min(GQA_SPLIT_MAX, tiles, GQA_SPLIT_TARGET // max(1, n_tiles * kv_heads)))


def paged_gqa_attention(q, k_cache, v_cache, block_tables, qstart, qlen, ctx, tile_seq, tile_tok0,
                        gate: Optional[torch.Tensor] = None, mfma: bool = False, splits: int = 1, window: int = 0,
                        out_f32: bool = False, keep_first: int = 0, sink: float = 0.0,
                        all_rows: bool = False, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal softmax attention over paged keys / values of any head widths (f32 scores, online
    softmax), output times sigmoid(gate).  ``tile_seq`` / ``tile_tok0``: one entry per
    ``gqa_tokens_per_tile(heads, kv_heads, mfma)`` new tokens of a sequence.  ``splits`` > 1
    (matrix-core kernel): a row's keys are split over that many workgroups and merged.
    ``window`` > 0: a position sees itself and the ``window - 1`` keys before it (older key tiles are
    not read), and with ``keep_first`` > 0 also the keys j < keep_first at any distance (their tiles
    are read as well).  ``sink`` > 0: one more term of score 0 and that weight in every softmax
    denominator, with no value.  A value cache with fewer heads than the key cache is shared by
    neighbouring key heads.  ``out_f32``: the output stays f32 whatever the model dtype.  ``all_rows``:
    the tiles cover every row of q (no padding rows), so the output needs no zero fill.  ``out``: a
    prepared output [T, heads * vdim] (its padding rows already cleared)."""
    ext = _native(q)
    if ext is None:
        return ref.paged_gqa_attention(q, k_cache, v_cache, block_tables, qstart, qlen, ctx, gate, window, out_f32,
                                       keep_first, sink)
    dv = v_cache.shape[2]
    if out is None:
        out = (torch.empty if all_rows else torch.zeros)((q.shape[0], q.shape[1] * dv),
                                                         dtype=torch.float32 if out_f32 else q.dtype, device=q.device)
    splits = int(splits) if mfma else 1
    part = None
    if splits > 1:
        part = torch.empty(int(tile_seq.numel()) * k_cache.shape[1] * splits * GQA_ROWS_MFMA * (dv + 2),
                           dtype=torch.float32, device=q.device)
    ext.paged_gqa_attention(q, k_cache, v_cache, block_tables, qstart, qlen, ctx, tile_seq, tile_tok0, gate, out,
                            bool(mfma), splits, part, int(window), int(keep_first), float(sink))
    return out


# ----------------------------------------------------------------------------- differential attention

def qk_norm_prep(proj, bias, heads, kv_heads, maps, dim, vdim, qnorm_w, knorm_w, cos_sin, rot_dims, eps, qscale,
                 positions, slots, k_cache, v_cache) -> torch.Tensor:
    """Attention inputs with a weighted RMS norm of every q / k vector BEFORE its rotation, biases,
    and ``maps`` score maps per head (differential attention: 2).  proj [T, q | k | v] (+ ``bias``
    f32 over the same columns); returns q [T, heads maps, dim], scaled by ``qscale``, the query rows
    of one key/value head ordered (map, head in group), so that the grouped-query kernels pair row r
    with key row r // (heads / kv_heads) of k_cache [blocks, kv_heads maps, block, dim].  v goes to
    v_cache [blocks, kv_heads, vdim, block].  ``k_cache`` None (a layer that reads another layer's
    keys and values): proj holds q alone."""
    ext = _native(proj)
    if ext is None:
        return ref.qk_norm_prep(proj, bias, heads, kv_heads, maps, dim, vdim, qnorm_w, knorm_w, cos_sin, rot_dims, eps,
                                qscale, positions, slots, k_cache, v_cache)
    q = torch.empty((proj.shape[0], heads * maps, dim), dtype=proj.dtype, device=proj.device)     # every row is written
    ext.qk_norm_prep(proj, bias, int(heads), int(kv_heads), int(maps), int(dim), int(vdim), qnorm_w, knorm_w, cos_sin,
                     int(rot_dims), float(eps), float(qscale), positions, slots, k_cache, v_cache, q)
    return q


def diff_combine(a, heads, kv_heads, vdim, lam, eps, out_scale, out_dtype) -> torch.Tensor:
    """The two maps of differential attention into one output per head: a [T, 2 heads vdim] f32 in
    the row order ``qk_norm_prep`` gives; o = a1 - lam a2, unit RMS over vdim, times ``out_scale``."""
    ext = _native(a)
    if ext is None:
        return ref.diff_combine(a, heads, kv_heads, vdim, lam, eps, out_scale, out_dtype)
    out = torch.empty((a.shape[0], heads * vdim), dtype=out_dtype, device=a.device)
    ext.diff_combine(a, int(heads), int(kv_heads), int(vdim), float(lam), float(eps), float(out_scale), out)
    return out


# ----------------------------------------------------------------------------- gated outer-product recurrences (Mamba-2, mLSTM)

SCAN_COLS = 16      # value columns of one (sequence, head) a workgroup of the recurrence kernels owns


def scan_col_blocks(vdim: int) -> int:
    """Workgroups per (sequence, head) of ``ssd_scan`` / ``mlstm``; an mLSTM keeps one copy of its
    normaliser state per block."""
    return (int(vdim) + SCAN_COLS - 1) // SCAN_COLS


def ssd_scan(xbc, proj, dt_col, heads, vdim, n_state, groups, dt_bias, neg_a, D, state, qstart, qlen, ctx,
             rows) -> torch.Tensor:
    """Mamba-2 recurrence (scalar decay per head, B / C per group of heads): xbc [T, x | B | C]
    convolved and activated, step logits in proj[:, dt_col:dt_col + heads]; dt = softplus(. + bias),
    S <- exp(neg_a dt) S + dt B x^T, y = S^T C + D x.  state [slots, heads, N, vdim] f32; returns y f32."""
    ext = _native(xbc)
    if ext is None:
        return ref.ssd_scan(xbc, proj, dt_col, heads, vdim, n_state, groups, dt_bias, neg_a, D, state, qstart, qlen, ctx,
                            rows)
    out = torch.zeros((xbc.shape[0], heads * vdim), dtype=torch.float32, device=xbc.device)
    ext.ssd_scan(xbc, proj, int(dt_col), int(heads), int(vdim), int(n_state), int(groups), dt_bias, neg_a, D, state,
                 qstart, qlen, ctx, rows, out)
    return out


def gated_group_norm(y, z, w, groups, eps, out_dtype) -> torch.Tensor:
    """rmsnorm over each of ``groups`` equal parts of ``y silu(z)``, times w: y f32 [T, n], z the first
    n columns of a [T, >= n] activation; the gate comes before the norm."""
    ext = _native(y)
    if ext is None:
        return ref.gated_group_norm(y, z, w, groups, eps, out_dtype)
    out = torch.empty(y.shape, dtype=out_dtype, device=y.device)
    ext.gated_group_norm(y, z, w, int(groups), float(eps), out)
    return out


def mlstm(proj, heads, dim, vdim, gate_b, cap, state, nm, eps, norm_w, qstart, qlen, ctx, rows) -> torch.Tensor:
    """Matrix-memory LSTM over proj [T, q | k | v | output gate | input-gate logits | forget-gate
    logits] (``gate_b``: the two gates' biases): capped exponential input gate, sigmoid forget gate in
    log space, running maximum from 0, normaliser max(|n . q|, exp(-m)) + 1e-6; heads to unit RMS times
    ``norm_w`` times sigmoid(gate).  state [slots, heads, dim, vdim] f32, nm [slots, heads,
    scan_col_blocks(vdim), dim + 1] f32 (n and m)."""
    ext = _native(proj)
    if ext is None:
        return ref.mlstm(proj, heads, dim, vdim, gate_b, cap, state, nm, eps, norm_w, qstart, qlen, ctx, rows)
    T = proj.shape[0]
    raw = torch.zeros((T, heads * vdim), dtype=torch.float32, device=proj.device)
    out = torch.empty((T, heads * vdim), dtype=proj.dtype, device=proj.device)      # the finish kernel writes every row
    ext.mlstm(proj, int(heads), int(dim), int(vdim), gate_b, float(cap), state, nm, float(eps), norm_w, qstart, qlen,
              ctx, rows, raw, out)
    return out


# ----------------------------------------------------------------------------- PolyNorm, grouped sigmoid router, SwiGLU experts

def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """a N(z) + b N(z^2) + c N(z^3) + e per row with N the scaling to unit RMS; coef f32 (a, b, c, e)."""
    ext = _native(z)
    if ext is None:
        return ref.polynorm(z, coef, eps)
    y = torch.empty_like(z)
    ext.polynorm(z, coef, float(eps), y)
    return y


def route_topk(logits: torch.Tensor, n_out: int, top: int, count: int = 1, keep: int = 1, score: str = "sigmoid",
               group_score: str = "top2", correction: Optional[torch.Tensor] = None,
               real: Optional[int] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Group-limited top-k routing over the first ``n_out`` columns of f32 logits [T, >= n_out]
    (further columns, e.g. a gate logit made by the same GEMM, are not read).  Scores s: sigmoid or
    softmax of the logits; the choice is made on s + ``correction`` (f32 [n_out]); ``count`` groups of
    neighbouring outputs, a group scores the sum of its two best choice scores ("top2") or its best
    ("max"); the ``top`` best outputs of the ``keep`` best groups are chosen; weights = their s, not
    renormalised.  Outputs from ``real`` on are identity experts: their weights are summed per token
    into ``idw`` and left 0 in ``w`` (the expert kernels then add nothing for them).
    -> ids [T, top] int32, w [T, top] f32, idw [T] f32."""
    ext = _native(logits)
    if ext is None:
        return ref.route_topk(logits, n_out, top, count, keep, score, group_score, correction, real)
    T = logits.shape[0]
    ids = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    w = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    idw = torch.empty((T,), dtype=torch.float32, device=logits.device)
    ext.route_topk(logits, int(n_out), int(top), int(count), int(keep), 0 if score == "sigmoid" else 1,
                   0 if group_score == "top2" else 1, correction, int(n_out if real is None else real), ids, w, idw)
    return ids, w, idw


def group_router(logits: torch.Tensor, top: int, count: int, keep: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Sigmoid scores of f32 router logits [T, E]; ``count`` groups of neighbouring experts, a group
    scores the sum of its two best, the ``top`` best experts of the ``keep`` best groups are chosen;
    weights = their scores, not renormalised.  -> ids [T, top] int32, weights [T, top] f32."""
    ids, w, _ = route_topk(logits, logits.shape[1], top, count, keep)
    return ids, w


def swiglu_scale(gu: torch.Tensor, gate: torch.Tensor, ff: int) -> torch.Tensor:
    """Dense form of routed SwiGLU experts: gu [T, E 2 ff] (per expert its gate columns, then its up
    columns) -> [T, E ff] = silu(gate) * up * gate[t, expert]."""
    ext = _native(gu)
    if ext is None:
        return ref.swiglu_scale(gu, gate, ff)
    y = torch.empty((gu.shape[0], gu.shape[1] // 2), dtype=gu.dtype, device=gu.device)
    ext.swiglu_scale(gu, gate, int(ff), y)
    return y


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """cap * tanh(x / cap), f32 out."""
    ext = _native(x)
    if ext is None:
        return ref.softcap(x, cap)
    y = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    ext.softcap(x, float(cap), y)
    return y


# ----------------------------------------------------------------------------- lightning attention, gated delta rule

def lightning_attention(qkvg, heads, dim, vdim, decay, state, eps, norm_w, qstart, qlen, ctx, rows,
                        chunked: Optional[bool] = None) -> torch.Tensor:
    """Decayed linear attention over SiLU'd q, k, v (no rotation, no key scale); a token's heads are
    normed together and gated by a sigmoid.  Runs the retention kernels (token by token for decode
    steps, chunked for prompt portions) in their raw-output form, then one norm-and-gate launch."""
    ext = _native(qkvg)
    if ext is None:
        return ref.lightning_attention(qkvg, heads, dim, vdim, decay, state, eps, norm_w, qstart, qlen, ctx, rows)
    T = qkvg.shape[0]
    out = torch.empty((T, heads * vdim), dtype=qkvg.dtype, device=qkvg.device)     # the finish kernel writes every row
    if chunked is None:
        chunked = T >= RETENTION_CHUNK_MIN * qstart.numel()
    if not chunked and retention_step_lds(dim, vdim) > 150 * 1024:
        chunked = True
    raw = torch.empty((T, heads, vdim), dtype=torch.float32, device=qkvg.device)    # read for live tokens only
    ext.lightning_attention(qkvg, int(heads), int(dim), int(vdim), decay, state, float(eps), norm_w, qstart, qlen, ctx,
                            rows, out, raw, bool(chunked))
    return out


def conv_state_refill(x, conv_state, qstart, qlen, ctx, rows) -> None:
    """Keep each sequence's last ``taps - 1`` convolution inputs in its slot."""
    ext = _native(x)
    if ext is None:
        return ref.conv_state_refill(x, conv_state, qstart, qlen, ctx, rows)
    ext.conv_state_refill(x, conv_state, qstart, qlen, ctx, rows)


def delta_rule(qkv, gba, heads, kv_heads, dim, vdim, neg_a, dt_bias, norm_w, eps, state, qstart, qlen, ctx,
               rows) -> torch.Tensor:
    """Gated delta rule over convolved q | k | v with the gate, beta and decay logits in ``gba``;
    unit q / k, decay, beta, the state [slots, heads, vdim, dim] and the per-head output norm in f32."""
    ext = _native(qkv)
    if ext is None:
        return ref.delta_rule(qkv, gba, heads, kv_heads, dim, vdim, neg_a, dt_bias, norm_w, eps, state, qstart, qlen,
                              ctx, rows)
    out = torch.empty((qkv.shape[0], heads * vdim), dtype=qkv.dtype, device=qkv.device)     # the finish kernel writes every row
    ext.delta_rule(qkv, gba, int(heads), int(kv_heads), int(dim), int(vdim), neg_a, dt_bias, norm_w, float(eps), state,
                   qstart, qlen, ctx, rows, out)
    return out


# ----------------------------------------------------------------------------- layer-norm layers with layer scale, wide q/k norms, gated activations

def ls_resadd_ln(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float, out_dtype,
                 y: Optional[torch.Tensor] = None, ls: Optional[torch.Tensor] = None,
                 bias: Optional[torch.Tensor] = None, y2: Optional[torch.Tensor] = None,
                 g2: Optional[torch.Tensor] = None, h: Optional[torch.Tensor] = None,
                 hw: Optional[torch.Tensor] = None) -> torch.Tensor:
    """A pre-norm sublayer's tail and the next layer norm in one launch: the f32 stream x [T, width]
    (in place) += ls * (y + bias + sigmoid(g2) y2 + hw h), every term after y optional (``g2`` f32,
    one logit per token, may be a column of a wider matrix; ``hw`` f32 [T]); returns
    layernorm(x) * w + b (mean and variance over the row) in ``out_dtype``.  Without y: the norm alone."""
    ext = _native(x)
    if ext is None:
        return ref.ls_resadd_ln(x, w, b, eps, out_dtype, y, ls, bias, y2, g2, h, hw)
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    ext.ls_resadd_ln(x, w, b, float(eps), out, y, ls, bias, y2, g2, h, hw)
    return out


def proj_norm_prep(proj, heads, kv_heads, dim, vdim, qnorm_w, knorm_w, cos_sin, rot_dims, interleaved, eps, qscale,
                   vnorm, positions, slots, k_cache, v_cache, zero_rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention inputs with the q / k RMS norm taken over the whole projection (all heads together,
    weights of that length) before the rotation; rotary pairs (2i, 2i + 1) when ``interleaved`` else
    (i, i + rot_dims / 2) on the first ``rot_dims`` dims of every head; q times ``qscale[head]`` (f32);
    ``vnorm``: every value head to unit RMS.  proj [T, q | k | v]; k and v go to their page slots
    (k_cache [blocks, kv_heads, block, dim], v_cache [blocks, kv_heads, vdim, block]); ``k_cache``
    None (a layer that reads another layer's keys and values): proj holds q alone.  ``zero_rows``
    [T, n] (the activations' dtype) is cleared in the same launch: the attention output of a step with
    padding rows.  Returns q [T, heads, dim]."""
    ext = _native(proj)
    if ext is None:
        if zero_rows is not None:
            zero_rows.zero_()
        return ref.proj_norm_prep(proj, heads, kv_heads, dim, vdim, qnorm_w, knorm_w, cos_sin, rot_dims, interleaved,
                                  eps, qscale, vnorm, positions, slots, k_cache, v_cache)
    q = torch.empty((proj.shape[0], heads, dim), dtype=proj.dtype, device=proj.device)     # every row is written
    ext.proj_norm_prep(proj, int(heads), int(kv_heads), int(dim), int(vdim), qnorm_w, knorm_w, cos_sin, int(rot_dims),
                       bool(interleaved), float(eps), qscale, bool(vnorm), positions, slots, k_cache, v_cache, q, zero_rows)
    return q


def glu_act(gu: torch.Tensor, bias: Optional[torch.Tensor] = None, mode: str = "swiglu", limit: float = 0.0,
            alpha: float = 1.0) -> torch.Tensor:
    """Gated activation of gu [T, 2 ff] (gate columns, then up columns; ``bias`` f32 over the same
    columns) -> [T, ff]: "swiglu" silu(g) u, or "clamped": g <- min(g, limit), u <- clamp(u, -limit,
    limit), g sigmoid(alpha g) (u + 1)."""
    ext = _native(gu)
    if ext is None:
        return ref.glu_act(gu, bias, mode, limit, alpha)
    y = torch.empty((gu.shape[0], gu.shape[1] // 2), dtype=gu.dtype, device=gu.device)
    ext.glu_act(gu, bias, 0 if mode == "swiglu" else 1, float(limit), float(alpha), y)
    return y
