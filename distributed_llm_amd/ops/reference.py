"""Plain-PyTorch (f32 math) reference implementations of every kernel in csrc/kernels.

Used (a) on CPU tensors (tests, CPU-only runs) and (b) as the numerics oracle the GPU kernel
tests compare against.  Layout contracts are identical to the HIP kernels.
"""
from __future__ import annotations

import math
from typing import List, Optional, Tuple

import torch

BS = 16


def rms_norm(x, w, eps, residual=None):
    if residual is not None:
        r = (x.float() + residual.float()).to(x.dtype)
        residual.copy_(r)
        x = r
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    return y.to(x.dtype)


def layer_norm(x, w, b, eps, residual=None):
    if residual is not None:
        r = (x.float() + residual.float()).to(x.dtype)
        residual.copy_(r)
        x = r
    y = torch.nn.functional.layer_norm(x.float(), (x.shape[-1],), w.float(), b.float(), eps)
    return y.to(x.dtype)


def llama3_scale_inv_freq(inv: torch.Tensor, sc: dict) -> torch.Tensor:
    factor = sc.get("factor", 8.0)
    lo = sc.get("low_freq_factor", 1.0)
    hi = sc.get("high_freq_factor", 4.0)
    old = sc.get("original_max_position_embeddings", 8192)
    wl = 2 * math.pi / inv
    lo_wl, hi_wl = old / lo, old / hi
    out = torch.where(wl > lo_wl, inv / factor, inv)
    smooth = (old / wl - lo) / (hi - lo)
    mid = (1 - smooth) * inv / factor + smooth * inv
    is_mid = (wl <= lo_wl) & (wl >= hi_wl)
    return torch.where(is_mid, mid, out)


def _rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    # x [T, h, d] f32; cos/sin [T, d/2]
    h = x.shape[-1] // 2
    x1, x2 = x[..., :h], x[..., h:]
    c, s = cos[:, None, :], sin[:, None, :]
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)


def rope_and_cache(qkv, positions, cos_sin, slots, k_cache, v_cache, nq, nkv, d):
    T = qkv.shape[0]
    f = qkv[:, : (nq + 2 * nkv) * d].float()
    q = f[:, : nq * d].view(T, nq, d)
    k = f[:, nq * d:(nq + nkv) * d].view(T, nkv, d)
    v = qkv[:, (nq + nkv) * d:(nq + 2 * nkv) * d].view(T, nkv, d)
    cs = cos_sin[positions.long()].float()
    cos, sin = cs[:, : d // 2], cs[:, d // 2:]
    q = _rope(q, cos, sin).to(qkv.dtype)
    k = _rope(k, cos, sin).to(qkv.dtype)
    kv_write(k, v, slots, k_cache, v_cache)
    return q.contiguous()


def kv_write(k, v, slots, k_cache, v_cache):
    sl = slots.long()
    ok = sl >= 0
    if not bool(ok.any()):
        return
    sl, k, v = sl[ok], k[ok], v[ok]
    blk, off = sl // BS, sl % BS
    k_cache[blk, :, off, :] = k.to(k_cache.dtype)
    v_cache[blk, :, :, off] = v.to(v_cache.dtype)


def write_newest_v(v_new, v_cache, block_tables, seq_qstart, seq_ctx):
    """Decode hand-over (attention.hip AttnArgs.v_new): each sequence's newest key ctx - 1 takes V
    row ``v_new[qstart]`` ([T, nkv * d] row-major) in the V^T cache."""
    nkv, d = v_cache.shape[1], v_cache.shape[2]
    for s in range(block_tables.shape[0]):
        ctx, qs = int(seq_ctx[s]), int(seq_qstart[s])
        if ctx <= 0:
            continue
        key = ctx - 1
        blk = int(block_tables[s, key // BS])
        v_cache[blk, :, :, key % BS] = v_new[qs].view(nkv, d).to(v_cache.dtype)


def gather_kv(k_cache, v_cache, block_table, n):
    """Dense K, V [n, nkv, d] of one sequence from the paged caches."""
    nb = (n + BS - 1) // BS
    blocks = block_table[:nb].long()
    k = k_cache[blocks]                       # [nb, nkv, 16, d]
    v = v_cache[blocks].transpose(2, 3)       # [nb, nkv, 16, d]
    k = k.permute(0, 2, 1, 3).reshape(nb * BS, k.shape[1], k.shape[3])[:n]
    v = v.permute(0, 2, 1, 3).reshape(nb * BS, v.shape[1], v.shape[3])[:n]
    return k, v


def paged_attention(q, k_cache, v_cache, block_tables, seq_qstart, seq_qlen, seq_ctx, scale, causal=True):
    out = torch.zeros_like(q)
    nq, d = q.shape[1], q.shape[2]
    nkv = k_cache.shape[1]
    G = nq // nkv
    for s in range(block_tables.shape[0]):
        ql, ctx, qs = int(seq_qlen[s]), int(seq_ctx[s]), int(seq_qstart[s])
        if ql == 0 or ctx == 0:
            continue
        k, v = gather_kv(k_cache, v_cache, block_tables[s], ctx)
        k = k.float().repeat_interleave(G, dim=1)  # [ctx, nq, d]
        v = v.float().repeat_interleave(G, dim=1)
        qq = q[qs:qs + ql].float()                 # [ql, nq, d]
        sc = torch.einsum("qhd,khd->hqk", qq, k) * scale
        if causal:
            pos = torch.arange(ctx - ql, ctx, device=q.device)[:, None]
            keys = torch.arange(ctx, device=q.device)[None, :]
            sc = sc.masked_fill((keys > pos)[None], float("-inf"))
        p = torch.softmax(sc, dim=-1)
        o = torch.einsum("hqk,khd->qhd", p, v)
        out[qs:qs + ql] = o.to(q.dtype)
    return out


def silu_mul(gu):
    I = gu.shape[1] // 2
    g, u = gu[:, :I].float(), gu[:, I:].float()
    return (torch.nn.functional.silu(g) * u).to(gu.dtype)


def gelu(x):
    return torch.nn.functional.gelu(x.float()).to(x.dtype)


def encoder_attention(qkv, lens, B, S, nh, d, scale):
    """Bidirectional attention of a padded batch: qkv [B*S, 3 nh d] -> [B*S, nh d]; keys >= lens[b]
    masked (csrc/kernels/encoder.hip)."""
    x = qkv.float().view(B, S, 3, nh, d).permute(2, 0, 3, 1, 4)   # [3, B, nh, S, d]
    q, k, v = x[0], x[1], x[2]
    s = (q @ k.transpose(-1, -2)) * scale
    keymask = torch.arange(S, device=qkv.device)[None, :] < lens.to(qkv.device).long()[:, None]
    s = s.masked_fill(~keymask[:, None, None, :], float("-inf"))
    p = torch.softmax(s, dim=-1).nan_to_num(0.0)
    o = (p @ v).permute(0, 2, 1, 3).reshape(B * S, nh * d)
    return o.to(qkv.dtype)


def embed_ln(ids, word, pos, type0, w, b, S, eps):
    """LayerNorm(word[ids] + pos[t % S] + type0) for flattened [B*S] ids (csrc/kernels/encoder.hip)."""
    T = ids.numel()
    p = pos[:S].float().repeat(T // S, 1)
    x = word[ids.long().reshape(-1)].float() + p + type0.float()
    y = torch.nn.functional.layer_norm(x, (x.shape[-1],), w.float(), b.float(), eps)
    return y.to(word.dtype)


def mean_pool_l2(x, lens):
    B, S, H = x.shape
    m = (torch.arange(S)[None, :].to(x.device) < lens.to(x.device)[:, None]).float()
    s = (x.float() * m[..., None]).sum(1) / m.sum(1, keepdim=True).clamp(min=1.0)
    return torch.nn.functional.normalize(s, dim=-1, eps=1e-12)


def moe_gate(logits, k):
    lf = logits.float()
    vals, ids = torch.topk(lf, k, dim=-1)
    w = torch.softmax(vals, dim=-1)
    return ids.to(torch.int32), w


def moe_ffn(x, ids, wts, w13, w2):
    """sum_j wts[t, j] * (silu(x w13_e[:I]^T) * (x w13_e[I:]^T)) w2_e^T  with e = ids[t, j] (f32 math,
    bf16 rounding of the activation like the kernel).  Ids outside [0, E) are clamped like the
    kernel's routing does (callers give such pairs the weight 0)."""
    T, H = x.shape
    I = w13.shape[1] // 2
    ids = ids.clamp(0, w13.shape[0] - 1)
    out = torch.zeros((T, H), dtype=torch.float32, device=x.device)
    xf = x.float()
    for j in range(ids.shape[1]):
        for e in ids[:, j].unique().tolist():
            sel = (ids[:, j] == e).nonzero().flatten()
            gu = xf[sel] @ w13[e].float().t()
            act = (torch.nn.functional.silu(gu[:, :I]) * gu[:, I:]).to(x.dtype).float()
            out[sel] += wts[sel, j:j + 1].float() * (act @ w2[e].float().t())
    return out.to(x.dtype)


def sample_top_p(vals, idx, temperature, top_p, uniform):
    t = temperature.float().clamp(min=1e-5)[:, None]
    p = torch.softmax(vals.float() / t, dim=-1)
    c = torch.cumsum(p, dim=-1)
    # keep the smallest prefix whose mass reaches top_p
    keep = (c - p) < top_p.float()[:, None]
    keep[:, 0] = True
    p = p * keep
    p = p / p.sum(-1, keepdim=True)
    cdf = torch.cumsum(p, dim=-1)
    pick = torch.searchsorted(cdf, uniform.float()[:, None].clamp(max=0.999999), right=True).clamp(max=vals.shape[1] - 1)
    return torch.gather(idx, 1, pick).view(-1).to(torch.int32)


def row_uniform(seed: int, rows: int) -> torch.Tensor:
    """Counter-based uniforms u[row] in [0, 1) — the same hash as sample_rows_kernel."""
    M = 0xFFFFFFFF
    out = []
    for r in range(rows):
        h = (seed + r * 0x9E3779B9) & M
        h ^= h >> 16
        h = (h * 0x7FEB352D) & M
        h ^= h >> 15
        h = (h * 0x846CA68B) & M
        h ^= h >> 16
        out.append((h >> 8) / 16777216.0)
    return torch.tensor(out, dtype=torch.float32)


def sample_rows(logits, temperature, top_p, top_k, seed: int):
    """Reference of the fused row sampler: greedy rows -> arg-max (lowest index on ties); sampled
    rows -> top-k (value desc, index asc; k <= 0 -> 256) -> temperature -> nucleus -> draw."""
    lg = logits.float()
    B, V = lg.shape
    u = row_uniform(int(seed) & 0xFFFFFFFF, B)
    out = torch.empty(B, dtype=torch.int32)
    for r in range(B):
        t = float(temperature[r])
        if not t > 0.0:
            out[r] = int(torch.argmax(lg[r]))
            continue
        k = int(top_k[r])
        k = 256 if k <= 0 or k > 256 else k
        k = min(k, V)
        order = sorted(range(V), key=lambda i: (-float(lg[r, i]), i))[:k]
        vals = lg[r, order]
        w = torch.exp((vals - vals[0]) / max(t, 1e-5))
        c = torch.cumsum(w, 0)
        s = float(c[-1])
        cut = k
        for i in range(k):
            if float(c[i]) >= float(top_p[r]) * s:
                cut = i + 1
                break
        target = float(u[r]) * float(c[cut - 1])
        pick = cut - 1
        for i in range(cut):
            if float(c[i]) > target:
                pick = i
                break
        out[r] = order[pick]
    return out


def _draw_ranked(vals, ids, t: float, top_p: float, k: int, u: float) -> int:
    """sample_rows' draw over candidates already ranked (value desc, id asc)."""
    if not t > 0.0:
        return int(ids[0])
    k = 256 if k <= 0 or k > 256 else k
    k = min(k, len(ids))
    vals = torch.as_tensor(vals[:k], dtype=torch.float32)
    w = torch.exp((vals - vals[0]) / max(t, 1e-5))
    c = torch.cumsum(w, 0)
    s = float(c[-1])
    cut = k
    for i in range(k):
        if float(c[i]) >= top_p * s:
            cut = i + 1
            break
    target = u * float(c[cut - 1])
    pick = cut - 1
    for i in range(cut):
        if float(c[i]) > target:
            pick = i
            break
    return int(ids[pick])


def tp_candidates(logits, start: int, kc: int = 256):
    """Reference of tp_cands_kernel: [S, kc, 2] int32 (value f32 bits, global id)."""
    lg = logits.float().cpu()
    S, V = lg.shape
    out = torch.empty((S, kc, 2), dtype=torch.int32)
    out[:, :, 0] = torch.tensor([float("-inf")], dtype=torch.float32).view(torch.int32)
    out[:, :, 1] = 2 ** 31 - 1
    _, order = torch.sort(-lg, dim=1, stable=True)          # value desc, index asc
    n = min(kc, V)
    for r in range(S):
        idx = order[r, :n]
        out[r, :n, 0] = lg[r, idx].contiguous().view(torch.int32)
        out[r, :n, 1] = (idx + start).to(torch.int32)
    return out.to(logits.device)


def tp_sample(cands, temperature, top_p, top_k, seed: int):
    """Reference of tp_sample_kernel over all-gathered candidates [tp, S, kc, 2]."""
    c = cands.cpu()
    tp, S, kc, _ = c.shape
    u = row_uniform(int(seed) & 0xFFFFFFFF, S)
    out = torch.empty(S, dtype=torch.int32)
    for r in range(S):
        v = c[:, r, :, 0].reshape(-1).contiguous().view(torch.float32)
        ids = c[:, r, :, 1].reshape(-1)
        keep = ids != 2 ** 31 - 1
        v, ids = v[keep], ids[keep]
        order = sorted(range(len(ids)), key=lambda i: (-float(v[i]), int(ids[i])))
        out[r] = _draw_ranked([float(v[i]) for i in order], [int(ids[i]) for i in order], float(temperature[r]),
                              float(top_p[r]), int(top_k[r]), float(u[r]))
    return out


def cosine_scores(q, c):
    qn = q.float()
    cn = c.float()
    num = qn @ cn.T
    den = qn.norm(dim=-1, keepdim=True) * cn.norm(dim=-1)[None, :]
    return torch.where(den < 1e-9, torch.zeros_like(num), num / den.clamp(min=1e-30))


def masked_cosine_argmax(q, table, norms, ctx, cid, thr) -> Tuple[int, float]:
    qf = q.float().reshape(-1)
    nq = float(qf.norm())
    if nq < 1e-9 or table.shape[0] == 0:
        return -1, 0.0
    mask = (ctx == cid) & (norms >= 1e-9)
    if not bool(mask.any()):
        return -1, 0.0
    sims = (table.float() @ qf) / (norms.float().clamp(min=1e-30) * nq)
    sims = torch.where(mask, sims, torch.full_like(sims, -float("inf")))
    j = int(torch.argmax(sims))
    s = float(sims[j])
    return (j, s) if s >= thr else (-1, 0.0)


def cache_scan(queries, cids, table, ctx, n_rows, thr) -> List[Tuple[int, float]]:
    """fp32 reference of ops.cache_scan: per query, the row of its context id with the highest
    cosine >= thr (lowest row on ties; rows or queries of norm < 1e-9 never match) or (-1, 0.0)."""
    t = table[:n_rows].float()
    c = ctx[:n_rows]
    rn = t.norm(dim=-1)
    out = []
    for q, cid in zip(queries, cids):
        qf = q.float().reshape(-1)
        nq = float(qf.norm())
        mask = (c == int(cid)) & (rn >= 1e-9)
        if nq < 1e-9 or not bool(mask.any()):
            out.append((-1, 0.0))
            continue
        sims = (t @ qf) / (rn.clamp(min=1e-30) * nq)
        sims = torch.where(mask, sims, torch.full_like(sims, -float("inf")))
        j = int(torch.argmax(sims))
        s = float(sims[j])
        out.append((j, s) if s >= thr else (-1, 0.0))
    return out


def embedding(ids, table, lo=0):
    """fp32-free reference of ops.embedding (exact row copies, zero rows outside the shard)."""
    local = ids.reshape(-1).long() - lo
    ok = (local >= 0) & (local < table.shape[0])
    return table[local.clamp(0, table.shape[0] - 1)] * ok.unsqueeze(-1).to(table.dtype)


# ----------------------------------------------------------------------------- sequence mixers
#
# Shared conventions of the recurrent / latent mixers (csrc/kernels/seqmix.hip, latent.hip): a step
# is a packed batch of S sequences; sequence s brings tokens [qstart[s], qstart[s] + qlen[s]) at
# positions [ctx[s] - qlen[s], ctx[s]) and keeps its recurrent state in slot rows[s].  A sequence
# whose first new position is 0 starts from a zero state whatever its slot holds.

def _seq_meta(qstart, qlen, ctx, rows):
    qs, ql, cx = qstart.tolist(), qlen.tolist(), ctx.tolist()
    rw = rows.tolist() if rows is not None else list(range(len(qs)))
    return [(qs[i], ql[i], cx[i], rw[i]) for i in range(len(qs)) if ql[i] > 0]


def rms_rows(x, w, eps, out_dtype=None, groups=1):
    """``groups`` > 1: each of that many equal consecutive parts of a row by its own root mean square."""
    xf = x.float()
    if groups > 1:
        xf = xf.reshape(*x.shape[:-1], groups, x.shape[-1] // groups)
    y = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).reshape(x.shape)
    if w is not None:
        y = y * w.float()
    return y.to(out_dtype or x.dtype)


def norm_resadd(y, w, eps, x, x_lp=None, groups=1, bias=None):
    """x (f32 residual stream, in place) += rmsnorm(y (+ bias)) * w; ``x_lp`` receives x rounded to its dtype."""
    x += rms_rows(y if bias is None else y.float() + bias.float(), w, eps, torch.float32, groups)
    if x_lp is not None:
        x_lp.copy_(x)
    return x


def causal_conv_silu(x, w, b, conv_state, qstart, qlen, ctx, rows, act="silu"):
    """y[t, c] = silu(b[c] + sum_k w[c, k] u[t - K + 1 + k, c]) over each sequence's inputs u (the
    slot's last K - 1 inputs before its new tokens, zeros before position 0).  x [T, >= C] (first C
    columns), conv_state [slots, K - 1, C].  The state is NOT updated (selective_scan does).
    ``act`` "residual": no activation, y = x + (b + the convolution)."""
    C, K = w.shape
    y = torch.zeros((x.shape[0], C), dtype=x.dtype, device=x.device)
    wf = w.float()
    for q0, n, cx, row in _seq_meta(qstart, qlen, ctx, rows):
        hist = conv_state[row].float() if cx - n > 0 else torch.zeros((K - 1, C), dtype=torch.float32, device=x.device)
        u = torch.cat([hist, x[q0:q0 + n, :C].float()], 0)
        acc = b.float()[None, :].expand(n, C).clone()
        for k in range(K):
            acc += u[k:k + n] * wf[:, k][None, :]
        y[q0:q0 + n] = (torch.nn.functional.silu(acc) if act == "silu" else acc + x[q0:q0 + n, :C].float()).to(x.dtype)
    return y


def selective_scan(xc, dt_raw, dt_bias, A, dbc, dt_rank, D, xz, ssm_state, conv_state, qstart, qlen, ctx, rows):
    """Mamba-1 recurrence with the output gate.  xc [T, C] (convolved, activated), dt_raw [T, C],
    A [C, N] f32 (negative), dbc [T, dt_rank + 2N] (B at dt_rank, C at dt_rank + N), xz [T, 2C]
    (x | z: z gates, x refills the convolution state).  Per channel: S <- exp(dt A) S + dt x B,
    y = S . C + D x, out = y silu(z).  Updates ssm_state [slots, C, N] f32 and conv_state."""
    C, N = A.shape
    Km1 = conv_state.shape[1]
    out = torch.zeros_like(xc)
    for q0, n, cx, row in _seq_meta(qstart, qlen, ctx, rows):
        S = ssm_state[row].clone() if cx - n > 0 else torch.zeros((C, N), dtype=torch.float32, device=xc.device)
        dt = torch.nn.functional.softplus(dt_raw[q0:q0 + n].float() + dt_bias.float()[None, :], threshold=30.0)
        xs = xc[q0:q0 + n].float()
        Bm = dbc[q0:q0 + n, dt_rank:dt_rank + N].float()
        Cm = dbc[q0:q0 + n, dt_rank + N:dt_rank + 2 * N].float()
        ys = torch.empty((n, C), dtype=torch.float32, device=xc.device)
        for t in range(n):
            S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * xs[t])[:, None] * Bm[t][None, :]
            ys[t] = S @ Cm[t] + D.float() * xs[t]
        z = xz[q0:q0 + n, C:2 * C].float()
        out[q0:q0 + n] = (ys * torch.nn.functional.silu(z)).to(xc.dtype)
        ssm_state[row] = S
        if Km1 > 0:
            hist = conv_state[row].float() if cx - n > 0 else torch.zeros((Km1, C), dtype=torch.float32, device=xc.device)
            u = torch.cat([hist, xz[q0:q0 + n, :C].float()], 0)
            conv_state[row] = u[-Km1:].to(conv_state.dtype)
    return out


def _rot_table(cos_sin, pos, half):
    """cos, sin [n, half] of positions ``pos`` from a [max_pos, 2 * half] table (cos | sin)."""
    t = cos_sin.index_select(0, pos.long())
    return t[:, :half], t[:, half:2 * half]


def retention(qkvg, heads, dim, vdim, cos_sin, rot_dims, decay, state, eps, positions, qstart, qlen, ctx, rows):
    """Decayed linear attention with rotate-half positions on the first ``rot_dims`` dims of q and k,
    k scaled by dim^-1/2, unit-RMS heads and a SiLU gate.  qkvg [T, 2 heads dim + 2 heads vdim]
    (q | k | v | gate); state [slots, heads, dim, vdim] f32; returns [T, heads * vdim]."""
    T = qkvg.shape[0]
    H, d, dv = heads, dim, vdim
    out = torch.zeros((T, H * dv), dtype=qkvg.dtype, device=qkvg.device)
    half = rot_dims // 2
    dec = decay.float()
    for q0, n, cx, row in _seq_meta(qstart, qlen, ctx, rows):
        blk = qkvg[q0:q0 + n].float()
        q = blk[:, :H * d].reshape(n, H, d).clone()
        k = blk[:, H * d:2 * H * d].reshape(n, H, d).clone()
        v = blk[:, 2 * H * d:2 * H * d + H * dv].reshape(n, H, dv)
        g = blk[:, 2 * H * d + H * dv:]
        if half > 0:
            c, s = _rot_table(cos_sin, positions[q0:q0 + n], half)
            c, s = c[:, None, :], s[:, None, :]
            for t_ in (q, k):
                u, w_ = t_[..., :half].clone(), t_[..., half:2 * half].clone()
                t_[..., :half] = u * c - w_ * s
                t_[..., half:2 * half] = w_ * c + u * s
        k = k * (d ** -0.5)
        S = state[row].clone() if cx - n > 0 else torch.zeros((H, d, dv), dtype=torch.float32, device=qkvg.device)
        o = torch.empty((n, H, dv), dtype=torch.float32, device=qkvg.device)
        for t in range(n):
            S = dec[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
            o[t] = torch.einsum("hdv,hd->hv", S, q[t])
        state[row] = S
        o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
        out[q0:q0 + n] = (o.reshape(n, H * dv) * torch.nn.functional.silu(g)).to(qkvg.dtype)
    return out


def _rope_interleaved(x, c, s):
    u, w_ = x[..., 0::2], x[..., 1::2]
    out = torch.empty_like(x)
    out[..., 0::2] = u * c - w_ * s
    out[..., 1::2] = w_ * c + u * s
    return out


def latent_kv_write(ckv, rank, norm_w, eps, positions, cos_sin, slots, cache):
    """cache[slot] = [rmsnorm(ckv[:, :rank]) * norm_w | interleaved-rotated ckv[:, rank:]]."""
    dr = ckv.shape[1] - rank
    c = rms_rows(ckv[:, :rank], norm_w, eps, torch.float32)
    cs, sn = _rot_table(cos_sin, positions, dr // 2)
    kr = _rope_interleaved(ckv[:, rank:].float(), cs, sn)
    ok = slots >= 0
    cache.view(-1, cache.shape[-1])[slots[ok].long()] = torch.cat([c, kr], 1)[ok].to(cache.dtype)


def latent_attention(qa, q, dim, rot_dim, positions, cos_sin, cache, block_tables, qstart, qlen, ctx, scale):
    """Causal softmax attention over a shared latent: row (t, h) scores key j as
    (qa[h, t] . c_j + rot(q[t, h, dim:]) . kr_j) * scale and returns sum_j p_j c_j.
    qa [heads, T, rank], q [T, heads * (dim + rot_dim)], cache [blocks, 16, rank + rot_dim]."""
    Hh, T, r = qa.shape
    out = torch.zeros((Hh, T, r), dtype=qa.dtype, device=qa.device)
    flat = cache.view(-1, cache.shape[-1])
    qs, ql, cx = qstart.tolist(), qlen.tolist(), ctx.tolist()
    for s in range(len(qs)):
        n = ql[s]
        if n <= 0:
            continue
        q0, L = qs[s], cx[s]
        nb = (L + BS - 1) // BS
        idx = (block_tables[s, :nb].long()[:, None] * BS + torch.arange(BS, device=cache.device)[None, :]).reshape(-1)[:L]
        kv = flat[idx].float()
        cs, sn = _rot_table(cos_sin, positions[q0:q0 + n], rot_dim // 2)
        qr = q[q0:q0 + n].float().reshape(n, Hh, dim + rot_dim)[..., dim:]
        qr = _rope_interleaved(qr, cs[:, None, :], sn[:, None, :])
        sc = (torch.einsum("htr,jr->htj", qa[:, q0:q0 + n].float(), kv[:, :r]) +
              torch.einsum("thr,jr->htj", qr, kv[:, r:])) * scale
        pos = positions[q0:q0 + n].long()
        mask = torch.arange(L, device=cache.device)[None, :] <= pos[:, None]
        sc = sc.masked_fill(~mask[None], float("-inf"))
        p = torch.softmax(sc, -1)
        out[:, q0:q0 + n] = torch.einsum("htj,jr->htr", p, kv[:, :r]).to(qa.dtype)
    return out


def relu2_scale(x, gate=None, ff=0):
    """relu(x)^2, optionally times gate[t, column // ff] (dense routed experts: a token's weight of
    the column's expert, zero for experts it does not use)."""
    y = torch.relu(x.float()) ** 2
    if gate is not None:
        y = y * gate.float().repeat_interleave(ff, dim=1)
    return y.to(x.dtype)


def moe_ffn_relu2(x, ids, wts, w1, w2):
    """sum_j wts[t, j] * relu(x w1_e^T)^2 w2_e^T with e = ids[t, j] (w1 [E, I, H], w2 [E, H, I])."""
    T, H = x.shape
    out = torch.zeros((T, H), dtype=torch.float32, device=x.device)
    xf = x.float()
    for j in range(ids.shape[1]):
        for e in ids[:, j].unique().tolist():
            sel = (ids[:, j] == e).nonzero().flatten()
            act = (torch.relu(xf[sel] @ w1[e].float().t()) ** 2).to(x.dtype).float()
            out[sel] += wts[sel, j:j + 1].float() * (act @ w2[e].float().t())
    return out.to(x.dtype)


def dense_gate(ids, wts, E):
    """[T, E] f32: wts scattered to their experts' columns, zero elsewhere."""
    g = torch.zeros((ids.shape[0], E), dtype=torch.float32, device=ids.device)
    g.scatter_(1, ids.long(), wts.float())
    return g


# ----------------------------------------------------------------------------- pre/post-norm layers, depth average

def resadd_norm(a, w_post, eps, x, w_next=None, x_next=None, b=None, wa=None, wb=None):
    """x (f32 stream, in place) += rmsnorm(y) * w_post with y = a, or, with a second branch,
    y = (rmsnorm(a) wa + rmsnorm(b) wb) / 2; ``x_next`` receives rmsnorm(x) * w_next (the plain
    rounding of x when ``w_next`` is None)."""
    y = a.float() if b is None else 0.5 * (rms_rows(a, wa, eps, torch.float32) + rms_rows(b, wb, eps, torch.float32))
    x += rms_rows(y, w_post, eps, torch.float32)
    if x_next is not None:
        x_next.copy_(x if w_next is None else rms_rows(x, w_next, eps, torch.float32))
    return x


def depth_mix(X, w, n, w_next=None, eps=0.0, out_next=None):
    """X[n] = sum over j < n of w[j] X[j] (X [slots, T, width] f32); ``out_next`` receives
    rmsnorm(X[n]) * w_next."""
    X[n] = torch.einsum("j,jtw->tw", w[:n].float(), X[:n])
    if out_next is not None:
        out_next.copy_(X[n] if w_next is None else rms_rows(X[n], w_next, eps, torch.float32))
    return X[n]


def gelu_erf(x):
    return torch.nn.functional.gelu(x.float()).to(x.dtype)


# ----------------------------------------------------------------------------- grouped-query attention, paged

def attn_prep(proj, heads, kv_heads, dim, vdim, cos_sin, rot_dims, eps, qscale, positions, slots, k_cache, v_cache):
    """proj [T, >= heads dim + kv_heads (dim + vdim)] (q | k | v).  q and k: rotate-half positions on
    the first ``rot_dims`` dims of each head, then each head to unit RMS; q times ``qscale[head]``.
    k and v go to their page slots (k_cache [blocks, kv_heads, block, dim], v_cache [blocks,
    kv_heads, vdim, block]: values transposed inside a page); returns q [T, heads, dim]."""
    T, H, G, d, dv = proj.shape[0], heads, kv_heads, dim, vdim
    pf = proj.float()
    q = pf[:, :H * d].reshape(T, H, d).clone()
    k = pf[:, H * d:(H + G) * d].reshape(T, G, d).clone()
    v = pf[:, (H + G) * d:(H + G) * d + G * dv].reshape(T, G, dv)
    half = rot_dims // 2
    if half > 0:
        c, s = _rot_table(cos_sin, positions, half)
        c, s = c[:, None, :], s[:, None, :]
        for t_ in (q, k):
            u, w_ = t_[..., :half].clone(), t_[..., half:2 * half].clone()
            t_[..., :half] = u * c - w_ * s
            t_[..., half:2 * half] = w_ * c + u * s
    q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * qscale.float()[None, :, None]
    k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps)
    live = slots >= 0
    sl = slots[live].long()
    BSz = k_cache.shape[2]
    k_cache[sl // BSz, :, sl % BSz] = k[live].to(k_cache.dtype)
    v_cache[sl // BSz, :, :, sl % BSz] = v[live].to(v_cache.dtype)
    return q.to(proj.dtype)


def paged_gqa_attention(q, k_cache, v_cache, block_tables, qstart, qlen, ctx, gate=None, window=0, out_f32=False,
                        keep_first=0, sink=0.0):
    """Causal softmax attention of q [T, heads, dim] (already scaled) over paged keys / values;
    query head h reads key head h // (heads / kv_heads); the output [T, heads * vdim] is
    multiplied by sigmoid(gate) when a gate [T, heads * vdim] is given.  ``window`` > 0: position i
    sees keys i - window < j <= i, and the keys j < ``keep_first`` whatever their distance.  A value
    cache with fewer heads than the key cache is shared by neighbouring key heads (key head g reads
    value head g // (key heads / value heads)).  ``sink``: weight of one more term of score 0 in
    every softmax denominator (it has no value): p_j = exp(s_j) / (sink + sum exp(s_j))."""
    T, H, d = q.shape
    G, BSz, dv = k_cache.shape[1], k_cache.shape[2], v_cache.shape[2]
    vrep = G // v_cache.shape[1]
    out = torch.zeros((T, H * dv), dtype=torch.float32 if out_f32 else q.dtype, device=q.device)
    qs, ql, cx = qstart.tolist(), qlen.tolist(), ctx.tolist()
    for s in range(len(qs)):
        n, c = ql[s], cx[s]
        if n <= 0:
            continue
        nb = (c + BSz - 1) // BSz
        blocks = block_tables[s, :nb].long()
        K = k_cache[blocks].transpose(1, 2).reshape(nb * BSz, G, d)[:c].float().repeat_interleave(H // G, 1)
        V = v_cache[blocks].permute(0, 3, 1, 2).reshape(nb * BSz, G // vrep, dv)[:c].float().repeat_interleave(
            vrep * (H // G), 1)
        qq = q[qs[s]:qs[s] + n].float()
        sc = torch.einsum("thd,uhd->htu", qq, K)
        pos = torch.arange(c - n, c, device=q.device)
        mask = torch.arange(c, device=q.device)[None, :] > pos[:, None]
        if window > 0:
            keys = torch.arange(c, device=q.device)[None, :]
            mask = mask | ((keys <= pos[:, None] - window) & (keys >= keep_first))
        sc = sc.masked_fill(mask[None], float("-inf"))
        if sink > 0:
            mx = sc.max(-1, keepdim=True).values.clamp_min(0.0)
            e = torch.exp(sc - mx)
            pr = e / (e.sum(-1, keepdim=True) + sink * torch.exp(-mx))
        else:
            pr = torch.softmax(sc, -1)
        o = torch.einsum("htu,uhv->thv", pr, V).reshape(n, H * dv)
        if gate is not None:
            o = o * torch.sigmoid(gate[qs[s]:qs[s] + n].float())
        out[qs[s]:qs[s] + n] = o.to(out.dtype)
    return out


# ----------------------------------------------------------------------------- lightning attention, gated delta rule

def lightning_attention(qkvg, heads, dim, vdim, decay, state, eps, norm_w, qstart, qlen, ctx, rows):
    """Linear attention with a fixed decay per head over SiLU'd q, k, v: S <- decay S + k v^T,
    o = S^T q; the heads of a token are RMS-normed together (weight ``norm_w``) and multiplied by
    sigmoid(gate).  qkvg [T, >= 2 heads dim + 2 heads vdim] (q | k | v | gate); state
    [slots, heads, dim, vdim] f32."""
    T, H, d, dv = qkvg.shape[0], heads, dim, vdim
    out = torch.zeros((T, H * dv), dtype=qkvg.dtype, device=qkvg.device)
    dec = decay.float()
    silu = torch.nn.functional.silu
    for q0, n, cx, row in _seq_meta(qstart, qlen, ctx, rows):
        blk = qkvg[q0:q0 + n].float()
        q = silu(blk[:, :H * d]).reshape(n, H, d)
        k = silu(blk[:, H * d:2 * H * d]).reshape(n, H, d)
        v = silu(blk[:, 2 * H * d:2 * H * d + H * dv]).reshape(n, H, dv)
        g = blk[:, 2 * H * d + H * dv:2 * H * d + 2 * H * dv]
        S = state[row].clone() if cx - n > 0 else torch.zeros((H, d, dv), dtype=torch.float32, device=qkvg.device)
        o = torch.empty((n, H, dv), dtype=torch.float32, device=qkvg.device)
        for t in range(n):
            S = dec[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
            o[t] = torch.einsum("hdv,hd->hv", S, q[t])
        state[row] = S
        o = rms_rows(o.reshape(n, H * dv), norm_w, eps, torch.float32)
        out[q0:q0 + n] = (o * torch.sigmoid(g)).to(qkvg.dtype)
    return out


def conv_state_refill(x, conv_state, qstart, qlen, ctx, rows):
    """conv_state[slot] <- the last K - 1 inputs of each sequence (x [T, >= C], state [slots, K - 1, C])."""
    Km1, C = conv_state.shape[1], conv_state.shape[2]
    for q0, n, cx, row in _seq_meta(qstart, qlen, ctx, rows):
        hist = conv_state[row].float() if cx - n > 0 else torch.zeros((Km1, C), dtype=torch.float32, device=x.device)
        u = torch.cat([hist, x[q0:q0 + n, :C].float()], 0)
        conv_state[row] = u[u.shape[0] - Km1:].to(conv_state.dtype)


def delta_rule(qkv, gba, heads, kv_heads, dim, vdim, neg_a, dt_bias, norm_w, eps, state, qstart, qlen, ctx, rows):
    """Gated delta rule.  qkv [T, 2 kv_heads dim + heads vdim] (q | k | v, convolved and activated);
    gba [T, >= heads vdim + 2 heads] (output gate | beta logits | decay logits).  Per head, with q
    and k made unit vectors (sum of squares + 1e-6), q times dim^-1/2, beta = sigmoid(.),
    g = exp(neg_a softplus(. + dt_bias)):  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;
    o = S^T q.  Each head's o to unit RMS times ``norm_w`` times silu(gate).  state
    [slots, heads, vdim, dim] f32 (transposed: a value column's state is contiguous)."""
    T, H, G, d, dv = qkv.shape[0], heads, kv_heads, dim, vdim
    out = torch.zeros((T, H * dv), dtype=qkv.dtype, device=qkv.device)
    rep = H // G
    for q0, n, cx, row in _seq_meta(qstart, qlen, ctx, rows):
        blk = qkv[q0:q0 + n].float()
        q = blk[:, :G * d].reshape(n, G, d)
        k = blk[:, G * d:2 * G * d].reshape(n, G, d)
        v = blk[:, 2 * G * d:2 * G * d + H * dv].reshape(n, H, dv)
        q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * (d ** -0.5)
        k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
        q, k = q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1)
        z = gba[q0:q0 + n].float()
        gate, beta = z[:, :H * dv], torch.sigmoid(z[:, H * dv:H * dv + H])
        g = torch.exp(neg_a.float()[None, :] * torch.nn.functional.softplus(z[:, H * dv + H:H * dv + 2 * H] + dt_bias.float()[None, :]))
        S = state[row].clone() if cx - n > 0 else torch.zeros((H, dv, d), dtype=torch.float32, device=qkv.device)
        o = torch.empty((n, H, dv), dtype=torch.float32, device=qkv.device)
        for t in range(n):
            S = g[t][:, None, None] * S
            u = beta[t][:, None] * (v[t] - torch.einsum("hvd,hd->hv", S, k[t]))
            S = S + u[:, :, None] * k[t][:, None, :]
            o[t] = torch.einsum("hvd,hd->hv", S, q[t])
        state[row] = S
        o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()[None, None, :]
        out[q0:q0 + n] = (o.reshape(n, H * dv) * torch.nn.functional.silu(gate)).to(qkv.dtype)
    return out


# ----------------------------------------------------------------------------- differential attention

def qk_norm_prep(proj, bias, heads, kv_heads, maps, dim, vdim, qnorm_w, knorm_w, cos_sin, rot_dims, eps, qscale,
                 positions, slots, k_cache, v_cache):
    """proj [T, >= heads maps dim (+ kv_heads maps dim + kv_heads vdim)] (q | k | v) plus ``bias``
    (f32, same columns).  Every (head, map) vector of q and k: RMS norm over ``dim`` times the shared
    weight, then rotate-half positions on its first ``rot_dims`` dims; q times ``qscale``.  q comes
    back as [T, heads maps, dim] with the heads of a key/value head ordered (map, head in group), so
    that query row r reads key row r // (heads / kv_heads) of k_cache [blocks, kv_heads maps, block,
    dim]; v goes to v_cache [blocks, kv_heads, vdim, block].  Without caches (a layer that reads
    another layer's) only q is made."""
    T, H, G, M, d, dv = proj.shape[0], heads, kv_heads, maps, dim, vdim
    nq, nk = H * M * d, G * M * d
    pf = proj.float()
    if bias is not None:
        pf = pf[:, :bias.numel()] + bias.float()[None, :]
    half = rot_dims // 2
    c, s = _rot_table(cos_sin, positions, half) if half > 0 else (None, None)

    def norm_rot(t, w):
        t = t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps) * w.float()
        if half > 0:
            u, w_ = t[..., :half].clone(), t[..., half:2 * half].clone()
            t[..., :half] = u * c[:, None, :] - w_ * s[:, None, :]
            t[..., half:2 * half] = w_ * c[:, None, :] + u * s[:, None, :]
        return t

    q = norm_rot(pf[:, :nq].reshape(T, H * M, d).clone(), qnorm_w) * qscale
    q = q.view(T, G, H // G, M, d).transpose(2, 3).reshape(T, H * M, d)
    if k_cache is not None:
        k = norm_rot(pf[:, nq:nq + nk].reshape(T, G * M, d).clone(), knorm_w)
        v = pf[:, nq + nk:nq + nk + G * dv].reshape(T, G, dv)
        live = slots >= 0
        sl = slots[live].long()
        BSz = k_cache.shape[2]
        k_cache[sl // BSz, :, sl % BSz] = k[live].to(k_cache.dtype)
        v_cache[sl // BSz, :, :, sl % BSz] = v[live].to(v_cache.dtype)
    return q.to(proj.dtype)


def diff_combine(a, heads, kv_heads, vdim, lam, eps, out_scale, out_dtype):
    """a [T, 2 heads vdim] f32: per key/value head the first-map outputs of its query heads, then the
    second-map outputs.  o = a1 - lam a2 per head, to unit RMS over vdim, times ``out_scale``."""
    T, R = a.shape[0], heads // kv_heads
    a = a.float().view(T, kv_heads, 2, R, vdim)
    o = (a[:, :, 0] - lam * a[:, :, 1]).reshape(T, heads, vdim)
    o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * out_scale
    return o.reshape(T, heads * vdim).to(out_dtype)


# ----------------------------------------------------------------------------- gated outer-product recurrences

def ssd_scan(xbc, proj, dt_col, heads, vdim, n_state, groups, dt_bias, neg_a, D, state, qstart, qlen, ctx, rows):
    """Mamba-2 recurrence.  xbc [T, heads vdim + 2 groups N] (x | B | C, convolved and activated),
    step logits in proj[:, dt_col : dt_col + heads].  dt = softplus(. + dt_bias); per head (B, C of
    group head // (heads / groups)):  S <- exp(neg_a dt) S + dt B x^T,  y = S^T C + D x.  state
    [slots, heads, N, vdim] f32; returns y [T, heads vdim] f32."""
    T, H, dv, N, G = xbc.shape[0], heads, vdim, n_state, groups
    out = torch.zeros((T, H * dv), dtype=torch.float32, device=xbc.device)
    rep = H // G
    for q0, n, cx, row in _seq_meta(qstart, qlen, ctx, rows):
        blk = xbc[q0:q0 + n].float()
        x = blk[:, :H * dv].reshape(n, H, dv)
        B = blk[:, H * dv:H * dv + G * N].reshape(n, G, N).repeat_interleave(rep, 1)
        C = blk[:, H * dv + G * N:H * dv + 2 * G * N].reshape(n, G, N).repeat_interleave(rep, 1)
        dt = torch.nn.functional.softplus(proj[q0:q0 + n, dt_col:dt_col + H].float() + dt_bias.float()[None, :])
        dA = torch.exp(neg_a.float()[None, :] * dt)
        S = state[row].clone() if cx - n > 0 else torch.zeros((H, N, dv), dtype=torch.float32, device=xbc.device)
        y = torch.empty((n, H, dv), dtype=torch.float32, device=xbc.device)
        for t in range(n):
            S = dA[t][:, None, None] * S + (dt[t][:, None] * B[t])[:, :, None] * x[t][:, None, :]
            y[t] = torch.einsum("hnv,hn->hv", S, C[t]) + D.float()[:, None] * x[t]
        state[row] = S
        out[q0:q0 + n] = y.reshape(n, H * dv)
    return out


def gated_group_norm(y, z, w, groups, eps, out_dtype):
    """rmsnorm over each of ``groups`` equal parts of y silu(z), times w (y f32 [T, n], z [T, >= n])."""
    g = y.float() * torch.nn.functional.silu(z[:, :y.shape[1]].float())
    return rms_rows(g, w, eps, out_dtype, groups)


def mlstm(proj, heads, dim, vdim, gate_b, cap, state, nm, eps, norm_w, qstart, qlen, ctx, rows):
    """Matrix-memory LSTM.  proj [T, 2 heads dim + 2 heads vdim + 2 heads] (q | k | v | output gate |
    input-gate logits | forget-gate logits), gate_b f32 [2 heads].  q times dim^-1/2;
    i = cap tanh(. / cap), f = logsigmoid(cap tanh(. / cap)); with a running maximum m (0 at the
    start):  m' = max(f + m, i),  S <- exp(f + m - m') S + exp(i - m') k v^T,  n likewise with k,
    o = S^T q / (max(|n . q|, exp(-m')) + 1e-6).  Each head's o to unit RMS, times norm_w, times
    sigmoid(gate).  state [slots, heads, dim, vdim] f32; nm [slots, heads, copies, dim + 1] f32
    holds n and, last, m (every copy the same: the kernel keeps one per block of value columns)."""
    T, H, d, dv = proj.shape[0], heads, dim, vdim
    out = torch.zeros((T, H * dv), dtype=proj.dtype, device=proj.device)
    logsig = torch.nn.functional.logsigmoid
    for q0, n_, cx, row in _seq_meta(qstart, qlen, ctx, rows):
        blk = proj[q0:q0 + n_].float()
        q = blk[:, :H * d].reshape(n_, H, d) * (d ** -0.5)
        k = blk[:, H * d:2 * H * d].reshape(n_, H, d)
        v = blk[:, 2 * H * d:2 * H * d + H * dv].reshape(n_, H, dv)
        g = blk[:, 2 * H * d + H * dv:2 * H * d + 2 * H * dv]
        z = blk[:, 2 * H * d + 2 * H * dv:2 * H * d + 2 * H * dv + 2 * H] + gate_b.float()[None, :]
        ig = cap * torch.tanh(z[:, :H] / cap)
        fg = logsig(cap * torch.tanh(z[:, H:] / cap))
        if cx - n_ > 0:
            S, nv, m = state[row].clone(), nm[row, :, 0, :d].clone(), nm[row, :, 0, d].clone()
        else:
            S = torch.zeros((H, d, dv), dtype=torch.float32, device=proj.device)
            nv, m = torch.zeros((H, d), dtype=torch.float32, device=proj.device), torch.zeros(H, device=proj.device)
        o = torch.empty((n_, H, dv), dtype=torch.float32, device=proj.device)
        for t in range(n_):
            m2 = torch.maximum(fg[t] + m, ig[t])
            a, b = torch.exp(fg[t] + m - m2), torch.exp(ig[t] - m2)
            S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
            nv = a[:, None] * nv + b[:, None] * k[t]
            m = m2
            den = torch.maximum((nv * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
            o[t] = torch.einsum("hdv,hd->hv", S, q[t]) / den[:, None]
        state[row] = S
        nm[row, :, :, :d] = nv[:, None, :]
        nm[row, :, :, d] = m[:, None]
        o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
        out[q0:q0 + n_] = (o.reshape(n_, H * dv) * norm_w.float()[None, :] * torch.sigmoid(g)).to(proj.dtype)
    return out


# ----------------------------------------------------------------------------- PolyNorm, grouped sigmoid router, SwiGLU experts

def polynorm(z, coef, eps):
    """a N(z) + b N(z^2) + c N(z^3) + e per row, N(u) = u / sqrt(mean(u^2) + eps); coef = (a, b, c, e) f32."""
    zf = z.float()
    a, b, c, e = coef.float().tolist()
    N = lambda u: u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps)
    return (a * N(zf) + b * N(zf * zf) + c * N(zf * zf * zf) + e).to(z.dtype)


def route_topk(logits, n_out, top, count=1, keep=1, score="sigmoid", group_score="top2", correction=None, real=None):
    """Group-limited top-k routing over the first ``n_out`` columns of f32 logits [T, >= n_out].
    Scores s = sigmoid or softmax of the logits; the choice is made on s + ``correction`` (f32
    [n_out]).  The outputs form ``count`` groups of neighbours; a group scores the sum of its two best
    choice scores ("top2") or its best ("max"); the ``top`` best outputs inside the ``keep`` best
    groups are chosen (ties: the lower index); weights = their scores s as they are.  ``real`` < n_out:
    the outputs from ``real`` on are identity experts; their weights are summed per token into the
    third result and left as 0 in the second.  -> ids [T, top] int32, w [T, top] f32, idw [T] f32."""
    z = logits[:, :n_out].float()
    s = torch.sigmoid(z) if score == "sigmoid" else torch.softmax(z, -1)
    ch = s if correction is None else s + correction.float()[None, :]
    T, E = s.shape
    per = E // count
    allowed = torch.ones((T, E), dtype=torch.bool, device=s.device)
    if count > 1 and keep < count:
        gv = ch.view(T, count, per)
        gs = gv.topk(min(2, per), -1).values.sum(-1) if group_score == "top2" else gv.max(-1).values
        order = torch.sort(gs, dim=-1, descending=True, stable=True).indices[:, :keep]
        ok = torch.zeros((T, count), dtype=torch.bool, device=s.device)
        ok.scatter_(1, order, True)
        allowed = ok.repeat_interleave(per, 1)
    masked = torch.where(allowed, ch, torch.full_like(ch, float("-inf")))
    ids = torch.sort(masked, dim=-1, descending=True, stable=True).indices[:, :top]
    w = s.gather(1, ids)
    idw = torch.zeros(T, dtype=torch.float32, device=s.device)
    if real is not None and real < n_out:
        ident = ids >= real
        idw = torch.where(ident, w, torch.zeros_like(w)).sum(-1)
        w = torch.where(ident, torch.zeros_like(w), w)
    return ids.to(torch.int32), w, idw


def group_router(logits, top, count, keep):
    """Sigmoid scores, a group scores the sum of its two best experts, weights = the chosen scores
    (``route_topk`` with its defaults).  -> ids [T, top] int32, w [T, top] f32."""
    ids, w, _ = route_topk(logits, logits.shape[1], top, count, keep)
    return ids, w


def swiglu_scale(gu, gate, ff):
    """Dense form of routed SwiGLU experts: gu [T, E 2 ff] (per expert: gate columns, then up columns)
    -> [T, E ff] = silu(gate part) * up part * gate[t, expert] (zero for experts the token does not use)."""
    T = gu.shape[0]
    g = gu.float().view(T, -1, 2, ff)
    y = torch.nn.functional.silu(g[:, :, 0]) * g[:, :, 1] * gate.float()[:, :, None]
    return y.reshape(T, -1).to(gu.dtype)


def softcap(x, cap):
    """cap * tanh(x / cap) in f32."""
    return cap * torch.tanh(x.float() / cap)


# ----------------------------------------------------------------------------- layer-norm layers with layer scale, wide q/k norms, gated activations

def ls_resadd_ln(x, w, b, eps, out_dtype, y=None, ls=None, bias=None, y2=None, g2=None, h=None, hw=None):
    """The tail of a sublayer of a pre-norm model and the layer norm ahead of the next one:
    x (f32 stream, in place) += ls * (y + bias + sigmoid(g2) y2 + hw h), every term after y optional
    (``g2`` and ``hw`` hold one number per token), then returns layernorm(x) * w + b in ``out_dtype``
    (mean and variance over the row, eps inside the root).  Without y the stream is only normed."""
    if y is not None:
        t = y.float()
        if bias is not None:
            t = t + bias.float()
        if y2 is not None:
            t = t + (y2.float() if g2 is None else torch.sigmoid(g2.float()).reshape(-1, 1) * y2.float())
        if h is not None:
            t = t + hw.float().reshape(-1, 1) * h.float()
        x += t if ls is None else t * ls.float()
    return torch.nn.functional.layer_norm(x, (x.shape[-1],), w.float(), b.float(), eps).to(out_dtype)


def proj_norm_prep(proj, heads, kv_heads, dim, vdim, qnorm_w, knorm_w, cos_sin, rot_dims, interleaved, eps, qscale,
                   vnorm, positions, slots, k_cache, v_cache):
    """Attention inputs whose q / k norm runs over the whole projection: proj [T, >= heads dim
    (+ kv_heads dim + kv_heads vdim)] (q | k | v).  q (all heads together) and k (all key heads
    together) get an RMS norm with weights of that length, then rotary positions on the first
    ``rot_dims`` dims of every head, pairs (2i, 2i + 1) when ``interleaved`` else (i, i + rot_dims/2);
    q times ``qscale[head]``.  With ``vnorm`` every value head is divided by its root mean square.
    k and v go to their page slots (k_cache [blocks, kv_heads, block, dim], v_cache [blocks,
    kv_heads, vdim, block]); without caches (a layer that reads another layer's) only q is made.
    Returns q [T, heads, dim]."""
    T, H, G, d, dv = proj.shape[0], heads, kv_heads, dim, vdim
    pf = proj.float()
    half = rot_dims // 2
    c, s = _rot_table(cos_sin, positions, half) if half > 0 else (None, None)

    def norm_rot(t, w, n):
        t = (t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps) * w.float()).reshape(T, n, d).clone()
        if half > 0:
            cc, ss = c[:, None, :], s[:, None, :]
            if interleaved:
                u, w_ = t[..., 0:rot_dims:2].clone(), t[..., 1:rot_dims:2].clone()
                t[..., 0:rot_dims:2] = u * cc - w_ * ss
                t[..., 1:rot_dims:2] = w_ * cc + u * ss
            else:
                u, w_ = t[..., :half].clone(), t[..., half:2 * half].clone()
                t[..., :half] = u * cc - w_ * ss
                t[..., half:2 * half] = w_ * cc + u * ss
        return t

    q = norm_rot(pf[:, :H * d], qnorm_w, H) * qscale.float()[None, :, None]
    if k_cache is not None:
        k = norm_rot(pf[:, H * d:(H + G) * d], knorm_w, G)
        v = pf[:, (H + G) * d:(H + G) * d + G * dv].reshape(T, G, dv)
        if vnorm:
            v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
        live = slots >= 0
        sl = slots[live].long()
        BSz = k_cache.shape[2]
        k_cache[sl // BSz, :, sl % BSz] = k[live].to(k_cache.dtype)
        v_cache[sl // BSz, :, :, sl % BSz] = v[live].to(v_cache.dtype)
    return q.to(proj.dtype)


def glu_act(gu, bias=None, mode="swiglu", limit=0.0, alpha=1.0):
    """gu [T, 2 ff] (gate columns, then up columns), ``bias`` f32 over the same columns -> [T, ff].
    "swiglu": silu(g) u.  "clamped": g <- min(g, limit), u <- clamp(u, -limit, limit), then
    g sigmoid(alpha g) (u + 1)."""
    f = gu.float()
    if bias is not None:
        f = f + bias.float()
    ff = f.shape[1] // 2
    g, u = f[:, :ff], f[:, ff:]
    if mode == "swiglu":
        return (torch.nn.functional.silu(g) * u).to(gu.dtype)
    g = g.clamp(max=limit)
    u = u.clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)
