"""Slow float64 oracle of the Pebodra design, one function per mechanism, written from the design's
equations and sharing no code with the product path.

Notation: h is a sublayer's input [T, width]; positions count from 0; a layer is
x <- x + gnorm(mixer(x)) and then x <- x + gnorm(ff(x)) with gnorm the RMS norm taken separately
over equal consecutive parts of the vector.  Weights come as a dict under the checkpoint's names
('l<i>.mix.<name>', 'l<i>.mlp.<name>'), the configuration as the parsed config.json.
"""
import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x, w, groups, eps):
    """RMS norm of each of ``groups`` equal consecutive parts of the last axis, then times w."""
    T, n = x.shape
    return rms(x.view(T, groups, n // groups), eps).reshape(T, n) * w


def silu(x):
    return x * torch.sigmoid(x)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def logsigmoid(x):
    return -softplus(-x)


def gelu_tanh(x):
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))


def rotate_half(x, pos, dims, base):
    """Rotate the first ``dims`` entries of the last axis of x [T, ..., d]; entry i pairs with
    i + dims/2; angle = position * base^(-2i/dims)."""
    half = dims // 2
    if half == 0:
        return x
    f = base ** (-2.0 * torch.arange(half, dtype=F64) / dims)
    a = pos.to(F64)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(a).view(shape), torch.sin(a).view(shape)
    out = x.clone()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half], out[..., half:dims] = u * c - v * s, v * c + u * s
    return out


def short_conv(x, w, b):
    """Causal convolution per channel, zeros before the start: x [T, C], w [C, taps] whose last
    column multiplies the current token."""
    T, C = x.shape
    K = w.shape[1]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=F64), x], 0)
    return torch.stack([(padded[t:t + K] * w.T).sum(0) for t in range(T)]) + b


def attention_keys(h, W, p, m, eps):
    """Keys (normed, rotated) [T, G, 2, dim] and values [T, G, vdim] of an attention layer."""
    T, G, d, dv = h.shape[0], m["kv_heads"], m["dim"], m["vdim"]
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, 2, d)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, dv)
    k = rms(k, eps) * W[p + "k.norm"]
    rot = m.get("rot")
    if rot:
        k = rotate_half(k, torch.arange(T), rot["dims"], rot["base"])
    return k, v


def diff_attention(h, W, p, m, eps, kv):
    """Two softmax maps per head over a sliding window and shared values, combined as
    a1 - lambda a2, each head to unit RMS times (1 - diff)."""
    T, H, G, d, dv = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    k, v = kv
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, 2, d)
    q = rms(q, eps) * W[p + "q.norm"]
    rot = m.get("rot")
    if rot:
        q = rotate_half(q, torch.arange(T), rot["dims"], rot["base"])
    lam = (torch.exp((W[p + "lq1"] * W[p + "lk1"]).sum()) - torch.exp((W[p + "lq2"] * W[p + "lk2"]).sum())
           + m["diff"])
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    seen = (i - j >= 0) & (i - j < m["mask"]["size"]) if m.get("mask") else i - j >= 0
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        a = []
        for c in range(2):
            s = (q[:, hh, c] @ k[:, g, c].T) * m["scale"]
            s = s.masked_fill(~seen, float("-inf"))
            a.append(torch.softmax(s, -1) @ v[:, g])
        out[:, hh] = rms(a[0] - lam * a[1], eps) * (1.0 - m["diff"])
    return out.reshape(T, H * dv) @ W[p + "o"].T + W[p + "o.b"]


def mamba2(h, W, p, m, eps):
    """State-space duality layer: scalar decay per head, B and C shared by groups of heads."""
    T, H, dv, N, G = h.shape[0], m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * dv
    u = h @ W[p + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    xbc = silu(short_conv(xbc, W[p + "conv"], W[p + "conv.b"]))
    x = xbc[:, :inner].view(T, H, dv)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + W[p + "dt_bias"])
    A = torch.exp(W[p + "A_log"])
    y = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        S = torch.zeros(N, dv, dtype=F64)
        for t in range(T):
            S = torch.exp(-A[hh] * dt[t, hh]) * S + dt[t, hh] * torch.outer(B[t, g], x[t, hh])
            y[t, hh] = S.T @ C[t, g] + W[p + "D"][hh] * x[t, hh]
    y = y.reshape(T, inner) * silu(z)
    return group_norm(y, W[p + "norm"], m["norm_groups"], eps) @ W[p + "o"].T


def mlstm(h, W, p, m, eps):
    """Matrix memory with exponential input gate, sigmoid forget gate in log space and a running
    maximum that starts at zero."""
    T, H, d, dv, cap = h.shape[0], m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ W[p + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, d)
    v = (h @ W[p + "v"].T).view(T, H, dv)
    ig = cap * torch.tanh((h @ W[p + "i"].T + W[p + "i.b"]) / cap)
    fg = logsigmoid(cap * torch.tanh((h @ W[p + "f"].T + W[p + "f.b"]) / cap))
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        S, n, mx = torch.zeros(d, dv, dtype=F64), torch.zeros(d, dtype=F64), torch.zeros((), dtype=F64)
        for t in range(T):
            m_new = torch.maximum(fg[t, hh] + mx, ig[t, hh])
            a, b = torch.exp(fg[t, hh] + mx - m_new), torch.exp(ig[t, hh] - m_new)
            S = a * S + b * torch.outer(k[t, hh], v[t, hh])
            n = a * n + b * k[t, hh]
            mx = m_new
            den = torch.maximum((n @ q[t, hh]).abs(), torch.exp(-mx)) + 1e-6
            out[t, hh] = (S.T @ q[t, hh]) / den
    o = rms(out, eps).reshape(T, H * dv) * W[p + "norm"] * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def dense_ff(h, W, p, eps):
    """W_down act(W_up h), act = a N(z) + b N(z^2) + c N(z^3) + e with N the unit-RMS scaling."""
    z = h @ W[p + "up"].T
    a, b, c, e = W[p + "act"].tolist()
    act = a * rms(z, eps) + b * rms(z ** 2, eps) + c * rms(z ** 3, eps) + e
    return act @ W[p + "down"].T


def route(h, W, p, r):
    """Sigmoid scores; a group of neighbouring experts scores the sum of its two best; the ``top``
    best experts of the ``keep`` best groups, weights = their scores.  Returns [T, experts]."""
    g = r.get("groups") or {"count": 1, "keep": 1}
    E, top, cnt, keep = r["experts"], r["top"], g["count"], g["keep"]
    s = torch.sigmoid(h @ W[p + "router"].T)
    T = s.shape[0]
    gs = s.view(T, cnt, E // cnt).topk(min(2, E // cnt), -1).values.sum(-1)
    best = gs.topk(keep, -1).indices
    allowed = torch.zeros(T, cnt, dtype=torch.bool)
    allowed.scatter_(1, best, True)
    masked = s.masked_fill(~allowed.repeat_interleave(E // cnt, 1), float("-inf"))
    ids = masked.topk(top, -1).indices
    w = torch.zeros(T, E, dtype=F64)
    w.scatter_(1, ids, s.gather(1, ids))
    return w


def moe_ff(h, W, p, f):
    w = route(h, W, p, f["router"])
    out = torch.zeros_like(h)
    for e in range(f["router"]["experts"]):
        q = f"{p}e{e}."
        y = (silu(h @ W[q + "gate"].T) * (h @ W[q + "up"].T)) @ W[q + "down"].T
        out = out + w[:, e:e + 1] * y
    return out


def forward(cfg, W, tokens, taps=None):
    """Logits [T, vocab] of one sequence from position 0; ``taps`` collects the stream after every layer."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    x = W["embed"][torch.tensor(tokens)]
    kvs = {}
    for i, L in enumerate(cfg["layers"]):
        p, m, kind = f"l{i}.mix.", L["mixer"], L["type"]
        if kind == "attention":
            src = m.get("kv_from")
            if src is None:
                kvs[i] = attention_keys(x, W, p, m, eps)
            y = diff_attention(x, W, p, m, eps, kvs[i if src is None else src])
        elif kind == "mamba2":
            y = mamba2(x, W, p, m, eps)
        elif kind == "mlstm":
            y = mlstm(x, W, p, m, eps)
        else:
            raise ValueError(kind)
        x = x + group_norm(y, W[f"l{i}.norm1"], groups, eps)
        f = L.get("mlp")
        if f:
            y = dense_ff(x, W, f"l{i}.mlp.", eps) if f["kind"] == "dense" else moe_ff(x, W, f"l{i}.mlp.", f)
            x = x + group_norm(y, W[f"l{i}.norm2"], groups, eps)
        if taps is not None:
            taps.append(x.clone())
    lg = group_norm(x, W["final.norm"], groups, eps) @ W["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(lg / cap) if cap else lg


def greedy(cfg, W, prompt, n):
    """n arg-max continuations of a prompt (the whole sequence is recomputed for every token)."""
    seq, out = list(prompt), []
    for _ in range(n):
        out.append(int(forward(cfg, W, seq)[-1].argmax()))
        seq.append(out[-1])
    return out
