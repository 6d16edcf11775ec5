"""Slow float64 oracle of the Dogilorn design, one function per mechanism, written from the design's
equations and sharing no code with the product path.

Notation: x is the residual stream [T, width] of ONE sequence, positions 0 .. T-1; a layer is
x <- x + ls1 * mixer(canon(LN1(x))) and then x <- x + ls2 * ff(LN2(x)), with LN a layer norm with
weight and bias, ls a learned vector and canon(h) = h + a short causal convolution of h over time.
Weights come as a dict under the checkpoint's names ('l<i>.mix.<name>', 'l<i>.mlp.<name>'), the
configuration as the parsed config.json.
"""
import torch

F64 = torch.float64


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def canon(h, w):
    """h + conv(h): per channel, conv(h)[t] = sum_j w[:, j] h[t - taps + 1 + j], zeros before the
    start.  h [T, C], w [C, taps]."""
    T, C = h.shape
    K = w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(K):
            s = t - K + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def rotate_pairs(x, pos, dims, base):
    """Rotate neighbouring pairs (2i, 2i + 1), i < dims / 2, of the last axis of x [T, heads, d] by
    the angle pos * base^(-2i / dims); entries from ``dims`` on pass unchanged."""
    out = x.clone()
    for i in range(dims // 2):
        a = pos.to(F64) * base ** (-2.0 * i / dims)
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def attention_kv(h, W, p, m, eps):
    """What an attention layer caches: keys [T, G, dim] (normed over the whole projection, rotated)
    and values [T, G, vdim] (every head at unit RMS)."""
    T, G, d, dv = h.shape[0], m["kv_heads"], m["dim"], m["vdim"]
    k = unit_rms(h @ W[p + "k"].T, eps) * W[p + "k.norm"]
    k = rotate_pairs(k.view(T, G, d), torch.arange(T), m["rot"]["dims"], m["rot"]["base"])
    v = unit_rms((h @ W[p + "v"].T).view(T, G, dv), eps)
    return k, v


def visible(i, j, size, keep_first):
    """Does position i see position j?"""
    return j <= i and (i - j < size or j < keep_first)


def sink_attention(h, W, p, m, eps, kv):
    """Grouped-query attention inside a sliding window that also keeps the first tokens; the softmax
    has one more term of score 0 in its denominator and no value for it."""
    T, H, G, d, dv = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    k, v = kv
    q = unit_rms(h @ W[p + "q"].T, eps) * W[p + "q.norm"]
    q = rotate_pairs(q.view(T, H, d), torch.arange(T), m["rot"]["dims"], m["rot"]["base"])
    size, first = m["mask"]["size"], m["mask"]["keep_first"]
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        tau = m["scale"] * W[p + "temp"][hd]
        for i in range(T):
            js = torch.tensor([j for j in range(i + 1) if visible(i, j, size, first)])
            e = torch.exp((k[js, g] @ q[i, hd]) * tau)
            pr = e / (1.0 + e.sum())
            out[i, hd] = pr @ v[js, g]
    return out.reshape(T, H * dv) @ W[p + "o"].T


def clamped_glu(h, W, p, f):
    """Dense feed-forward: g = min(Wg h + bg, limit), u = clamp(Wu h + bu, +-limit),
    W_down (g sigmoid(1.702 g) (u + 1)) + b."""
    lim = f["limit"]
    g = torch.clamp(h @ W[p + "gate"].T + W[p + "gate.b"], max=lim)
    u = torch.clamp(h @ W[p + "up"].T + W[p + "up.b"], min=-lim, max=lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T + W[p + "down.b"]


def swiglu(h, W, p):
    g = h @ W[p + "gate"].T
    return (g * torch.sigmoid(g) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(z, corr, top, count, keep):
    """One token's router logits z [R] -> (chosen indices, weights).  Scores are the softmax of z;
    the choice is made on scores + corr inside the ``keep`` groups (of ``count`` equal groups of
    neighbours) whose largest choice score is largest; the weights are the plain scores."""
    R = z.numel()
    s = torch.softmax(z, -1)
    c = s + corr
    n = R // count
    gs = torch.stack([c[g * n:(g + 1) * n].max() for g in range(count)])
    kept = sorted(range(count), key=lambda g: (-float(gs[g]), g))[:keep]
    allowed = [e for e in range(R) if e // n in kept]
    chosen = sorted(allowed, key=lambda e: (-float(c[e]), e))[:top]
    return chosen, [s[e] for e in chosen]


def experts(h, W, p, f):
    """Routed experts; the last ``identity`` router outputs stand for experts that return their
    input.  A shared expert, if any, is added times sigmoid(W_sg h)."""
    r = f["router"]
    E = r["experts"]
    g = r.get("groups") or {}
    T = h.shape[0]
    z = h @ W[p + "router"].T
    out = torch.zeros_like(h)
    for t in range(T):
        ids, ws = route(z[t], W[p + "correction"], r["top"], g.get("count", 1), g.get("keep", g.get("count", 1)))
        for e, w in zip(ids, ws):
            out[t] += w * (h[t] if e >= E else swiglu(h[t:t + 1], W, p + f"e{e}.")[0])
    if f.get("shared"):
        gate = torch.sigmoid(h @ W[p + "shared.sg"].T)
        out = out + gate * swiglu(h, W, p + "shared.")
    return out


def forward(tokens, W, cfg, taps=None):
    """Logits [T, vocab] of one sequence; ``taps`` (a list) receives the stream after every layer."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    cache = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        assert L["type"] == "attention"
        h = canon(layer_norm(x, W[p + "norm1"], W[p + "norm1.b"], eps), W[p + "canon1"])
        src = m.get("kv_from")
        if src is None:
            cache[i] = attention_kv(h, W, p + "mix.", m, eps)
        x = x + W[p + "ls1"] * sink_attention(h, W, p + "mix.", m, eps, cache[i if src is None else src])
        f = L.get("mlp")
        if f:
            h = layer_norm(x, W[p + "norm2"], W[p + "norm2.b"], eps)
            y = clamped_glu(h, W, p + "mlp.", f) if f["kind"] == "dense" else experts(h, W, p + "mlp.", f)
            x = x + W[p + "ls2"] * y
        if taps is not None:
            taps.append(x.clone())
    return layer_norm(x, W["final.norm"], W["final.norm.b"], eps) @ W["embed"].T


def greedy(tokens, W, cfg, n):
    """n arg-max continuations of a prompt (the whole sequence is recomputed for every token)."""
    seq, out = list(tokens), []
    for _ in range(n):
        out.append(int(forward(seq, W, cfg)[-1].argmax()))
        seq.append(out[-1])
    return out
