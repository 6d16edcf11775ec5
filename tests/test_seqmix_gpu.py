"""Numerics of the sequence-mixer HIP kernels (csrc/kernels/seqmix.hip, latent.hip, the squared-ReLU
expert mode of moe.hip) against the plain-PyTorch f32 references of the same ops (ops.reference),
in bf16 and f32, over packed batches of unequal sequences that continue from state slots."""
import pytest
import torch

from distributed_llm_amd import ops
from distributed_llm_amd.ops import reference as ref
from distributed_llm_amd.ops import seqmix

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.bfloat16, torch.float32]


@pytest.fixture(autouse=True, scope="module")
def _native():
    assert ops.native_available(), "HIP extension must be built for GPU tests"


def tol(dt):
    return dict(atol=2e-2, rtol=2e-2) if dt == torch.bfloat16 else dict(atol=2e-5, rtol=2e-5)


def i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def batch(qlens, starts):
    """Packed metadata of sequences with ``qlens`` new tokens after ``starts`` old ones; slots are
    given out of order on purpose."""
    qstart, t = [], 0
    for n in qlens:
        qstart.append(t)
        t += n
    ctx = [a + n for a, n in zip(starts, qlens)]
    rows = list(reversed(range(len(qlens))))
    pos = [p for a, n in zip(starts, qlens) for p in range(a, a + n)]
    return t, i32(qstart), i32(qlens), i32(ctx), i32(rows), i32(pos)


CASES = [([5, 1, 0, 19], [0, 7, 3, 2]), ([1, 1, 1], [4, 0, 33]), ([70], [0]), ([2, 3], [1, 0])]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("n", [24, 104, 328, 1000])
def test_rms_rows_and_resadd(dt, n):
    torch.manual_seed(0)
    x = torch.randn(13, n + 8, device=DEV).to(dt)[:, 3:3 + n]      # a column slice
    w = torch.randn(n, device=DEV)
    torch.testing.assert_close(seqmix.rms_rows(x, w, 1e-6).float(), ref.rms_rows(x, w, 1e-6).float(), **tol(dt))
    torch.testing.assert_close(seqmix.rms_rows(x, None, 1e-5, torch.float32), ref.rms_rows(x, None, 1e-5, torch.float32),
                               atol=1e-5, rtol=1e-5)
    y = torch.randn(13, n, device=DEV).to(dt)
    r1 = torch.randn(13, n, device=DEV)
    r2 = r1.clone()
    l1 = torch.empty(13, n, device=DEV, dtype=dt) if dt == torch.bfloat16 else None
    l2 = l1.clone() if l1 is not None else None
    seqmix.norm_resadd(y, w, 1e-6, r1, l1)
    ref.norm_resadd(y, w, 1e-6, r2, l2)
    torch.testing.assert_close(r1, r2, atol=1e-5, rtol=1e-5)
    if l1 is not None:
        torch.testing.assert_close(l1.float(), l2.float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("C,N,K,R", [(40, 20, 3, 5), (128, 16, 4, 8), (72, 1, 2, 3), (64, 40, 1, 4)])
def test_conv_and_scan(dt, case, C, N, K, R):
    torch.manual_seed(1)
    qlens, starts = case
    T, qstart, qlen, ctx, rows, _ = batch(qlens, starts)
    slots = len(qlens) + 1
    xz = torch.randn(T, 2 * C, device=DEV).to(dt)
    w, b = torch.randn(C, K, device=DEV) * 0.5, torch.randn(C, device=DEV) * 0.1
    conv0 = torch.randn(slots, K - 1, C, device=DEV).to(dt)
    ssm0 = torch.randn(slots, C, N, device=DEV)
    y = seqmix.causal_conv_silu(xz, w, b, conv0, qstart, qlen, ctx, rows)
    yr = ref.causal_conv_silu(xz, w, b, conv0, qstart, qlen, ctx, rows)
    torch.testing.assert_close(y.float(), yr.float(), **tol(dt))
    dbc = torch.randn(T, R + 2 * N + 3, device=DEV).to(dt)[:, :R + 2 * N]
    dt_raw = (torch.randn(T, C, device=DEV) * 2).to(dt)
    dtb = torch.randn(C, device=DEV)
    A = -torch.exp(torch.randn(C, N, device=DEV))
    D = torch.randn(C, device=DEV)
    c1, s1, c2, s2 = conv0.clone(), ssm0.clone(), conv0.clone(), ssm0.clone()
    o1 = seqmix.selective_scan(yr, dt_raw, dtb, A, dbc, R, D, xz, s1, c1, qstart, qlen, ctx, rows)
    o2 = ref.selective_scan(yr, dt_raw, dtb, A, dbc, R, D, xz, s2, c2, qstart, qlen, ctx, rows)
    torch.testing.assert_close(o1.float(), o2.float(), **tol(dt))
    torch.testing.assert_close(s1, s2, atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(c1.float(), c2.float(), atol=0, rtol=0)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("chunked", [False, True])
@pytest.mark.parametrize("H,d,dv,rot", [(2, 64, 48, 32), (3, 32, 24, 16), (1, 16, 80, 0), (4, 128, 128, 64)])
def test_retention(dt, case, H, d, dv, rot, chunked):
    torch.manual_seed(2)
    qlens, starts = case
    T, qstart, qlen, ctx, rows, pos = batch(qlens, starts)
    qkvg = torch.randn(T, 2 * H * d + 2 * H * dv, device=DEV).to(dt)
    table = ops.rope_cos_sin(128, max(rot, 2), 10000.0, DEV)
    decay = torch.tensor([1.0 - 2.0 ** (-2 - h) for h in range(H)], device=DEV)
    st0 = torch.randn(len(qlens) + 1, H, d, dv, device=DEV)
    s1, s2 = st0.clone(), st0.clone()
    o1 = seqmix.retention(qkvg, H, d, dv, table, rot, decay, s1, 1e-6, pos, qstart, qlen, ctx, rows, chunked=chunked)
    o2 = ref.retention(qkvg, H, d, dv, table, rot, decay, s2, 1e-6, pos, qstart, qlen, ctx, rows)
    torch.testing.assert_close(o1.float(), o2.float(), **tol(dt))
    torch.testing.assert_close(s1, s2, atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("splits", [1, 3, 16])
@pytest.mark.parametrize("mfma", [False, True, 32])
@pytest.mark.parametrize("H,dim,rot,rank", [(8, 32, 16, 96), (3, 16, 8, 40), (20, 32, 16, 128), (1, 8, 64, 512), (2, 8, 6, 70)])
def test_latent_attention(dt, case, H, dim, rot, rank, splits, mfma):
    if mfma and dt != torch.bfloat16:
        pytest.skip("the matrix-core kernel serves bf16 models")
    wg_rows = 32 if mfma == 32 else 16
    torch.manual_seed(3)
    qlens, starts = case
    T, qstart, qlen, ctx, rows, pos = batch(qlens, starts)
    S, nblk = len(qlens), 12
    table = ops.rope_cos_sin(256, rot, 10000.0, DEV)
    perm = torch.randperm(S * nblk, device=DEV).to(torch.int32).view(S, nblk)       # scattered pages
    cache1 = torch.zeros(S * nblk, 16, rank + rot, device=DEV, dtype=dt)
    cache2 = cache1.clone()
    # every sequence's earlier tokens, then this step's, through the cache-write kernel
    for lo, hi in ((0, None), (None, 0)):
        ps, sl = [], []
        for s, (a, n) in enumerate(zip(starts, qlens)):
            rng = range(0, a) if hi is None else range(a, a + n)
            for p_ in rng:
                ps.append(p_)
                sl.append(int(perm[s, p_ // 16]) * 16 + p_ % 16)
        if not ps:
            continue
        ckv = torch.randn(len(ps), rank + rot + 5, device=DEV).to(dt)[:, 5:]
        wn = torch.rand(rank, device=DEV) + 0.5
        seqmix.latent_kv_write(ckv, rank, wn, 1e-6, i32(ps), table, i32(sl), cache1)
        ref.latent_kv_write(ckv, rank, wn, 1e-6, i32(ps), table, i32(sl), cache2)
    torch.testing.assert_close(cache1.float(), cache2.float(), **tol(dt))
    qa = (torch.randn(H, T, rank, device=DEV) * 0.3).to(dt)
    q = torch.randn(T, H * (dim + rot), device=DEV).to(dt)
    from distributed_llm_amd.models.llama import AttnMeta
    meta = AttnMeta(slots=None, block_tables=perm, qstart=qstart, qlen=qlen, ctx=ctx, tile_seq=None, tile_tok0=None,
                    last_idx=None, host_qlen=qlens)
    ts, tt = meta.latent_tiles(H, DEV, wg_rows)
    o1 = seqmix.latent_attention(qa, q, dim, rot, pos, table, cache2, perm, qstart, qlen, ctx, ts, tt, 0.2, splits=splits, mfma=bool(mfma), rows=wg_rows)
    o2 = ref.latent_attention(qa, q, dim, rot, pos, table, cache2, perm, qstart, qlen, ctx, 0.2)
    torch.testing.assert_close(o1.float(), o2.float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
def test_relu2_and_dense_gate(dt):
    torch.manual_seed(4)
    T, E, ff, k = 9, 6, 20, 3
    x = torch.randn(T, E * ff, device=DEV).to(dt)
    ids = torch.stack([torch.randperm(E, device=DEV)[:k] for _ in range(T)]).to(torch.int32)
    w = torch.rand(T, k, device=DEV)
    g = seqmix.dense_gate(ids, w, E)
    torch.testing.assert_close(g, ref.dense_gate(ids, w, E))
    torch.testing.assert_close(seqmix.relu2_scale(x, g, ff).float(), ref.relu2_scale(x, g, ff).float(), **tol(dt))
    torch.testing.assert_close(seqmix.relu2_scale(x).float(), ref.relu2_scale(x).float(), **tol(dt))


@pytest.mark.parametrize("T", [1, 7, 200])
def test_moe_relu2_grouped(T):
    torch.manual_seed(5)
    H, I, E, k = 256, 96, 6, 2
    x = (torch.randn(T, H, device=DEV)).to(torch.bfloat16)
    w1 = (torch.randn(E, I, H, device=DEV) * H ** -0.5).to(torch.bfloat16)
    w2 = (torch.randn(E, H, I, device=DEV) * I ** -0.5).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(E, device=DEV)[:k] for _ in range(T)]).to(torch.int32)
    w = torch.rand(T, k, device=DEV)
    assert seqmix.moe_ffn_relu2_ok(x, w1)
    y = seqmix.moe_ffn_relu2(x, ids, w, w1, w2)
    torch.testing.assert_close(y.float(), ref.moe_ffn_relu2(x, ids, w, w1, w2).float(), atol=3e-2, rtol=3e-2)


# ----------------------------------------------------------------------------- pre/post-norm tails, depth average, GELU

@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("n", [24, 200, 1032])
@pytest.mark.parametrize("pair", [False, True])
def test_resadd_norm(dt, n, pair):
    torch.manual_seed(2)
    a = torch.randn(9, n + 5, device=DEV).to(dt)[:, 2:2 + n]
    b = torch.randn(9, n, device=DEV).to(dt) if pair else None
    wa, wb, wp, wn = (torch.randn(n, device=DEV) for _ in range(4))
    for w_next in (wn, None):
        x1 = torch.randn(9, n, device=DEV)
        x2 = x1.clone()
        h1, h2 = torch.empty(9, n, device=DEV, dtype=dt), torch.empty(9, n, device=DEV, dtype=dt)
        kw = dict(b=b, wa=wa, wb=wb) if pair else {}
        seqmix.resadd_norm(a, wp, 1e-5, x1, w_next, h1, **kw)
        ref.resadd_norm(a, wp, 1e-5, x2, w_next, h2, **kw)
        torch.testing.assert_close(x1, x2, atol=2e-5, rtol=2e-5)
        torch.testing.assert_close(h1.float(), h2.float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("pair", [False, True])
def test_resadd_norm_with_depth_average(dt, pair):
    """The layer-ending form: the residual update and the weighted sum over the stack in one launch."""
    torch.manual_seed(8)
    T, n = 7, 136
    X1 = torch.randn(5, T, n, device=DEV)
    X2 = X1.clone()
    a, b = torch.randn(T, n, device=DEV).to(dt), torch.randn(T, n, device=DEV).to(dt)
    wa, wb, wp, wn, dw = (torch.randn(k, device=DEV) for k in (n, n, n, n, 4))
    kw = dict(b=b, wa=wa, wb=wb) if pair else {}
    for slot in (1, 3):
        h1, h2 = torch.empty(T, n, device=DEV, dtype=dt), torch.empty(T, n, device=DEV, dtype=dt)
        o1 = seqmix.resadd_norm(a, wp, 1e-5, X1[slot], wn, h1, depth=(X1, dw, slot + 1), **kw)
        o2 = ref.resadd_norm(a, wp, 1e-5, X2[slot], None, None, **kw)
        o2 = ref.depth_mix(X2, dw, slot + 1, wn, 1e-5, h2)
        torch.testing.assert_close(X1, X2, atol=2e-5, rtol=2e-5)
        torch.testing.assert_close(o1, X1[slot + 1], atol=0, rtol=0)
        torch.testing.assert_close(h1.float(), h2.float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
def test_depth_mix_and_gelu(dt):
    torch.manual_seed(3)
    X1 = torch.randn(6, 11, 72, device=DEV)
    X2 = X1.clone()
    w, wn = torch.randn(5, device=DEV), torch.randn(72, device=DEV)
    h1, h2 = torch.empty(11, 72, device=DEV, dtype=dt), torch.empty(11, 72, device=DEV, dtype=dt)
    for n in (1, 3, 5):
        seqmix.depth_mix(X1, w, n, wn, 1e-5, h1)
        ref.depth_mix(X2, w, n, wn, 1e-5, h2)
        torch.testing.assert_close(X1, X2, atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(h1.float(), h2.float(), **tol(dt))
    x = (torch.randn(7, 100, device=DEV) * 3).to(dt)
    torch.testing.assert_close(seqmix.gelu_erf(x).float(), ref.gelu_erf(x).float(), **tol(dt))


# ----------------------------------------------------------------------------- grouped-query attention over pages

def _pages(case, G, d, dv, dt, BSz=16):
    qlens, starts = case
    T, qstart, qlen, ctx, rows, pos = batch(qlens, starts)
    nb = max((a + n + BSz - 1) // BSz for a, n in zip(starts, qlens))
    S = len(qlens)
    perm = torch.randperm(S * nb + 3, device=DEV)[:S * nb].to(torch.int32).view(S, nb)     # pages out of order
    kc = (torch.randn(S * nb + 3, G, BSz, d, device=DEV) * 0.5).to(dt)
    vc = torch.randn(S * nb + 3, G, dv, BSz, device=DEV).to(dt)
    slots = i32([int(perm[i, p // BSz]) * BSz + p % BSz for i, (a, n) in enumerate(zip(starts, qlens)) for p in range(a, a + n)])
    return T, qstart, qlen, ctx, pos, perm.contiguous(), kc, vc, slots


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CASES + [([40, 3], [90, 130])])
@pytest.mark.parametrize("H,G,d,dv,rot", [(4, 2, 16, 8, 8), (6, 2, 88, 56, 20), (3, 3, 40, 72, 40), (34, 2, 8, 5, 0),
                                          (8, 1, 64, 64, 32), (2, 1, 136, 200, 64)])
def test_attn_prep_and_paged_gqa(dt, case, H, G, d, dv, rot):
    from distributed_llm_amd.models.llama import AttnMeta
    torch.manual_seed(4)
    T, qstart, qlen, ctx, pos, bt, kc, vc, slots = _pages(case, G, d, dv, dt)
    proj = torch.randn(T, (H + G) * d + G * dv + H * dv + 3, device=DEV).to(dt)
    table = ops.rope_cos_sin(256, max(rot, 2), 100.0, DEV)
    qscale = torch.rand(H, device=DEV) * 2 + 0.5
    kc2, vc2 = kc.clone(), vc.clone()
    q1 = seqmix.attn_prep(proj, H, G, d, dv, table, rot, 1e-5, qscale, pos, slots, kc, vc)
    q2 = ref.attn_prep(proj, H, G, d, dv, table, rot, 1e-5, qscale, pos, slots, kc2, vc2)
    torch.testing.assert_close(q1.float(), q2.float(), **tol(dt))
    torch.testing.assert_close(kc.float(), kc2.float(), **tol(dt))
    torch.testing.assert_close(vc.float(), vc2.float(), atol=0, rtol=0)
    gate = proj[:, (H + G) * d + G * dv:(H + G) * d + G * dv + H * dv]
    want = ref.paged_gqa_attention(q2, kc2, vc2, bt, qstart, qlen, ctx, gate).float()
    meta = AttnMeta(slots=None, block_tables=bt, qstart=qstart, qlen=qlen, ctx=ctx, tile_seq=None, tile_tok0=None,
                    last_idx=None, host_qlen=case[0])
    forms = [False] + ([True] if seqmix.gqa_use_mfma(q2, H, G, d, dv, 16) else [])
    for mfma in forms:
        ts, tt = meta.latent_tiles(1, DEV, seqmix.gqa_tokens_per_tile(H, G, mfma))
        for splits in ((1, 2, 7) if mfma else (1,)):      # 7: more splits than some rows have key tiles, and than value dims
            got = seqmix.paged_gqa_attention(q2, kc2, vc2, bt, qstart, qlen, ctx, ts, tt, gate, mfma, splits).float()
            torch.testing.assert_close(got, want, **tol(dt))


def test_paged_gqa_mfma_keeps_small_weights():
    """One key carries almost all of a row's weight; the others' weights are ~1e-3 and their values
    large: the hi + lo split of the weights keeps their sum (a bf16-only weight would lose ~0.4 %)."""
    from distributed_llm_amd.models.llama import AttnMeta
    torch.manual_seed(5)
    H, G, d, dv, n = 2, 1, 64, 64, 200
    dt = torch.bfloat16
    T, qstart, qlen, ctx, pos, bt, kc, vc, slots = _pages(([n], [0]), G, d, dv, dt)
    q = (torch.randn(n, H, d, device=DEV) * 0.6).to(dt)
    vc = (vc.float() * 50).to(dt)
    want = ref.paged_gqa_attention(q, kc, vc, bt, qstart, qlen, ctx).float()
    meta = AttnMeta(slots=None, block_tables=bt, qstart=qstart, qlen=qlen, ctx=ctx, tile_seq=None, tile_tok0=None,
                    last_idx=None, host_qlen=[n])
    ts, tt = meta.latent_tiles(1, DEV, seqmix.gqa_tokens_per_tile(H, G, True))
    got = seqmix.paged_gqa_attention(q, kc, vc, bt, qstart, qlen, ctx, ts, tt, None, True).float()
    assert float((got - want).abs().max()) < 0.02 * float(want.abs().max())
    torch.testing.assert_close(got, want, atol=0.35, rtol=8e-3)      # outputs rounded to bf16 at |o| ~ 50


# ----------------------------------------------------------------------------- lightning attention, gated delta rule

@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("H,d,dv", [(2, 8, 6), (4, 48, 40), (1, 40, 130), (3, 128, 128)])
@pytest.mark.parametrize("chunked", [False, True])
def test_lightning_attention(dt, case, H, d, dv, chunked):
    torch.manual_seed(6)
    T, qstart, qlen, ctx, rows, pos = batch(*case)
    qkvg = torch.randn(T, 2 * H * d + 2 * H * dv + 5, device=DEV).to(dt)
    decay = torch.tensor([0.6, 0.9, 0.99, 1.0][:H], device=DEV)
    st1 = torch.randn(len(case[0]), H, d, dv, device=DEV) * 0.3
    st2 = st1.clone()
    nw = torch.randn(H * dv, device=DEV)
    got = seqmix.lightning_attention(qkvg, H, d, dv, decay, st1, 1e-5, nw, qstart, qlen, ctx, rows, chunked=chunked)
    want = ref.lightning_attention(qkvg, H, d, dv, decay, st2, 1e-5, nw, qstart, qlen, ctx, rows)
    torch.testing.assert_close(got.float(), want.float(), **tol(dt))
    torch.testing.assert_close(st1, st2, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("H,G,d,dv,K", [(4, 2, 8, 6, 3), (6, 2, 72, 24, 5), (1, 1, 20, 33, 1), (2, 1, 200, 18, 2), (2, 2, 128, 128, 4)])
def test_delta_rule_and_conv_refill(dt, case, H, G, d, dv, K):
    torch.manual_seed(7)
    T, qstart, qlen, ctx, rows, pos = batch(*case)
    C = 2 * G * d + H * dv
    S = len(case[0])
    proj = torch.randn(T, C + H * dv + 2 * H, device=DEV).to(dt)
    qkv = torch.nn.functional.silu(torch.randn(T, C, device=DEV)).to(dt)
    neg_a, dtb, nw = -torch.rand(H, device=DEV) * 2, torch.randn(H, device=DEV), torch.randn(dv, device=DEV)
    st1 = torch.randn(S, H, dv, d, device=DEV) * 0.3
    st2 = st1.clone()
    got = seqmix.delta_rule(qkv, proj[:, C:], H, G, d, dv, neg_a, dtb, nw, 1e-5, st1, qstart, qlen, ctx, rows)
    want = ref.delta_rule(qkv, proj[:, C:], H, G, d, dv, neg_a, dtb, nw, 1e-5, st2, qstart, qlen, ctx, rows)
    torch.testing.assert_close(got.float(), want.float(), **tol(dt))
    torch.testing.assert_close(st1, st2, atol=1e-4, rtol=1e-4)
    c1 = torch.randn(S, K - 1, C, device=DEV).to(dt)
    c2 = c1.clone()
    seqmix.conv_state_refill(proj, c1, qstart, qlen, ctx, rows)
    ref.conv_state_refill(proj, c2, qstart, qlen, ctx, rows)
    torch.testing.assert_close(c1.float(), c2.float(), atol=0, rtol=0)
    if max(case[0]) <= 1:      # a step of single tokens: the convolution refills the slots in its own launch
        w, b = torch.randn(C, K, device=DEV), torch.randn(C, device=DEV)
        c3 = c1.clone()
        y1 = seqmix.causal_conv_silu(proj, w, b, c3, qstart, qlen, ctx, rows, refill=True)
        y2 = ref.causal_conv_silu(proj, w, b, c1, qstart, qlen, ctx, rows)
        ref.conv_state_refill(proj, c1, qstart, qlen, ctx, rows)
        torch.testing.assert_close(y1.float(), y2.float(), **tol(dt))
        torch.testing.assert_close(c3.float(), c1.float(), atol=0, rtol=0)


# ----------------------------------------------------------------------------- differential attention, Mamba-2, mLSTM, PolyNorm, grouped router

@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("n,groups", [(24, 1), (96, 4), (328, 2), (1000, 5), (66, 33)])
def test_group_norms(dt, n, groups):
    torch.manual_seed(9)
    x = torch.randn(11, n + 8, device=DEV).to(dt)[:, 3:3 + n]
    w = torch.randn(n, device=DEV)
    torch.testing.assert_close(seqmix.rms_rows(x, w, 1e-6, groups=groups).float(),
                               ref.rms_rows(x, w, 1e-6, groups=groups).float(), **tol(dt))
    y, bias = torch.randn(11, n, device=DEV).to(dt), torch.randn(n, device=DEV)
    for b in (None, bias):
        r1 = torch.randn(11, n, device=DEV)
        r2 = r1.clone()
        l1 = torch.empty(11, n, device=DEV, dtype=dt)
        l2 = l1.clone()
        seqmix.norm_resadd(y, w, 1e-6, r1, l1, groups=groups, bias=b)
        ref.norm_resadd(y, w, 1e-6, r2, l2, groups=groups, bias=b)
        torch.testing.assert_close(r1, r2, atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(l1.float(), l2.float(), **tol(dt))
    yy, z = torch.randn(11, n, device=DEV), torch.randn(11, n + 5, device=DEV).to(dt)
    torch.testing.assert_close(seqmix.gated_group_norm(yy, z, w, groups, 1e-6, dt).float(),
                               ref.gated_group_norm(yy, z, w, groups, 1e-6, dt).float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CASES + [([40, 3], [90, 130])])
@pytest.mark.parametrize("H,G,d,dv,rot,win", [(4, 2, 16, 8, 8, 5), (6, 2, 88, 56, 20, 64), (3, 3, 40, 72, 40, 1), (8, 1, 64, 64, 32, 100),
                                              (4, 1, 56, 88, 28, 70), (2, 1, 136, 200, 64, 0), (5, 5, 24, 40, 0, 17)])
def test_diff_attention_kernels(dt, case, H, G, d, dv, rot, win):
    """Prep (bias, weighted norm before rotation, two maps a head), windowed attention with shared
    values in both kernel forms and every split count, and the combination of the maps."""
    from distributed_llm_amd.models.llama import AttnMeta
    torch.manual_seed(14)
    T, qstart, qlen, ctx, pos, bt, kc, _, slots = _pages(case, 2 * G, d, dv, dt)
    vc = torch.randn(kc.shape[0], G, dv, 16, device=DEV).to(dt)
    cols = 2 * H * d + 2 * G * d + G * dv
    proj = torch.randn(T, cols + 3, device=DEV).to(dt)
    bias = torch.randn(cols, device=DEV) * 0.3
    qw, kw = torch.rand(d, device=DEV) + 0.5, torch.rand(d, device=DEV) + 0.5
    table = ops.rope_cos_sin(256, max(rot, 2), 100.0, DEV)
    kc2, vc2 = kc.clone(), vc.clone()
    q1 = seqmix.qk_norm_prep(proj, bias, H, G, 2, d, dv, qw, kw, table, rot, 1e-5, 0.3, pos, slots, kc, vc)
    q2 = ref.qk_norm_prep(proj, bias, H, G, 2, d, dv, qw, kw, table, rot, 1e-5, 0.3, pos, slots, kc2, vc2)
    torch.testing.assert_close(q1.float(), q2.float(), **tol(dt))
    torch.testing.assert_close(kc.float(), kc2.float(), **tol(dt))
    torch.testing.assert_close(vc.float(), vc2.float(), **tol(dt))
    q3 = seqmix.qk_norm_prep(proj, bias[:2 * H * d], H, G, 2, d, dv, qw, kw, table, rot, 1e-5, 0.3, pos, slots, None, None)
    torch.testing.assert_close(q3.float(), q2.float(), **tol(dt))       # a layer that reads another layer's pages
    want = ref.paged_gqa_attention(q2, kc2, vc2, bt, qstart, qlen, ctx, None, win, True)
    meta = AttnMeta(slots=None, block_tables=bt, qstart=qstart, qlen=qlen, ctx=ctx, tile_seq=None, tile_tok0=None,
                    last_idx=None, host_qlen=case[0])
    forms = [False] + ([True] if seqmix.gqa_use_mfma(q2, 2 * H, 2 * G, d, dv, 16) else [])
    for mfma in forms:
        ts, tt = meta.latent_tiles(1, DEV, seqmix.gqa_tokens_per_tile(2 * H, 2 * G, mfma))
        for splits in ((1, 2, 7) if mfma else (1,)):
            got = seqmix.paged_gqa_attention(q2, kc2, vc2, bt, qstart, qlen, ctx, ts, tt, None, mfma, splits, window=win,
                                             out_f32=True)
            assert got.dtype == torch.float32
            torch.testing.assert_close(got, want, **tol(dt))
    o1 = seqmix.diff_combine(want, H, G, dv, 0.37, 1e-5, 0.7, dt)
    o2 = ref.diff_combine(want, H, G, dv, 0.37, 1e-5, 0.7, dt)
    torch.testing.assert_close(o1.float(), o2.float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("H,dv,N,G", [(4, 32, 24, 2), (3, 40, 20, 3), (2, 8, 128, 1), (6, 70, 5, 2), (1, 64, 300, 1)])
def test_ssd_scan(dt, case, H, dv, N, G):
    torch.manual_seed(15)
    qlens, starts = case
    T, qstart, qlen, ctx, rows, _ = batch(qlens, starts)
    slots = len(qlens) + 1
    inner = H * dv
    xbc = torch.randn(T, inner + 2 * G * N, device=DEV).to(dt)
    proj = torch.randn(T, 2 * inner + 2 * G * N + H + 3, device=DEV).to(dt)
    dt_col = 2 * inner + 2 * G * N
    dt_b, neg_a, D = torch.randn(H, device=DEV), -torch.rand(H, device=DEV) * 2, torch.randn(H, device=DEV)
    s1 = torch.randn(slots, H, N, dv, device=DEV)
    s2 = s1.clone()
    y1 = seqmix.ssd_scan(xbc, proj, dt_col, H, dv, N, G, dt_b, neg_a, D, s1, qstart, qlen, ctx, rows)
    y2 = ref.ssd_scan(xbc, proj, dt_col, H, dv, N, G, dt_b, neg_a, D, s2, qstart, qlen, ctx, rows)
    torch.testing.assert_close(y1, y2, atol=2e-3, rtol=2e-4)
    torch.testing.assert_close(s1, s2, atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("H,d,dv", [(4, 40, 48), (3, 20, 40), (2, 128, 8), (1, 7, 70), (2, 200, 64)])
def test_mlstm(dt, case, H, d, dv):
    torch.manual_seed(16)
    qlens, starts = case
    T, qstart, qlen, ctx, rows, _ = batch(qlens, starts)
    slots = len(qlens) + 1
    proj = torch.randn(T, 2 * H * (d + dv + 1) + 5, device=DEV).to(dt)
    proj[:, 2 * H * (d + dv):] *= 4          # gate logits across the cap's bend
    gate_b = torch.randn(2 * H, device=DEV)
    w = torch.rand(H * dv, device=DEV) + 0.5
    s1 = torch.randn(slots, H, d, dv, device=DEV)
    nm1 = torch.randn(slots, H, 1, d + 1, device=DEV).repeat(1, 1, seqmix.scan_col_blocks(dv), 1).contiguous()
    s2, nm2 = s1.clone(), nm1.clone()
    o1 = seqmix.mlstm(proj, H, d, dv, gate_b, 3.0, s1, nm1, 1e-5, w, qstart, qlen, ctx, rows)
    o2 = ref.mlstm(proj, H, d, dv, gate_b, 3.0, s2, nm2, 1e-5, w, qstart, qlen, ctx, rows)
    torch.testing.assert_close(o1.float(), o2.float(), **(tol(dt) if dt == torch.bfloat16 else dict(atol=2e-4, rtol=2e-4)))
    torch.testing.assert_close(s1, s2, atol=2e-4, rtol=2e-4)
    torch.testing.assert_close(nm1, nm2, atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("dt", DTYPES)
def test_polynorm_swiglu_softcap(dt):
    torch.manual_seed(17)
    for n in (24, 344, 1000):
        z = (torch.randn(9, n + 4, device=DEV) * 2).to(dt)[:, 1:1 + n]
        coef = torch.tensor([0.7, -0.4, 0.2, 0.1], device=DEV)
        torch.testing.assert_close(seqmix.polynorm(z, coef, 1e-6).float(), ref.polynorm(z, coef, 1e-6).float(), **tol(dt))
    E, ff = 6, 20
    gu = torch.randn(9, E * 2 * ff, device=DEV).to(dt)
    gate = torch.rand(9, E, device=DEV) * (torch.rand(9, E, device=DEV) > 0.5)
    torch.testing.assert_close(seqmix.swiglu_scale(gu, gate, ff).float(), ref.swiglu_scale(gu, gate, ff).float(), **tol(dt))
    x = (torch.randn(9, 77, device=DEV) * 40).to(dt)
    torch.testing.assert_close(seqmix.softcap(x, 25.0), ref.softcap(x, 25.0), atol=1e-4, rtol=1e-5)


@pytest.mark.parametrize("E,top,count,keep", [(16, 3, 2, 1), (16, 4, 1, 1), (12, 3, 4, 2), (64, 8, 8, 3), (5, 5, 5, 5), (6, 1, 6, 1),
                                              (200, 6, 4, 4)])
def test_group_router(E, top, count, keep):
    torch.manual_seed(18)
    logits = torch.randn(37, E, device=DEV) * 2
    i1, w1 = seqmix.group_router(logits, top, count, keep)
    i2, w2 = ref.group_router(logits, top, count, keep)
    assert torch.equal(i1, i2)
    torch.testing.assert_close(w1, w2, atol=1e-6, rtol=1e-6)


# ----------------------------------------------------------------------------- layer-norm layers, input convolution, wide q/k norms, sink attention

@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("n", [24, 104, 328, 1000, 4104, 8200])
@pytest.mark.parametrize("pad", [3, 8])      # rows of y that are, or are not, whole 16-byte vectors
@pytest.mark.parametrize("terms", ["none", "y", "y+bias", "all", "all-no-gate"])
def test_ls_resadd_ln(dt, n, terms, pad):
    torch.manual_seed(21)
    T = 11
    x1 = torch.randn(T, n, device=DEV) * 3 + 0.7
    x2 = x1.clone()
    w, b, ls, bias = (torch.randn(n, device=DEV) for _ in range(4))
    kw = {}
    if terms != "none":
        kw = dict(y=torch.randn(T, n + pad, device=DEV).to(dt)[:, :n], ls=ls)
    if terms in ("y+bias", "all"):
        kw["bias"] = bias
    if terms.startswith("all"):
        z = torch.randn(T, 5, device=DEV)
        kw.update(y2=torch.randn(T, n, device=DEV).to(dt), h=torch.randn(T, n, device=DEV).to(dt), hw=torch.rand(T, device=DEV))
        if terms == "all":
            kw["g2"] = z[:, 3]      # a column of a wider matrix
    got = seqmix.ls_resadd_ln(x1, w, b, 1e-5, dt, **kw)
    want = ref.ls_resadd_ln(x2, w, b, 1e-5, dt, **kw)
    torch.testing.assert_close(x1, x2, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(got.float(), want.float(), **tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CASES + [([300, 2, 41], [5, 0, 16])])
@pytest.mark.parametrize("C,K", [(40, 3), (128, 4), (72, 1), (64, 7), (1032, 5), (36, 2)])
def test_input_convolution(dt, case, C, K):
    """y = x + conv(x) without an activation; decode steps refill the slot in the same launch."""
    torch.manual_seed(22)
    T, qstart, qlen, ctx, rows, pos = batch(*case)
    x = torch.randn(T, C + 5, device=DEV).to(dt)
    w, b = torch.randn(C, K, device=DEV) * 0.5, torch.zeros(C, device=DEV)
    st1 = torch.randn(len(case[0]), K - 1, C, device=DEV).to(dt)
    st2, st3 = st1.clone(), st1.clone()
    single = max(case[0]) <= 1
    got = seqmix.causal_conv_silu(x, w, b, st1, qstart, qlen, ctx, rows, refill=single, act="residual")
    want = ref.causal_conv_silu(x, w, b, st2, qstart, qlen, ctx, rows, act="residual")
    torch.testing.assert_close(got.float(), want.float(), **tol(dt))
    if not single:
        seqmix.conv_state_refill(x, st1, qstart, qlen, ctx, rows)
    ref.conv_state_refill(x, st2, qstart, qlen, ctx, rows)
    torch.testing.assert_close(st1.float(), st2.float(), atol=0, rtol=0)
    if single:      # the same step with the output written over the input
        xc = x[:, :C].contiguous()
        out = seqmix.causal_conv_silu(xc, w, b, st3, qstart, qlen, ctx, rows, refill=True, act="residual", inplace=True)
        assert out.data_ptr() == xc.data_ptr()
        torch.testing.assert_close(out.float(), want.float(), **tol(dt))
        torch.testing.assert_close(st3.float(), st2.float(), atol=0, rtol=0)


@pytest.mark.parametrize("dt", DTYPES)
def test_glu_act(dt):
    torch.manual_seed(23)
    for ff in (70, 72, 1024):      # 72, 1024: rows of whole 16-byte vectors
        gu = (torch.randn(33, 2 * ff + 8, device=DEV) * 3).to(dt)[:, :2 * ff]
        bias = torch.randn(2 * ff, device=DEV)
        for kw in (dict(), dict(bias=bias), dict(bias=bias, mode="clamped", limit=1.5, alpha=1.702), dict(mode="clamped", limit=0.3, alpha=1.0)):
            torch.testing.assert_close(seqmix.glu_act(gu, **kw).float(), ref.glu_act(gu, **kw).float(), **tol(dt))


@pytest.mark.parametrize("score", ["softmax", "sigmoid"])
@pytest.mark.parametrize("group_score", ["max", "top2"])
@pytest.mark.parametrize("R,real,top,count,keep", [(16, 12, 3, 2, 1), (16, 16, 4, 1, 1), (12, 7, 3, 4, 2), (64, 60, 8, 8, 3), (5, 0, 5, 5, 5),
                                                   (6, 5, 1, 6, 1), (200, 190, 6, 4, 4)])
def test_route_topk(score, group_score, R, real, top, count, keep):
    torch.manual_seed(24)
    logits = torch.randn(37, R + 2, device=DEV) * 2
    for corr in (None, torch.randn(R, device=DEV) * 0.3 - 0.2):
        a = seqmix.route_topk(logits, R, top, count, keep, score, group_score, corr, real)
        b = ref.route_topk(logits, R, top, count, keep, score, group_score, corr, real)
        assert torch.equal(a[0], b[0])
        torch.testing.assert_close(a[1], b[1], atol=1e-6, rtol=1e-5)
        torch.testing.assert_close(a[2], b[2], atol=1e-6, rtol=1e-5)
        assert bool(((a[0] >= real) == (a[1] == 0)).all())


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", CASES + [([40, 3], [90, 130]), ([1, 1], [300, 77]), ([150], [170])])
@pytest.mark.parametrize("H,G,d,dv,rot,win,keep", [(4, 2, 16, 8, 8, 5, 3), (6, 2, 88, 56, 20, 64, 70), (3, 3, 40, 72, 40, 1, 0),
                                                   (8, 1, 80, 112, 20, 100, 9), (4, 1, 56, 88, 28, 70, 1), (2, 1, 136, 200, 64, 0, 9),
                                                   (5, 5, 24, 40, 0, 17, 130), (8, 2, 64, 64, 64, 3, 64)])
def test_sink_attention_kernels(dt, case, H, G, d, dv, rot, win, keep):
    """Prep (norm over the whole q / k projection before an interleaved rotation, unit-RMS values),
    then attention with a window, kept first keys and a sink, in both kernel forms and every split
    count; a layer that reads another layer's pages makes the same queries."""
    from distributed_llm_amd.models.llama import AttnMeta
    torch.manual_seed(25)
    T, qstart, qlen, ctx, pos, bt, kc, vc, slots = _pages(case, G, d, dv, dt)
    cols = H * d + G * (d + dv)
    proj = torch.randn(T, cols + 3, device=DEV).to(dt)
    qw, kw = torch.rand(H * d, device=DEV) + 0.5, torch.rand(G * d, device=DEV) + 0.5
    qscale = torch.rand(H, device=DEV) * 0.6 + 0.2
    table = ops.rope_cos_sin(512, max(rot, 2), 100.0, DEV)
    for inter in (True, False):
        kc2, vc2 = kc.clone(), vc.clone()
        kc1, vc1 = kc.clone(), vc.clone()
        q1 = seqmix.proj_norm_prep(proj, H, G, d, dv, qw, kw, table, rot, inter, 1e-5, qscale, inter, pos, slots, kc1, vc1)
        q2 = ref.proj_norm_prep(proj, H, G, d, dv, qw, kw, table, rot, inter, 1e-5, qscale, inter, pos, slots, kc2, vc2)
        torch.testing.assert_close(q1.float(), q2.float(), **tol(dt))
        torch.testing.assert_close(kc1.float(), kc2.float(), **tol(dt))
        torch.testing.assert_close(vc1.float(), vc2.float(), **tol(dt))
        stale = torch.full((T, H * dv), float("nan"), device=DEV).to(dt)
        q3 = seqmix.proj_norm_prep(proj, H, G, d, dv, qw, qw, table, rot, inter, 1e-5, qscale, inter, pos, slots, None, None,
                                   zero_rows=stale)
        torch.testing.assert_close(q3.float(), q2.float(), **tol(dt))
        assert float(stale.float().abs().max()) == 0.0 if T else True
    meta = AttnMeta(slots=None, block_tables=bt, qstart=qstart, qlen=qlen, ctx=ctx, tile_seq=None, tile_tok0=None,
                    last_idx=None, host_qlen=case[0])
    forms = [False] + ([True] if seqmix.gqa_use_mfma(q2, H, G, d, dv, 16) else [])
    for sink in (1.0, 0.0):
        want = ref.paged_gqa_attention(q2, kc2, vc2, bt, qstart, qlen, ctx, None, win, False, keep, sink).float()
        for mfma in forms:
            ts, tt = meta.latent_tiles(1, DEV, seqmix.gqa_tokens_per_tile(H, G, mfma))
            for splits in ((1, 2, 7) if mfma else (1,)):
                got = seqmix.paged_gqa_attention(q2, kc2, vc2, bt, qstart, qlen, ctx, ts, tt, None, mfma, splits, window=win,
                                                 keep_first=keep, sink=sink).float()
                torch.testing.assert_close(got, want, **tol(dt))
