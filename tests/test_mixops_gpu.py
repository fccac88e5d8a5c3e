"""HIP kernels of the fp32-residual / delta-rule / talking-attention ops
against their plain PyTorch fp32 references (production_stack_amd.ops.
reference), in bfloat16 and float32, on shapes that exercise padding,
strided views, page borders, chunk/window edges and slot reuse."""

import math

import pytest
import torch

from production_stack_amd import ops
from production_stack_amd.ops import reference

pytestmark = pytest.mark.gpu

DTYPES = [torch.bfloat16, torch.float32]


def tol(dtype):
    return dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(
        rtol=2e-5, atol=2e-5)


def test_native_library_loaded():
    from production_stack_amd.ops import native

    assert native.load() is not None


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed_scale(dtype):
    g = torch.Generator().manual_seed(0)
    emb = torch.randn(97, 200, generator=g).to(dtype)
    tok = torch.randint(0, 97, (33,), generator=g)
    want = reference.embed_scale(tok, emb, 3.25)
    got = ops.embed_scale(tok.cuda(), emb.cuda(), 3.25)
    assert got.dtype == torch.float32
    torch.testing.assert_close(got.cpu(), want, rtol=0, atol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("ndelta", [0, 1, 2])
def test_add_rms_norm32(dtype, ndelta):
    g = torch.Generator().manual_seed(1)
    T, W = 19, 328
    x = torch.randn(T, W, generator=g) * 3
    w = torch.randn(W, generator=g)
    deltas = [torch.randn(T, W, generator=g).to(dtype)
              for _ in range(ndelta)]
    xr = x.clone()
    want = reference.add_rms_norm32(xr, deltas, w, 1e-5, dtype)
    xg = x.cuda()
    got = ops.add_rms_norm32(xg, [d.cuda() for d in deltas], w.cuda(), 1e-5,
                             dtype)
    torch.testing.assert_close(xg.cpu(), xr, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind,limit", [("silu", 0.0), ("gelu_tanh", 0.0),
                                        ("clamped_swish", 1.25)])
def test_gated_act_strided(dtype, kind, limit):
    g = torch.Generator().manual_seed(2)
    T, F = 11, 300
    proj = (torch.randn(T, 2 * F + 7, generator=g) * 2).to(dtype)
    want = reference.gated_act(proj[:, 3:3 + F], proj[:, 3 + F:3 + 2 * F],
                               kind, limit, dtype)
    pg = proj.cuda()
    buf = torch.zeros(T, F + 5, dtype=dtype, device="cuda")
    ops.gated_act(pg[:, 3:3 + F], pg[:, 3 + F:3 + 2 * F], kind, limit,
                  out=buf[:, 5:])
    torch.testing.assert_close(buf[:, 5:].cpu().float(), want.float(),
                               **tol(dtype))
    assert float(buf[:, :5].abs().sum()) == 0.0


def _paged(T_total, G, D, DV, bs, dtype, gen, n_seqs):
    """Random paged caches with scattered, non-monotonic block tables."""
    per = (T_total + bs - 1) // bs
    nb = per * n_seqs + 3
    perm = torch.randperm(nb, generator=gen)
    tables = perm[: per * n_seqs].view(n_seqs, per).to(torch.int32)
    kc = torch.randn(nb, G, bs, D, generator=gen).to(dtype)
    vc = torch.randn(nb, G, bs, DV, generator=gen).to(dtype)
    return kc, vc, tables


@pytest.mark.parametrize("dtype", DTYPES)
def test_kv_append_distinct_widths(dtype):
    g = torch.Generator().manual_seed(3)
    G, D, DV, bs = 3, 40, 24, 16
    kc, vc, tables = _paged(50, G, D, DV, bs, dtype, g, 1)
    T = 21
    proj = torch.randn(T, G * D + G * DV + 9, generator=g).to(dtype)
    pos = torch.arange(7, 7 + T)
    slots = tables[0].long()[pos // bs] * bs + pos % bs
    kr, vr = kc.clone(), vc.clone()
    reference.kv_append(proj[:, 4:4 + G * D].reshape(T, G, D),
                        proj[:, 4 + G * D:4 + G * D + G * DV].reshape(
                            T, G, DV), kr, vr, slots)
    kg, vg, pg = kc.cuda(), vc.cuda(), proj.cuda()
    ops.kv_append(pg[:, 4:4 + G * D], pg[:, 4 + G * D:4 + G * D + G * DV],
                  kg, vg, slots.cuda())
    assert torch.equal(kg.cpu(), kr) and torch.equal(vg.cpu(), vr)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("variant", [1, 2, 4, 41, 43])
@pytest.mark.parametrize("H,G,D,DV,chunk,window,sink,talk", [
    (4, 2, 40, 40, 24, 0, True, True),
    (6, 3, 40, 24, 40, 0, True, True),
    (3, 1, 32, 64, 0, 0, False, False),
    (4, 4, 16, 16, 0, 20, True, False),
    (8, 2, 64, 32, 37, 0, False, True),
    (32, 8, 128, 128, 64, 0, True, True),
    (16, 4, 72, 96, 0, 50, True, True),
    (5, 5, 24, 24, 30, 0, True, True),
])
def test_talk_attention(dtype, variant, H, G, D, DV, chunk, window, sink,
                        talk):
    g = torch.Generator().manual_seed(4)
    bs, n_seqs, L = 16, 3, 150
    kc, vc, tables = _paged(L, G, D, DV, bs, dtype, g, n_seqs)
    # ragged batch: a long portion, a portion crossing chunk/page edges,
    # single tokens at edges
    token_seq, token_pos = [], []
    for s, (a, b) in enumerate([(0, 70), (90, 131), (149, 150)]):
        token_seq += [s] * (b - a)
        token_pos += list(range(a, b))
    edge = chunk or window or bs
    for p in (edge - 1, edge, edge + 1, 2 * edge - 1, 2 * edge):
        token_seq.append(1)
        token_pos.append(p)
    # single tokens of different sequences side by side (decode rows)
    for s, p in ((0, 69), (2, 149), (1, 130), (2, 0), (0, 0), (1, 1)):
        token_seq.append(s)
        token_pos.append(p)
    T = len(token_seq)
    q = torch.randn(T, H * D + 5, generator=g).to(dtype)
    tk = (torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)) if talk \
        else None
    ts = torch.tensor(token_seq, dtype=torch.int32)
    tp = torch.tensor(token_pos, dtype=torch.int32)
    scale = 1.0 / math.sqrt(D)
    want = reference.talk_attention(
        q[:, :H * D].float().reshape(T, H, D), kc.float(), vc.float(),
        tables, ts, tp, scale, chunk, window, sink, tk)
    got = ops.talk_attention(
        q.cuda()[:, :H * D], kc.cuda(), vc.cuda(), tables.cuda(), ts.cuda(),
        tp.cuda(), scale, H, chunk=chunk, window=window, sink=sink,
        talk=tk.cuda() if tk is not None else None,
        # 41 / 43: the split-key kernel with one / three workgroups a token
        variant=min(variant, 4), splits=variant - 40 if variant > 4 else 0)
    torch.testing.assert_close(got.cpu().float().view(T, H, DV), want,
                               **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D", [(2, 56), (3, 16), (1, 72), (2, 128),
                                 (1, 160)])
def test_delta_rule(dtype, H, D):
    g = torch.Generator().manual_seed(5)
    HD = H * D
    slots = 5
    # segments: fresh long one (tile remainder), continuing ones (slot
    # state kept), a fresh single token in a slot holding stale state
    segs = [(0, 37, 0, 3), (37, 1, 9, 1), (38, 18, 4, 0), (56, 1, 0, 4),
            (57, 2, 100, 2)]
    T = 59
    proj = torch.randn(T, 6 * HD + 3, generator=g).to(dtype)
    views = [proj[:, i * HD:(i + 1) * HD] for i in range(6)]
    w0 = torch.randn(HD, generator=g)
    ab = torch.randn(HD, generator=g)
    nw = torch.randn(HD, generator=g)
    state = torch.randn(slots, H, D, D, generator=g) * 0.3
    rows = torch.tensor(segs, dtype=torch.int32)
    sr = state.clone()
    sh = (T, H, D)
    want = reference.delta_rule(
        *[v.float().reshape(sh) for v in views], w0, ab, nw, sr, rows,
        1e-5, 0.6, torch.float32)
    sg = state.cuda()
    pg = proj.cuda()
    gviews = [pg[:, i * HD:(i + 1) * HD] for i in range(6)]
    got = ops.delta_rule(*gviews, w0.cuda(), ab.cuda(), nw.cuda(), sg,
                         rows.cuda(), H, 1e-5, 0.6)
    t = tol(dtype)
    torch.testing.assert_close(got.cpu().float().view(sh), want, **t)
    torch.testing.assert_close(sg.cpu(), sr, rtol=1e-4, atol=1e-4)
