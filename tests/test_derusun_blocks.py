"""Each Derusun mechanism alone: the engine's ops and mixer modules (with a
paged cache / state-slot harness) against the float64 oracle in
tests/oracle_derusun.py. CPU runs the reference ops, the gpu-marked
variants run the HIP kernels."""

import math

import pytest
import torch

import oracle_derusun as O
from derusun_util import (TOL, cdelta, lattn, make_cfg, make_weights,
                          rel_err, wattn)
from production_stack_amd import ops
from production_stack_amd.engine.models.ffn import GatedMLP
from production_stack_amd.engine.models.llama import BatchMeta

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DTYPES = ["float32", "bfloat16"]
TD = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F64 = torch.float64

pytestmark = pytest.mark.filterwarnings("ignore::UserWarning")


def rnd(shape, seed, scale=1.0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def seq_rows(parts, device):
    """parts: [(rows, first position, slot)] -> (seq_rows, token_seq)."""
    rows, tseq, r0 = [], [], 0
    for i, (n, p0, slot) in enumerate(parts):
        rows.append([r0, n, p0, slot])
        tseq += [i] * n
        r0 += n
    return (torch.tensor(rows, dtype=torch.int32, device=device),
            torch.tensor(tseq, dtype=torch.int32, device=device))


def cuts(total, sizes):
    out, at = [], 0
    for s in sizes:
        s = total - at if s is None else min(s, total - at)
        if s > 0:
            out.append((at, at + s))
            at += s
    assert at == total
    return out


PORTIONS = [[None], [1] * 12 + [None], [2, 3, 2, 17, 5, None],
            [16, 16, 1, 1, None], [31, 2, None]]


# ---------------------------------------------------------------------------
# stream ops
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("groups", [1, 3, 4])
@pytest.mark.parametrize("sizes", PORTIONS)
def test_group_norm_and_token_shift(device, groups, sizes):
    """Two sequences side by side in differently cut portions; slot 1 holds
    another sequence's stale row first."""
    W, T = 48, 40
    x = [rnd((T, W), 1 + s, 2.0, torch.float32) for s in range(2)]
    w = 1.0 + 0.2 * rnd((W,), 3, 1.0, torch.float32)
    mu = torch.rand(W, generator=torch.Generator().manual_seed(4))
    want = [O.token_shift(O.group_rms_norm(xx, w, 1e-5, groups), mu)
            for xx in x]
    state = rnd((3, W), 5, 3.0, torch.float32).to(device)    # garbage
    got = [[], []]
    ca, cb = cuts(T, sizes), cuts(T, [7, None])
    for step in range(max(len(ca), len(cb))):
        parts, rows = [], []
        for s, cc in ((0, ca), (1, cb)):
            if step < len(cc):
                a, b = cc[step]
                parts.append((b - a, a, 2 - s))
                rows.append((s, x[s][a:b]))
        sr, ts = seq_rows(parts, device)
        h = ops.group_norm_shift(
            torch.cat([r for _, r in rows]).to(device), w.to(device), 1e-5,
            groups, torch.float32, mu.to(device), state, ts, sr)
        r0 = 0
        for s, r in rows:
            got[s].append(h[r0:r0 + len(r)])
            r0 += len(r)
    for s in range(2):
        assert rel_err(torch.cat(got[s]), want[s]) < 1e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("groups", [1, 2, 5])
@pytest.mark.parametrize("dtype", DTYPES)
def test_add_and_group_norm(device, groups, dtype):
    T, W = 9, 40
    x = rnd((T, W), 1, 2.0, torch.float32)
    d = rnd((T, W), 2, 1.0)
    w = 1.0 + 0.2 * rnd((W,), 3, 1.0, torch.float32)
    out32 = torch.full((T, W), 7.0).to(device)
    h = ops.add_rms_norm32(x.to(device), [d.to(TD[dtype]).to(device)],
                           w.to(device), 1e-5, TD[dtype], groups, out32)
    want = x.double() + d.double()
    assert rel_err(out32, want) < 1e-6
    assert rel_err(h, O.group_rms_norm(want, w, 1e-5, groups)) < TOL[dtype]


@pytest.mark.parametrize("device", DEVICES)
def test_depth_weighted_sum(device):
    n, T, W = 5, 7, 24
    hist = rnd((n, T, W), 1, 1.0, torch.float32).to(device)
    wts = rnd((n,), 2, 1.0, torch.float32)
    base = rnd((T, W), 3, 1.0, torch.float32)
    delta = rnd((T, W), 4, 1.0)
    for k in (1, 3, 5):
        hh = hist.clone()
        out = ops.depth_mix(hh, k, wts.to(device), base.to(device),
                            delta.float().to(device))
        streams = [hist[j].cpu() for j in range(k - 1)] + [
            base.double() + delta.double()]
        assert rel_err(out, O.depth_average(streams, wts)) < 1e-5
        assert rel_err(hh[k - 1], streams[-1]) < 1e-6
        assert torch.equal(hh[k:], hist[k:])          # later rows untouched


# ---------------------------------------------------------------------------
# short convolution
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
@pytest.mark.parametrize("sizes", PORTIONS + [[70, 1, 65, None]])
def test_short_convolution(device, dtype, taps, sizes):
    """Portions shorter than the taps reach back over several earlier
    portions; the second sequence runs beside it in a slot that held a
    third one's tail."""
    C, T = 37, 150
    x = [rnd((T, C), 1 + s, 1.0) for s in range(2)]
    w = rnd((C, taps), 3, 0.6).float()
    want = [O.causal_conv_silu(xx, w) for xx in x]
    state = rnd((3, taps - 1, C), 5, 3.0).to(TD[dtype]).to(device)
    got = [[], []]
    ca, cb = cuts(T, sizes), cuts(T, [5, 1, None])
    for step in range(max(len(ca), len(cb))):
        parts, rows = [], []
        for s, cc in ((0, ca), (1, cb)):
            if step < len(cc):
                a, b = cc[step]
                parts.append((b - a, a, 2 - s))
                rows.append((s, x[s][a:b]))
        sr, _ = seq_rows(parts, device)
        y = ops.short_conv_silu(
            torch.cat([r for _, r in rows]).to(TD[dtype]).to(device),
            w.to(device), state, sr)
        r0 = 0
        for s, r in rows:
            got[s].append(y[r0:r0 + len(r)])
            r0 += len(r)
    for s in range(2):
        assert rel_err(torch.cat(got[s]), want[s]) < TOL[dtype]


# ---------------------------------------------------------------------------
# feed-forward
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_clamped_feed_forward(device, dtype):
    width, ff, limit = 40, 72, 0.9
    W = {"gate": rnd((ff, width), 1, 0.4), "up": rnd((ff, width), 2, 0.4),
         "down": rnd((width, ff), 3, 0.2)}
    h = rnd((13, width), 4, 1.5)
    want = O.clamped_ff(h, W["gate"], W["up"], W["down"], limit)
    # both clamps must bite for the test to mean anything
    assert float(O.lin(W["gate"], h).max()) > limit
    assert float(O.lin(W["up"], h).min()) < -limit
    m = GatedMLP(width, ff, "clamped_swish", limit, TD[dtype])
    with torch.no_grad():
        m.gate_up.copy_(torch.cat([W["gate"], W["up"]]))
        m.down.copy_(W["down"])
    m = m.to(device)
    assert rel_err(m(h.to(TD[dtype]).to(device)), want) < TOL[dtype]


# ---------------------------------------------------------------------------
# mixers: a tiny paged cache / slot harness
# ---------------------------------------------------------------------------
class Harness:
    """Drives one mixer module over chosen portions of chosen sequences,
    with scattered block tables and state slots, as the runner would. Every
    page and slot starts with garbage: stale keys and states must never be
    read."""

    def __init__(self, mixer, device, dtype, n_seqs=3, max_len=400, bs=16,
                 slots=4):
        self.mixer, self.device, self.bs = mixer, device, bs
        per = (max_len + bs - 1) // bs
        g = torch.Generator().manual_seed(99)
        nb = per * n_seqs + 5
        perm = torch.randperm(nb, generator=g)
        self.tables = perm[:per * n_seqs].view(n_seqs, per).to(torch.int32)

        def alloc(d):
            if d[0] == "kv":
                return (torch.randn(nb, d[1], bs, d[2], generator=g)
                        .to(dtype).to(device),
                        torch.randn(nb, d[1], bs, d[3], generator=g)
                        .to(dtype).to(device))
            if d[0] == "paged":
                return torch.randn(nb, d[1], bs, d[2], generator=g).to(
                    dtype).to(device)
            if d[0] == "state":
                return torch.randn(slots, d[1], d[2], d[3],
                                   generator=g).to(device)
            if d[0] == "slots":
                return torch.randn(slots, *d[1], generator=g).to(
                    d[2] or dtype).to(device)
            return tuple(alloc(c) for c in d[1])

        self.cache = alloc(mixer.cache_shape())

    def run(self, parts, slot_of=None, shared=None):
        """parts: [(seq index, first position, inputs [n, width])]; returns
        the mixer's outputs (before W_o), one tensor per part."""
        bs, dev = self.bs, self.device
        order = sorted(range(len(parts)),
                       key=lambda i: parts[i][2].shape[0] == 1)
        if order != list(range(len(parts))):
            res = self.run([parts[i] for i in order], slot_of, shared)
            back = [None] * len(parts)
            for k, i in enumerate(order):
                back[i] = res[k]
            return back
        n_multi = sum(p.shape[0] for _, _, p in parts if p.shape[0] > 1)
        h = torch.cat([p for _, _, p in parts]).to(dev)
        pos, tseq, slots, rows = [], [], [], []
        r0 = 0
        for i, (s, p0, p) in enumerate(parts):
            n = p.shape[0]
            for t in range(n):
                pp = p0 + t
                pos.append(pp)
                tseq.append(i)
                slots.append(int(self.tables[s][pp // bs]) * bs + pp % bs)
            rows.append([r0, n, p0, (slot_of or {}).get(s, s)])
            r0 += n
        meta = BatchMeta(
            positions=torch.tensor(pos, dtype=torch.int32, device=dev),
            slot_mapping=torch.tensor(slots, dtype=torch.long, device=dev),
            num_prefill_tokens=n_multi, prefill_token_seq=None,
            prefill_token_pos=None, prefill_block_tables=None,
            num_decode_seqs=0, decode_seq_lens=None,
            decode_block_tables=None,
            block_tables=torch.stack(
                [self.tables[s] for s, _, _ in parts]).to(dev),
            token_seq=torch.tensor(tseq, dtype=torch.int32, device=dev),
            seq_rows=torch.tensor(rows, dtype=torch.int32, device=dev))
        out = self.mixer(h, meta, self.cache,
                         shared if shared is not None else {})
        res, r0 = [], 0
        for _, _, p in parts:
            res.append(out[r0:r0 + p.shape[0]])
            r0 += p.shape[0]
        return res


def build(layer, width, W, dtype, device):
    """The layer's mixer, loaded as the engine loads it: a one-layer
    checkpoint folder read through the registry."""
    import tempfile

    from derusun_util import save_checkpoint
    from production_stack_amd.engine.models import registry

    cfg = make_cfg([(layer, None)], width=width)
    with tempfile.TemporaryDirectory() as d:
        save_checkpoint(d, cfg, W)
        mcfg = registry.config_from_dir(d)
        model = registry.build_model(mcfg, dtype)
        registry.load_weights(model, d)
    return model.layers[0].mixer.to(device)


def finish(mixer, outs):
    return torch.nn.functional.linear(torch.cat(outs), mixer.out_weight)


def run_portions(hs, h, sizes, dtype, s=0, slot_of=None, shared_of=None):
    outs = []
    for a, b in cuts(h.shape[0], sizes):
        sh = shared_of(a, b) if shared_of else None
        outs += hs.run([(s, a, h[a:b].to(TD[dtype]))], slot_of, sh)
    return outs


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", PORTIONS)
@pytest.mark.parametrize("shape", [(4, 2, 16, 24, 3), (3, 3, 40, 8, 4),
                                   (2, 1, 20, 68, 2)])
def test_channel_delta(device, dtype, sizes, shape):
    layer = cdelta(*shape)
    width, T = 48, 50
    W = make_weights(make_cfg([(layer, None)], width=width), seed=11)
    h = rnd((T, width), 12, 1.0)
    want = O.channel_delta(h, W, "l0.mix.", layer["mixer"], 1e-5)
    mixer = build(layer, width, W, dtype, device)
    hs = Harness(mixer, device, TD[dtype])
    got = finish(mixer, run_portions(hs, h, sizes, dtype))
    assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("device", DEVICES)
def test_channel_delta_state_survives_and_slots_are_reused(device):
    """340 tokens decoded one by one after a short portion (what the
    portion wrote still shows dozens of tokens later); then another
    sequence takes the same slot and must start from zero."""
    layer = cdelta(2, 1, 16, 24, 4)
    width = 32
    W = make_weights(make_cfg([(layer, None)], width=width), seed=13)
    # slow decay: what the first tokens wrote must still matter at the end
    W["l0.mix.dt_bias"] = (W["l0.mix.dt_bias"].float() - 6.0).to(
        torch.bfloat16)
    mixer = build(layer, width, W, "float32", device)
    hs = Harness(mixer, device, torch.float32, max_len=352)
    h = rnd((350, width), 14, 1.0)
    want = O.channel_delta(h, W, "l0.mix.", layer["mixer"], 1e-5)
    cut = h.clone()
    cut[:5] = 0
    far = O.channel_delta(cut, W, "l0.mix.", layer["mixer"], 1e-5)
    assert rel_err(far[40:41], want[40:41]) > 1e-3  # the test has teeth
    got = finish(mixer, run_portions(hs, h, [10] + [1] * 340, "float32",
                                     slot_of={0: 3}))
    assert rel_err(got, want) < TOL["float32"]
    h2 = rnd((9, width), 15, 1.0)
    want2 = O.channel_delta(h2, W, "l0.mix.", layer["mixer"], 1e-5)
    got2 = finish(mixer, run_portions(hs, h2, [4, 1, None], "float32", s=1,
                                      slot_of={1: 3}))
    assert rel_err(got2, want2) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_channel_delta_ragged_batch(device):
    layer = cdelta(4, 2, 16, 24, 3)
    width = 48
    W = make_weights(make_cfg([(layer, None)], width=width), seed=16)
    mixer = build(layer, width, W, "float32", device)
    hs = Harness(mixer, device, torch.float32)
    hh = [rnd((n, width), 20 + i, 1.0) for i, n in enumerate((33, 7, 21))]
    want = [O.channel_delta(x, W, "l0.mix.", layer["mixer"], 1e-5)
            for x in hh]
    f32 = [x.float() for x in hh]
    o1 = hs.run([(0, 0, f32[0][:17]), (1, 0, f32[1][:1]),
                 (2, 0, f32[2][:20])])
    o2 = hs.run([(0, 17, f32[0][17:]), (1, 1, f32[1][1:]),
                 (2, 20, f32[2][20:])])
    for i in range(3):
        got = finish(mixer, [o1[i], o2[i]])
        assert rel_err(got, want[i]) < TOL["float32"], i


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", PORTIONS)
@pytest.mark.parametrize("shape", [
    (6, 2, 16, 24, 20, 3, 0.3, 8.0), (3, 3, 40, 8, 33, 0, 0.2, 0.0),
    (5, 1, 12, 20, 7, 9, 0.25, 3.0), (2, 1, 136, 24, 0, 0, 0.1, 5.0)])
def test_window_attention(device, dtype, sizes, shape):
    """Also a head width above 128 (the plain kernel) and no window."""
    layer = wattn(*shape, v_mix=True)
    width, T = 48, 50
    W = make_weights(make_cfg([(layer, None)], width=width), seed=21)
    h = rnd((T, width), 22, 1.0)
    m = layer["mixer"]
    v_first = rnd((T, m["kv_heads"], m["vdim"]), 23, 1.0)
    want, _ = O.attention(h, W, "l0.mix.", m, 1e-5, v_first)
    mixer = build(layer, width, W, dtype, device)
    hs = Harness(mixer, device, TD[dtype])
    flat = v_first.reshape(T, -1).to(TD[dtype]).to(device)
    got = finish(mixer, run_portions(
        hs, h, sizes, dtype,
        shared_of=lambda a, b: {"v_first": flat[a:b]}))
    assert rel_err(got, want) < TOL[dtype]
    # without earlier values the layer publishes its own, unblended
    shared = {}
    want0, v0 = O.attention(h, W, "l0.mix.", m, 1e-5, None)
    got0 = finish(mixer, hs.run([(1, 0, h.to(TD[dtype]))], shared=shared))
    assert rel_err(got0, want0) < TOL[dtype]
    assert rel_err(shared["v_first"].float(), v0.reshape(T, -1)) < TOL[dtype]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", PORTIONS)
@pytest.mark.parametrize("shape", [
    (3, 16, 8, 12, 24, 0.2, 10000.0, None), (5, 8, 12, 20, 16, 0.3, 50.0, 6),
    (2, 24, 16, 8, 120, 0.15, 1e6, None)])
def test_latent_attention(device, dtype, sizes, shape):
    """Also cached rows wider than 128 entries (the plain kernel)."""
    layer = lattn(*shape)
    width, T = 48, 50
    W = make_weights(make_cfg([(layer, None)], width=width), seed=31)
    h = rnd((T, width), 32, 1.0)
    want = O.latent_attention(h, W, "l0.mix.", layer["mixer"], 1e-5)
    mixer = build(layer, width, W, dtype, device)
    hs = Harness(mixer, device, TD[dtype])
    got = finish(mixer, run_portions(hs, h, sizes, dtype))
    assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("device", DEVICES)
def test_latent_attention_far_positions(device):
    """A small rotary base makes every pair turn many times over 300
    positions; decoding one by one must agree with the oracle's angles."""
    layer = lattn(2, 8, 8, 8, 16, 0.3, 20.0)
    width, T = 32, 300
    W = make_weights(make_cfg([(layer, None)], width=width), seed=33)
    h = rnd((T, width), 34, 1.0)
    want = O.latent_attention(h, W, "l0.mix.", layer["mixer"], 1e-5)
    mixer = build(layer, width, W, "float32", device)
    hs = Harness(mixer, device, torch.float32)
    got = finish(mixer, run_portions(hs, h, [250] + [1] * 50, "float32"))
    assert rel_err(got, want) < TOL["float32"]


# ---------------------------------------------------------------------------
# the attention op with keys made to stand out
# ---------------------------------------------------------------------------
def needle_case(T, H, G, D, DV, needle, seed):
    """Random small queries/keys; the key at `needle` points along the last
    query of every head of its group, so where it is visible it takes
    almost all the weight; its value is far from all others."""
    g = torch.Generator().manual_seed(seed)
    q = 0.3 * torch.randn(T, H, D, generator=g)
    k = 0.3 * torch.randn(T, G, D, generator=g)
    v = 0.3 * torch.randn(T, G, DV, generator=g)
    rep = H // G
    for gi in range(G):
        d = torch.randn(D, generator=g)
        d = d / d.norm()
        k[needle, gi] = 60.0 * d
        # every head of the group sees the needle the same way
        q[T - 1, gi * rep:(gi + 1) * rep] = d
    v[needle] = 25.0 * (1.0 - 2.0 * (torch.arange(DV) % 2))
    return q, k, v


def oracle_attend(q, k, v, scale, size, keep, cap, sink):
    T, H, _ = q.shape
    rep = H // k.shape[1]
    s = torch.einsum("ihd,jhd->hij", q.double(),
                     k.double().repeat_interleave(rep, 1)) * scale
    if cap:
        s = cap * torch.tanh(s / cap)
    p = O.sink_softmax(s, O.window_visibility(T, size or T, keep), sink)
    return torch.einsum("hij,jhv->ihv", p,
                        v.double().repeat_interleave(rep, 1)), p


def paged(q, k, v, device, bs=16, sizes=(None,), variant_last=None,
          dtype=torch.float32, **kw):
    """Run ops.talk_attention over a scattered paged cache, in portions;
    the last portion may force a kernel variant."""
    T, H, D = q.shape
    G, DV = k.shape[1], v.shape[2]
    per = (T + bs - 1) // bs
    g = torch.Generator().manual_seed(7)
    table = torch.randperm(per + 3, generator=g)[:per].to(torch.int32)
    kc = torch.randn(per + 3, G, bs, D, generator=g).to(dtype).to(device)
    vc = torch.randn(per + 3, G, bs, DV, generator=g).to(dtype).to(device)
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    outs = []
    cc = cuts(T, sizes)
    for n, (a, b) in enumerate(cc):
        pos = torch.arange(a, b, dtype=torch.int32)
        slots = (table[(pos // bs).long()].long() * bs + pos % bs)
        ops.kv_append(k[a:b].reshape(b - a, -1).to(device),
                      v[a:b].reshape(b - a, -1).to(device), kc, vc,
                      slots.to(device))
        variant = 3 if b - a == 1 else 0
        if n == len(cc) - 1 and variant_last is not None:
            variant = variant_last
        outs.append(ops.talk_attention(
            q[a:b].reshape(b - a, -1).to(device), kc, vc,
            table[None].to(device),
            torch.zeros(b - a, dtype=torch.int32, device=device),
            pos.to(device), heads=H, variant=variant, **kw))
    return torch.cat(outs).view(T, H, DV).float()


NEEDLE_MODES = [((None,), None), ((None,), 1), ((0, 1), None), ((0, 1), 4),
                ((0, 1), 1), ((0, 2), None)]


def _sizes(T, mode):
    """mode (0, n): everything but the last n tokens in one portion, then
    those n in one portion."""
    if mode[0] is None:
        return [None]
    return [T - mode[1], None]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("mode,variant", NEEDLE_MODES)
@pytest.mark.parametrize("T,size,keep,needle,seen", [
    (200, 48, 0, 152, True),      # just inside the window
    (200, 48, 0, 151, False),     # just outside
    (200, 48, 5, 4, True),        # last kept first key
    (200, 48, 5, 5, False),       # first key that is not kept
    (209, 64, 0, 145, True),      # inside, query first on a page, key last
    (209, 64, 0, 144, False),     # on a page's last entry, outside
    (330, 0, 0, 1, True),         # no window: hundreds of keys back
    (193, 32, 40, 39, True),      # more kept keys than the window holds
    (50, 64, 3, 0, True),         # window larger than the sequence
])
def test_needle_at_window_edges(device, mode, variant, T, size, keep, needle,
                                seen):
    """The last query against a key that dominates wherever it is visible:
    in a whole prompt, as the last token decoded alone and in a two-token
    portion, through every kernel variant."""
    H, G, D, DV = 4, 2, 16, 24
    q, k, v = needle_case(T, H, G, D, DV, needle, seed=T + needle)
    sink = torch.tensor([0.5, -1.0, 2.0, 0.0])
    want, p = oracle_attend(q, k, v, 0.25, size, keep, 30.0, sink)
    assert (float(p[:, T - 1, needle].min()) > 0.9) == seen
    assert float(p[:, T - 1, needle].max()) < 1e-9 or seen
    got = paged(q, k, v, device, sizes=_sizes(T, mode), variant_last=variant,
                scale=0.25, window=size, keep_first=keep, softcap=30.0,
                sink=True, sink_vals=sink.to(device))
    assert rel_err(got.reshape(T, -1), want.reshape(T, -1)) < 1e-4
    assert (float(got[T - 1].abs().mean()) > 20.0) == seen


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("mode,variant", NEEDLE_MODES)
def test_sink_takes_the_weight(device, mode, variant):
    """A large learned sink leaves almost nothing for the keys; a very
    negative one changes nothing; the sink is neither scaled nor capped."""
    T, H, G, D, DV = 70, 4, 4, 8, 8
    q, k, v = needle_case(T, H, G, D, DV, 3, seed=5)
    for sv, small in ((torch.tensor([60.0, 60.0, 60.0, 60.0]), True),
                      (torch.tensor([-60.0, 9.0, -60.0, 9.0]), False)):
        want, _ = oracle_attend(q, k, v, 0.5, 0, 0, 7.0, sv)
        got = paged(q, k, v, device, sizes=_sizes(T, mode),
                    variant_last=variant, scale=0.5, softcap=7.0, sink=True,
                    sink_vals=sv.to(device))
        assert rel_err(got.reshape(T, -1), want.reshape(T, -1)) < 1e-4
        assert (float(got.abs().max()) < 1e-6) == small


@pytest.mark.parametrize("device", DEVICES)
def test_values_read_from_key_rows(device):
    """Keys that carry their values: the value is the leading part of the
    key row, one cache for both."""
    T, H, D, DV = 45, 3, 24, 16
    g = torch.Generator().manual_seed(3)
    q = torch.randn(T, H, D, generator=g)
    k = torch.randn(T, 1, D, generator=g)
    sink = torch.tensor([0.0, 1.0, -1.0])
    want, _ = oracle_attend(q, k, k[..., :DV], 0.2, 0, 0, 0.0, sink)
    bs, per = 16, 3
    table = torch.tensor([2, 0, 3], dtype=torch.int32)
    kc = torch.randn(5, 1, bs, D, generator=g)
    pos = torch.arange(T, dtype=torch.int32)
    slots = table[(pos // bs).long()].long() * bs + pos % bs
    kc[(slots // bs), 0, slots % bs] = k[:, 0]
    kc = kc.to(device)
    for variant in (0, 1, 3):
        got = ops.talk_attention(
            q.reshape(T, -1).to(device), kc, kc, table[None].to(device),
            torch.zeros(T, dtype=torch.int32, device=device), pos.to(device),
            0.2, H, sink=True, sink_vals=sink.to(device), vdim=DV,
            variant=variant)
        assert got.shape == (T, H * DV)
        assert rel_err(got, want.reshape(T, -1)) < 1e-4, variant
    assert per * bs >= T and not math.isnan(float(got.sum()))


# ---------------------------------------------------------------------------
# the matrix-core kernel (bfloat16 on the GPU only)
# ---------------------------------------------------------------------------
def bf(x):
    return x.to(torch.bfloat16).float()


MC_SHAPES = [(4, 2, 16, 24), (8, 1, 40, 72), (64, 2, 32, 160)]
MC_MODES = [((None,), 0, 5), ((0, 1), 0, 5), ((0, 1), 3, 5), ((0, 2), 0, 5),
            ((0, 7), 0, 5), ((None,), 0, 6), ((0, 7), 0, 6),
            ((0, 150), 0, 6)]
# the 128-row form (variant 6) holds at most 128 value columns
MC_CASES = [(m, sh) for m in MC_MODES for sh in MC_SHAPES
            if not (m[2] == 6 and sh[3] > 128)]


@pytest.mark.gpu
@pytest.mark.parametrize("T,size,keep,needle,seen", [
    (200, 48, 0, 152, True), (200, 48, 0, 151, False),
    (200, 48, 5, 4, True), (200, 48, 5, 5, False),
    (209, 64, 0, 145, True), (209, 64, 0, 144, False),
    (330, 0, 0, 1, True), (193, 32, 40, 39, True), (50, 64, 3, 0, True)])
@pytest.mark.parametrize("case", MC_CASES)
def test_matrix_core_attention_needles(case, T, size, keep, needle, seen):
    """The same stand-out keys through the matrix-core kernel: 2, 8 and 32
    heads per KV head, key widths that need zero padding, value widths over
    several column blocks, portions of 1, 2 and 7 tokens, split keys; the
    128-row form (variant 6) on whole prompts and portions."""
    (mode, splits, variant), (H, G, D, DV) = case
    q, k, v = needle_case(T, H, G, D, DV, needle, seed=T + needle)
    q, k, v = bf(q), bf(k), bf(v)
    sink = torch.linspace(-1.0, 2.0, H)
    want, p = oracle_attend(q, k, v, 0.25, size, keep, 30.0, sink)
    assert (float(p[:, T - 1, needle].min()) > 0.9) == seen
    got = paged(q, k, v, "cuda", sizes=_sizes(T, mode), variant_last=variant,
                dtype=torch.bfloat16, scale=0.25, window=size,
                keep_first=keep, softcap=30.0, sink=True,
                sink_vals=sink.cuda(), splits=splits)
    # the output is rounded to bfloat16 once
    assert rel_err(got.reshape(T, -1), want.reshape(T, -1)) < 6e-3
    assert (float(got[T - 1].abs().mean()) > 20.0) == seen


@pytest.mark.gpu
@pytest.mark.parametrize("H,D,DV", [(8, 136, 96), (32, 288, 256),
                                    (2, 48, 48), (16, 584, 512)])
@pytest.mark.parametrize("splits", [0, 4])
def test_matrix_core_values_in_key_rows(H, D, DV, splits):
    """Latent-attention shapes: one KV head, rows of up to 584 entries whose
    leading entries are the values; prompt rows and single tokens."""
    T = 75
    g = torch.Generator().manual_seed(H + D)
    q = bf(torch.randn(T, H, D, generator=g))
    k = bf(torch.randn(T, 1, D, generator=g))
    sink = torch.linspace(-1.0, 1.0, H)
    scale = 2.0 / D ** 0.5
    want, _ = oracle_attend(q, k, k[..., :DV], scale, 0, 0, 0.0, sink)
    bs = 16
    table = torch.tensor([4, 0, 3, 1, 5], dtype=torch.int32)
    kc = torch.randn(6, 1, bs, D, generator=g)
    pos = torch.arange(T, dtype=torch.int32)
    slots = table[(pos // bs).long()].long() * bs + pos % bs
    kc[(slots // bs), 0, slots % bs] = k[:, 0]
    kc = kc.to(torch.bfloat16).cuda()
    tq = q.reshape(T, -1).to(torch.bfloat16).cuda()
    zero = torch.zeros(T, dtype=torch.int32, device="cuda")
    got = ops.talk_attention(
        tq, kc, kc, table[None].cuda(), zero, pos.cuda(), scale, H,
        sink=True, sink_vals=sink.cuda(), vdim=DV, variant=5)
    assert rel_err(got.float(), want.reshape(T, -1)) < 6e-3
    # the last rows again, one token per launch row, keys split
    got1 = ops.talk_attention(
        tq[-9:], kc, kc, table[None].cuda(), zero[-9:], pos[-9:].cuda(),
        scale, H, sink=True, sink_vals=sink.cuda(), vdim=DV, variant=5,
        splits=splits)
    assert rel_err(got1.float(), want.reshape(T, -1)[-9:]) < 6e-3
