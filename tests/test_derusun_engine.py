"""Derusun through the engine: checkpoint folder -> registry -> runner ->
scheduler / block manager / state slots, against the float64 oracle in
tests/oracle_derusun.py. Every test builds its own small configuration and
random weights. CPU runs the reference ops; gpu-marked variants run the HIP
kernels."""

import json
import os

import pytest
import torch

import oracle_derusun as O
from derusun_util import (TOL, cdelta, close, dense, lattn, make_cfg,
                          make_engine, make_weights, rel_err,
                          save_checkpoint, wattn)
from production_stack_amd.engine.models import registry
from production_stack_amd.engine.sampling import SamplingParams

pytestmark = pytest.mark.filterwarnings("ignore::UserWarning")

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DTYPES = ["float32", "bfloat16"]

# head counts, group sizes and widths differ by layer; key width != value
# width; a recurrent layer with and one without feed-forward; windows of 20
# and 33 positions keeping 3 and 1 first keys; three value-mixing layers of
# which the first sits behind a non-mixing one; pages of 16
STACK = [
    (cdelta(4, 2, 16, 24, 3), None),
    (wattn(6, 2, 16, 24, 20, 3, 0.3, 8.0, False), dense(72, 1.5)),
    (wattn(4, 2, 8, 24, 33, 1, 0.4, 5.0, True), None),
    (lattn(3, 16, 8, 12, 24, 0.2, 10000.0), dense(40, 0.8)),
    (cdelta(2, 2, 24, 8, 4), dense(56, 2.5)),
    (wattn(2, 2, 24, 24, 20, 0, 0.25, 0.0, True), dense(48, 1.0)),
    (wattn(4, 2, 16, 24, 0, 0, 0.3, 6.0, True), None),
]
VOCAB = 97


@pytest.fixture(scope="module")
def ckpt(tmp_path_factory):
    cfg = make_cfg(STACK, width=64, vocab=VOCAB, groups=2)
    W = make_weights(cfg, seed=5)
    path = save_checkpoint(tmp_path_factory.mktemp("dr") / "m", cfg, W)
    return path, cfg, W


def tokens(n, seed, vocab=VOCAB):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def replay(eng, rid, toks, sizes):
    """Feed toks in portions of the given sizes (None = the rest); returns
    logits at every position."""
    out, at = [], 0
    for s in sizes:
        s = len(toks) - at if s is None else min(s, len(toks) - at)
        if s <= 0:
            continue
        last = at + s == len(toks)
        out.append(eng.replay_step(
            [(rid, toks[at:at + s], list(range(s)))],
            end=[rid] if last else []))
        at += s
    assert at == len(toks)
    return torch.cat(out)


# ---------------------------------------------------------------------------
def test_registry_reads_checkpoint_folder(ckpt):
    path, cfg, W = ckpt
    mc = registry.config_from_dir(path)
    assert mc.family == "derusun" and mc.vocab_size == VOCAB
    assert mc.hidden_size == 64 and len(mc.layer_specs) == len(STACK)
    assert mc.norm_groups == 2 and mc.has_recurrent_state
    s0, s1, s2, s3 = mc.layer_specs[:4]
    m0 = s0.mixer
    assert (m0.kind, m0.heads, m0.kv_heads, m0.dim, m0.vdim, m0.conv) == (
        "channel_delta", 4, 2, 16, 24, 3)
    assert (m0.decay_rank, m0.gate_rank) == (6, 5)   # tensor shapes
    assert s0.mlp is None and s0.token_shift and s0.depth_average
    m1 = s1.mixer
    assert (m1.window, m1.keep_first, m1.softcap, m1.v_mix) == (
        20, 3, 8.0, False)
    assert m1.learned_sink and m1.qk_norm and m1.bias and not m1.rope
    assert (s1.mlp.act, s1.mlp.limit) == ("clamped_swish", 1.5)
    assert s2.mixer.v_mix and s2.mixer.keep_first == 1
    m3 = s3.mixer
    assert (m3.kind, m3.kv_rank, m3.rot_dim, m3.rot_dims, m3.rot_base) == (
        "latent_attention", 24, 8, 8, 10000.0)
    last = mc.layer_specs[-1].mixer
    assert last.window == 0 and last.keep_first == 0      # no mask entry
    assert "derusun" in registry.FP32_FAMILIES


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_whole_prompt_and_every_layer(ckpt, device, dtype):
    path, cfg, W = ckpt
    toks = tokens(70, 1)
    layers = []
    want = O.forward(cfg, W, toks, layers)
    eng = make_engine(path, dtype, device)
    seen = {}
    eng.runner.model.residual_hook = lambda i, x: seen.__setitem__(
        i, x.detach().clone())
    got = replay(eng, "a", toks, [None])
    assert close(got, want, dtype)
    assert sorted(seen) == list(range(len(STACK)))
    for i in range(len(STACK)):
        assert seen[i].dtype == torch.float32     # fp32 residual streams
        assert close(seen[i], layers[i], dtype), i


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_first_tokens_and_single_token_prompt(ckpt, device, dtype):
    path, cfg, W = ckpt
    eng = make_engine(path, dtype, device)
    for n in (1, 2, 3, 5):
        toks = tokens(n, 10 + n)
        want = O.forward(cfg, W, toks)
        assert close(replay(eng, f"p{n}", toks, [None]), want, dtype)
        assert close(replay(eng, f"q{n}", toks, [1] * n), want, dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [
    [1] * 90, [2] * 45, [3, 2, 17, 2, 31, 2, None], [19, 1, 1, 1, None],
    [20, 20, 13, None], [33, 1, 33, None], [16, 16, 16, 16, 16, None]])
def test_portions_match_whole_prompt(ckpt, device, dtype, sizes):
    """Prefill against token-by-token decoding, and portions of several
    sizes down to two tokens, cut inside pages and windows and exactly on
    their edges (windows of 20 and 33 positions, pages of 16, convolutions
    of 3 and 4 taps reaching back over a cut)."""
    path, cfg, W = ckpt
    toks = tokens(90, 2)
    want = O.forward(cfg, W, toks)
    eng = make_engine(path, dtype, device)
    assert close(replay(eng, "a", toks, sizes), want, dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_past_many_windows(ckpt, device):
    path, cfg, W = ckpt
    toks = tokens(260, 3)
    want = O.forward(cfg, W, toks)
    eng = make_engine(path, "float32", device)
    got = replay(eng, "a", toks, [37] + [1] * 223)
    assert rel_err(got, want) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_mixed_batches_reuse_pages_and_slots(ckpt, device, dtype):
    """Up to three live requests of unequal length per step, portions
    beside single tokens; the pool (3 slots, 12 pages) is smaller than the
    sum of all requests, so pages and slots (recurrent state, convolution
    tail, shift row) pass from finished requests to new ones. Every request
    must equal itself alone."""
    path, cfg, W = ckpt
    lens = {"a": 61, "b": 5, "c": 40, "d": 1, "e": 47, "f": 22}
    toks = {k: tokens(n, 30 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: O.forward(cfg, W, v) for k, v in toks.items()}
    eng = make_engine(path, dtype, device, blocks=12, max_seqs=3)
    plan = [
        [("a", 17), ("b", 2), ("c", 3)],
        [("a", 1), ("b", 3), ("c", 16)],          # b ends
        [("a", 2), ("d", 1), ("c", 1)],           # d: one-token request
        [("c", 20), ("e", 31)],                   # a sits out; c ends
        [("a", 41), ("e", 1), ("f", 2)],          # a ends
        [("e", 15), ("f", 20)],                   # both end
    ]
    at = {k: 0 for k in toks}
    got = {k: [] for k in toks}
    for step in plan:
        entries, end = [], []
        for rid, n in step:
            lo = at[rid]
            entries.append((rid, toks[rid][lo:lo + n], list(range(n))))
            at[rid] += n
            if at[rid] == lens[rid]:
                end.append(rid)
        out = eng.replay_step(entries, end=end)
        r0 = 0
        for rid, n in step:
            got[rid].append(out[r0:r0 + n])
            r0 += n
    assert at == lens
    bm = eng.block_manager
    assert bm.num_free == 12 and len(bm.free_slots) == 3   # all given back
    for k in toks:
        assert close(torch.cat(got[k]), want[k], dtype), k


def oracle_greedy(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(O.forward(cfg, W, toks)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("budget,blocks", [(1 << 20, 64), (7, 64), (24, 9)])
def test_greedy_generation_through_the_scheduler(ckpt, device, budget,
                                                 blocks):
    """LLMEngine.generate: the scheduler's own chunking (token budgets of
    7 and 24 cut the prompts into portions), continuous batching of three
    unequal requests, and with 9 pages preemption with recomputation, must
    all give the oracle's greedy continuation."""
    path, cfg, W = ckpt
    prompts = [tokens(45, 50), tokens(3, 51), tokens(28, 52)]
    n_new = 10
    want = [oracle_greedy(cfg, W, p, n_new) for p in prompts]
    eng = make_engine(path, "float32", device, blocks=blocks, max_seqs=3,
                      budget=budget)
    out = eng.generate(prompts, SamplingParams(
        max_tokens=n_new, temperature=0.0, ignore_eos=True))
    for i in range(3):
        assert out[f"offline-{i}"] == want[i], i
    assert eng.block_manager.num_free == blocks
    assert len(eng.block_manager.free_slots) == 3


OTHER_STACKS = [
    # attention first and last; one group of every kind (kv_heads 1); one
    # norm group; rotary on half of the rotated part; a convolution of two
    # taps and one of a single tap; a window of one position; no value
    # mixing anywhere; width no multiple of 64
    ([(wattn(3, 1, 24, 8, 1, 0, 0.2, 0.0, False), dense(40, 3.0)),
      (cdelta(3, 1, 8, 8, 2), dense(24, 0.5)),
      (lattn(5, 8, 12, 20, 16, 0.3, 500.0, 6), None),
      (cdelta(1, 1, 40, 16, 1), None),
      (wattn(8, 4, 8, 16, 64, 70, 0.35, 3.0, False), dense(32, 1.2))],
     72, 53, 1, 3e-4, (3, 2)),
    # head widths that are no multiple of 8, five query heads on one kv
    # head, seven taps, three norm groups, exactly one value-mixing layer,
    # a large rotary base, kept keys beyond the window size
    ([(cdelta(2, 1, 20, 12, 7), dense(36, 2.0)),
      (wattn(5, 1, 20, 12, 7, 9, 0.22, 4.0, True), None),
      (lattn(2, 12, 4, 20, 12, 0.25, 1e6), dense(28, 1.0)),
      (wattn(7, 7, 12, 20, 50, 2, 0.3, 0.0, False), dense(28, 0.7))],
     60, 71, 3, 1e-6, (4, 7)),
    # one layer only; a single head everywhere
    ([(cdelta(1, 1, 16, 16, 4), None)], 24, 19, 4, 1e-5, (2, 2)),
    ([(wattn(1, 1, 16, 16, 5, 1, 0.25, 2.0, True), None)], 16, 23, 1,
     1e-5, (2, 2)),
    ([(lattn(1, 8, 8, 8, 8, 0.3, 100.0), dense(16, 1.0))], 16, 23, 2,
     1e-5, (2, 2)),
]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", range(len(OTHER_STACKS)))
def test_other_orders_and_sizes(tmp_path, device, dtype, which):
    stack, width, vocab, groups, eps, ranks = OTHER_STACKS[which]
    cfg = make_cfg(stack, width=width, vocab=vocab, eps=eps, groups=groups)
    W = make_weights(cfg, seed=40 + which, ranks=ranks)
    path = save_checkpoint(tmp_path / f"o{which}", cfg, W)
    toks = tokens(80, 70 + which, vocab=vocab)
    want = O.forward(cfg, W, toks)
    eng = make_engine(path, dtype, device)
    assert close(replay(eng, "a", toks, [None]), want, dtype)
    assert close(replay(eng, "b", toks, [6, 1, 2, 30, 1, 1, None]), want,
                 dtype)
    # two requests side by side, cut differently
    half = replay_two(eng, toks, [9, 40, None], [33, 2, None])
    assert close(half[0], want, dtype) and close(half[1], want, dtype)


def replay_two(eng, toks, sizes_a, sizes_b):
    """The same tokens as two requests in shared steps with different
    cuts; returns both requests' logits at every position."""
    def cuts(sizes):
        out, at = [], 0
        for s in sizes:
            s = len(toks) - at if s is None else min(s, len(toks) - at)
            if s > 0:
                out.append((at, at + s))
                at += s
        return out
    ca, cb = cuts(sizes_a), cuts(sizes_b)
    got = {"x": [], "y": []}
    for step in range(max(len(ca), len(cb))):
        entries, end = [], []
        for rid, cc in (("x", ca), ("y", cb)):
            if step < len(cc):
                a, b = cc[step]
                entries.append((rid, toks[a:b], list(range(b - a))))
                if b == len(toks):
                    end.append(rid)
        out = eng.replay_step(entries, end=end)
        r0 = 0
        for rid, t, _ in entries:
            got[rid].append(out[r0:r0 + len(t)])
            r0 += len(t)
    return torch.cat(got["x"]), torch.cat(got["y"])


def test_value_mixing_reads_the_first_mixing_layer(tmp_path):
    """Guards the oracle and the engine together: changing the FIRST
    value-mixing layer's value projection must move the logits even when
    that layer's own output projection is zero, because later mixing layers
    blend its values in; the first layer's own blend weight must not
    matter."""
    stack = [(wattn(2, 1, 8, 8, 12, 1, 0.3, 0.0, True), None),
             (wattn(2, 1, 8, 8, 12, 1, 0.3, 0.0, True), None)]
    cfg = make_cfg(stack, width=32, vocab=31, groups=1)
    W = make_weights(cfg, seed=3)
    W["l0.mix.o"] = torch.zeros_like(W["l0.mix.o"])
    toks = tokens(30, 5, 31)
    base = O.forward(cfg, W, toks)
    W2 = dict(W)
    W2["l0.mix.vmix"] = torch.tensor(0.9).to(torch.bfloat16)
    assert rel_err(O.forward(cfg, W2, toks), base) == 0.0
    W3 = dict(W)
    W3["l0.mix.v"] = (W["l0.mix.v"].float() * 1.5).to(torch.bfloat16)
    assert rel_err(O.forward(cfg, W3, toks), base) > 1e-3
    for k, w in enumerate((W, W3)):
        path = save_checkpoint(tmp_path / f"v{k}", cfg, w)
        eng = make_engine(path, "float32", "cpu")
        got = replay(eng, "a", toks, [7, 1, None])
        assert rel_err(got, O.forward(cfg, w, toks)) < 2e-4


def test_named_config_generates_deterministically():
    from production_stack_amd.engine.config import (CacheConfig,
                                                    EngineConfig,
                                                    SchedulerConfig)
    from production_stack_amd.engine.engine import LLMEngine

    def run(budget):
        eng = LLMEngine(EngineConfig(
            model="tiny-derusun", dtype="float32", max_model_len=256,
            cache=CacheConfig(num_gpu_blocks=32),
            scheduler=SchedulerConfig(max_num_seqs=3,
                                      max_num_batched_tokens=budget)),
            device="cpu")
        return eng.generate(
            [tokens(50, 1, 384), tokens(9, 2, 384)],
            SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True))

    a, b = run(256), run(11)
    assert a == b and all(len(v) == 6 for v in a.values())


def test_trace_run_command(ckpt, tmp_path):
    """bin/trace_run end to end: JSON lines in, 'done' lines and logit
    files out, pool sized by --max-tokens, requests ended and replaced."""
    import subprocess
    import sys

    import numpy as np

    path, cfg, W = ckpt
    root = os.path.join(os.path.dirname(__file__), "..")
    ta, tb, tc = tokens(40, 80), tokens(7, 81), tokens(21, 82)
    steps = [
        {"step": 0, "entries": [
            {"id": "a", "tokens": ta[:33], "want": [0, 32]},
            {"id": "b", "tokens": tb, "want": [6]}], "end": ["b"]},
        {"step": 1, "entries": [
            {"id": "a", "tokens": ta[33:34], "want": []}], "end": []},
        {"step": 2, "entries": [
            {"id": "c", "tokens": tc, "want": [20]},
            {"id": "a", "tokens": ta[34:], "want": [5]}],
         "end": ["a", "c"]},
    ]
    out = tmp_path / "out"
    r = subprocess.run(
        [sys.executable, os.path.join(root, "bin", "trace_run"), "--model",
         path, "--dtype", "float32", "--out", str(out), "--max-tokens", "128",
         "--max-seqs", "2", "--device", "cpu"],
        input="\n".join(json.dumps(s) for s in steps) + "\n",
        capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    done = [ln for ln in r.stdout.splitlines() if ln.startswith("done ")]
    assert done == ["done 0", "done 1", "done 2"]
    assert not (out / "1.f32").exists()
    wa, wb, wc = (O.forward(cfg, W, t) for t in (ta, tb, tc))
    g0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4")
                          .reshape(3, -1).copy())
    g2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4")
                          .reshape(2, -1).copy())
    assert rel_err(g0, torch.stack([wa[0], wa[32], wb[6]])) < 2e-4
    assert rel_err(g2, torch.stack([wc[20], wa[39]])) < 2e-4


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_decode_graph_replays_match_eager(ckpt, dtype):
    """Single-token steps replay a captured hipGraph (padded to a batch
    bucket, padding rows parked on the spare state slot). Three requests of
    unequal length join and leave, so bucket sizes, padding rows and slots
    change between replays; eager prompt portions run in between. Every
    step's logits must match the eager engine's."""
    from production_stack_amd.engine.config import (CacheConfig,
                                                    EngineConfig,
                                                    SchedulerConfig)
    from production_stack_amd.engine.engine import LLMEngine

    path, cfg, W = ckpt

    def make(eager):
        return LLMEngine(EngineConfig(
            model=path, dtype=dtype, max_model_len=256, enforce_eager=eager,
            cache=CacheConfig(num_gpu_blocks=48, block_size=16,
                              enable_prefix_caching=False),
            scheduler=SchedulerConfig(max_num_seqs=4,
                                      max_num_batched_tokens=64)),
            device="cuda")

    graph, eager = make(False), make(True)
    assert graph.runner.graphs is not None and eager.runner.graphs is None
    prompts = [tokens(37, 90), tokens(5, 91), tokens(70, 92)]
    lens = [9, 14, 6]
    outs = []
    for eng in (graph, eager):
        got = {}
        seen = []
        orig = eng.runner.sample

        def spy(logits, seqs, _orig=orig, _seen=seen):
            _seen.append(logits.detach().float().cpu().clone())
            return _orig(logits, seqs)

        eng.runner.sample = spy
        for i, (p, n) in enumerate(zip(prompts, lens)):
            eng.add_request(f"r{i}", p, SamplingParams(
                max_tokens=n, temperature=0.0, ignore_eos=True))
        while eng.has_unfinished():
            for o in eng.step():
                got.setdefault(o.request_id, []).extend(o.new_token_ids)
        outs.append((got, seen))
    (g_tok, g_log), (e_tok, e_log) = outs
    assert len(g_log) == len(e_log) and len(g_log) >= max(lens)
    if dtype == "float32":
        assert g_tok == e_tok
    for a, b in zip(g_log, e_log):
        assert a.shape == b.shape
        if dtype == "float32":
            assert rel_err(a, b) < 2e-4
    want = [oracle_greedy(cfg, W, p, n) for p, n in zip(prompts, lens)]
    if dtype == "float32":
        assert [g_tok[f"r{i}"] for i in range(3)] == want
