"""Nanurax through the engine: checkpoint folder -> registry -> runner ->
scheduler / block manager / state slots, against the float64 oracle. Every
test builds its own small configuration and random weights. CPU runs the
reference ops; gpu-marked variants run the HIP kernels."""

import json

import pytest
import torch

import oracle_nanurax as O
from nanurax_util import (TOL, attn, delta, dense, make_cfg, make_engine,
                          make_weights, moe, rel_err, save_checkpoint)
from nanurax_util import close
from production_stack_amd.engine.block_manager import BlockManager
from production_stack_amd.engine.models import registry
from production_stack_amd.engine.sampling import SamplingParams
from production_stack_amd.engine.sequence import Sequence

pytestmark = pytest.mark.filterwarnings("ignore::UserWarning")

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DTYPES = ["float32", "bfloat16"]

# a stack that differs from any single-valued choice: head counts and dims
# vary by layer, group sizes 3 and 1, value width != key width, two and
# three experts per token, a layer without feed-forward, routed layers with
# and without a shared expert, attention first and last
STACK = [
    (attn(6, 2, 16, 24, 20, 0.3), dense(72)),
    (delta(3, 16), moe(24, 1.75, 5, 2, (40, 1.25))),
    (delta(2, 24), None),
    (attn(3, 3, 8, 8, 33, 0.45), moe(16, 0.9, 4, 3, None)),
    (delta(1, 40), dense(56)),
]


@pytest.fixture(scope="module")
def ckpt(tmp_path_factory):
    cfg = make_cfg(STACK, width=64, vocab=97)
    W = make_weights(cfg, seed=5, rank=6)
    path = save_checkpoint(tmp_path_factory.mktemp("nx") / "m", cfg, W)
    return path, cfg, W


def tokens(n, seed, vocab=97):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def replay(eng, rid, toks, sizes, want_all=True):
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
    assert mc.family == "nanurax" and mc.vocab_size == 97
    assert mc.hidden_size == 64 and len(mc.layer_specs) == len(STACK)
    s0, s1, s2, s3 = mc.layer_specs[:4]
    assert (s0.mixer.kind, s0.mixer.heads, s0.mixer.kv_heads,
            s0.mixer.vdim, s0.mixer.chunk) == ("attention", 6, 2, 24, 20)
    assert s0.mixer.sink and s0.mixer.talking_heads and not s0.mixer.rope
    assert s1.mixer.decay_rank == 6          # read off the tensor's shape
    assert (s1.mlp.experts, s1.mlp.top, s1.mlp.shared_ff,
            s1.mlp.shared_limit) == (5, 2, 40, 1.25)
    assert s1.mlp.score == "sigmoid" and not s1.mlp.renormalize
    assert s2.mlp is None and s3.mlp.shared_ff == 0
    assert mc.has_recurrent_state
    with open(path + "/config.json") as f:
        bad = json.load(f)
    bad["architecture"] = "Nope"
    import os
    os.makedirs(path + "_bad", exist_ok=True)
    with open(path + "_bad/config.json", "w") as f:
        json.dump(bad, f)
    with pytest.raises(ValueError):
        registry.config_from_dir(path + "_bad")


def test_state_slot_pool():
    bm = BlockManager(32, 16, enable_prefix_caching=True, num_state_slots=2)
    assert not bm.enable_prefix_caching   # recurrent state: no prefix reuse
    sp = SamplingParams(max_tokens=1)
    a, b, c = (Sequence(n, [1] * 20, sp) for n in "abc")
    bm.allocate_prompt(a)
    bm.allocate_prompt(b)
    assert {a.state_slot, b.state_slot} == {0, 1}
    assert not bm.can_allocate_prompt(c)  # blocks are free, slots are not
    with pytest.raises(RuntimeError):
        bm.allocate_prompt(c)
    assert bm.num_free == 32 - 4          # the failed admission leaked none
    freed = a.state_slot
    bm.free_seq(a)
    assert a.state_slot is None and bm.can_allocate_prompt(c)
    bm.allocate_prompt(c)
    assert c.state_slot == freed


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_whole_prompt_and_every_layer(ckpt, device, dtype):
    path, cfg, W = ckpt
    toks = tokens(70, 1)
    want, layers = O.forward(cfg, W, toks, return_layers=True)
    eng = make_engine(path, dtype, device)
    seen = {}
    eng.runner.model.residual_hook = lambda i, x: seen.__setitem__(
        i, x.detach().clone())
    got = replay(eng, "a", toks, [None])
    assert close(got, want, dtype)
    assert sorted(seen) == list(range(len(STACK)))
    for i in range(len(STACK)):
        assert seen[i].dtype == torch.float32     # fp32 residual stream
        assert close(seen[i], layers[i], dtype), i


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_first_tokens_and_single_token_prompt(ckpt, device, dtype):
    path, cfg, W = ckpt
    eng = make_engine(path, dtype, device)
    for n in (1, 2, 3):
        toks = tokens(n, 10 + n)
        want = O.forward(cfg, W, toks)
        assert close(replay(eng, f"p{n}", toks, [None]), want, dtype)
        assert close(replay(eng, f"q{n}", toks, [1] * n), want, dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [
    [1] * 90, [2] * 45, [3, 2, 17, 2, 31, 2, None], [19, 1, 1, 1, None],
    [20, 20, 13, None], [33, 33, None], [16, 16, 16, 16, 16, None]])
def test_portions_match_whole_prompt(ckpt, device, dtype, sizes):
    """Prefill against token-by-token decoding, and portions of several
    sizes down to two tokens, cut inside pages and chunks and exactly on
    their edges (chunks of 20 and 33 positions, pages of 16)."""
    path, cfg, W = ckpt
    toks = tokens(90, 2)
    want = O.forward(cfg, W, toks)
    eng = make_engine(path, dtype, device)
    assert close(replay(eng, "a", toks, sizes), want, dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_past_many_chunks(ckpt, device):
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
    sum of all requests, so pages and slots pass from finished requests to
    new ones. Every request must equal itself alone."""
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


def test_replay_refuses_a_plan_that_does_not_fit(ckpt):
    path, cfg, W = ckpt
    eng = make_engine(path, "float32", "cpu", blocks=4, max_seqs=2)
    eng.replay_step([("a", tokens(10, 1), []), ("b", tokens(10, 2), [])])
    with pytest.raises(RuntimeError):
        eng.replay_step([("c", tokens(3, 3), [])])       # no slot left
    with pytest.raises(RuntimeError):
        eng.replay_step([("a", tokens(60, 4), [])])      # no pages left


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
    n_new = 12
    want = [oracle_greedy(cfg, W, p, n_new) for p in prompts]
    eng = make_engine(path, "float32", device, blocks=blocks, max_seqs=3,
                      budget=budget)
    out = eng.generate(prompts, SamplingParams(
        max_tokens=n_new, temperature=0.0, ignore_eos=True))
    for i in range(3):
        assert out[f"offline-{i}"] == want[i], i
    assert eng.block_manager.num_free == blocks
    assert len(eng.block_manager.free_slots) == 3


@pytest.mark.parametrize("device", DEVICES)
def test_other_layer_orders_and_sizes(tmp_path, device):
    """A second stack: recurrent layers only at the ends, one expert per
    token beside many, a chunk of one position (a key sees only itself),
    width that is no multiple of 64."""
    stack = [
        (delta(4, 8), moe(8, 2.5, 7, 1, (8, 0.5))),
        (attn(2, 1, 24, 16, 1, 0.2), None),
        (attn(8, 4, 8, 16, 64, 0.35), dense(40)),
        (delta(2, 32), dense(24)),
    ]
    cfg = make_cfg(stack, width=72, vocab=53, eps=3e-4, scale=2.25)
    W = make_weights(cfg, seed=9, rank=3)
    path = save_checkpoint(tmp_path / "m2", cfg, W)
    toks = tokens(80, 60, vocab=53)
    want = O.forward(cfg, W, toks)
    eng = make_engine(path, "float32", device)
    assert rel_err(replay(eng, "a", toks, [None]), want) < 2e-4
    assert rel_err(replay(eng, "b", toks, [5, 2, 60, 1, None]), want) < 2e-4


ODD_STACKS = [
    # head widths that are no multiple of 8 or 16, five query heads on one
    # kv head, a chunk of 7 positions, every expert chosen, delta heads of
    # 20 and 100 channels
    ([(attn(5, 1, 20, 12, 7, 0.22), moe(12, 1.5, 3, 3, (20, 2.0))),
      (delta(2, 20), dense(36)),
      (delta(1, 100), None),
      (attn(7, 7, 12, 20, 50, 0.3), dense(28))], 60, 71),
    # one layer only; a single head everywhere
    ([(delta(1, 16), moe(8, 3.0, 2, 1, None))], 24, 19),
    ([(attn(1, 1, 16, 16, 5, 0.25), None)], 16, 23),
]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("which", range(len(ODD_STACKS)))
def test_odd_shapes(tmp_path, device, which):
    stack, width, vocab = ODD_STACKS[which]
    cfg = make_cfg(stack, width=width, vocab=vocab, eps=1e-6, scale=3.0)
    W = make_weights(cfg, seed=40 + which, rank=5)
    path = save_checkpoint(tmp_path / f"odd{which}", cfg, W)
    toks = tokens(64, 70 + which, vocab=vocab)
    want = O.forward(cfg, W, toks)
    eng = make_engine(path, "float32", device)
    assert rel_err(replay(eng, "a", toks, [None]), want) < 2e-4
    assert rel_err(replay(eng, "b", toks, [6, 1, 2, 30, 1, 1, None]),
                   want) < 2e-4
    # two requests side by side, cut differently
    half = replay_two(eng, toks, [9, 40, None], [33, 2, None])
    assert rel_err(half[0], want) < 2e-4 and rel_err(half[1], want) < 2e-4


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


def test_named_config_generates_deterministically():
    from production_stack_amd.engine.config import (CacheConfig,
                                                    EngineConfig,
                                                    SchedulerConfig)
    from production_stack_amd.engine.engine import LLMEngine

    def run(budget):
        eng = LLMEngine(EngineConfig(
            model="tiny-nanurax", dtype="float32", max_model_len=256,
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
    import os
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
    done = [l for l in r.stdout.splitlines() if l.startswith("done ")]
    assert done == ["done 0", "done 1", "done 2"]
    assert not (out / "1.f32").exists()
    wa, wb, wc = (O.forward(cfg, W, t) for t in (ta, tb, tc))
    g0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4")
                          .reshape(3, -1).copy())
    g2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4")
                          .reshape(2, -1).copy())
    assert rel_err(g0, torch.stack([wa[0], wa[32], wb[6]])) < 2e-4
    assert rel_err(g2, torch.stack([wc[20], wa[39]])) < 2e-4
