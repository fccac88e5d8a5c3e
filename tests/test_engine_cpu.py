"""CPU end-to-end tests of the engine (tiny model, torch-reference ops)."""

import torch

from production_stack_amd.engine.config import (
    CacheConfig,
    EngineConfig,
    SchedulerConfig,
)
from production_stack_amd.engine.engine import LLMEngine
from production_stack_amd.engine.sampling import SamplingParams


def make_engine(**kw):
    cfg = EngineConfig(
        model="tiny-llama",
        max_model_len=kw.pop("max_model_len", 256),
        cache=CacheConfig(
            num_gpu_blocks=kw.pop("num_gpu_blocks", 128), block_size=16
        ),
        scheduler=SchedulerConfig(
            max_num_seqs=kw.pop("max_num_seqs", 8),
            max_num_batched_tokens=kw.pop("max_num_batched_tokens", 128),
        ),
        **kw,
    )
    return LLMEngine(cfg, device="cpu")


def test_greedy_deterministic():
    eng = make_engine()
    p = SamplingParams(max_tokens=8, temperature=0.0, ignore_eos=True)
    o1 = eng.generate([[5, 6, 7, 8, 9]], p)["offline-0"]
    o2 = eng.generate([[5, 6, 7, 8, 9]], p)["offline-0"]
    assert o1 == o2
    assert len(o1) == 8


def test_chunked_prefill_matches_single_shot():
    """Chunked prefill must produce identical greedy outputs."""
    prompt = list(range(10, 90))  # 80 tokens
    p = SamplingParams(max_tokens=5, temperature=0.0, ignore_eos=True)
    big = make_engine(max_num_batched_tokens=256)
    out_big = big.generate([prompt], p)["offline-0"]
    small = make_engine(max_num_batched_tokens=16)  # forces 5 chunks
    out_small = small.generate([prompt], p)["offline-0"]
    assert out_big == out_small


def test_prefix_cache_consistency():
    """A cached-prefix run must produce the same tokens as a cold run."""
    prompt = list(range(10, 60))  # 50 tokens: 3 full blocks cacheable
    p = SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True)
    eng = make_engine()
    cold = eng.generate([prompt], p)["offline-0"]
    assert eng.block_manager.prefix_hits == 0
    warm = eng.generate([prompt], p)["offline-0"]
    assert eng.block_manager.prefix_hits >= 3
    assert cold == warm


def test_batched_matches_sequential():
    prompts = [list(range(10, 30)), list(range(200, 240)), [7, 8, 9]]
    p = SamplingParams(max_tokens=4, temperature=0.0, ignore_eos=True)
    eng = make_engine(enforce_eager=True)
    batched = eng.generate(prompts, p)
    for i, prompt in enumerate(prompts):
        eng2 = make_engine(enforce_eager=True)
        solo = eng2.generate([prompt], p)["offline-0"]
        assert batched[f"offline-{i}"] == solo, f"prompt {i} diverged"


def test_streaming_outputs_and_ttft():
    eng = make_engine()
    eng.add_request(
        "r1", list(range(40)), SamplingParams(max_tokens=4, ignore_eos=True,
                                              temperature=0.0)
    )
    seen = []
    first = None
    while eng.has_unfinished():
        for out in eng.step():
            if out.first_token:
                first = out
            seen.extend(out.new_token_ids)
    assert len(seen) == 4
    assert first is not None and first.num_prompt_tokens == 40


def test_stop_token():
    eng = make_engine()
    p = SamplingParams(max_tokens=64, temperature=0.0)
    out = eng.generate([[3, 4, 5]], p)["offline-0"]
    # find what the 2nd token would be, then use it as a stop token
    eng2 = make_engine()
    p2 = SamplingParams(max_tokens=64, temperature=0.0,
                        stop_token_ids=[out[1]] if len(out) > 1 else [out[0]])
    out2 = eng2.generate([[3, 4, 5]], p2)["offline-0"]
    assert len(out2) <= len(out)


def test_sampling_with_temperature_runs():
    eng = make_engine()
    p = SamplingParams(max_tokens=6, temperature=0.8, top_p=0.9, top_k=50,
                       ignore_eos=True)
    out = eng.generate([[1, 2, 3, 4]], p)["offline-0"]
    assert len(out) == 6
    assert all(0 <= t < eng.model_cfg.vocab_size for t in out)


def test_metrics_surface():
    eng = make_engine()
    m = eng.engine_metrics()
    for key in (
        "num_requests_running",
        "num_requests_waiting",
        "gpu_cache_usage_perc",
        "gpu_prefix_cache_hits_total",
        "gpu_prefix_cache_queries_total",
    ):
        assert key in m


def test_concurrent_add_abort_step_thread_safety():
    """Engine lock: concurrent add/abort from another thread while the step
    loop runs must not corrupt block accounting."""
    import threading

    eng = make_engine(max_num_seqs=8, max_num_batched_tokens=256)
    stop = threading.Event()
    errors = []

    def chaos():
        i = 0
        try:
            while not stop.is_set() and i < 200:
                rid = f"c{i}"
                with eng.lock:
                    eng.add_request(
                        rid, list(range(10, 42)),
                        SamplingParams(max_tokens=6, temperature=0.0,
                                       ignore_eos=True),
                    )
                if i % 3 == 0:
                    with eng.lock:
                        eng.abort_request(rid)
                i += 1
        except Exception as e:  # pragma: no cover
            errors.append(e)

    t = threading.Thread(target=chaos)
    t.start()
    import time as _t

    deadline = _t.time() + 3
    while _t.time() < deadline:
        eng.step()
    stop.set()
    t.join()
    assert not errors
    # drain (bounded chaos: <=200 requests x ~8 steps each)
    for _ in range(3000):
        if not eng.has_unfinished():
            break
        eng.step()
    assert not eng.has_unfinished()
    bm = eng.block_manager
    assert bm.num_free == bm.num_blocks


def test_mistral_sliding_window_family():
    """tiny-mistral (window=48): generates; beyond the window the output
    must differ from an identical-weight full-attention model, while a
    short prompt (inside the window) matches it exactly."""
    from production_stack_amd.engine.config import ARCHITECTURES
    import dataclasses

    def mk(model, window):
        cfg = EngineConfig(
            model=model,
            max_model_len=256,
            seed=3,
            cache=CacheConfig(num_gpu_blocks=128, block_size=16),
            scheduler=SchedulerConfig(max_num_seqs=4,
                                      max_num_batched_tokens=256),
        )
        eng = LLMEngine(cfg, device="cpu")
        return eng

    p = SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True)
    swa = mk("tiny-mistral", 48)
    # tiny-mistral and tiny-llama share shapes; copy weights for a
    # full-attention control
    full = mk("tiny-llama", None)
    full.runner.model.load_state_dict(swa.runner.model.state_dict())

    short = list(range(10, 40))  # 30 tokens < window
    assert swa.generate([short], p)["offline-0"] == \
        full.generate([short], p)["offline-0"]

    long = list(range(5, 105))  # 100 tokens > window 48
    out_swa = swa.generate([long], p)["offline-0"]
    out_full = full.generate([long], p)["offline-0"]
    assert len(out_swa) == 6
    assert out_swa != out_full, "window must change long-context attention"


def test_qwen2_bias_and_tied_embeddings():
    """tiny-qwen2: qkv biases load/save through the HF format and change
    the output; lm_head is the embedding matrix (tied)."""
    import torch as _t

    from production_stack_amd.engine.weights import (
        load_safetensors,
        save_hf_safetensors,
    )

    cfg = EngineConfig(
        model="tiny-qwen2",
        max_model_len=256,
        seed=11,
        cache=CacheConfig(num_gpu_blocks=64, block_size=16),
        scheduler=SchedulerConfig(max_num_seqs=4,
                                  max_num_batched_tokens=256),
    )
    eng = LLMEngine(cfg, device="cpu")
    m = eng.runner.model
    assert m.lm_head is m.embed, "tie_word_embeddings must share storage"
    assert m.layers[0].qkv_bias is not None

    p = SamplingParams(max_tokens=5, temperature=0.0, ignore_eos=True)
    out1 = eng.generate([[4, 5, 6, 7]], p)["offline-0"]

    import tempfile

    with tempfile.TemporaryDirectory() as d:
        save_hf_safetensors(m, d)
        eng2 = LLMEngine(cfg, device="cpu")
        load_safetensors(eng2.runner.model, d)
        out2 = eng2.generate([[4, 5, 6, 7]], p)["offline-0"]
    assert out1 == out2, "bias round-trip through HF format"

    # zeroing the bias changes generation (bias actually applies)
    with _t.no_grad():
        for layer in m.layers:
            layer.qkv_bias.zero_()
    out3 = eng.generate([[4, 5, 6, 7]], p)["offline-0"]
    assert len(out3) == 5


def test_sampling_penalties_and_logit_bias():
    """presence/frequency/repetition penalties reduce repeats; logit_bias
    forces a token; min_tokens suppresses EOS."""
    eng = make_engine()
    base = SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True)
    out_base = eng.generate([[3, 4, 5]], base)["offline-0"]

    # logit_bias strong enough to force one specific token every step
    forced = 7
    p_bias = SamplingParams(max_tokens=4, temperature=0.0, ignore_eos=True,
                            logit_bias={forced: 1000.0})
    out_bias = make_engine().generate([[3, 4, 5]], p_bias)["offline-0"]
    assert out_bias == [forced] * 4

    # heavy frequency penalty must not emit the same token 3x in a row
    p_pen = SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True,
                           frequency_penalty=2.0, presence_penalty=2.0,
                           repetition_penalty=1.5)
    out_pen = make_engine().generate([[3, 4, 5]], p_pen)["offline-0"]
    assert len(out_pen) == 10
    assert out_pen != out_base or len(set(out_base)) == len(out_base)

    # min_tokens: generation may not stop at EOS before the floor
    eos = eng.model_cfg.eos_token_id
    p_min = SamplingParams(max_tokens=8, temperature=0.0, min_tokens=8,
                           logit_bias={eos: 1000.0})  # EOS otherwise wins
    out_min = make_engine().generate([[3, 4, 5]], p_min)["offline-0"]
    assert len(out_min) == 8
    assert all(t != eos for t in out_min[:-1])


def test_speculative_ngram_matches_plain_greedy():
    """n-gram speculative decoding must be a pure latency optimization:
    greedy outputs identical to the plain engine, with drafts actually
    proposed and accepted on self-repeating context."""
    def mk(spec):
        cfg = EngineConfig(
            model="tiny-llama",
            max_model_len=512,
            seed=5,
            cache=CacheConfig(num_gpu_blocks=128, block_size=16),
            scheduler=SchedulerConfig(
                max_num_seqs=4, max_num_batched_tokens=256,
                num_speculative_tokens=4 if spec else 0,
            ),
        )
        return LLMEngine(cfg, device="cpu")

    p = SamplingParams(max_tokens=24, temperature=0.0, ignore_eos=True)
    # strongly periodic prompt: the model's continuation repeats too, so
    # prompt-lookup drafts hit
    prompt = [7, 8, 9, 10] * 8
    plain = mk(False)
    want = plain.generate([prompt], p)["offline-0"]
    spec = mk(True)
    spec.runner.model.load_state_dict(plain.runner.model.state_dict())
    got = spec.generate([prompt], p)["offline-0"]
    assert got == want, f"spec {got} != plain {want}"
    assert spec.runner.spec_proposed > 0
    # on periodic context at least SOME drafts must be accepted
    assert spec.runner.spec_accepted > 0

    # random prompt: still identical (drafts may all be rejected)
    prompt2 = list(range(60, 120))
    plain2 = mk(False)
    want2 = plain2.generate([prompt2], p)["offline-0"]
    spec2 = mk(True)
    spec2.runner.model.load_state_dict(plain2.runner.model.state_dict())
    got2 = spec2.generate([prompt2], p)["offline-0"]
    assert got2 == want2


def test_speculative_respects_stops_and_length():
    cfg = EngineConfig(
        model="tiny-llama",
        max_model_len=512,
        seed=5,
        cache=CacheConfig(num_gpu_blocks=128, block_size=16),
        scheduler=SchedulerConfig(
            max_num_seqs=4, max_num_batched_tokens=256,
            num_speculative_tokens=4,
        ),
    )
    eng = LLMEngine(cfg, device="cpu")
    p = SamplingParams(max_tokens=7, temperature=0.0, ignore_eos=True)
    out = eng.generate([[1, 2, 3] * 6], p)["offline-0"]
    assert len(out) == 7  # acceptance bursts must not overshoot max_tokens


def test_async_scheduling_matches_sync_exactly():
    """One-step-lagged sampling must be invisible: identical greedy
    outputs (including EOS/stop behaviour) vs the synchronous engine."""
    def mk(async_on):
        cfg = EngineConfig(
            model="tiny-llama",
            max_model_len=256,
            seed=5,
            async_scheduling=async_on,
            cache=CacheConfig(num_gpu_blocks=128, block_size=16),
            scheduler=SchedulerConfig(max_num_seqs=8,
                                      max_num_batched_tokens=128),
        )
        return LLMEngine(cfg, device="cpu")

    prompts = [list(range(10, 60)), list(range(200, 230)), [7, 8, 9]]
    for params in (
        SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True),
        SamplingParams(max_tokens=40, temperature=0.0),  # EOS may fire
    ):
        sync = mk(False)
        want = sync.generate(prompts, params)
        a = mk(True)
        a.runner.model.load_state_dict(sync.runner.model.state_dict())
        got = a.generate(prompts, params)
        assert got == want, f"{got} != {want}"


def test_async_scheduling_nongreedy_fallback():
    """Non-greedy requests silently take the synchronous path."""
    cfg = EngineConfig(
        model="tiny-llama",
        max_model_len=256,
        seed=5,
        async_scheduling=True,
        cache=CacheConfig(num_gpu_blocks=128, block_size=16),
        scheduler=SchedulerConfig(max_num_seqs=8,
                                  max_num_batched_tokens=128),
    )
    eng = LLMEngine(cfg, device="cpu")
    p = SamplingParams(max_tokens=6, temperature=0.8, top_p=0.9,
                       ignore_eos=True)
    out = eng.generate([[1, 2, 3, 4]], p)["offline-0"]
    assert len(out) == 6
    bm = eng.block_manager
    assert bm.num_free == bm.num_blocks


def test_async_scheduling_preemption_consistency():
    """Tight KV cache forces preemption while a step is in flight; async
    must still match sync exactly."""
    def mk(async_on):
        cfg = EngineConfig(
            model="tiny-llama",
            max_model_len=256,
            seed=9,
            async_scheduling=async_on,
            cache=CacheConfig(num_gpu_blocks=24, block_size=16,
                              enable_prefix_caching=False),
            scheduler=SchedulerConfig(max_num_seqs=4,
                                      max_num_batched_tokens=64),
        )
        return LLMEngine(cfg, device="cpu")

    prompts = [list(range(5, 85)), list(range(100, 170)),
               list(range(300, 350))]
    p = SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True)
    sync = mk(False)
    want = sync.generate(prompts, p)
    a = mk(True)
    a.runner.model.load_state_dict(sync.runner.model.state_dict())
    got = a.generate(prompts, p)
    assert got == want, f"{got} != {want}"
    bm = a.block_manager
    assert bm.num_free == bm.num_blocks


def test_async_scheduling_abort_and_chaos():
    """Aborting requests while a step is in flight must not corrupt
    accounting; bounded add/abort chaos drains clean."""
    import threading
    import time as _t

    cfg = EngineConfig(
        model="tiny-llama",
        max_model_len=256,
        seed=3,
        async_scheduling=True,
        cache=CacheConfig(num_gpu_blocks=128, block_size=16),
        scheduler=SchedulerConfig(max_num_seqs=8,
                                  max_num_batched_tokens=256),
    )
    eng = LLMEngine(cfg, device="cpu")
    p = SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True)
    # abort while pending
    eng.add_request("a1", list(range(30)), p)
    eng.step()  # launches, pending in flight
    eng.abort_request("a1")
    for _ in range(5):
        eng.step()
    assert not eng.has_unfinished()

    errors = []

    def chaos():
        try:
            for i in range(100):
                rid = f"c{i}"
                with eng.lock:
                    eng.add_request(rid, list(range(10, 42)), p)
                if i % 3 == 0:
                    with eng.lock:
                        eng.abort_request(rid)
        except Exception as e:  # pragma: no cover
            errors.append(e)

    t = threading.Thread(target=chaos)
    t.start()
    deadline = _t.time() + 3
    while _t.time() < deadline:
        eng.step()
    t.join()
    assert not errors
    for _ in range(2000):
        if not eng.has_unfinished():
            break
        eng.step()
    assert not eng.has_unfinished()
    bm = eng.block_manager
    assert bm.num_free == bm.num_blocks


def test_fp8_weight_quantization_cpu():
    """--quantization fp8: engine runs with fp8 weights (dequant matmul
    reference on CPU); early greedy tokens agree with bf16."""
    def mk(q):
        cfg = EngineConfig(
            model="tiny-llama",
            max_model_len=256,
            seed=5,
            quantization=q,
            cache=CacheConfig(num_gpu_blocks=128, block_size=16),
            scheduler=SchedulerConfig(max_num_seqs=8,
                                      max_num_batched_tokens=128),
        )
        return LLMEngine(cfg, device="cpu")

    p = SamplingParams(max_tokens=8, temperature=0.0, ignore_eos=True)
    want = mk(None).generate([[5, 6, 7, 8, 9]], p)["offline-0"]
    got = mk("fp8").generate([[5, 6, 7, 8, 9]], p)["offline-0"]
    assert len(got) == 8
    agree = sum(a == b for a, b in zip(want[:4], got[:4]))
    assert agree >= 2, (want, got)


def test_llama31_rope_scaling():
    """Llama-3.1 frequency remap: high-frequency dims untouched,
    low-frequency wavelengths divided by the scale factor."""
    import torch

    from production_stack_amd.engine.models.llama import build_cos_sin_cache

    N = 65536
    base = build_cos_sin_cache(128, N, 500000.0)
    scaled = build_cos_sin_cache(128, N, 500000.0, (8.0, 1.0, 4.0, 8192))
    diff = (base - scaled).abs().view(N, 2, 64).amax(dim=(0, 1))
    assert diff[:4].max() < 1e-5, f"high-freq dims changed: {diff[:4]}"
    assert diff[-4:].min() > 0.1, f"low-freq dims unscaled: {diff[-4:]}"

    # engine-level: llama-3.1 config constructs and generates
    from production_stack_amd.engine.config import ARCHITECTURES
    assert ARCHITECTURES["llama-3.1-8b"].rope_scaling is not None


def test_incremental_detokenization_bpe():
    """streamed text_delta must equal the suffix diff of
    the full decode — single-token BPE decode loses word-boundary markers
    and a forced per-token space corrupts streams. Train a tiny byte-level
    BPE in-process (no network) and check the accumulated stream_decode
    output equals decode(all ids) exactly."""
    import tempfile

    from tokenizers import Tokenizer, models, pre_tokenizers, decoders, trainers

    from production_stack_amd.engine.tokenizer import HFTokenizer

    tk = Tokenizer(models.BPE(unk_token=None))
    tk.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False)
    tk.decoder = decoders.ByteLevel()
    corpus = [
        "the quick brown fox jumps over the lazy dog",
        "hello world, streaming detokenization must round-trip",
        "naïve café déjà vu — unicode splits across byte tokens",
    ] * 50
    tk.train_from_iterator(
        corpus, trainers.BpeTrainer(vocab_size=400, min_frequency=1,
                                    initial_alphabet=pre_tokenizers.ByteLevel.alphabet())
    )
    with tempfile.NamedTemporaryFile(suffix=".json", delete=False) as f:
        tk.save(f.name)
        hf = HFTokenizer(f.name)

    for text in [
        "the quick brown fox jumps over the lazy dog",
        "hello world, streaming must round-trip",
        "naïve café déjà vu — unicode",
    ]:
        ids = hf.encode(text)
        full = hf.decode(ids)
        state: dict = {}
        acc = ""
        for i in range(1, len(ids) + 1):
            acc += hf.stream_decode(ids[:i], state)
        assert acc == full, (acc, full)
        # per-token single decode would differ (word boundaries lost) —
        # the accumulated stream matches the batch decode instead.


def test_per_request_seed_determinism():
    """SamplingParams.seed gives per-request reproducible
    sampling — two requests with the same seed produce identical tokens
    even when batched alongside unseeded traffic."""
    def engine():
        cfg = EngineConfig(
            model="tiny-llama", max_model_len=256, seed=7,
            cache=CacheConfig(block_size=16, num_gpu_blocks=128),
            scheduler=SchedulerConfig(max_num_seqs=8,
                                      max_num_batched_tokens=128),
        )
        return LLMEngine(cfg, device="cpu")

    prompt = [5, 6, 7, 8, 9, 10]
    p_seeded = SamplingParams(max_tokens=12, temperature=1.0, seed=99,
                              ignore_eos=True)
    p_noise = SamplingParams(max_tokens=12, temperature=1.0,
                             ignore_eos=True)

    e1 = engine()
    out1 = e1.generate([prompt, list(range(20, 30))],
                       [p_seeded, p_noise])["offline-0"]
    # different engine, different unseeded companions, same seed -> same ids
    e2 = engine()
    out2 = e2.generate(
        [list(range(40, 52)), prompt],
        [SamplingParams(max_tokens=12, temperature=1.0, ignore_eos=True),
         SamplingParams(max_tokens=12, temperature=1.0, seed=99,
                        ignore_eos=True)],
    )["offline-1"]
    assert out1 == out2, (out1, out2)

    # and a different seed diverges (overwhelmingly likely over 12 draws)
    e3 = engine()
    out3 = e3.generate([prompt], [SamplingParams(
        max_tokens=12, temperature=1.0, seed=100, ignore_eos=True)])[
        "offline-0"]
    assert out3 != out1


def test_speculative_stochastic_rejection_preserves_distribution():
    """Rejection-sampling acceptance (point-mass draft): the emitted
    token at a draft position must stay marginally distributed exactly
    as the target distribution p — accept draft d w.p. p(d), else a
    residual resample from p with d removed."""
    import numpy as np

    from production_stack_amd.engine.sampling import SamplingParams
    from production_stack_amd.engine.scheduler import (
        ScheduledSeq,
        SchedulerOutput,
    )
    from production_stack_amd.engine.sequence import Sequence

    cfg = EngineConfig(
        model="tiny-llama",
        max_model_len=128,
        seed=11,
        cache=CacheConfig(num_gpu_blocks=32, block_size=16),
        scheduler=SchedulerConfig(max_num_seqs=2,
                                  max_num_batched_tokens=64),
    )
    eng = LLMEngine(cfg, device="cpu")
    runner = eng.runner
    V = 8
    logits_row = torch.tensor(
        [2.0, 1.0, 0.5, 0.0, -1.0, -2.0, -3.0, -4.0])
    p_target = torch.softmax(logits_row, dim=-1)
    draft = 1  # p(draft) ~ 0.23: both branches exercised often

    params = SamplingParams(max_tokens=4, temperature=1.0)
    counts = np.zeros(V)
    trials = 4000
    for _ in range(trials):
        seq = Sequence("r0", [1, 2, 3], params)
        out = SchedulerOutput(scheduled=[
            ScheduledSeq(seq, 2, draft_tokens=[draft])])
        logits = torch.stack([logits_row, logits_row])
        # bonus row's own sample (never read for position 0)
        toks = torch.tensor([0, 0], dtype=torch.long)
        fixed = runner._spec_stochastic_fix(out, [seq, seq], logits, toks)
        counts[int(fixed[0])] += 1
    freq = counts / trials
    assert abs(freq[draft] - float(p_target[draft])) < 0.03
    for t in range(V):
        assert abs(freq[t] - float(p_target[t])) < 0.03, (t, freq[t])


def test_speculative_stochastic_end_to_end():
    """Spec decoding with temperature > 0: runs, proposes and accepts
    drafts on periodic context, respects max_tokens, and per-request
    seeding keeps the run deterministic."""
    def mk():
        cfg = EngineConfig(
            model="tiny-llama",
            max_model_len=512,
            seed=5,
            cache=CacheConfig(num_gpu_blocks=128, block_size=16),
            scheduler=SchedulerConfig(
                max_num_seqs=4, max_num_batched_tokens=256,
                num_speculative_tokens=4,
            ),
        )
        return LLMEngine(cfg, device="cpu")

    def fresh_params():
        # a fresh object per run: the per-request seeded generator is
        # cached on the params instance (one request = one instance in
        # the server), so sharing one across engines would carry state
        # near-greedy temperature: the continuation stays periodic so
        # prompt-lookup drafts actually fire, while still exercising the
        # stochastic (rejection-sampling) acceptance path
        return SamplingParams(max_tokens=20, temperature=0.05,
                              seed=7, ignore_eos=True)

    prompt = [7, 8, 9, 10] * 8
    a = mk()
    got = a.generate([prompt], fresh_params())["offline-0"]
    assert len(got) == 20
    assert a.runner.spec_proposed > 0
    b = mk()
    b.runner.model.load_state_dict(a.runner.model.state_dict())
    assert b.generate([prompt], fresh_params())["offline-0"] == got


def test_prompt_logprobs_chunking_invariant():
    """params.prompt_logprobs: [None, lp...] over the prompt, identical
    whether the prefill ran as one chunk or many."""
    def run(batched):
        cfg = EngineConfig(
            model="tiny-llama",
            max_model_len=256,
            seed=4,
            cache=CacheConfig(num_gpu_blocks=64, block_size=16),
            scheduler=SchedulerConfig(
                max_num_seqs=2, max_num_batched_tokens=batched),
        )
        eng = LLMEngine(cfg, device="cpu")
        p = SamplingParams(max_tokens=2, temperature=0.0,
                           ignore_eos=True, prompt_logprobs=1)
        eng.add_request("plp", list(range(30, 70)), p)
        got = None
        while eng.has_unfinished():
            for out in eng.step():
                if out.prompt_logprobs is not None:
                    got = out.prompt_logprobs
        return eng, got

    ref_eng, one = run(256)   # whole prompt in one chunk
    assert one is not None and one[0] is None
    assert len(one) == 40     # one entry per prompt position
    assert all(v <= 0 for v in one[1:])
    eng2, many = run(16)      # forced chunked prefill
    eng2.runner.model.load_state_dict(ref_eng.runner.model.state_dict())
    # rerun chunked with identical weights for the comparison
    p = SamplingParams(max_tokens=2, temperature=0.0,
                       ignore_eos=True, prompt_logprobs=1)
    eng2.add_request("plp2", list(range(30, 70)), p)
    got2 = None
    while eng2.has_unfinished():
        for out in eng2.step():
            if out.prompt_logprobs is not None:
                got2 = out.prompt_logprobs
    assert got2 is not None
    for a, b in zip(one[1:], got2[1:]):
        assert abs(a - b) < 1e-3, (a, b)


def test_one_token_prompt_chunk_samples_nothing():
    """A token budget that leaves ONE token for a prompt in the middle of
    its prefill must not be taken for a decode step: nothing is sampled
    until the prompt's last token has run."""
    prompts = [list(range(10, 55)), [7, 8, 9], list(range(100, 128))]
    p = SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True)
    big = make_engine(max_num_batched_tokens=256).generate(prompts, p)
    small = make_engine(max_num_batched_tokens=7).generate(prompts, p)
    assert big == small
