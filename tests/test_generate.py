"""Generation through the entry points: greedy and temperature sampling against the plain
implementation, portions and preemption through the scheduler, the sampling options, the
command line."""
import os
import subprocess
import sys

import pytest
import torch

import helpers as H
import plain_llama4 as plain

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, cfg in H.CONFIGS.items():
        d = str(tmp_path_factory.mktemp("gen") / name)
        out[name] = (d, H.make_model(d, cfg, seed=11, dtype="float32"), cfg)
    return out


def engine(d, **kw):
    from spite_amd import Engine
    args = dict(dtype="float32", page_size=16, cache_tokens=1024, max_requests=8, max_batch_tokens=64)
    args.update(kw)
    return Engine(d, **args)


def plain_generate(cfg, weights, prompt, n, temperature=0.0, seed=0, **opts):
    toks, state = list(prompt), seed
    for _ in range(n):
        logits = plain.forward(cfg, weights, toks)[-1]
        t, state = plain.sample(logits, toks, state, temperature, **opts)
        toks.append(t)
    return toks[len(prompt):]


def test_greedy_generation_equals_the_plain_implementation(models):
    # the workload of the first tiny configuration: prompts of 5, 23 and 40 tokens, 16 new tokens each
    d, w, cfg = models["A"]
    prompts = [H.random_tokens(cfg["vocab_size"], n, 40 + n) for n in (5, 23, 40)]
    got = engine(d).generate(prompts, max_tokens=16, temperature=0.0)
    for p, g in zip(prompts, got):
        assert g == plain_generate(cfg, w, p, 16)


def test_temperature_sampling_in_mixed_batches_equals_the_plain_sampler(models):
    # the workload of the second: prompts of 1, 7, 16, 33 and 70 tokens, portions of prompts beside
    # decoded tokens (the budget of 24 tokens a step cuts the prompts), temperature 0.8, fixed seed
    d, w, cfg = models["B"]
    prompts = [H.random_tokens(cfg["vocab_size"], n, 60 + n) for n in (1, 7, 16, 33, 70)]
    stats = {}
    got = engine(d, page_size=8, max_batch_tokens=24).generate(prompts, max_tokens=12, temperature=0.8, seed=1234,
                                                               stats=stats)
    assert stats["steps"] > 12          # the prompts did not fit one step each
    for i, (p, g) in enumerate(zip(prompts, got)):
        assert g == plain_generate(cfg, w, p, 12, temperature=0.8, seed=1234 ^ i)


def test_tokens_do_not_depend_on_the_other_requests(models):
    d, w, cfg = models["B"]
    prompts = [H.random_tokens(cfg["vocab_size"], n, 80 + n) for n in (9, 30, 3)]
    eng = engine(d, page_size=8)
    together = eng.generate(prompts, max_tokens=10, temperature=1.0, seed=5)
    for i, p in enumerate(prompts):
        alone = eng.generate([p], max_tokens=10, temperature=1.0, seed=5 ^ i)
        assert alone[0] == together[i]


def test_preemption_changes_nothing(models):
    d, w, cfg = models["A"]
    prompts = [H.random_tokens(cfg["vocab_size"], n, 90 + n) for n in (20, 28, 12)]
    roomy = engine(d).generate(prompts, max_tokens=24, temperature=0.0)
    stats = {}
    tight = engine(d, page_size=4, num_pages=22, max_batch_tokens=32).generate(prompts, max_tokens=24, temperature=0.0,
                                                                               stats=stats)
    assert stats["preemptions"] >= 1, "the pool was not tight enough to preempt"
    assert tight == roomy


def test_bfloat16_generation_through_mixed_steps_and_preemption(tmp_path):
    """bfloat16 through the scheduler: prompts cut into portions beside decoded tokens, and a pool so
    tight that requests are preempted and computed again.  bfloat16 products pick their kernel from
    the step's rows, so the two runs agree to rounding, not bit for bit: every token that either run
    chose must be the plain implementation's choice at that place (fed the run's own tokens), or
    within rounding of it; and where the plain implementation's choice is clear the runs agree."""
    cfg = H.TINY_C
    d = str(tmp_path / "C16")
    w = H.make_model(d, cfg, seed=11, dtype="bfloat16")
    V = cfg["vocab_size"]
    prompts = [H.random_tokens(V, n, 70 + n) for n in (40, 60, 30, 50)]
    n_new = 40
    roomy = engine(d, dtype="bfloat16", page_size=32, cache_tokens=2048, max_batch_tokens=256)
    assert not roomy.slow_paths                   # sizes that the MFMA kernels take
    runs = {"roomy": roomy.generate(prompts, max_tokens=n_new, temperature=0.0)}
    stats = {}
    tight = engine(d, dtype="bfloat16", page_size=32, num_pages=5, max_batch_tokens=48)
    runs["tight"] = tight.generate(prompts, max_tokens=n_new, temperature=0.0, stats=stats)
    assert stats["preemptions"] >= 1, "the pool was not tight enough to preempt"
    assert stats["steps"] > n_new + 4             # prompts went in portions beside decoded tokens
    worst = 0.0
    clear = {}
    for name, run in runs.items():
        for r, (p, g) in enumerate(zip(prompts, run)):
            assert len(g) == n_new
            logits = plain.forward(cfg, w, p + g)[len(p) - 1:-1]
            scale = float(logits.abs().max())
            for i, t in enumerate(g):
                top = torch.topk(logits[i], 2).values
                worst = max(worst, float(top[0] - logits[i, t]) / scale)
                # a place where the runner-up is far behind, and all tokens before it agree with the other run
                clear[(name, r, i)] = float(top[0] - top[1]) > 0.08 * scale
    print(f"largest distance of a chosen token from the plain implementation's best: {worst:.4f} of the logits' scale")
    assert worst <= 0.04, worst
    for r in range(len(prompts)):
        for i in range(n_new):
            if runs["roomy"][r][:i] != runs["tight"][r][:i]:
                break
            if clear[("roomy", r, i)]:
                assert runs["roomy"][r][i] == runs["tight"][r][i], (r, i)


def test_finish_reasons(models):
    d, w, cfg = models["A"]
    eng = engine(d)
    p = H.random_tokens(cfg["vocab_size"], 12, 7)
    free = eng.generate([p], max_tokens=10, temperature=0.0)[0]
    # greedy decoding of random weights repeats itself: stop at the first appearance of a token
    new = [k for k in range(1, 10) if free[k] not in free[:k]]
    assert len(new) >= 2, free
    k1, k2 = new[-1], new[0]
    res = eng.generate([p], max_tokens=10, temperature=0.0, eos_token_ids=[free[k1]], details=True)[0]
    assert res.tokens == free[:k1] and res.finish_reason == "EosToken"         # the end token is not emitted
    res = eng.generate([p], max_tokens=10, temperature=0.0, stop_token_ids=[free[k2]], details=True)[0]
    assert res.tokens == free[:k2] and res.finish_reason == "StopToken"
    res = eng.generate([p], max_tokens=10, temperature=0.0, max_context=15, details=True)[0]
    assert res.tokens == free[:3] and res.finish_reason == "ContextLimit"      # 12 + 3 positions
    res = eng.generate([p], max_tokens=3, temperature=0.0, details=True)[0]
    assert res.tokens == free[:3] and res.finish_reason == "MaxTokens"
    for g in range(eng.cache.n_groups()):
        assert eng.cache.free_pages(g) == eng.cache.total_pages(g)


def test_sampling_options(models):
    d, w, cfg = models["A"]
    eng = engine(d)
    p = H.random_tokens(cfg["vocab_size"], 10, 3)
    greedy = eng.generate([p], max_tokens=8, temperature=0.0)[0]
    assert eng.generate([p], max_tokens=8, temperature=1.0, top_k=1, seed=9)[0] == greedy
    assert eng.generate([p], max_tokens=8, temperature=1.0, top_p=1e-6, seed=9)[0] == greedy
    assert eng.generate([p], max_tokens=8, temperature=1.0, min_p=0.999, seed=9)[0] == greedy
    hot = eng.generate([p], max_tokens=8, temperature=1.5, seed=9)[0]
    assert hot == eng.generate([p], max_tokens=8, temperature=1.5, seed=9)[0] and hot != greedy
    for opts in (dict(top_k=5), dict(top_p=0.7), dict(min_p=0.05), dict(repetition_penalty=1.3, repeat_last_n=4)):
        got = eng.generate([p], max_tokens=8, temperature=0.9, seed=3, **opts)[0]
        assert got == plain_generate(cfg, w, p, 8, temperature=0.9, seed=3, **opts), opts
    # a penalty reaches greedy decoding too (crates/spite-executor/src/lib.rs:814-828)
    pen = eng.generate([p], max_tokens=8, temperature=0.0, repetition_penalty=1.5, repeat_last_n=0)[0]
    assert pen == plain_generate(cfg, w, p, 8, repetition_penalty=1.5, repeat_last_n=0)


def test_errors_are_raised_before_anything_runs(models):
    from spite_amd import EngineError, StepEntry
    from spite_amd.engine.scheduler import SchedulerError
    d, w, cfg = models["A"]
    eng = engine(d)
    with pytest.raises(SchedulerError, match="empty prompt"):
        eng.generate([[]], max_tokens=2)
    with pytest.raises(SchedulerError, match="context limit"):
        eng.generate([[1] * 20], max_tokens=2, max_context=10)
    s = eng.admit()
    with pytest.raises(EngineError, match="outside the vocabulary"):
        eng.step([StepEntry(s, [3, cfg["vocab_size"]], [1])])
    with pytest.raises(EngineError, match="twice"):
        eng.step([StepEntry(s, [3], [0]), StepEntry(s, [4], [0])])
    with pytest.raises(EngineError, match="wanted place"):
        eng.step([StepEntry(s, [3], [1])])
    assert eng.cache.cached(s) == 0                      # a refused step wrote nothing
    eng.release(s)
    with pytest.raises(EngineError, match="holds no request"):
        eng.step([StepEntry(s, [3], [0])])


def test_command_line(models):
    d, w, cfg = models["A"]
    p = H.random_tokens(cfg["vocab_size"], 9, 21)
    want = engine(d).generate([p], max_tokens=6, temperature=0.0)[0]
    out = subprocess.run([sys.executable, os.path.join(H.ROOT, "bin", "spite"), "run", "-m", d, "--prompt-ids",
                          ",".join(map(str, p)), "--max-tokens", "6", "--temperature", "0", "--dtype", "fp32",
                          "--ctx", "64", "--page-size", "16"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    assert out.stdout.strip().splitlines()[-1].split() == [str(t) for t in want]
    assert "generate     : 9 prompt + 6 new tokens" in out.stderr and "tok/s" in out.stderr
    assert "max tokens   : 6" in out.stdout and "temperature  : 0.0" in out.stdout


@pytest.mark.parametrize("name", ["A", "B"])
def test_random_weights_mode_of_the_engine_holds_the_model_of_the_folder_of_that_seed(name, tmp_path):
    # the engine draws on the GPU; the folder writer draws on the host; the plain implementation
    # reads the tensors back from the engine and must generate the engine's tokens
    from spite_amd import Engine
    from spite_amd.weights.random_init import write_random_model
    cfg = dict(H.CONFIGS[name], torch_dtype="float32")
    eng = Engine(cfg, dtype="float32", random_weights=True, seed=4, init_std=0.08, page_size=16, cache_tokens=256,
                 max_requests=2)
    d = write_random_model(str(tmp_path / "m"), cfg, seed=4, std=0.08)
    stored = H.read_weights(d)
    assert sorted(stored) == sorted(eng.tensor_names())
    for n, t in stored.items():
        assert torch.equal(eng.get_tensor(n).double(), t), n
    prompts = [H.random_tokens(cfg["vocab_size"], n, 2 + n) for n in (12, 31)]
    got = eng.generate(prompts, max_tokens=6)
    for p, g in zip(prompts, got):
        assert g == plain_generate(cfg, stored, p, 6)
    assert Engine(d, dtype="float32", page_size=16, cache_tokens=256, max_requests=2).generate(prompts, max_tokens=6) == got
    # a bfloat16 folder rounds every tensor once; the engine that draws does the same
    cfg16 = dict(cfg, torch_dtype="bfloat16")
    e16 = Engine(cfg16, dtype="bfloat16", random_weights=True, seed=4, page_size=16, cache_tokens=64, max_requests=1)
    d16 = write_random_model(str(tmp_path / "m16"), cfg16, seed=4)
    for n, t in H.read_weights(d16).items():
        assert torch.equal(e16.get_tensor(n).double(), t), n


def test_tensors_and_cache_can_be_looked_at(models):
    from spite_amd import Engine
    from spite_amd.engine.engine import EngineError, StepEntry
    d, w, cfg = models["A"]
    eng = engine(d)
    names = eng.tensor_names()
    assert "lm_head.weight" in names and "model.layers.1.feed_forward.router.weight" in names
    assert torch.equal(eng.get_tensor("model.layers.0.self_attn.q_proj.weight"), w["model.layers.0.self_attn.q_proj.weight"])
    with pytest.raises(KeyError):
        eng.get_tensor("no.such.tensor")
    # pages: 40 positions take three pages of 16 in the full group; the chunked group (chunks of 32) keeps one
    slot = eng.admit()
    free = [eng.cache.free_pages(g) for g in range(eng.cache.n_groups())]
    eng.step([StepEntry(slot, H.random_tokens(cfg["vocab_size"], 40, 1), [39])])
    held = [free[g] - eng.cache.free_pages(g) for g in range(eng.cache.n_groups())]
    assert sorted(held) == [1, 3]
    assert sorted(sum(p >= 0 for p in eng.cache.block_table(slot, g)) for g in range(eng.cache.n_groups())) == [1, 3]
    eng.release(slot)
    assert [eng.cache.free_pages(g) for g in range(eng.cache.n_groups())] == free
