"""Letarax through the package (checkpoint reader, executor, cache and state slots, trace replay, scheduler) against
the plain model in `letarax_oracle`. Every test runs on the torch executor on the CPU; the same tests run on the HIP
executor, in fp32 and in bf16, under the `gpu` marker."""
import numpy as np
import pytest
import torch

import letarax_oracle as O
from letarax_util import SAME, STACKS, TOL, alone, oracle_logits, random_tokens, rel_err, replay, save_model, session

BACKENDS = [pytest.param("torch", "fp32", id="torch"),
            pytest.param("hip", "fp32", id="hip-fp32", marks=pytest.mark.gpu),
            pytest.param("hip", "bf16", id="hip-bf16", marks=pytest.mark.gpu)]


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for i, (name, cfg) in enumerate(STACKS.items()):
        W = O.random_weights(cfg, seed=10 + i)
        out[name] = (cfg, W, save_model(str(tmp_path_factory.mktemp(name)), cfg, W))
    return out


def check(got, ref, dtype, what="", same_as=None):
    e = rel_err(got, ref)
    assert e < TOL[dtype], f"{what}: error {e:.3g} over {TOL[dtype]}"
    if same_as is not None:
        e = rel_err(got, same_as.astype(np.float64))
        assert e < SAME[dtype], f"{what}: differs from the whole prompt run alone by {e:.3g}, over {SAME[dtype]}"


@pytest.mark.parametrize("backend,dtype", BACKENDS)
@pytest.mark.parametrize("stack", list(STACKS))
def test_whole_prompt(models, stack, backend, dtype):
    cfg, W, path = models[stack]
    toks = random_tokens(cfg, 75, 1)
    sess = session(path, backend, dtype)
    got = replay(sess, {"a": toks}, [[("a", len(toks))]])["a"]
    sess.close()
    check(got, oracle_logits(cfg, W, toks), dtype, stack)


@pytest.mark.parametrize("backend,dtype", BACKENDS)
@pytest.mark.parametrize("stack", ["mixed", "delta_first", "odd_sizes", "mfma_heads"])
def test_prefill_then_token_by_token(models, stack, backend, dtype):
    """A prompt, then decoding one token a step past every window of the stack and over several cache blocks."""
    cfg, W, path = models[stack]
    toks = random_tokens(cfg, 110, 2)
    sess = session(path, backend, dtype)
    got = replay(sess, {"a": toks}, [[("a", 30)]] + [[("a", 1)]] * 80)["a"]
    sess.close()
    check(got, oracle_logits(cfg, W, toks), dtype, stack, alone(path, backend, dtype, toks))


@pytest.mark.parametrize("backend,dtype", BACKENDS)
@pytest.mark.parametrize("stack", ["mixed", "delta_first", "odd_sizes", "only_delta"])
def test_first_tokens_alone(models, stack, backend, dtype):
    """A sequence that starts token by token: the convolutions' inputs before the start are zero, windows are not full."""
    cfg, W, path = models[stack]
    toks = random_tokens(cfg, 12, 3)
    sess = session(path, backend, dtype)
    got = replay(sess, {"a": toks}, [[("a", 1)]] * 12)["a"]
    sess.close()
    check(got, oracle_logits(cfg, W, toks), dtype, stack, alone(path, backend, dtype, toks))


@pytest.mark.parametrize("backend,dtype", BACKENDS)
@pytest.mark.parametrize("stack,cuts", [("mixed", [2, 2, 3, 1, 29, 2, 31, 33, 2, 1, 5]), ("delta_first", [31, 2, 2, 36, 1, 3, 2, 34]),
                                        ("odd_sizes", [1, 2, 30, 3, 64, 2, 9]), ("wide_heads", [33, 2, 40, 2, 30]),
                                        ("mfma_heads", [2, 31, 2, 1, 97, 3, 130, 2, 33])])
def test_portions(models, stack, cuts, backend, dtype):
    """Prompts cut into portions of changing size, down to two tokens, across block and window edges."""
    cfg, W, path = models[stack]
    toks = random_tokens(cfg, sum(cuts), 4)
    sess = session(path, backend, dtype)
    got = replay(sess, {"a": toks}, [[("a", c)] for c in cuts])["a"]
    sess.close()
    check(got, oracle_logits(cfg, W, toks), dtype, stack, alone(path, backend, dtype, toks))


@pytest.mark.parametrize("backend,dtype", BACKENDS)
@pytest.mark.parametrize("stack", ["mixed", "delta_first", "odd_sizes", "mfma_heads"])
def test_mixed_batches_and_reuse(models, stack, backend, dtype):
    """Unequal requests share steps (portions beside single tokens), more requests than slots over time, a pool that
    only holds the live ones: slots and blocks change hands. Every request must come out as if it ran alone."""
    cfg, W, path = models[stack]
    reqs = {n: random_tokens(cfg, ln, 20 + i) for i, (n, ln) in enumerate([("a", 70), ("b", 9), ("c", 41), ("d", 100), ("e", 35), ("f", 66), ("g", 3)])}
    sched = [[("a", 33), ("b", 2)], [("a", 1), ("b", 7), ("c", 30)], [("a", 30), ("c", 1), ("d", 64)],
             [("a", 1), ("c", 1), ("d", 1), ("e", 35)],                      # b ended: e takes its slot; e ends at once
             [("a", 5), ("c", 9), ("d", 30), ("f", 2)], [("d", 1), ("f", 62), ("g", 1)], [("d", 2), ("f", 1), ("g", 2)],
             [("d", 2), ("f", 1)]]
    sess = session(path, backend, dtype, max_tokens=352, slots=4)
    got = replay(sess, reqs, sched)
    assert sess.alloc.used == 0 and all(r is None for r in sess.rows)
    sess.close()
    for name, toks in reqs.items():
        check(got[name], oracle_logits(cfg, W, toks), dtype, f"{stack}/{name}", alone(path, backend, dtype, toks))


@pytest.mark.parametrize("backend,dtype", BACKENDS)
def test_slot_taken_over_starts_clean(models, backend, dtype):
    """One slot, one request after another: the second must not see the first one's recurrent state, carried
    convolution inputs or cache rows."""
    cfg, W, path = models["delta_first"]
    a, b = random_tokens(cfg, 50, 31), random_tokens(cfg, 20, 32)
    sess = session(path, backend, dtype, max_tokens=64, slots=1)
    got = replay(sess, {"a": a, "b": b}, [[("a", 50)], [("b", 1)], [("b", 2)], [("b", 17)]])
    sess.close()
    check(got["b"], oracle_logits(cfg, W, b), dtype, "second", alone(path, backend, dtype, b))
    check(got["a"], oracle_logits(cfg, W, a), dtype, "first", alone(path, backend, dtype, a))


@pytest.mark.parametrize("d", [16, 64])
@pytest.mark.parametrize("backend,dtype", BACKENDS)
def test_window_edges_and_far_keys(tmp_path, backend, dtype, d):
    """One attention layer whose keys and queries are shaped so that a single key stands out: the one a query must
    still see at the far edge of its window, or the one it must no longer see, hundreds of tokens back, across block
    edges; in a prompt, in portions and in decoding. A window that is one token off moves the logits by far more than
    the tolerance; so does a sink that is left out, because the far key's weight against the sink decides the output."""
    window = 130
    cfg = O.make_config([O.attention_layer(1, 1, d, d, window=window, scale=1.0, v_mix=False, ff=0)], vocab=40, width=32)
    W = O.random_weights(cfg, seed=5)
    # token 7 is the beacon: its key is large along one direction; token 9 asks along it, every other token looks away
    # (queries and keys come from the biases, so the mixer's input hardly matters)
    for n in ("l0.mix.q", "l0.mix.k"):
        W[n] = torch.zeros_like(W[n])
    W["l0.mix.q.b"] = torch.zeros(d, dtype=torch.bfloat16)
    W["l0.mix.k.b"] = torch.zeros(d, dtype=torch.bfloat16)
    W["l0.mix.q"][0] = (W["embed"][9].float() * 0.5).to(torch.bfloat16)      # q[0] large for token 9 only ...
    W["l0.mix.k"][0] = (W["embed"][7].float() * 0.5).to(torch.bfloat16)      # ... k[0] large for token 7 only
    path = save_model(str(tmp_path / "m"), cfg, W)
    base = [t for t in random_tokens(cfg, 400, 6) if t not in (7, 9)][:300]
    for beacon, ask in [(20, 20 + window - 1), (20, 20 + window), (95, 95 + window - 1), (96, 96 + window), (31, 160), (32, 162)]:
        toks = list(base)
        toks[beacon], toks[ask] = 7, 9
        ref = oracle_logits(cfg, W, toks)
        for sched in ([[("a", 300)]], [[("a", ask - 1)], [("a", 2)], [("a", 300 - ask - 1)]], [[("a", ask)]] + [[("a", 1)]] * 3):
            n = sum(c for step in sched for _, c in step)
            sess = session(path, backend, dtype, max_tokens=352, slots=1)
            got = replay(sess, {"a": toks[:n]}, sched)["a"]
            sess.close()
            check(got, ref[:n], dtype, f"beacon {beacon} asked at {ask}")
    # the asked position's logits do depend on whether the beacon is inside the window
    inside = oracle_logits(cfg, W, [7 if i == 20 else 9 if i == 20 + window - 1 else t for i, t in enumerate(base)])[20 + window - 1]
    outside = oracle_logits(cfg, W, [7 if i == 19 else 9 if i == 20 + window - 1 else t for i, t in enumerate(base)])[20 + window - 1]
    assert rel_err(inside[None], outside[None]) > 0.05


@pytest.mark.parametrize("stack,buckets", [("mixed", []), ("mfma_heads", []), ("mixed", [2])])
@pytest.mark.parametrize("backend,dtype", BACKENDS)
def test_greedy_generation_through_the_scheduler(models, backend, dtype, stack, buckets):
    """Requests of unequal length through the engine's own entry point: scheduler, continuous batching, sampling
    (greedy), on the HIP executor with captured decode steps (also with a second, smaller step size, whose steps are
    captured at bring-up and between which the scheduler would pack rows if their state did not live in their slots).
    The tokens are those of the plain model's argmax."""
    from distributed_llm_inference_amd.config import EngineConfig
    from distributed_llm_inference_amd.parallel.launcher import LocalPipeline
    from distributed_llm_inference_amd.runtime.sampler import SamplingParams
    cfg, W, path = models[stack]
    prompts = [random_tokens(cfg, n, 40 + n) for n in (5, 37, 64, 11, 90, 2)]
    new = 24
    ecfg = EngineConfig(model=path, dtype=dtype, pp_size=1, max_batch=4, num_micro_batches=1, max_seq_len=256, prefill_chunk=48,
                        kv_blocks=24, device="cuda" if backend == "hip" else "cpu", backend=backend, seed=0, decode_buckets=buckets)
    pipe = LocalPipeline(ecfg)
    try:
        reqs = [pipe.engine.submit(p, SamplingParams(temperature=0.0, max_new_tokens=new, stop_on_eos=False)) for p in prompts]
        outs = [r.wait(120).output for r in reqs]
        if backend == "hip":
            assert pipe.executors[0].graph_replays > 0, "decode did not go through the captured steps"
    finally:
        pipe.close()
    for p, out in zip(prompts, outs):
        assert len(out) == new
        # teacher-forced: the plain model, fed the engine's own tokens, must agree with every choice (or hold a near tie)
        lg = oracle_logits(cfg, W, p + out)[len(p) - 1:-1]
        for t, row in zip(out, lg):
            best = float(row.max())
            assert row[t] >= best - (1e-3 if dtype == "fp32" else 0.35) * max(1.0, abs(best)), (t, int(row.argmax()))


@pytest.mark.parametrize("backend,dtype,model", [pytest.param("torch", "fp32", "tiny-letarax-test", id="torch"),
                                                 pytest.param("hip", "bf16", "tiny-letarax-gpu-test", id="hip-bf16", marks=pytest.mark.gpu)])
def test_builtin_stack_samples_reproducibly(backend, dtype, model):
    """A built-in Letarax stack (random weights, no checkpoint) through the engine with temperature / top-k / top-p
    sampling: the same seeds give the same tokens on a second pipeline, different seeds do not. (Random weights with a
    tied head put a token's own logit far above the rest; the temperature is what makes the draw a draw here.)"""
    from distributed_llm_inference_amd.config import EngineConfig
    from distributed_llm_inference_amd.parallel.launcher import LocalPipeline
    from distributed_llm_inference_amd.runtime.sampler import SamplingParams

    def run(seeds):
        ecfg = EngineConfig(model=model, dtype=dtype, pp_size=1, max_batch=4, num_micro_batches=1, max_seq_len=128, prefill_chunk=32,
                            kv_blocks=16, device="cuda" if backend == "hip" else "cpu", backend=backend, seed=3)
        pipe = LocalPipeline(ecfg)
        try:
            reqs = [pipe.engine.submit(list(range(3, 3 + n)), SamplingParams(temperature=40.0, top_k=40, top_p=0.95, max_new_tokens=12,
                                                                              seed=s, stop_on_eos=False))
                    for n, s in zip((4, 21, 40), seeds)]
            return [r.wait(120).output for r in reqs]
        finally:
            pipe.close()

    a, b, c = run((1, 2, 3)), run((1, 2, 3)), run((4, 5, 6))
    assert all(len(o) == 12 for o in a)
    assert a == b
    assert a != c


def _random_stack(seed: int):
    """A stack drawn at random: 2 to 6 layers of either kind in any order, head counts 1 to 9 with any grouping, key and
    value sizes from 8 to 128 (equal or not), windows from 1 to beyond the prompt, 1 to 6 taps, feed-forward widths that
    are multiples of 8 or not, or none; widths and vocabularies that are powers of two or not."""
    import random
    rng = random.Random(seed)
    layers, vshape = [], None
    for _ in range(rng.randint(2, 6)):
        heads = rng.choice([1, 2, 3, 4, 6, 8])
        kv = rng.choice([k for k in (1, 2, 3, 4, 6, 8) if heads % k == 0])
        dim = rng.choice([8, 12, 16, 24, 32, 40, 64, 80, 128])
        vdim = rng.choice([dim, dim, rng.choice([8, 16, 24, 64, 128])])
        ff = rng.choice([0, 24, 40, 64, 128, 200])
        if rng.random() < 0.6:
            mixes = rng.random() < 0.7
            if mixes:                                  # layers that mix values share the shape of their values
                if vshape is None:
                    vshape = (kv, vdim)
                else:
                    kv, vdim = vshape
                    heads = kv * rng.choice([1, 2, 3])
            layers.append(O.attention_layer(heads, kv, dim, vdim, window=rng.choice([1, 2, 5, 31, 32, 33, 64, 97, 150]),
                                            scale=rng.choice([dim ** -0.5, 0.2, 0.05]), v_mix=mixes, ff=ff))
        else:
            layers.append(O.delta_layer(heads, kv, dim, vdim, conv=rng.randint(1, 6), ff=ff))
    cfg = O.make_config(layers, vocab=rng.choice([33, 64, 100, 257]), width=rng.choice([24, 40, 64, 96, 136, 160, 200, 256, 384]),
                        eps=rng.choice([1e-5, 1e-6]))
    cuts, left = [], 110
    while left > 0:
        cuts.append(min(left, rng.choice([1, 2, 3, 7, 31, 32, 33, 50])))
        left -= cuts[-1]
    return cfg, cuts


@pytest.mark.parametrize("backend,dtype", BACKENDS)
@pytest.mark.parametrize("seed", [11, 12, 13, 14, 15])
def test_random_stacks(tmp_path, seed, backend, dtype):
    cfg, cuts = _random_stack(seed)
    W = O.random_weights(cfg, seed=seed)
    path = save_model(str(tmp_path / "m"), cfg, W)
    toks = random_tokens(cfg, sum(cuts) + 15, seed)
    sess = session(path, backend, dtype)
    got = replay(sess, {"a": toks}, [[("a", c)] for c in cuts] + [[("a", 1)]] * 15)["a"]
    sess.close()
    if dtype == "fp32":
        check(got, oracle_logits(cfg, W, toks), dtype, f"seed {seed}", alone(path, backend, dtype, toks))
    else:   # (a random stack can put a position where bf16 rounding is magnified past any fixed bound: the schedule check stays)
        e = rel_err(got, alone(path, backend, dtype, toks).astype(np.float64))
        assert e < 0.1, f"seed {seed}: differs from the whole prompt run alone by {e:.3g}"


def test_trace_run_executable(models, tmp_path):
    """The executable itself: JSON steps on stdin, `done <step>` lines on stdout, one file of little-endian fp32 logits
    per step in which something is wanted, exit code 0 when the input ends. (CPU: torch executor.)"""
    import json
    import os
    import subprocess
    import sys
    cfg, W, path = models["delta_first"]
    a, b = random_tokens(cfg, 40, 71), random_tokens(cfg, 9, 72)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:33], "want": [0, 32]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:2], "want": []}, {"id": "a", "tokens": a[33:34], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[34:], "want": [5]}, {"id": "b", "tokens": b[2:], "want": [6]}], "end": ["a", "b"]}]
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "trace_run")
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, exe, "--model", path, "--dtype", "float32", "--out", str(out), "--max-tokens", "128",
                        "--backend", "torch", "--device", "cpu"], input="".join(json.dumps(s) + "\n" for s in steps),
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done ")] == ["done 0", "done 1", "done 2"]
    ra, rb = oracle_logits(cfg, W, a), oracle_logits(cfg, W, b)
    V = cfg["vocab"]
    got = {n: np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, V) for n in (0, 1, 2)}
    check(got[0], ra[[0, 32]], "fp32")
    check(got[1], ra[[33]], "fp32")
    check(got[2], np.stack([ra[39], rb[8]]), "fp32")
