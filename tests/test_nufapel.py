"""Nufapel through the package (checkpoint reader, executor, per-run caches and state slots, trace replay, scheduler) against
the plain model in `nufapel_oracle`. Every test runs on the torch executor on the CPU; the same tests run on the HIP executor,
in fp32 and in bf16, under the `gpu` marker."""
import numpy as np
import pytest
import torch

import nufapel_oracle as O
from nufapel_util import (STACKS, alone, dense, gd_layer, make_config, moe, oracle_logits, par_layer, random_tokens, random_weights,
                          rel_err, replay, save, session)

BACKENDS = [pytest.param("torch", "fp32", id="torch"),
            pytest.param("hip", "fp32", id="hip-fp32", marks=pytest.mark.gpu),
            pytest.param("hip", "bf16", id="hip-bf16", marks=pytest.mark.gpu)]
# fp32 executors agree with the plain model to rounding. In bf16 a tiny random stack magnifies single roundings, so the sharp
# check there is SAME: however a request was cut into steps and whatever shared its batches, its logits agree with the same
# executor's run of the whole prompt alone.
# (bf16 against the plain model: nine positions in ten. A router is a discontinuity: where two experts' scores nearly tie,
# one bf16 rounding picks the other expert and that position's logits move as a whole.)
TOL = {"fp32": 3e-4, "bf16": 0.35}
SAME = {"fp32": 1e-4, "bf16": 8e-2}


def pos_errs(got, ref):
    d = got.astype(np.float64) - ref
    d = d - d.mean(-1, keepdims=True)
    r = ref - ref.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt((r ** 2).mean(-1)).mean()


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for i, (name, cfg) in enumerate(STACKS.items()):
        W = random_weights(cfg, seed=30 + i)
        out[name] = (cfg, W, save(str(tmp_path_factory.mktemp(name)), cfg, W))
    return out


def check(got, ref, dtype, what="", same_as=None):
    e = pos_errs(got, ref)
    e = float(e.max() if dtype == "fp32" else np.quantile(e, 0.9))
    assert e < TOL[dtype], f"{what}: error {e:.3g} over {TOL[dtype]}"
    if same_as is not None:
        e = pos_errs(got, same_as.astype(np.float64))
        e = float(e.max() if dtype == "fp32" else np.quantile(e, 0.9))      # (bf16: kernels of another shape round otherwise, a near tie flips)
        assert e < SAME[dtype], f"{what}: differs from the whole prompt run alone by {e:.3g}, over {SAME[dtype]}"


def test_config_round_trip_and_runs():
    from distributed_llm_inference_amd.models.spec import ModelSpec
    from nufapel_util import config_json
    for name, cfg in STACKS.items():
        spec = ModelSpec.from_hf_config(config_json(cfg))
        assert spec.family == "nufapel" and spec.has_recurrent_state
        assert [(li, p if p >= 0 else None) for li, p in spec.layer_runs()] == [(li, p) for li, p, _ in O.layer_runs(cfg)], name
        again = ModelSpec.from_hf_config(spec.hf_config())
        assert again.layer_runs() == spec.layer_runs() and again.logit_softcap == spec.logit_softcap


@pytest.mark.parametrize("backend,dtype", BACKENDS)
@pytest.mark.parametrize("stack", list(STACKS))
def test_whole_prompt(models, stack, backend, dtype):
    cfg, W, path = models[stack]
    toks = random_tokens(cfg, 70, 1)
    sess = session(path, backend, dtype)
    got = replay(sess, {"a": toks}, [[("a", len(toks))]])["a"]
    sess.close()
    check(got, oracle_logits(cfg, W, toks), dtype, stack)


@pytest.mark.parametrize("backend,dtype", BACKENDS)
@pytest.mark.parametrize("stack", ["loop_mid", "no_loop", "packed", "mfma_heads"])
def test_prefill_then_long_decoding(models, stack, backend, dtype):
    """A prompt, then one token a step over several cache blocks and past every edge of the bias tables."""
    cfg, W, path = models[stack]
    toks = random_tokens(cfg, 120, 2)
    sess = session(path, backend, dtype)
    got = replay(sess, {"a": toks}, [[("a", 30)]] + [[("a", 1)]] * 90)["a"]
    sess.close()
    check(got, oracle_logits(cfg, W, toks), dtype, stack, alone(path, backend, dtype, toks))


@pytest.mark.parametrize("backend,dtype", BACKENDS)
@pytest.mark.parametrize("stack", ["loop_mid", "once", "whole_loop"])
def test_first_tokens_alone(models, stack, backend, dtype):
    """A sequence that starts token by token: states start from zero, the running maximum from 0, the sink counts from the first token."""
    cfg, W, path = models[stack]
    toks = random_tokens(cfg, 10, 3)
    sess = session(path, backend, dtype)
    got = replay(sess, {"a": toks}, [[("a", 1)]] * 10)["a"]
    sess.close()
    check(got, oracle_logits(cfg, W, toks), dtype, stack, alone(path, backend, dtype, toks))


@pytest.mark.parametrize("backend,dtype", BACKENDS)
@pytest.mark.parametrize("stack,cuts", [("loop_mid", [2, 2, 3, 1, 29, 2, 31, 33, 2, 1, 5]), ("no_loop", [31, 2, 2, 36, 1, 3, 2, 17]),
                                        ("once", [1, 2, 30, 3, 16, 17, 2, 9]), ("packed", [2, 31, 2, 1, 60, 3, 18, 2, 33]), ("mfma_heads", [2, 31, 2, 1, 97, 3, 130, 2, 33])])
def test_portions(models, stack, cuts, backend, dtype):
    """Prompts cut into portions of changing size, down to two tokens, across block edges and the recurrences' chunk edges."""
    cfg, W, path = models[stack]
    toks = random_tokens(cfg, sum(cuts), 4)
    sess = session(path, backend, dtype)
    got = replay(sess, {"a": toks}, [[("a", c)] for c in cuts])["a"]
    sess.close()
    check(got, oracle_logits(cfg, W, toks), dtype, stack, alone(path, backend, dtype, toks))


@pytest.mark.parametrize("backend,dtype", BACKENDS)
@pytest.mark.parametrize("stack", ["loop_mid", "no_loop", "packed", "mfma_heads"])
def test_mixed_batches_and_reuse(models, stack, backend, dtype):
    """Unequal requests share steps (portions beside single tokens), more requests than slots over time, a pool that only holds
    the live ones: slots and blocks change hands. Every request must come out as if it ran alone."""
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
def test_long_prompt(tmp_path, backend, dtype):
    """A prompt long enough that the routed feed-forward takes its many-row path (128-row expert tiles on the GPU in bf16), the
    recurrences walk dozens of chunks and the attention spans twenty cache blocks; whole, and in two portions."""
    cfg = dict(STACKS["packed"], max_positions=1024)
    W = random_weights(cfg, seed=77)
    path = save(str(tmp_path / "m"), cfg, W)
    toks = random_tokens(cfg, 640, 9)
    ref = oracle_logits(cfg, W, toks)
    whole = alone(path, backend, dtype, toks)
    check(whole, ref, dtype, "whole")
    sess = session(path, backend, dtype, max_tokens=704)
    got = replay(sess, {"a": toks}, [[("a", 300)], [("a", 340)]])["a"]
    sess.close()
    check(got, ref, dtype, "two portions", whole)


@pytest.mark.parametrize("backend,dtype", BACKENDS)
def test_slot_taken_over_starts_clean(models, backend, dtype):
    """One slot, one request after another: the second must not see the first one's states, running maxima or cache rows."""
    cfg, W, path = models["loop_mid"]
    a, b = random_tokens(cfg, 50, 31), random_tokens(cfg, 20, 32)
    sess = session(path, backend, dtype, max_tokens=64, slots=1)
    got = replay(sess, {"a": a, "b": b}, [[("a", 50)], [("b", 1)], [("b", 2)], [("b", 17)]])
    sess.close()
    check(got["b"], oracle_logits(cfg, W, b), dtype, "second", alone(path, backend, dtype, b))
    check(got["a"], oracle_logits(cfg, W, a), dtype, "first", alone(path, backend, dtype, a))


@pytest.mark.parametrize("d", [16, 64])
@pytest.mark.parametrize("backend,dtype", BACKENDS)
def test_far_keys_bucket_edges_and_sink(tmp_path, backend, dtype, d):
    """A parallel layer whose attention weights are shaped so that one far key stands out: token 7's key is large along one
    direction, token 9 asks along it, nobody else does. The bias table is steep, so a distance that lands in the neighbouring
    row, a key that is lost, or a sink that is left out moves the asked position's logits by far more than the tolerance. The
    beacon sits at every edge of the table's rows (the linear rows, the first logarithmic ones, the last row's start), hundreds
    of tokens back across cache blocks; in a prompt, in portions and in decoding."""
    rows, far = 12, 96
    cfg = make_config([par_layer(2, 1, d, d, 1, 8, 8, None, scale=1.0, rows=rows, bias_max=far)], vocab=40, width=32)
    W = random_weights(cfg, seed=5)
    for n in ("l0.mix.left.q", "l0.mix.left.k"):
        W[n] = torch.zeros_like(W[n])
    # (the norm keeps the sign pattern of a token's embedding + position; positions are switched off so that tokens are told apart)
    W["pos"] = torch.zeros_like(W["pos"])
    h7 = O.dyt(W["embed"][7].double(), W["l0.norm1"].double(), W["l0.norm1.b"].double(), W["l0.norm1.alpha"].double())
    h9 = O.dyt(W["embed"][9].double(), W["l0.norm1"].double(), W["l0.norm1.b"].double(), W["l0.norm1.alpha"].double())
    W["l0.mix.left.k"][0] = (h7 * 0.6).to(torch.bfloat16)
    W["l0.mix.left.q"][0] = (h9 * 0.6).to(torch.bfloat16)
    W["l0.mix.left.q"][d] = (h9 * 0.6).to(torch.bfloat16)
    W["l0.mix.left.rel"] = (torch.arange(rows).float().view(-1, 1) * torch.tensor([[1.5, -1.5]])).to(torch.bfloat16)
    W["l0.mix.left.sink"] = torch.tensor([24.0, 7.0], dtype=torch.bfloat16)
    path = save(str(tmp_path / "m"), cfg, W)
    base = [t for t in random_tokens(cfg, 500, 6) if t not in (7, 9)][:330]
    edges = sorted({n for n in range(1, 300) if O.distance_bucket(n, rows, far) != O.distance_bucket(n - 1, rows, far)})
    assert len(edges) == rows - 1
    for dist in [edges[4], edges[5] - 1, edges[5], edges[7] - 1, edges[7], edges[-1] - 1, edges[-1], 200, 290]:
        ask = 300
        toks = list(base)
        toks[ask - dist], toks[ask] = 7, 9
        ref = oracle_logits(cfg, W, toks)
        for sched in ([[("a", 330)]], [[("a", ask - 1)], [("a", 2)], [("a", 29)]], [[("a", ask)]] + [[("a", 1)]] * 3):
            n = sum(c for step in sched for _, c in step)
            sess = session(path, backend, dtype, max_tokens=352, slots=1)
            got = replay(sess, {"a": toks[:n]}, sched)["a"]
            sess.close()
            check(got, ref[:n], dtype, f"beacon {dist} back")
    # what the check rests on: the asked position's logits depend on the beacon, on its row of the table and on the sink
    def at(toks, Wx):
        return oracle_logits(cfg, Wx, toks)[300][None]
    toks = list(base); toks[300 - edges[5]], toks[300] = 7, 9
    moved = list(base); moved[300 - edges[5] + 1], moved[300] = 7, 9
    none = list(base); none[300] = 9
    nosink = dict(W); nosink["l0.mix.left.sink"] = torch.tensor([-30.0, -30.0], dtype=torch.bfloat16)
    assert rel_err(at(toks, W), at(moved, W)) > 0.02 and rel_err(at(toks, W), at(none, W)) > 0.02 and rel_err(at(toks, W), at(toks, nosink)) > 0.02


@pytest.mark.parametrize("stack,buckets", [("loop_mid", []), ("packed", []), ("no_loop", [2]), ("mfma_heads", [])])
@pytest.mark.parametrize("backend,dtype", BACKENDS)
def test_greedy_generation_through_the_scheduler(models, backend, dtype, stack, buckets):
    """Requests of unequal length through the engine's own entry point: scheduler, continuous batching, chunked prompts, greedy
    sampling; on the HIP executor with captured decode steps. The tokens are those of the plain model's argmax."""
    from distributed_llm_inference_amd.config import EngineConfig
    from distributed_llm_inference_amd.parallel.launcher import LocalPipeline
    from distributed_llm_inference_amd.runtime.sampler import SamplingParams
    cfg, W, path = models[stack]
    prompts = [random_tokens(cfg, n, 40 + n) for n in (5, 37, 64, 11, 90, 2)]
    new = 20
    ecfg = EngineConfig(model=path, dtype=dtype, pp_size=1, max_batch=4, num_micro_batches=1, max_seq_len=256, prefill_chunk=48,
                        kv_blocks=24, device="cuda" if backend == "hip" else "cpu", backend=backend, seed=0, decode_buckets=buckets)
    pipe = LocalPipeline(ecfg)
    try:
        reqs = [pipe.engine.submit(p, SamplingParams(temperature=0.0, max_new_tokens=new, stop_on_eos=False)) for p in prompts]
        outs = [r.wait(180).output for r in reqs]
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


@pytest.mark.parametrize("backend,dtype,model", [pytest.param("torch", "fp32", "tiny-nufapel-test", id="torch"),
                                                 pytest.param("hip", "bf16", "tiny-nufapel-gpu-test", id="hip-bf16", marks=pytest.mark.gpu)])
def test_builtin_stack_samples_reproducibly(backend, dtype, model):
    """A built-in stack (random weights drawn by the package, no checkpoint) through the engine with temperature / top-k / top-p
    sampling: the same seeds give the same tokens on a second pipeline, other seeds do not."""
    from distributed_llm_inference_amd.config import EngineConfig
    from distributed_llm_inference_amd.parallel.launcher import LocalPipeline
    from distributed_llm_inference_amd.runtime.sampler import SamplingParams

    def run(seeds):
        ecfg = EngineConfig(model=model, dtype=dtype, pp_size=1, max_batch=4, num_micro_batches=1, max_seq_len=128, prefill_chunk=32,
                            kv_blocks=16, device="cuda" if backend == "hip" else "cpu", backend=backend, seed=3)
        pipe = LocalPipeline(ecfg)
        try:
            reqs = [pipe.engine.submit(list(range(3, 3 + n)), SamplingParams(temperature=3.0, top_k=40, top_p=0.95, max_new_tokens=12,
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
    """A stack drawn at random: 2 to 5 layers of either kind in any order, any stretch repeated 1 to 3 times or none, head counts,
    groupings and sizes of all kinds, every feed-forward kind."""
    import random
    rng = random.Random(seed)

    def mlp():
        k = rng.choice(["none", "dense", "moe", "moe"])
        if k == "none":
            return None
        if k == "dense":
            return dense(rng.choice([24, 40, 64, 100]))
        groups = rng.choice([1, 2, 3, 4])
        per = rng.choice([1, 2, 3])
        keep = rng.randint(1, groups)
        return moe(groups * per, rng.randint(1, keep * per), rng.choice([8, 24, 40]), groups, keep, rng.choice([1.0, 2.5]), rng.choice([0.5, 1.5, 7.0]))

    layers = []
    for _ in range(rng.randint(2, 5)):
        if rng.random() < 0.4:
            layers.append(gd_layer(rng.choice([1, 2, 3, 4]), rng.choice([8, 16, 24, 40, 64, 80]), mlp(), rank=rng.choice([2, 8, 12, 32])))
        else:
            heads = rng.choice([1, 2, 3, 4, 6, 8])
            kv = rng.choice([k for k in (1, 2, 3, 4, 6, 8) if heads % k == 0])
            dim = rng.choice([8, 12, 16, 24, 40, 64])
            rows = rng.choice([4, 8, 14, 32])
            layers.append(par_layer(heads, kv, dim, rng.choice([dim, 8, 24, 64]), rng.choice([1, 2, 3]), rng.choice([8, 16, 24, 72]),
                                    rng.choice([8, 16, 40, 64]), mlp(), scale=rng.choice([None, 0.2]), rows=rows,
                                    bias_max=rng.choice([rows, 3 * rows, 500]), gate_cap=rng.choice([3.0, 15.0])))
    n = len(layers)
    loop = None
    if rng.random() < 0.7:
        start = rng.randint(0, n - 1)
        loop = (start, rng.randint(start + 1, n), rng.randint(1, 3))
    cfg = make_config(layers, vocab=rng.choice([33, 64, 100, 257]), width=rng.choice([24, 40, 64, 96, 136, 160, 256]), loop=loop,
                      eps=rng.choice([1e-5, 1e-6]), softcap=rng.choice([5.0, 30.0]))
    cuts, left = [], 90
    while left > 0:
        cuts.append(min(left, rng.choice([1, 2, 3, 7, 16, 31, 32, 33, 50])))
        left -= cuts[-1]
    return cfg, cuts


@pytest.mark.parametrize("backend,dtype", BACKENDS)
@pytest.mark.parametrize("seed", [11, 12, 13, 14, 15, 16])
def test_random_stacks(tmp_path, seed, backend, dtype):
    cfg, cuts = _random_stack(seed)
    W = random_weights(cfg, seed=seed)
    path = save(str(tmp_path / "m"), cfg, W)
    toks = random_tokens(cfg, sum(cuts) + 12, seed)
    sess = session(path, backend, dtype)
    got = replay(sess, {"a": toks}, [[("a", c)] for c in cuts] + [[("a", 1)]] * 12)["a"]
    sess.close()
    if dtype == "fp32":
        check(got, oracle_logits(cfg, W, toks), dtype, f"seed {seed}", alone(path, backend, dtype, toks))
    else:   # (a random stack can put a position where bf16 rounding is magnified past any fixed bound: the schedule check stays)
        e = float(np.quantile(pos_errs(got, alone(path, backend, dtype, toks).astype(np.float64)), 0.9))
        assert e < 0.1, f"seed {seed}: differs from the whole prompt run alone by {e:.3g}"


def test_trace_run_executable(models, tmp_path):
    """The executable on a Nufapel checkpoint: the model class is chosen by config.json, steps arrive as JSON lines, logits
    leave as little-endian fp32 files. (CPU: torch executor.)"""
    import json
    import os
    import subprocess
    import sys
    cfg, W, path = models["no_loop"]
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
