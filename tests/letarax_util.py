"""Helpers of the Letarax tests: random models written as checkpoints (config.json + model.safetensors), run through
the package's own loader, executor and trace replay, and compared with the plain model of `letarax_oracle`."""
from __future__ import annotations

import json
import os
from typing import Dict, List, Sequence

import numpy as np
import torch

import letarax_oracle as O


def save_model(path: str, cfg: dict, W: Dict[str, torch.Tensor]) -> str:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return path


def random_tokens(cfg: dict, n: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def session(model_dir: str, backend: str, dtype: str = "fp32", max_tokens: int = 1024, slots: int = 4):
    from distributed_llm_inference_amd.runtime.trace_runner import TraceSession
    return TraceSession(model_dir, dtype, max_tokens, slots, device="cuda" if backend == "hip" else "cpu", backend=backend)


def replay(sess, requests: Dict[str, List[int]], schedule: Sequence[Sequence[tuple]]) -> Dict[str, np.ndarray]:
    """Runs `schedule` (steps of (request, token count) pairs) and returns every request's logits at all its
    positions. A request ends with the step that brings its last token."""
    at = {k: 0 for k in requests}
    got = {k: [] for k in requests}
    for step in schedule:
        entries, end = [], []
        for name, n in step:
            lo = at[name]
            hi = lo + n
            assert hi <= len(requests[name])
            entries.append({"id": name, "tokens": requests[name][lo:hi], "want": list(range(n))})
            at[name] = hi
            if hi == len(requests[name]):
                end.append(name)
        out = sess.step(entries, end)
        r = 0
        for name, n in step:
            got[name].append(out[r:r + n])
            r += n
    return {k: np.concatenate(v) for k, v in got.items() if v}


def oracle_logits(cfg: dict, W, tokens: List[int]) -> np.ndarray:
    return O.forward(cfg, W, tokens).numpy()


def rel_err(got: np.ndarray, ref: np.ndarray) -> float:
    """Largest per-position error: rms over the vocabulary of the difference (mean taken off), over the rms of the reference."""
    d = got.astype(np.float64) - ref
    d = d - d.mean(-1, keepdims=True)
    r = ref - ref.mean(-1, keepdims=True)
    return float((np.sqrt((d ** 2).mean(-1)) / np.sqrt((r ** 2).mean(-1)).mean()).max())


# Against the plain model: fp32 executors agree to rounding; in bf16 a tiny random model's worst position carries
# several per cent of rounding noise, so the sharp check of a bf16 run is `SAME`: however a request was cut into
# steps and whatever shared its batches, its logits agree with the same executor's run of the whole prompt alone
# (to a few roundings: GEMMs and attention kernels choose their blocking, split and kernel shape by the step's size;
# a random stack this small magnifies one bf16 rounding, 0.4 %, some tenfold on its way to the logits, which is also
# why its bf16 logits sit up to 20 % of their spread away from the plain model's at the worst position).
TOL = {"fp32": 2e-4, "bf16": 0.35}
SAME = {"fp32": 1e-4, "bf16": 8e-2}


def alone(model_dir: str, backend: str, dtype: str, tokens: List[int]) -> np.ndarray:
    sess = session(model_dir, backend, dtype, max_tokens=len(tokens) + 64, slots=1)
    out = replay(sess, {"x": tokens}, [[("x", len(tokens))]])["x"]
    sess.close()
    return out

# Stacks that differ from each other in everything a config can say: order and kind of the layers, head counts
# and groupings, key and value sizes (equal, unequal, not powers of two), window lengths (1, shorter and longer
# than a cache block, longer than the prompts), convolution lengths, layers with and without a feed-forward,
# feed-forward widths that are no multiple of 16, value mixing on all, some or one attention layer, widths that
# are no multiple of 8.
A, D = O.attention_layer, O.delta_layer
STACKS = {
    "mixed": (O.make_config([A(6, 3, 16, 16, window=8), D(6, 2, 16, 16, conv=4), A(6, 3, 16, 16, window=8), A(6, 3, 16, 16, window=8)],
                            vocab=96, width=48)),
    "delta_first": (O.make_config([D(2, 1, 24, 40, conv=2, ff=40), A(3, 3, 24, 8, window=37, scale=0.3, v_mix=False),
                                   D(6, 3, 8, 16, conv=5), A(6, 2, 8, 24, window=3, v_mix=True, ff=0)], vocab=70, width=72)),
    "odd_sizes": (O.make_config([A(2, 1, 12, 20, window=1, scale=0.5, ff=24), A(4, 1, 20, 20, window=200, scale=0.11, ff=56),
                                 A(2, 2, 6, 10, window=33, v_mix=False, ff=0), D(1, 1, 7, 9, conv=3, ff=16), A(4, 1, 36, 20, window=32, scale=0.2)],
                                vocab=51, width=36, eps=1e-6)),
    "only_delta": (O.make_config([D(4, 4, 32, 32, conv=4, ff=32), D(2, 2, 64, 16, conv=1)], vocab=64, width=64)),
    # key / value sizes and widths that the packed-weight GEMMs and the MFMA attention kernels take (bf16)
    "mfma_heads": (O.make_config([A(4, 2, 64, 64, window=40, scale=0.125, ff=128), A(4, 2, 64, 64, window=100, scale=0.125, ff=64),
                                  D(2, 1, 64, 64, conv=4), A(8, 1, 128, 128, window=5, scale=0.09, v_mix=False, ff=0)], vocab=90, width=128)),
    "wide_heads": (O.make_config([A(2, 1, 96, 128, window=64, scale=0.1), D(2, 1, 160, 72, conv=4), A(4, 1, 96, 128, window=48, scale=0.1)],
                                 vocab=80, width=128)),
}
