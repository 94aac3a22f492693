"""Helpers of the Nufapel tests: small configurations, random checkpoints in the design's tensor names, and the stacks the
model-level tests run. Sessions, replays and error measures are those of the other hybrid design's tests."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

import nufapel_oracle as O
from letarax_util import alone, random_tokens, rel_err, replay, save_model, session  # noqa: F401  (re-exported)

BF = torch.bfloat16


def dense(ff: int) -> dict:
    return {"kind": "dense", "ff": ff}


def moe(experts: int, top: int, ff: int, groups: int = 1, keep: int = 1, scale: float = 1.0, limit: float = 2.0) -> dict:
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "top": top, "scale": scale, "groups": {"count": groups, "keep": keep}}}


def gd_layer(heads: int, dim: int, mlp: Optional[dict] = None, rank: int = 8) -> dict:
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim}, "mlp": mlp, "_rank": rank}


def par_layer(heads: int, kv_heads: int, dim: int, vdim: int, r_heads: int, r_dim: int, r_vdim: int, mlp: Optional[dict] = None,
              scale: Optional[float] = None, bias_max: int = 64, rows: int = 12, gate_cap: float = 10.0) -> dict:
    return {"type": "parallel", "mlp": mlp, "_rows": rows,
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "bias_max": bias_max,
                               "scale": dim ** -0.5 if scale is None else scale},
                      "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "gate_cap": gate_cap}}}


def make_config(layers: List[dict], vocab: int, width: int, loop=None, eps: float = 1e-5, softcap: float = 20.0, max_positions: int = 512) -> dict:
    cfg = {"architecture": "Nufapel", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width,
           "max_positions": max_positions, "logit_softcap": softcap}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def config_json(cfg: dict) -> dict:
    """What goes to config.json: without the sizes that only the tensors' shapes give (decay rank, bias rows)."""
    return {**cfg, "layers": [{k: v for k, v in l.items() if not k.startswith("_")} for l in cfg["layers"]]}


def random_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors under the checkpoint's names, of sizes at which every mechanism moves the logits."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    rn = lambda *shape, std=1.0: (torch.randn(*shape, generator=g) * std).to(BF)
    one = lambda *shape, std=0.1: (1.0 + torch.randn(*shape, generator=g) * std).to(BF)
    t = {"embed": rn(V, W), "pos": rn(cfg["max_positions"], W, std=0.5), "head": rn(V, W, std=2.0 * W ** -0.5),
         "final.norm": one(W), "final.norm.b": rn(W, std=0.1), "final.norm.alpha": torch.tensor(0.7, dtype=BF)}
    if cfg.get("loop"):
        t["loop.step"] = rn(cfg["loop"]["times"], W, std=0.5)

    def norm(name, alpha):
        t[name], t[name + ".b"], t[name + ".alpha"] = one(W), rn(W, std=0.1), torch.tensor(alpha, dtype=BF)

    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        norm(p + "norm1", 0.5 + 0.1 * (i % 3))
        t[p + "rg1"], t[p + "rg1.b"] = rn(W, W, std=W ** -0.5), rn(W, std=0.5)
        x = p + "mix."
        if L["type"] == "general_delta":
            n, R = m["heads"] * m["dim"], L["_rank"]
            for k in "rkvga":
                t[x + k] = rn(n, W, std=W ** -0.5)
            t[x + "a.b"], t[x + "w1"], t[x + "w2"], t[x + "w0"] = rn(n, std=0.5), rn(R, W, std=W ** -0.5), rn(n, R, std=2.0 * R ** -0.5), rn(n, std=1.5)
            t[x + "norm"], t[x + "o"] = one(n), rn(W, n, std=n ** -0.5)
        else:
            a, b = m["left"], m["right"]
            t[x + "left.q"], t[x + "left.k"] = rn(a["heads"] * a["dim"], W, std=1.5 * W ** -0.5), rn(a["kv_heads"] * a["dim"], W, std=1.5 * W ** -0.5)
            t[x + "left.v"], t[x + "left.g"] = rn(a["kv_heads"] * a["vdim"], W, std=W ** -0.5), rn(a["heads"], W, std=W ** -0.5)
            t[x + "left.rel"], t[x + "left.temp"], t[x + "left.sink"] = rn(L["_rows"], a["heads"]), one(a["heads"], std=0.3), rn(a["heads"])
            t[x + "left.o"] = rn(W, a["heads"] * a["vdim"], std=(a["heads"] * a["vdim"]) ** -0.5)
            nk, nv = b["heads"] * b["dim"], b["heads"] * b["vdim"]
            t[x + "right.q"], t[x + "right.k"], t[x + "right.v"], t[x + "right.g"] = rn(nk, W, std=W ** -0.5), rn(nk, W, std=W ** -0.5), rn(nv, W, std=W ** -0.5), rn(nv, W, std=W ** -0.5)
            t[x + "right.i"], t[x + "right.f"] = rn(b["heads"], W, std=2.0 * W ** -0.5), rn(b["heads"], W, std=2.0 * W ** -0.5)
            t[x + "right.i.b"], t[x + "right.f.b"] = rn(b["heads"]), rn(b["heads"]) + 2.0
            t[x + "right.norm"], t[x + "right.o"] = one(nv), rn(W, nv, std=nv ** -0.5)
            t[x + "left.out"], t[x + "right.out"] = one(W), one(W)
        mlp = L.get("mlp")
        if mlp is None:
            continue
        norm(p + "norm2", 0.6)
        t[p + "rg2"], t[p + "rg2.b"] = rn(W, W, std=W ** -0.5), rn(W, std=0.5)
        if mlp["kind"] == "dense":
            t[p + "mlp.up"], t[p + "mlp.down"] = rn(mlp["ff"], W, std=W ** -0.5), rn(W, mlp["ff"], std=mlp["ff"] ** -0.5)
        else:
            f = mlp["expert"]["ff"]
            t[p + "mlp.router"] = rn(mlp["router"]["experts"], W, std=2.0 * W ** -0.5)
            for e in range(mlp["router"]["experts"]):
                t[f"{p}mlp.e{e}.gate"], t[f"{p}mlp.e{e}.up"] = rn(f, W, std=1.5 * W ** -0.5), rn(f, W, std=1.5 * W ** -0.5)
                t[f"{p}mlp.e{e}.down"] = rn(W, f, std=f ** -0.5)
    return t


def save(path: str, cfg: dict, W) -> str:
    return save_model(path, config_json(cfg), W)


def oracle_logits(cfg: dict, W, tokens: List[int]):
    return O.forward(cfg, W, tokens).numpy()


# Stacks that differ in what a config can say: order of the layers, which stretch repeats and how often (or none), layers
# without a feed-forward, dense and routed feed-forwards on either mixer, head counts and groupings, key / value sizes (equal,
# unequal, not powers of two; 64 and 128, which the MFMA attention kernels take in bf16), bias tables of several sizes and reaches, expert counts, group counts of 1 and of one expert
# each, a single chosen expert, decay ranks, widths that are no multiple of 8 and widths the packed-weight GEMMs take.
STACKS = {
    "loop_mid": make_config([par_layer(4, 2, 16, 16, 2, 16, 24, dense(48)), gd_layer(2, 32, moe(6, 2, 24, 3, 2, 1.5)),
                             par_layer(2, 2, 24, 8, 1, 32, 16, None, rows=8, bias_max=40), gd_layer(4, 16, dense(40), rank=4),
                             par_layer(6, 3, 8, 16, 3, 8, 8, moe(4, 1, 16, 1, 1, 2.5, limit=1.0), rows=16, bias_max=200)],
                            vocab=90, width=64, loop=(1, 3, 3)),
    "no_loop": make_config([gd_layer(3, 24, None, rank=5), par_layer(3, 1, 20, 12, 2, 12, 20, moe(8, 3, 20, 4, 2, 0.7), scale=0.3, rows=10, bias_max=30)],
                           vocab=51, width=72, eps=1e-6, softcap=8.0),
    "once": make_config([gd_layer(1, 48, dense(24), rank=3), par_layer(2, 2, 12, 12, 2, 24, 12, dense(36), gate_cap=4.0),
                         gd_layer(2, 16, moe(5, 2, 12, 5, 3, 1.0))], vocab=64, width=40, loop=(2, 3, 1)),
    "whole_loop": make_config([par_layer(4, 4, 8, 8, 4, 8, 8, moe(9, 3, 8, 3, 3, 3.0), rows=6, bias_max=12), gd_layer(2, 24, None)],
                              vocab=70, width=48, loop=(0, 2, 4)),
    # sizes the packed-weight GEMMs take in bf16 (inner sizes that are multiples of 128)
    "packed": make_config([gd_layer(2, 64, moe(8, 2, 128, 2, 1, 2.0), rank=16), par_layer(4, 2, 32, 32, 2, 64, 64, dense(256), rows=20, bias_max=300),
                           par_layer(8, 1, 16, 16, 1, 128, 128, moe(4, 2, 128, 2, 2, 1.0))], vocab=96, width=128, loop=(0, 2, 2)),
    "mfma_heads": make_config([par_layer(6, 2, 64, 64, 2, 64, 64, dense(128), rows=14, bias_max=100), gd_layer(2, 64, None, rank=16),
                               par_layer(8, 1, 128, 128, 1, 32, 48, moe(6, 2, 64, 3, 2, 1.5), scale=0.05, rows=24, bias_max=90)],
                              vocab=80, width=128, loop=(0, 3, 2)),
}
