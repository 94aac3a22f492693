"""A plain, slow model of the Letarax design, one function per mechanism, in float64 on the CPU.

It shares no code with the package: tests compare the package's executors (torch and HIP) with it.
A model is a config dictionary (the layout of the design's config.json) and a dictionary of tensors
under the checkpoint's names. Everything works on one sequence, token by token where the mechanism
is recurrent, with whole-sequence loops otherwise.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def offset_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * (1 + w): the weight is stored as its distance from one."""
    x = x.to(F64)
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * (1.0 + w.to(F64))


def plain_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    x = x.to(F64)
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w.to(F64)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def linear(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    y = x.to(F64) @ w.to(F64).t()
    return y if b is None else y + b.to(F64)


def sink_window_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv] of one sequence from its start. Token i attends to the
    tokens j with 0 <= i - j < window; the softmax has one more term in its denominator, a sink of
    score 0 that carries no value. Returns [T, H, dv]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for i in range(T):
        lo = max(0, i - window + 1)
        for h in range(H):
            g = h // (H // G)
            s = (k[lo:i + 1, g].to(F64) @ q[i, h].to(F64)) * scale
            m = max(float(s.max()), 0.0)
            e = torch.exp(s - m)
            p = e / (math.exp(-m) + e.sum())
            out[i, h] = p @ v[lo:i + 1, g].to(F64)
    return out


def mix_values(v: torch.Tensor, v_first: torch.Tensor, lam: float) -> torch.Tensor:
    return (1.0 - lam) * v.to(F64) + lam * v_first.to(F64)


def causal_short_conv(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, K]: y[t, c] = sum_j taps[c, j] * x[t - (K - 1 - j), c], zeros before the start."""
    T, C = x.shape
    K = taps.shape[1]
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(K):
            s = t - (K - 1 - j)
            if s >= 0:
                y[t] += taps[:, j].to(F64) * x[s].to(F64)
    return y


def unit_vectors(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def gated_delta_rule(q, k, v, beta, decay):
    """One head. q, k [T, d], v [T, dv], beta, decay [T]. S starts at zero; per token
    S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q (the read-out sees the write)."""
    T, d = q.shape
    S = torch.zeros(d, v.shape[1], dtype=F64)
    out = torch.zeros(T, v.shape[1], dtype=F64)
    for t in range(T):
        S = decay[t] * S
        u = beta[t] * (v[t] - S.t() @ k[t])
        S = S + torch.outer(k[t], u)
        out[t] = S.t() @ q[t]
    return out


def attention_mixer(h, W: Dict[str, torch.Tensor], p: str, m: dict, v_first):
    """Returns (output [T, width], this layer's values [T, G, dv] before mixing is applied downstream)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(h, W[p + "q"], W[p + "q.b"]).reshape(T, H, d)
    k = linear(h, W[p + "k"], W[p + "k.b"]).reshape(T, G, d)
    v = linear(h, W[p + "v"], W[p + "v.b"]).reshape(T, G, dv)
    first = v
    if m.get("v_mix"):
        if v_first is not None:
            v = mix_values(v, v_first, float(W[p + "vmix"]))
            first = v_first
    else:
        first = v_first
    o = sink_window_attention(q, k, v, float(m["scale"]), int(m["mask"]["size"]))
    return linear(o.reshape(T, H * dv), W[p + "o"]), first


def delta_mixer(h, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_short_conv(linear(h, W[p + "q"]), W[p + "q.conv"])).reshape(T, G, d)
    k = silu(causal_short_conv(linear(h, W[p + "k"]), W[p + "k.conv"])).reshape(T, G, d)
    v = silu(causal_short_conv(linear(h, W[p + "v"]), W[p + "v.conv"])).reshape(T, H, dv)
    q = unit_vectors(q) * d ** -0.5
    k = unit_vectors(k)
    beta = torch.sigmoid(linear(h, W[p + "b"]))                                   # [T, H]
    a = linear(h, W[p + "a"]) + W[p + "dt_bias"].to(F64)
    softplus = torch.where(a > 30, a, torch.log1p(torch.exp(torch.clamp(a, max=30.0))))
    decay = torch.exp(-torch.exp(W[p + "A_log"].to(F64)) * softplus)              # [T, H]
    gate = silu(linear(h, W[p + "g"])).reshape(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        o = gated_delta_rule(q[:, g], k[:, g], v[:, hh], beta[:, hh], decay[:, hh])
        out[:, hh] = plain_rmsnorm(o, W[p + "norm"], eps) * gate[:, hh]
    return linear(out.reshape(T, H * dv), W[p + "o"])


def dense_ff(h, W: Dict[str, torch.Tensor], p: str):
    a = gelu_tanh(linear(h, W[p + "gate"], W[p + "gate.b"])) * linear(h, W[p + "up"], W[p + "up.b"])
    return linear(a, W[p + "down"], W[p + "down.b"])


def forward(cfg: dict, W: Dict[str, torch.Tensor], tokens: List[int], return_layers: bool = False):
    """Logits [T, vocab] of one sequence (float64); with `return_layers` also the residual stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = W["embed"].to(F64)[torch.tensor(tokens, dtype=torch.long)]
    v_first = None
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = offset_rmsnorm(x, W[p + "norm1"], eps)
        if layer["type"] == "attention":
            y, v_first = attention_mixer(h, W, p + "mix.", layer["mixer"], v_first)
        elif layer["type"] == "delta":
            y = delta_mixer(h, W, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + offset_rmsnorm(y, W[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            y = dense_ff(offset_rmsnorm(x, W[p + "norm2"], eps), W, p + "mlp.")
            x = x + offset_rmsnorm(y, W[p + "norm2b"], eps)
        after.append(x.clone())
    logits = linear(offset_rmsnorm(x, W["final.norm"], eps), W["embed"])
    return (logits, torch.stack(after)) if return_layers else logits


# ---- random models for tests -----------------------------------------------------------------------------------

def attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, window=8, scale=0.25, v_mix=True, ff=64):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                           "mask": {"size": window}, "scale": scale, "v_mix": v_mix},
            "mlp": None if not ff else {"kind": "dense", "ff": ff}}


def delta_layer(heads=4, kv_heads=2, dim=16, vdim=16, conv=4, ff=0):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": None if not ff else {"kind": "dense", "ff": ff}}


def make_config(layers, vocab=96, width=48, eps=1e-5):
    return {"architecture": "Letarax", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}


def random_weights(cfg: dict, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random tensors under the checkpoint's names, rounded to `dtype` (what a checkpoint stores)."""
    g = torch.Generator().manual_seed(seed)
    D = cfg["width"]
    r = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std).to(dtype)
    W = {"embed": r(cfg["vocab"], D), "final.norm": r(D, std=0.2)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        W[p + "norm1"], W[p + "norm1b"] = r(D, std=0.2), r(D, std=0.2)
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        lin = lambda n, k: r(n, k, std=k ** -0.5)
        if layer["type"] == "attention":
            W[p + "mix.q"], W[p + "mix.q.b"] = lin(H * d, D), r(H * d, std=0.3)
            W[p + "mix.k"], W[p + "mix.k.b"] = lin(G * d, D), r(G * d, std=0.3)
            W[p + "mix.v"], W[p + "mix.v.b"] = lin(G * dv, D), r(G * dv, std=0.3)
            W[p + "mix.vmix"] = (torch.rand((), generator=g) * 0.6 + 0.2).to(dtype)
            W[p + "mix.o"] = lin(D, H * dv)
        else:
            K = m["conv"]
            W[p + "mix.q"], W[p + "mix.q.conv"] = lin(G * d, D), r(G * d, K, std=0.6)
            W[p + "mix.k"], W[p + "mix.k.conv"] = lin(G * d, D), r(G * d, K, std=0.6)
            W[p + "mix.v"], W[p + "mix.v.conv"] = lin(H * dv, D), r(H * dv, K, std=0.6)
            W[p + "mix.b"], W[p + "mix.a"] = lin(H, D), lin(H, D)
            W[p + "mix.A_log"], W[p + "mix.dt_bias"] = r(H, std=0.5), r(H, std=0.5)
            W[p + "mix.norm"] = (1.0 + 0.2 * torch.randn(dv, generator=g)).to(dtype)
            W[p + "mix.g"], W[p + "mix.o"] = lin(H * dv, D), lin(D, H * dv)
        if layer.get("mlp") is not None:
            Fd = layer["mlp"]["ff"]
            W[p + "norm2"], W[p + "norm2b"] = r(D, std=0.2), r(D, std=0.2)
            W[p + "mlp.gate"], W[p + "mlp.gate.b"] = r(Fd, D, std=D ** -0.5), r(Fd, std=0.2)
            W[p + "mlp.up"], W[p + "mlp.up.b"] = r(Fd, D, std=D ** -0.5), r(Fd, std=0.2)
            W[p + "mlp.down"], W[p + "mlp.down.b"] = r(D, Fd, std=Fd ** -0.5), r(D, std=0.2)
    return W
