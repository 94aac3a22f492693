"""A plain float64 model of the Nufapel design, written from its equations: one function per mechanism, whole
sequences only, no cache, nothing shared with the package. `forward(cfg, tensors, tokens)` takes the dict form
of a config.json, a dict of checkpoint tensors by name and one sequence of token ids.

Notation: x [T, W] is the residual stream, h a sublayer's input, sigma the logistic function.
"""
import math

import torch

F64 = torch.float64


def sigma(x):
    return 1.0 / (1.0 + torch.exp(-x))


def dyt(x, w, b, alpha):
    """Dynamic tanh in place of a norm: no statistics, y = tanh(alpha x) w + b."""
    return torch.tanh(alpha * x) * w + b


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_erf(x):
    return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))


def distance_bucket(n, rows, far):
    """Row of the bias table for a distance n >= 0: one row per distance below rows / 2, logarithmic rows up to `far`."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def biased_sink_attention(h, t, m, pre):
    """Causal grouped-query attention without rotation. score_ij = (q_i . k_j) scale temp_head + rel[bucket(i - j), head];
    the softmax's denominator has one more term exp(sink_head); each head's output is gated by sigma(W_g h)_head."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ t[pre + "q"].T).reshape(T, H, d)
    k = (h @ t[pre + "k"].T).reshape(T, G, d)
    v = (h @ t[pre + "v"].T).reshape(T, G, dv)
    gate = sigma(h @ t[pre + "g"].T)                              # [T, H]
    rel, temp, sink = t[pre + "rel"], t[pre + "temp"], t[pre + "sink"]
    rows = torch.tensor([distance_bucket(n, rel.shape[0], m["bias_max"]) for n in range(T)])
    pos = torch.arange(T)
    dist = pos.view(-1, 1) - pos.view(1, -1)                      # i - j
    hidden = dist < 0
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"] * temp[hd] + rel[:, hd][rows[dist.clamp(min=0)]]
        s = s.masked_fill(hidden, float("-inf"))
        s = torch.cat([s, sink[hd].expand(T, 1)], dim=1)          # the sink: a score without a key or a value
        p = torch.softmax(s, dim=1)[:, :T]
        out[:, hd] = (p @ v[:, g]) * gate[:, hd:hd + 1]
    return out.reshape(T, H * dv) @ t[pre + "o"].T


def matrix_memory(h, t, m, pre, eps):
    """A matrix memory with exponential gates stabilised by a running maximum mx whose initial value is 0, not -inf:
    mx_t = max(f + mx_(t-1), i); S_t = exp(f + mx_(t-1) - mx_t) S_(t-1) + exp(i - mx_t) k v^T, n_t the same with k alone;
    o_t = S_t^T q / (max(|n_t . q|, exp(-mx_t)) + 1e-6)."""
    T = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ t[pre + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ t[pre + "k"].T).reshape(T, H, d)
    v = (h @ t[pre + "v"].T).reshape(T, H, dv)
    li = cap * torch.tanh((h @ t[pre + "i"].T + t[pre + "i.b"]) / cap)
    lf = cap * torch.tanh((h @ t[pre + "f"].T + t[pre + "f.b"]) / cap)
    lf = -torch.log1p(torch.exp(-lf))                             # log sigma
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        S, n, mx = torch.zeros(d, dv, dtype=F64), torch.zeros(d, dtype=F64), 0.0
        for i in range(T):
            new = max(float(lf[i, hd]) + mx, float(li[i, hd]))
            keep, put = math.exp(float(lf[i, hd]) + mx - new), math.exp(float(li[i, hd]) - new)
            S = keep * S + put * torch.outer(k[i, hd], v[i, hd])
            n = keep * n + put * k[i, hd]
            mx = new
            out[i, hd] = (S.T @ q[i, hd]) / (max(abs(float(n @ q[i, hd])), math.exp(-mx)) + 1e-6)
    o = rms_unit(out, eps).reshape(T, H * dv) * t[pre + "norm"] * sigma(h @ t[pre + "g"].T)
    return o @ t[pre + "o"].T


def general_delta(h, t, m, pre, eps):
    """Generalised delta rule. Per head: S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T with the unit key u,
    decay w = exp(-exp(-1/2) sigma(W_w2 tanh(W_w1 h) + w0)), removal rate a = sigma(W_a h + b); o_t = S_t^T r_t."""
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    r = (h @ t[pre + "r"].T).reshape(T, H, d)
    k = (h @ t[pre + "k"].T).reshape(T, H, d)
    v = (h @ t[pre + "v"].T).reshape(T, H, d)
    w = torch.exp(-math.exp(-0.5) * sigma(torch.tanh(h @ t[pre + "w1"].T) @ t[pre + "w2"].T + t[pre + "w0"])).reshape(T, H, d)
    a = sigma(h @ t[pre + "a"].T + t[pre + "a.b"]).reshape(T, H, d)
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    out = torch.zeros(T, H, d, dtype=F64)
    for hd in range(H):
        S = torch.zeros(d, d, dtype=F64)
        for i in range(T):
            S = w[i, hd].unsqueeze(1) * S - torch.outer(a[i, hd] * u[i, hd], u[i, hd] @ S) + torch.outer(k[i, hd], v[i, hd])
            out[i, hd] = S.T @ r[i, hd]
    o = rms_unit(out, eps).reshape(T, H * d) * t[pre + "norm"] * sigma(h @ t[pre + "g"].T)
    return o @ t[pre + "o"].T


def parallel_mixer(h, t, m, pre, eps):
    left = biased_sink_attention(h, t, m["left"], pre + "left.")
    right = matrix_memory(h, t, m["right"], pre + "right.", eps)
    return 0.5 * (rms_unit(left, eps) * t[pre + "left.out"] + rms_unit(right, eps) * t[pre + "right.out"])


def dense_ff(h, t, pre):
    return gelu_erf(h @ t[pre + "up"].T) @ t[pre + "down"].T


def routed_ff(h, t, mlp, pre):
    """Every token runs `top` of the experts, chosen among the experts of the `keep` best groups (a group's score: its two
    largest expert scores added), weighted by their sigmoid scores normalised to `scale`."""
    r, lim = mlp["router"], mlp["expert"]["limit"]
    E, top, groups, keep = r["experts"], r["top"], r["groups"]["count"], r["groups"]["keep"]
    per = E // groups
    s = sigma(h @ t[pre + "router"].T)                            # [T, E]
    out = torch.zeros(h.shape[0], t[pre + "e0.down"].shape[0], dtype=F64)
    for i in range(h.shape[0]):
        gs = [sum(sorted(s[i, g * per:(g + 1) * per].tolist(), reverse=True)[:2]) for g in range(groups)]
        kept = sorted(range(groups), key=lambda g: (-gs[g], g))[:keep]
        allowed = [e for e in range(E) if e // per in kept]
        chosen = sorted(allowed, key=lambda e: (-float(s[i, e]), e))[:top]
        total = sum(float(s[i, e]) for e in chosen) + 1e-20
        for e in chosen:
            g = torch.clamp(t[f"{pre}e{e}.gate"] @ h[i], max=lim)
            u = torch.clamp(t[f"{pre}e{e}.up"] @ h[i], min=-lim, max=lim)
            y = g * sigma(1.702 * g) * (u + 1.0)
            out[i] += float(s[i, e]) / total * r["scale"] * (t[f"{pre}e{e}.down"] @ y)
    return out


def layer_runs(cfg):
    """[(layer, pass number or None, first of its pass)] in the order the layers run: a stretch of layers repeats with the
    same weights, each pass behind its own step vector."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    runs = [(i, None, False) for i in range(loop["start"])]
    for p in range(loop["times"]):
        runs += [(i, p, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None, False) for i in range(loop["stop"], n)]


def forward(cfg, tensors, tokens, keep_layers=False):
    """Logits [T, vocab] (float64) of one sequence; with `keep_layers` also the residual stream after every layer run."""
    t = {k: v.to(F64) for k, v in tensors.items()}
    eps = cfg["norm"]["eps"]
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x = t["embed"][ids] + t["pos"][: len(ids)]
    norm = lambda z, name: dyt(z, t[name], t[name + ".b"], t[name + ".alpha"])
    after = []
    for li, p, first in layer_runs(cfg):
        L, pre = cfg["layers"][li], f"l{li}."
        if first:
            x = x + t["loop.step"][p]
        h = norm(x, pre + "norm1")
        y = general_delta(h, t, L["mixer"], pre + "mix.", eps) if L["type"] == "general_delta" else parallel_mixer(h, t, L["mixer"], pre + "mix.", eps)
        x = x + sigma(h @ t[pre + "rg1"].T + t[pre + "rg1.b"]) * y
        if L.get("mlp") is not None:
            h = norm(x, pre + "norm2")
            y = dense_ff(h, t, pre + "mlp.") if L["mlp"]["kind"] == "dense" else routed_ff(h, t, L["mlp"], pre + "mlp.")
            x = x + sigma(h @ t[pre + "rg2"].T + t[pre + "rg2.b"]) * y
        after.append(x.clone())
    z = norm(x, "final.norm") @ t["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        z = cap * torch.tanh(z / cap)
    return (z, torch.stack(after)) if keep_layers else z
