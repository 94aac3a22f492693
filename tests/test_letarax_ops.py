"""Each mechanism of the Letarax design alone: the package's torch operations (CPU) and HIP kernels (`gpu` marker)
against the one-function-per-mechanism plain model in `letarax_oracle`, on sizes that are not powers of two."""
import math

import numpy as np
import pytest
import torch

import letarax_oracle as O
from distributed_llm_inference_amd.ops import reference as R

gpu = pytest.mark.gpu


def close(a, b, tol):
    a, b = a.double().cpu(), b.double().cpu()
    err = float((a - b).abs().max() / (b.abs().max() + 1e-12))
    assert err < tol, f"relative error {err:.3g} over {tol}"


def rnd(*shape, seed=0, std=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * std


# ---- torch operations (what the CPU executor is made of) -------------------------------------------------------------

def test_torch_offset_norm():
    x, w = rnd(5, 36), rnd(36, seed=1, std=0.3)
    close(R.rmsnorm(x, w, 1e-5, unit_offset=True), O.offset_rmsnorm(x, w, 1e-5), 1e-6)
    close(R.rmsnorm(x, w, 1e-5), O.plain_rmsnorm(x, w, 1e-5), 1e-6)


@pytest.mark.parametrize("window,ctx", [(1, 0), (5, 0), (5, 9), (40, 3), (100, 0)])
def test_torch_window_sink_attention(window, ctx):
    T, H, G, d, dv = 23, 4, 2, 12, 20
    q, k, v = rnd(T, H, d, seed=1), rnd(T, G, d, seed=2), rnd(T, G, dv, seed=3)
    ref = O.sink_window_attention(q, k, v, 0.3, window)
    got = R.attention(q[ctx:], k, v, ctx, 0.3, window=window, sink=True)
    close(got, ref[ctx:], 1e-5)


def test_torch_sink_takes_weight():
    """Scores far below zero: the sink holds the weight and the output vanishes (a plain softmax would return v)."""
    q, k, v = torch.full((1, 1, 4), 10.0), torch.full((1, 1, 4), -10.0), torch.ones(1, 1, 3)
    assert float(R.attention(q, k, v, 0, 1.0, window=4, sink=True).abs().max()) < 1e-6
    assert float(R.attention(q, k, v, 0, 1.0, window=4, sink=False).min()) > 0.99


@pytest.mark.parametrize("K", [1, 2, 4, 7])
def test_torch_short_conv_carried(K):
    x, taps = rnd(19, 10, seed=1), rnd(10, K, seed=2)
    ref = O.causal_short_conv(x, taps)
    prev = torch.zeros(K - 1, 10)
    outs = []
    for lo, hi in [(0, 1), (1, 3), (3, 4), (4, 12), (12, 19)]:
        y, prev = R.short_conv(x[lo:hi], prev, taps)
        outs.append(y)
    close(torch.cat(outs), ref, 1e-6)


def test_torch_delta_rule_carried():
    T, G, H, d, dv = 17, 2, 4, 7, 9
    q, k = O.unit_vectors(rnd(T, G, d, seed=1).double()).float(), O.unit_vectors(rnd(T, G, d, seed=2).double()).float()
    v, beta, decay = rnd(T, H, dv, seed=3), torch.sigmoid(rnd(T, H, seed=4)), torch.sigmoid(rnd(T, H, seed=5) + 2)
    S = torch.zeros(H, d, dv)
    outs = []
    for lo, hi in [(0, 5), (5, 6), (6, 17)]:
        o, S = R.gated_delta_rule(q[lo:hi], k[lo:hi], v[lo:hi], beta[lo:hi], decay[lo:hi], S)
        outs.append(o)
    got = torch.cat(outs)
    for h in range(H):
        ref = O.gated_delta_rule(q[:, h // 2].double(), k[:, h // 2].double(), v[:, h].double(), beta[:, h].double(), decay[:, h].double())
        close(got[:, h], ref, 1e-5)


# ---- HIP kernels -------------------------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def K():
    from distributed_llm_inference_amd import ops
    return ops.load()


def dev(t, dt=torch.float32):
    return t.to(device="cuda", dtype=dt).contiguous()


@gpu
@pytest.mark.parametrize("dt,tol", [(torch.float32, 2e-6), (torch.bfloat16, 1e-5)])
@pytest.mark.parametrize("M,N,Kd", [(1, 4, 36), (23, 48, 32), (70, 100, 52), (5, 322, 200), (129, 65, 7), (64, 64, 64), (300, 36, 136)])
def test_gemm_any(K, dt, tol, M, N, Kd):
    x, w, b = dev(rnd(M, Kd, seed=1), dt), dev(rnd(N, Kd, seed=2), dt), dev(rnd(N, seed=3))
    out = torch.zeros(M, N, device="cuda")
    K.gemm_any(out, x, w, b, 0)
    close(out, O.linear(x.cpu(), w.cpu(), b.cpu()), tol)
    if dt == torch.bfloat16:           # output in the operand type
        out16 = torch.zeros(M, N, device="cuda", dtype=dt)
        K.gemm_any(out16, x, w, None, 0)
        close(out16, O.linear(x.cpu(), w.cpu()), 1e-2)


@gpu
@pytest.mark.parametrize("dt,tol", [(torch.float32, 5e-6), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("M,F,Kd", [(9, 16, 36), (70, 48, 72), (3, 176, 200)])
def test_gemm_any_gated(K, dt, tol, M, F, Kd):
    from distributed_llm_inference_amd.ops.packing import interleave_gate_up
    x, wg, wu = dev(rnd(M, Kd, seed=1), dt), dev(rnd(F, Kd, seed=2, std=Kd ** -0.5), dt), dev(rnd(F, Kd, seed=3, std=Kd ** -0.5), dt)
    bg, bu = dev(rnd(F, seed=4)), dev(rnd(F, seed=5))
    w = interleave_gate_up(wg, wu).contiguous()
    b = interleave_gate_up(bg.unsqueeze(1), bu.unsqueeze(1)).reshape(-1).contiguous()
    out = torch.zeros(M, F, device="cuda", dtype=dt)
    K.gemm_any(out, x, w, b, 1)
    ref = O.gelu_tanh(O.linear(x.cpu(), wg.cpu(), bg.cpu())) * O.linear(x.cpu(), wu.cpu(), bu.cpu())
    close(out, ref, tol)


@gpu
@pytest.mark.parametrize("H", [36, 200, 1000])
def test_norm32_forms(K, H):
    T, eps = 7, 1e-5
    x, y = rnd(T, H, seed=1, std=3.0), rnd(T, H, seed=2, std=0.7)
    wb, wn = rnd(H, seed=3, std=0.3), rnd(H, seed=4, std=0.3)
    xd, out = dev(x), torch.zeros(T, H, device="cuda")
    K.norm32(out, xd, None, None, dev(wn), None, eps, 1.0)
    close(out, O.offset_rmsnorm(x, wn, eps), 2e-6)
    K.norm32(out, xd, dev(y), dev(wb), dev(wn), None, eps, 1.0)            # post-norm, add, next pre-norm
    x2 = x.double() + O.offset_rmsnorm(y, wb, eps)
    close(xd, x2, 2e-6)
    close(out, O.offset_rmsnorm(x2, wn, eps), 2e-6)
    xd2 = dev(x)
    K.norm32(None, xd2, dev(y), dev(wb), None, None, eps, 1.0)
    close(xd2, x2, 2e-6)
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device="cuda")
    out16 = torch.zeros(3, H, device="cuda", dtype=torch.bfloat16)
    K.norm32(out16, dev(x), None, None, dev(wn), rows, eps, 0.0)               # gathered rows, plain weight, bf16 out
    close(out16, O.plain_rmsnorm(x[[5, 0, 5]], wn, eps), 1e-2)


def paged(K, q, k, v, scale, window, sink, dt, chunks, blocks_perm=None):
    """Runs kv_store + window_attention over one sequence given in `chunks`, blocks handed out in a scrambled order."""
    T, H, d = q.shape
    G, dv = k.shape[1], v.shape[2]
    nb = (T + 31) // 32
    order = list(range(nb + 3))[::-1] if blocks_perm is None else blocks_perm
    table = torch.full((3, nb), -1, dtype=torch.int32)
    table[1, :nb] = torch.tensor(order[:nb], dtype=torch.int32)
    table = table.cuda()
    kc = torch.zeros(nb + 3, G, 32, d, device="cuda", dtype=dt)
    vc = torch.zeros(nb + 3, G, 32, dv, device="cuda", dtype=dt)
    outs, lo = [], 0
    for n in chunks:
        qkv = dev(torch.cat([q[lo:lo + n].reshape(n, -1), k[lo:lo + n].reshape(n, -1), v[lo:lo + n].reshape(n, -1)], dim=1))
        pos = torch.arange(lo, lo + n, dtype=torch.int32, device="cuda")
        seq = torch.ones(n, dtype=torch.int32, device="cuda")
        K.kv_store(qkv, None, None, 0, kc, vc, pos, seq, table, G, d, dv, H * d)
        out = torch.zeros(n, H * dv, device="cuda", dtype=dt)
        K.window_attention(out, qkv, kc, vc, pos, seq, table, H, G, d, dv, scale, window, sink)
        outs.append(out.float().cpu().reshape(n, H, dv))
        lo += n
    return torch.cat(outs)


@gpu
@pytest.mark.parametrize("dt,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("H,G,d,dv,window", [(4, 2, 12, 20, 5), (3, 3, 64, 64, 96), (2, 1, 7, 130, 1), (8, 2, 128, 32, 70), (1, 1, 36, 36, 1000)])
def test_window_attention_kernel(K, dt, tol, H, G, d, dv, window):
    T = 150
    q, k, v = rnd(T, H, d, seed=1), rnd(T, G, d, seed=2), rnd(T, G, dv, seed=3)
    if dt == torch.bfloat16:
        k, v = k.bfloat16().float(), v.bfloat16().float()
    ref = O.sink_window_attention(q, k, v, d ** -0.5, window)
    close(paged(K, q, k, v, d ** -0.5, window, True, dt, [150]), ref, tol)
    close(paged(K, q, k, v, d ** -0.5, window, True, dt, [31, 2, 1, 1, 64, 33, 18]), ref, tol)


@gpu
def test_window_attention_edge_and_sink(K):
    """One key with a large score right at the window's far edge (seen) and one step beyond (not seen), 200 tokens
    back across block edges; and scores so low that only the sink has weight."""
    T, d, window = 260, 8, 200
    for back, seen in [(window - 1, True), (window, False)]:
        q, k, v = torch.zeros(T, 1, d), torch.zeros(T, 1, d), rnd(T, 1, 4, seed=1)
        ask, beacon = 255, 255 - back
        q[ask, 0, 0], k[beacon, 0, 0] = 6.0, 6.0
        out = paged(K, q, k, v, 1.0, window, True, torch.float32, [250, 3, 1, 1, 1, 4])
        close(out, O.sink_window_attention(q, k, v, 1.0, window), 1e-5)
        near_beacon = float((out[ask, 0] - v[beacon, 0]).abs().max()) < 1e-3
        assert near_beacon == seen
    q, k, v = torch.full((40, 1, d), 3.0), torch.full((40, 1, d), -3.0), torch.ones(40, 1, 4)
    assert float(paged(K, q, k, v, 1.0, 16, True, torch.float32, [40]).abs().max()) < 1e-6
    assert float(paged(K, q, k, v, 1.0, 16, False, torch.float32, [40]).min()) > 0.999


@gpu
def test_value_mixing_in_store(K):
    T, G, d, dv, H = 5, 2, 8, 12, 2
    qkv1, qkv2 = dev(rnd(T, H * d + G * d + G * dv, seed=1)), dev(rnd(T, H * d + G * d + G * dv, seed=2))
    table = torch.tensor([[0]], dtype=torch.int32, device="cuda")
    pos, seq = torch.arange(T, dtype=torch.int32, device="cuda"), torch.zeros(T, dtype=torch.int32, device="cuda")
    kc, vc = torch.zeros(1, G, 32, d, device="cuda"), torch.zeros(1, G, 32, dv, device="cuda")
    vf, lam = torch.zeros(T * G * dv, device="cuda"), torch.tensor([0.3], device="cuda")
    K.kv_store(qkv1, vf, None, 1, kc, vc, pos, seq, table, G, d, dv, H * d)
    v1 = qkv1[:, H * d + G * d:].cpu()
    close(vc[0, :, :T].permute(1, 0, 2).reshape(T, -1), v1, 1e-7)
    K.kv_store(qkv2, vf, lam, 2, kc, vc, pos, seq, table, G, d, dv, H * d)
    close(vc[0, :, :T].permute(1, 0, 2).reshape(T, -1), O.mix_values(qkv2[:, H * d + G * d:].cpu(), v1, float(lam)), 1e-6)
    close(kc[0, :, :T].permute(1, 0, 2).reshape(T, -1), qkv2[:, H * d:H * d + G * d].cpu(), 1e-7)


def ragged(lens, ctxs, slots):
    qs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    t = lambda a: torch.tensor(np.asarray(a, dtype=np.int32), device="cuda")
    return t(qs), t(ctxs), t(slots)


@gpu
@pytest.mark.parametrize("Kt", [1, 2, 4, 9])
def test_short_conv_kernel(K, Kt):
    C, T = 70, 45
    x, taps = rnd(T, C + 6, seed=1), rnd(C, Kt, seed=2)
    ref = O.silu(O.causal_short_conv(x[:, :C], taps))
    carry = torch.full((3, max(Kt - 1, 1), C), 7.0, device="cuda")          # stale contents: a first step must not read them
    outs, lo = [], 0
    for n in [1, 1, 2, 20, 3, 18]:
        z = dev(x[lo:lo + n])
        y = torch.zeros(n, C, device="cuda")
        qs, ctx, sl = ragged([n], [lo], [2])
        K.short_conv(y, z, carry, dev(taps), qs, ctx, sl, n)
        outs.append(y.cpu())
        lo += n
    close(torch.cat(outs), ref, 1e-5)


@gpu
@pytest.mark.parametrize("G,H,d,dv", [(1, 1, 7, 9), (2, 4, 32, 32), (2, 6, 16, 48), (1, 2, 160, 72), (1, 1, 128, 128), (3, 3, 64, 20)])
def test_delta_rule_kernel(K, G, H, d, dv):
    T, C = 40, 2 * G * d + H * dv
    y = torch.cat([O.unit_vectors(rnd(T, G, d, seed=1).double()).float().reshape(T, -1) * d ** -0.5,
                   O.unit_vectors(rnd(T, G, d, seed=2).double()).float().reshape(T, -1), rnd(T, H * dv, seed=3)], dim=1)
    z = rnd(T, 5 + 2 * H, seed=4)                                            # [pad | beta logits | decay logits]
    A_log, dtb = rnd(H, seed=5, std=0.5), rnd(H, seed=6, std=0.5)
    state = torch.full((4, H, d, dv), 3.0, device="cuda")                    # stale
    outs, lo = [], 0
    for n in [1, 2, 17, 1, 19]:
        o = torch.zeros(n, H * dv, device="cuda")
        qs, ctx, sl = ragged([n], [lo], [3])
        K.delta_rule(o, dev(y[lo:lo + n]), dev(z[lo:lo + n]), state, dev(A_log), dev(dtb), qs, ctx, sl, G, H, d, dv, 5, 5 + H, n)
        outs.append(o.cpu())
        lo += n
    got = torch.cat(outs).reshape(T, H, dv)
    beta = torch.sigmoid(z[:, 5:5 + H].double())
    a = z[:, 5 + H:].double() + dtb.double()
    decay = torch.exp(-torch.exp(A_log.double()) * torch.log1p(torch.exp(a)))
    yq, yk, yv = y[:, :G * d].reshape(T, G, d), y[:, G * d:2 * G * d].reshape(T, G, d), y[:, 2 * G * d:].reshape(T, H, dv)
    for h in range(H):
        g = h // (H // G)
        ref = O.gated_delta_rule(yq[:, g].double(), yk[:, g].double(), yv[:, h].double(), beta[:, h], decay[:, h])
        close(got[:, h], ref, 2e-5)


@gpu
def test_unit_heads_and_gated_headnorm(K):
    T, heads, d = 6, 5, 13
    x = rnd(T, heads * d + 3, seed=1)
    xd = dev(x)
    K.unit_heads(xd[:, :heads * d], heads, d, 2, 0.25, 1e-6)
    ref = O.unit_vectors(x[:, :heads * d].reshape(T, heads, d).double())
    ref[:, :2] *= 0.25
    close(xd[:, :heads * d], ref.reshape(T, -1), 1e-6)
    close(xd[:, heads * d:], x[:, heads * d:], 1e-7)
    dv = 9
    o, gate, w = rnd(T, heads * dv, seed=2), rnd(T, heads * dv + 4, seed=3), rnd(dv, seed=4)
    out = torch.zeros(T, heads * dv, device="cuda")
    K.gated_headnorm(out, dev(o), dev(gate)[:, 2:2 + heads * dv], dev(w), heads, dv, 1e-5)
    ref = O.plain_rmsnorm(o.reshape(T, heads, dv), w, 1e-5) * O.silu(gate[:, 2:2 + heads * dv].double()).reshape(T, heads, dv)
    close(out, ref.reshape(T, -1), 1e-5)


def fragment_paged(K, q, k, v, scale, window, sink, chunks):
    """The MFMA attention path: bf16 fused q|k|v rows, fragment-ordered cache written without rotation, windowed kernel."""
    T, H, D = q.shape
    G = k.shape[1]
    nb = (T + 31) // 32
    table = torch.full((2, nb), -1, dtype=torch.int32)
    table[1] = torch.arange(nb - 1, -1, -1, dtype=torch.int32) + 2
    table = table.cuda()
    kv = torch.zeros(nb + 2, G, 2, 32 * D, device="cuda", dtype=torch.bfloat16)
    zero = torch.zeros(1, D // 2, device="cuda")
    outs, lo = [], 0
    for n in chunks:
        qkv = dev(torch.cat([q[lo:lo + n].reshape(n, -1), k[lo:lo + n].reshape(n, -1), v[lo:lo + n].reshape(n, -1)], dim=1), torch.bfloat16)
        pos = torch.arange(lo, lo + n, dtype=torch.int32, device="cuda")
        seq = torch.ones(n, dtype=torch.int32, device="cuda")
        K.rope_kvwrite(qkv, None, 1, None, kv, zero, zero, pos, seq, table, H, G, D, False)
        out = torch.zeros(n, H * D, device="cuda", dtype=torch.bfloat16)
        qs, ctx, sl = ragged([n], [lo], [1])
        K.paged_attention_window(out, qkv, kv, qs, ctx, table, sl, None, n, H, G, D, scale, 1, window, sink)
        outs.append(out.float().cpu().reshape(n, H, D))
        lo += n
    return torch.cat(outs)


@gpu
@pytest.mark.parametrize("H,G,D,window", [(4, 2, 64, 5), (4, 4, 64, 96), (8, 1, 128, 70), (3, 1, 128, 1), (2, 1, 64, 1000), (4, 2, 128, 33)])
def test_windowed_mfma_attention(K, H, G, D, window):
    T = 330
    bf = lambda t: t.bfloat16().float()
    q, k, v = bf(rnd(T, H, D, seed=1)), bf(rnd(T, G, D, seed=2)), bf(rnd(T, G, D, seed=3))
    ref = O.sink_window_attention(q, k, v, D ** -0.5, window)
    close(fragment_paged(K, q, k, v, D ** -0.5, window, True, [330]), ref, 2e-2)                       # prefill-shaped kernel
    close(fragment_paged(K, q, k, v, D ** -0.5, window, True, [200, 2, 1, 1, 1, 64, 33, 28]), ref, 2e-2)   # portions and single tokens


@gpu
def test_windowed_mfma_attention_edge_and_sink(K):
    T, D, window = 300, 64, 200
    for back, seen in [(window - 1, True), (window, False)]:
        for chunks in ([300], [290, 3, 1, 1, 1, 4]):
            q, k, v = torch.zeros(T, 1, D), torch.zeros(T, 1, D), rnd(T, 1, D, seed=1).bfloat16().float()
            ask, beacon = 294, 294 - back
            q[ask, 0, 0], k[beacon, 0, 0] = 6.0, 6.0
            out = fragment_paged(K, q, k, v, 1.0, window, True, chunks)
            close(out, O.sink_window_attention(q, k, v, 1.0, window), 2e-2)
            assert (float((out[ask, 0] - v[beacon, 0]).abs().max()) < 5e-2) == seen
    q, k, v = torch.full((40, 1, D), 1.0), torch.full((40, 1, D), -1.0), torch.ones(40, 1, D)
    assert float(fragment_paged(K, q, k, v, 1.0, 16, True, [40]).abs().max()) < 1e-6
    assert float(fragment_paged(K, q, k, v, 1.0, 16, False, [40]).min()) > 0.99


@gpu
def test_value_mix_kernel(K):
    T, cols, off = 5, 24, 40
    a, b = rnd(T, off + cols, seed=1).bfloat16(), rnd(T, off + cols, seed=2).bfloat16()
    vf, lam = torch.zeros(T * cols, device="cuda"), torch.tensor([0.3], device="cuda")
    ad, bd = a.cuda(), b.cuda()
    K.value_mix(ad, vf, None, 1, off, cols)
    close(vf.view(T, cols), a[:, off:].float(), 1e-7)
    K.value_mix(bd, vf, lam, 2, off, cols)
    close(bd[:, off:], O.mix_values(b[:, off:].float(), a[:, off:].float(), float(lam)), 1e-2)
    close(bd[:, :off], b[:, :off].float(), 1e-7)
