"""MI355X executor for hybrid stacks: models whose layers are listed one by one (`ModelSpec.layer_specs`),
each with its own token mixer — windowed softmax attention with a sink over the paged cache, or a gated
delta-rule recurrence over a per-sequence state — a norm on both sides of every sublayer, and a residual
stream in fp32.

It is a `GpuStage`: the same step descriptors, metadata upload, block table, slots, scoring / sampling head,
fixed-shape decode states and hipGraph capture. What differs is what a layer runs:

    h (fp32) -> norm -> [ qkv GEMM -> value mixing + cache write -> windowed attention
                        | input GEMM -> short conv + silu -> unit q, k -> delta rule -> per-head norm * gate ]
             -> o GEMM -> post-norm + residual add + the next pre-norm (one kernel)
             -> [ gate/up GEMM with the gelu * up epilogue -> down GEMM -> post-norm + add + next pre-norm ]

and what a sequence owns: besides its cache blocks (attention layers), one slot of every recurrent layer's
state arrays, indexed by the step descriptor's slot number (the row of the block table). A sequence's first
tokens (context length 0) start from a zero state inside the kernels, so a slot is reused without clearing.

Matrix products take bf16 operands (or fp32: `dtype="fp32"`, everything in true 32-bit) and accumulate in
fp32; norms, scores, softmax, value mixing, gates, decays and states are fp32 in both modes.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from ..ops import packing
from .partition import StagePlan
from .spec import LayerSpec, ModelSpec
from .stage_gpu import BLOCK, GpuStage
from .weights import StageWeights


@dataclass
class _HybridWork:
    """Activation workspaces of one step in flight (the eager path owns one, every decode micro-batch its own)."""
    h: torch.Tensor              # fp32 [T, H]   residual stream
    xn: torch.Tensor             # act  [T, H]   normalised input of the next GEMM
    z: torch.Tensor              # fp32 flat     output of a mixer's input projection (q|k|v, or q|k|v|gate|beta|decay)
    y: torch.Tensor              # fp32 flat     convolved q|k|v of a recurrent mixer
    o: torch.Tensor              # fp32 flat     raw read-out of a recurrent mixer
    mixed: torch.Tensor          # act  flat     mixer output ahead of the o projection
    yo: torch.Tensor             # fp32 [T, H]   sublayer output ahead of its post-norm
    act: torch.Tensor            # act  flat     gated feed-forward activation
    vfirst: torch.Tensor         # fp32 flat     values of the first value-mixing layer, for this step's tokens
    gu: torch.Tensor             # bf16 flat     gate | up pre-activations where the packed-weight GEMM produced them
    qkv16: torch.Tensor          # bf16 flat     fused q | k | v of the attention layers that run on the MFMA attention kernels
    ws: torch.Tensor             # fp32          split-K workspace of the packed-weight GEMMs (its last 4096 words: arrival counters)
    head_x: Optional[torch.Tensor]
    logits: Optional[torch.Tensor]
    cmax: Optional[torch.Tensor] = None
    guided: bool = False         # (the any-shape head GEMM leaves no chunk maxima: the sampler reads whole rows)


class HybridGpuStage(GpuStage):
    backend = "hip"

    def __init__(self, spec: ModelSpec, plan: StagePlan, weights: StageWeights, *, device="cuda", max_slots: int = 256,
                 max_seq_len: int = 2048, num_blocks: Optional[int] = None, max_tokens: int = 2048, max_batch: int = 64,
                 use_graphs: bool = True, kv_mem_fraction: float = 0.85, dtype: str = "bf16", decode_states: int = 1,
                 defer_kv: bool = False, graph_sizes: Optional[List[int]] = None):
        if not torch.cuda.is_available():
            raise RuntimeError("HybridGpuStage needs a GPU; use RefStage on CPU")
        if not spec.is_hybrid:
            raise ValueError("HybridGpuStage runs models described layer by layer")
        if not (plan.has_embed and plan.has_head):
            raise ValueError("a hybrid stack runs on one stage (its value mixing spans layers)")
        if dtype not in ("bf16", "fp32"):
            raise ValueError("hybrid stacks run in bf16 or fp32")
        self.kv8, self.wmode, self.w8 = False, dtype, False
        self.act_dtype = torch.float32 if dtype == "fp32" else torch.bfloat16
        self._init_limits(spec, plan, device, max_slots, max_seq_len, max_tokens, max_batch, use_graphs, graph_sizes)
        self.specs: List[LayerSpec] = [spec.layer_specs[i] for i in plan.layers]
        for i, ls in zip(plan.layers, self.specs):
            if max(ls.dim, ls.vdim) > 512:
                raise ValueError(f"layer {i}: head sizes up to 512 are supported")
            if ls.kind == "delta" and not 1 <= ls.conv <= 16:
                raise ValueError(f"layer {i}: 1 to 16 convolution taps are supported")
        mixers = [ls for ls in self.specs if ls.kind == "attention" and ls.v_mix]
        if len({(ls.kv_heads, ls.vdim) for ls in mixers}) > 1:
            raise ValueError("value mixing needs the same key / value heads and value size in every layer that mixes")
        dev, at = self.device, self.act_dtype
        f32 = lambda t: t.to(device=dev, dtype=torch.float32).contiguous()
        mat = lambda t: t.to(device=dev, dtype=at).contiguous()
        # Projections whose inner size is a multiple of 128 run on the library's packed-weight GEMMs (the weight-streaming
        # kernel up to 256 rows, the 256 x 256 tile kernel above), bf16 only; every other shape, and the fp32 mode, runs on
        # the any-shape kernel. DLIA_HYBRID_PACKED=0 keeps everything on the any-shape kernel (A/B).
        self._packed = dtype == "bf16" and os.environ.get("DLIA_HYBRID_PACKED", "1") != "0"
        self.decode_rows = 256
        self._shapes = []                        # (N, K, has_bias) of every packed GEMM, for the workspace
        # Attention layers whose keys and values have one size, 64 or 128, with up to 16 query heads per key / value head run
        # on the library's MFMA attention kernels (fragment-ordered cache, the windowed / sink instantiations), bf16 only;
        # other sizes, and the fp32 mode, on the any-size kernel. DLIA_HYBRID_MFMA_ATTN=0 keeps all on the any-size kernel (A/B).
        mfma_ok = dtype == "bf16" and os.environ.get("DLIA_HYBRID_MFMA_ATTN", "1") != "0"
        self.mfma_attn = [mfma_ok and ls.kind == "attention" and ls.dim == ls.vdim and ls.dim in (64, 128) and ls.group <= 16
                          for ls in self.specs]
        self._no_rope = {D: torch.zeros(1, D // 2, device=self.device) for D in (64, 128)}
        self.embed = mat(weights.embed)
        self.lm_head = self.embed
        self.lm_head_p = None
        self.pos_embed = None
        self.final_norm_w = f32(weights.final_norm_w)
        self.vocab_pad = packing.padded_n(spec.vocab_size)
        self.layers: List[Dict[str, torch.Tensor]] = []
        for i, ls in enumerate(self.specs):
            l = weights.layers[i]
            p: Dict[str, torch.Tensor] = {"ln1_w": f32(l["ln1_w"]), "ln1b_w": f32(l["ln1b_w"])}
            self._matrix(p, "w_o", mat(l["w_o"]), None)
            if ls.kind == "attention":
                self._matrix(p, "w_qkv", mat(l["w_qkv"]), f32(l["b_qkv"]))
                p["vmix"] = f32(l["vmix"]).reshape(1)
            else:
                self._matrix(p, "w_in", mat(l["w_in"]), None)
                p["conv_w"] = f32(l["conv_w"])
                p["A_log"], p["dt_bias"], p["o_norm_w"] = f32(l["A_log"]), f32(l["dt_bias"]), f32(l["o_norm_w"])
            if ls.ff:
                # gate and up rows interleaved in 16-row tiles, so that one wave holds both for the same output
                # columns; a width that is no multiple of 16 is padded with zero rows (their activations are zero
                # and meet zero columns of the down projection)
                pad = (-ls.ff) % 16
                padr = lambda t: torch.cat([t, t.new_zeros(pad, *t.shape[1:])]) if pad else t
                p["ln2_w"], p["ln2b_w"] = f32(l["ln2_w"]), f32(l["ln2b_w"])
                if self._packed and spec.hidden_size % 128 == 0 and ls.ff % 8 == 0:
                    # gate rows, then up rows, through the packed-weight GEMM; the gate is applied by a kernel of its own
                    self._matrix(p, "w_gu", torch.cat([mat(l["w_gate"]), mat(l["w_up"])]), torch.cat([f32(l["b_gate"]), f32(l["b_up"])]))
                    p["ff_cols"] = ls.ff
                else:
                    p["w_gu"] = packing.interleave_gate_up(padr(mat(l["w_gate"])), padr(mat(l["w_up"]))).contiguous()
                    p["b_gu"] = packing.interleave_gate_up(padr(f32(l["b_gate"])).unsqueeze(1), padr(f32(l["b_up"])).unsqueeze(1)).reshape(-1).contiguous()
                    p["ff_cols"] = ls.ff + pad
                wd = mat(l["w_down"])
                if "w_gu_p" not in p and pad:
                    wd = torch.cat([wd, wd.new_zeros(wd.shape[0], pad)], dim=1).contiguous()
                self._matrix(p, "w_down", wd, f32(l["b_down"]))
            self.layers.append(p)
            weights.layers[i] = {}
        if self._packed and spec.hidden_size % 128 == 0:
            self.lm_head_p = packing.pack_weight(self.embed)
            self._shapes.append((self.vocab_pad, spec.hidden_size, False))
        self._ws_floats = self._packed_ws_floats()
        self.keep_layer_outputs = False          # debugging aid: eager steps append the residual stream after every layer
        self.layer_outputs: List[torch.Tensor] = []
        self.wk0 = self._new_work(self.max_tokens)
        self._init_step_state(kv_mem_fraction, decode_states)
        # recurrent state, one slot per row of the block table (the null slot included: padding rows land there)
        self.rec: List[Optional[tuple]] = []
        for ls in self.specs:
            if ls.kind == "delta":
                C = 2 * ls.kv_heads * ls.dim + ls.heads * ls.vdim
                self.rec.append((torch.zeros(max_slots + 1, max(ls.conv - 1, 1), C, device=dev),
                                 torch.zeros(max_slots + 1, ls.heads, ls.dim, ls.vdim, device=dev)))
            else:
                self.rec.append(None)
        if not defer_kv:
            self.allocate_kv(num_blocks if num_blocks is not None else self.kv_budget_blocks())

    # ---- matrices: packed for the library's tuned GEMMs where the shape allows, row-major otherwise --------------
    def _matrix(self, p: Dict[str, torch.Tensor], name: str, w: torch.Tensor, bias: Optional[torch.Tensor]):
        """Stores W [N, K] (+ fp32 bias) under `name`: as the packed image `name_p` (N padded to a multiple of 4 with
        zero rows: `name_n`; bias in bf16, which a bf16 checkpoint's bias is anyway) when K is a multiple of 128, as the
        row-major matrix for the any-shape kernel otherwise."""
        N, K = w.shape
        if self._packed and K % 128 == 0:
            n4 = (N + 3) // 4 * 4
            if n4 != N:
                w = torch.cat([w, w.new_zeros(n4 - N, K)])
                bias = torch.cat([bias, bias.new_zeros(n4 - N)]) if bias is not None else None
            p[name + "_p"], p[name + "_n"] = packing.pack_weight(w.contiguous()), n4
            if bias is not None:
                p[name + "_b"] = bias.to(torch.bfloat16).contiguous()
            self._shapes.append((n4, K, bias is not None))
        else:
            p[name] = w
            if bias is not None:
                p["b_" + name[2:]] = bias

    def _cols(self, p, name: str) -> int:
        """Output columns of the projection stored under `name` (the padded count when it is packed)."""
        return p[name + "_n"] if name + "_p" in p else p[name].shape[0]

    def _mm(self, wk, out: torch.Tensor, x: torch.Tensor, p, name: str):
        """out = x . W^T (+ bias) for the projection stored under `name`."""
        wp = p.get(name + "_p")
        if wp is None:
            self.K.gemm_any(out, x, p[name], p.get("b_" + name[2:]), 0)
            return
        b = p.get(name + "_b")
        # more than 256 rows: the tile kernel, spread over the whole chip when a shape has few tiles
        self.K.gemm(out, x, wp, b, None, wk.ws, p[name + "_n"], 1 if b is not None else 0, 256 if x.shape[0] > self.decode_rows else 0, 0)

    def _packed_ws_floats(self) -> int:
        need = 1
        for (n_, k_, hb) in self._shapes:
            for m_ in range(1, self.decode_rows + 1):
                sk = int(self.K.gemm_config(m_, n_, k_, 1 if hb else 0, True)[1])
                if sk > 1:
                    need = max(need, sk * m_ * n_)
        return need

    # ---- workspaces ---------------------------------------------------------------------------------------
    def _new_work(self, rows: int) -> _HybridWork:
        s, dev, at = self.spec, self.device, self.act_dtype
        z = lambda n, dt=torch.float32: torch.zeros(max(int(n), 1), device=dev, dtype=dt)
        B = min(rows, self.max_batch)
        H = s.hidden_size
        zc = yc = oc = mc = ac = vc = 1
        for ls in self.specs:
            qn, kn, vn, on = ls.qk_heads * ls.dim, ls.kv_heads * ls.dim, ls.v_heads * ls.vdim, ls.heads * ls.vdim
            mc, ac = max(mc, on), max(ac, (ls.ff + 15) // 16 * 16)
            if ls.kind == "attention":
                zc = max(zc, qn + kn + vn + 3)
                vc = max(vc, vn if ls.v_mix else 1)
            else:
                zc, yc, oc = max(zc, qn + kn + vn + on + 2 * ls.heads + 3), max(yc, qn + kn + vn), max(oc, on)
        ws_floats = self._ws_floats
        if self._packed and rows > self.decode_rows:
            for m_ in {rows, min(rows, 512), min(rows, 1024)}:
                if m_ > self.decode_rows:
                    ws_floats = max([ws_floats] + [int(self.K.gemm_ws_floats(m_, n_, k_)) for n_, k_, _ in self._shapes])
        guc = max([2 * ls.ff for ls in self.specs if ls.ff] + [1]) if self._packed else 1
        qc = max([(ls.heads + 2 * ls.kv_heads) * ls.dim for ls, fast in zip(self.specs, self.mfma_attn) if fast] + [1])
        return _HybridWork(
            h=torch.zeros(rows, H, device=dev), xn=torch.zeros(rows, H, device=dev, dtype=at), z=z(rows * zc), y=z(rows * yc),
            o=z(rows * oc), mixed=z(rows * mc, at), yo=torch.zeros(rows, H, device=dev), act=z(rows * ac, at),
            vfirst=z(rows * vc), gu=z(rows * guc, torch.bfloat16), qkv16=z(rows * qc, torch.bfloat16), ws=z(ws_floats + 4096), head_x=torch.zeros(B, H, device=dev, dtype=at),
            logits=torch.zeros(B, self.vocab_pad, device=dev))

    # ---- cache and state sizing -------------------------------------------------------------------------
    def kv_block_bytes(self) -> int:
        e = 4 if self.act_dtype == torch.float32 else 2
        return max(1, sum(ls.kv_heads * BLOCK * (ls.dim + ls.vdim) * e for ls in self.specs if ls.kind == "attention"))

    def _decode_state_bytes(self) -> int:
        n = 0
        for B in self.graph_sizes:
            w = self.wk0
            per_row = sum(t.numel() * t.element_size() for t in (w.h, w.xn, w.z, w.y, w.o, w.mixed, w.yo, w.act, w.vfirst)) // self.max_tokens
            n += B * (per_row + 4 * self.vocab_pad + 4 * self.spec.hidden_size)
        return n

    def allocate_kv(self, num_blocks: int):
        dev, at = self.device, self.act_dtype
        self.num_blocks = int(num_blocks)
        # zero-filled: a row that was never written must hold finite values
        # (a layer on the MFMA attention kernels keeps K and V slabs of a block side by side, in fragment order)
        self.kv = [None if ls.kind != "attention" else
                   torch.zeros(self.num_blocks, ls.kv_heads, 2, BLOCK * ls.dim, device=dev, dtype=at) if fast else
                   (torch.zeros(self.num_blocks, ls.kv_heads, BLOCK, ls.dim, device=dev, dtype=at),
                    torch.zeros(self.num_blocks, ls.kv_heads, BLOCK, ls.vdim, device=dev, dtype=at))
                   for ls, fast in zip(self.specs, self.mfma_attn)]

    def _pick_splits(self, B: int, max_ctx: int) -> int:
        return 1

    def _capture(self, st):
        """Capturing a step runs it once for real beforehand (first-use initialisation must not happen under
        capture). A cache write of that run is harmless: the replay writes the same row again. A recurrent state is
        not idempotent: the same token applied twice is a different state. So the rows are parked on the null slot
        for the run and the capture (kernels read the slots from the static buffer at replay time, not now)."""
        saved = st.slots.clone()
        st.slots.fill_(self.null_slot)
        try:
            super()._capture(st)
        finally:
            st.slots.copy_(saved)

    # ---- the layer stack ----------------------------------------------------------------------------------
    def _embed_rows(self, wk, T: int, ids, pos):
        self.K.embed32(wk.h[:T], ids, self.embed)

    def _layers(self, wk: _HybridWork, T: int, B: int, tok_pos, tok_seq, q_start, ctx, slots, max_q: int, splits: int,
                alone: bool = False, lead_decode: int = 0):
        K, eps = self.K, self.spec.norm_eps
        h, xn, yo = wk.h[:T], wk.xn[:T], wk.yo[:T]
        view = lambda buf, cols: buf[:T * cols].view(T, cols)
        keep = self.keep_layer_outputs and not torch.cuda.is_current_stream_capturing()
        if keep:
            self.layer_outputs = []
        K.norm32(xn, h, None, None, self.layers[0]["ln1_w"], None, eps, 1.0)
        seen_mix = False
        n_layers = len(self.layers)
        for li, (ls, p) in enumerate(zip(self.specs, self.layers)):
            Hh, G, d, dv = ls.heads, ls.kv_heads, ls.dim, ls.vdim
            mixed = view(wk.mixed, Hh * dv)
            if ls.kind == "attention" and self.mfma_attn[li]:
                qkv = view(wk.qkv16, (Hh + 2 * G) * d)
                self._mm(wk, qkv, xn, p, "w_qkv")
                mix = 0 if not ls.v_mix else (2 if seen_mix else 1)
                seen_mix = seen_mix or ls.v_mix
                if mix:
                    K.value_mix(qkv, wk.vfirst, p["vmix"] if mix == 2 else None, mix, (Hh + G) * d, G * d)
                K.rope_kvwrite(qkv, None, 1, None, self.kv[li], self._no_rope[d], self._no_rope[d], tok_pos, tok_seq,
                               self.block_table, Hh, G, d, False)
                win = ls.window or 0
                if 0 < lead_decode < B and max_q > 1:
                    # single tokens riding in front of prompt portions: the decode-shaped kernel for them, the prefill-shaped for the rest
                    n = lead_decode
                    K.paged_attention_window(mixed, qkv, self.kv[li], q_start[:n + 1], ctx[:n], self.block_table, slots[:n], None,
                                             1, Hh, G, d, ls.scale, 1, win, ls.sink)
                    K.paged_attention_window(mixed, qkv, self.kv[li], q_start[n:], ctx[n:], self.block_table, slots[n:], None,
                                             max_q, Hh, G, d, ls.scale, 1, win, ls.sink)
                else:
                    K.paged_attention_window(mixed, qkv, self.kv[li], q_start, ctx, self.block_table, slots, None, max_q, Hh, G, d,
                                             ls.scale, 1, win, ls.sink)
            elif ls.kind == "attention":
                z = view(wk.z, self._cols(p, "w_qkv"))
                self._mm(wk, z, xn, p, "w_qkv")
                mix = 0 if not ls.v_mix else (2 if seen_mix else 1)
                seen_mix = seen_mix or ls.v_mix
                kc, vc = self.kv[li]
                z = z[:, :(Hh + G) * d + G * dv]
                K.kv_store(z, wk.vfirst if mix else None, p["vmix"] if mix == 2 else None, mix, kc, vc, tok_pos, tok_seq,
                           self.block_table, G, d, dv, Hh * d)
                K.window_attention(mixed, z, kc, vc, tok_pos, tok_seq, self.block_table, Hh, G, d, dv, ls.scale,
                                   ls.window or 0, ls.sink)
            else:
                qn, vn = G * d, Hh * dv
                C = 2 * qn + vn
                z = view(wk.z, self._cols(p, "w_in"))
                y, o = view(wk.y, C), view(wk.o, vn)
                carry, state = self.rec[li]
                self._mm(wk, z, xn, p, "w_in")
                K.short_conv(y, z, carry, p["conv_w"], q_start, ctx, slots, max_q)
                K.unit_heads(y[:, :2 * qn], 2 * G, d, G, d ** -0.5, 1e-6)
                K.delta_rule(o, y, z, state, p["A_log"], p["dt_bias"], q_start, ctx, slots, G, Hh, d, dv, C + vn, C + vn + Hh, max_q)
                K.gated_headnorm(mixed, o, z[:, C:C + vn], p["o_norm_w"], Hh, dv, eps)
            self._mm(wk, yo, mixed, p, "w_o")
            nxt = self.layers[li + 1]["ln1_w"] if li + 1 < n_layers else None
            after_mixer = p["ln2_w"] if ls.ff else nxt
            K.norm32(xn if after_mixer is not None else None, h, yo, p["ln1b_w"], after_mixer, None, eps, 1.0)
            if ls.ff:
                act = view(wk.act, p["ff_cols"])
                if "w_gu_p" in p:
                    gu = view(wk.gu, 2 * ls.ff)
                    self._mm(wk, gu, xn, p, "w_gu")
                    K.gated_gelu(act, gu)
                else:
                    K.gemm_any(act, xn, p["w_gu"], p["b_gu"], 1)
                self._mm(wk, yo, act, p, "w_down")
                K.norm32(xn if nxt is not None else None, h, yo, p["ln2b_w"], nxt, None, eps, 1.0)
            if keep:
                self.layer_outputs.append(h.clone())
        return None

    def _fold(self, wk, T: int, pend):
        return None

    def _head(self, wk: _HybridWork, rows_idx: torch.Tensor, R: int, T: int, pend):
        K = self.K
        hx = wk.head_x[:R]
        K.norm32(hx, wk.h[:T], None, None, self.final_norm_w, rows_idx[:R], self.spec.norm_eps, 1.0)
        if self.lm_head_p is not None:
            K.gemm(wk.logits[:R], hx, self.lm_head_p, None, None, wk.ws, self.vocab_pad, 0, 0, 0)
        else:
            K.gemm_any(wk.logits[:R, :self.spec.vocab_size], hx, self.lm_head, None, 0)
        return wk.logits[:R]

    def memory_report(self) -> Dict[str, float]:
        gib = 1 << 30
        size = lambda t: t.numel() * t.element_size()
        wbytes = size(self.embed) + sum(size(t) for l in self.layers for t in l.values())
        kvb = sum(sum(size(t) for t in (kv if isinstance(kv, tuple) else (kv,))) for kv in (self.kv or []) if kv is not None)
        rec = sum(size(c) + size(s) for r in self.rec if r is not None for c, s in [r])
        return {"weights_gib": wbytes / gib, "kv_gib": kvb / gib, "state_gib": rec / gib, "kv_blocks": self.num_blocks,
                "kv_tokens": self.num_blocks * BLOCK}
