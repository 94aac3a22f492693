"""Replaying a trace: given token ids go through the model step by step, logits come out, nothing is sampled.

A trace is a stream of JSON lines on standard input,

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

Every entry brings a request's next tokens (a whole prompt, a portion of one, or one decoded token); all entries
of a line are ONE ragged step of the engine: portions of prompts beside single tokens. `want` names the places
among the entry's tokens whose logits are written, as little-endian fp32 [wanted, vocab], to `<out>/<step>.f32`;
`end` lists the requests that are over after the step. After every step a line `done <step>` is printed.

The replay drives what generation drives: the stage executor's step function through `StageRuntime.execute`,
fed with `StepBatch` descriptors (scoring steps: `score_rows`), the native block allocator handing out cache
blocks on demand (a block whenever a request crosses a 32-token boundary), block tables travelling on the
descriptors, slots = rows of the one micro-batch, released through the same control descriptor. Only the
policy differs: which tokens run in which step comes from the trace instead of from the scheduler.
"""
from __future__ import annotations

import json
import os
import sys
from typing import Dict, List, Optional

import numpy as np
import torch

from ..config import EngineConfig
from ..ops.packing import KV_BLOCK
from .batch import KIND_RELEASE, StepBatch, control
from .kv_cache import BlockAllocator, blocks_for


class _Live:
    __slots__ = ("rid", "slot", "ctx", "blocks", "fresh")

    def __init__(self, rid: int, slot: int):
        self.rid, self.slot, self.ctx, self.blocks, self.fresh = rid, slot, 0, [], True


class TraceSession:
    """One single-stage pipeline whose cache pool holds `max_tokens` tokens and whose micro-batch has `slots` rows."""

    def __init__(self, model: str, dtype: str = "bf16", max_tokens: int = 4096, slots: int = 4, device: str = "auto",
                 backend: str = "auto", seed: int = 0):
        from ..parallel.launcher import build_executor, plans_for, resolve_spec
        from ..parallel.pipeline import StageRuntime
        from ..parallel.transport import make_loopback_links
        pool = max(KV_BLOCK, (int(max_tokens) + KV_BLOCK - 1) // KV_BLOCK * KV_BLOCK)
        self.cfg = EngineConfig(model=model, dtype=dtype, pp_size=1, max_batch=slots, num_micro_batches=1,
                                max_seq_len=pool, prefill_chunk=pool, kv_blocks=pool // KV_BLOCK, device=device,
                                backend=backend, use_graphs=False, seed=seed, transport="loopback")
        self.spec = resolve_spec(self.cfg)
        plan = plans_for(self.cfg, self.spec)[0]
        self.ex = build_executor(self.cfg, self.spec, plan)
        self.job = f"dlia_trace_{os.getpid()}"
        links = make_loopback_links(1, device=None, max_bytes=1 << 16, fb_bytes=1 << 10, job=self.job)
        self.rt = StageRuntime(self.ex, links[0], decode_streams=0)
        self.alloc = BlockAllocator(self.cfg.kv_blocks)
        self.rows: List[Optional[_Live]] = [None] * slots
        self.live: Dict[str, _Live] = {}
        self._rid = 0
        self._step = 0

    # ---- one step -----------------------------------------------------------------------------------------
    def step(self, entries: List[dict], end: List[str]) -> Optional[np.ndarray]:
        """Runs the entries as one ragged step. Returns the wanted logits [wanted, vocab] (fp32, in the order
        of the entries and of their `want`), or None when nothing is wanted."""
        self._step += 1
        d = StepBatch(step_id=self._step, micro_batch=0, token_ids=[], score_rows=[])
        # single decoded tokens ride in front of the prompt portions, as in the scheduler's mixed steps
        order = sorted(range(len(entries)), key=lambda i: 0 if (len(entries[i]["tokens"]) == 1 and entries[i]["id"] in self.live) else 1)
        where: Dict[int, int] = {}
        for i in order:
            e = entries[i]
            toks = [int(t) for t in e["tokens"]]
            if not toks:
                continue
            r = self.live.get(e["id"])
            if r is None:
                r = self._admit(e["id"])
            need = blocks_for(r.ctx + len(toks)) - len(r.blocks)
            if need > 0:
                got = self.alloc.take(r.rid, need)
                if got is None:
                    raise RuntimeError(f"the cache pool ({self.alloc.num_blocks} blocks) has no {need} blocks left for request {e['id']!r}")
                if not r.fresh:
                    for b in got:
                        d.grow_slots.append(r.slot); d.grow_pos.append(len(r.blocks)); d.grow_blocks.append(b)
                        r.blocks.append(b)
                else:
                    r.blocks += got
            if r.fresh:
                d.table_slots.append(r.slot); d.table_blocks.append(list(r.blocks))
                r.fresh = False
            where[i] = len(d.token_ids)
            d.slots.append(r.slot); d.q_lens.append(len(toks)); d.ctx_lens.append(r.ctx); d.sample.append(0)
            d.temperature.append(0.0); d.top_k.append(1); d.top_p.append(1.0); d.seeds.append(0); d.sample_steps.append(0)
            d.token_ids += toks
            r.ctx += len(toks)
        for i, e in enumerate(entries):
            if i in where:
                d.score_rows += [where[i] + int(w) for w in e.get("want", [])]
        out = None
        if d.slots:
            d.validate()
            res = self.rt.execute(d)
            if d.score_rows:
                out = res.detach().float().cpu().numpy()
        gone = []
        for name in end:
            r = self.live.pop(name, None)
            if r is not None:
                self.alloc.release(r.rid)
                self.rows[r.slot] = None
                gone.append(r.slot)
        if gone:
            self.rt.execute(control(KIND_RELEASE, gone))
        return out

    def _admit(self, name: str) -> _Live:
        if None not in self.rows:
            raise RuntimeError(f"no free slot for request {name!r} ({len(self.rows)} are live)")
        self._rid += 1
        slot = self.rows.index(None)
        r = _Live(self._rid, slot)
        self.rows[slot] = r
        self.live[name] = r
        return r

    def close(self):
        try:
            self.rt.drain()
            self.rt.links.close()
        except Exception:
            pass


def run(model: str, dtype: str, out_dir: str, max_tokens: int, slots: int = 4, device: str = "auto", backend: str = "auto",
        stdin=None, stdout=None) -> int:
    stdin, stdout = stdin or sys.stdin, stdout or sys.stdout
    dt = {"bfloat16": "bf16", "float32": "fp32", "bf16": "bf16", "fp32": "fp32"}[dtype]
    try:
        sess = TraceSession(model, dt, max_tokens, slots, device=device, backend=backend)
    except ValueError as e:
        if dt == "fp32" and "fp32" in str(e):
            print(f"refused: {e}", file=sys.stderr)
            return 3
        raise
    os.makedirs(out_dir, exist_ok=True)
    try:
        for line in stdin:
            line = line.strip()
            if not line:
                continue
            msg = json.loads(line)
            logits = sess.step(msg.get("entries", []), msg.get("end", []))
            if logits is not None:
                tmp = os.path.join(out_dir, f".{msg['step']}.part")
                with open(tmp, "wb") as f:
                    f.write(np.ascontiguousarray(logits, dtype="<f4").tobytes())
                os.replace(tmp, os.path.join(out_dir, f"{msg['step']}.f32"))
            stdout.write(f"done {msg['step']}\n")
            stdout.flush()
    finally:
        sess.close()
    return 0
