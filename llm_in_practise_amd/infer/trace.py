"""Replay of a token trace through the serving engine's own step functions, writing logits instead of sampling.

A trace is a stream of steps, one JSON object per line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

Every entry brings a request's next tokens; ``want`` lists the places among them whose logits are written to
``<out>/<step>.f32`` (little-endian float32 ``[wanted, vocab]``, in the order of the entries).  A request seen for the
first time takes a free slot of the engine and is prefilled with the other new requests of its step (one packed
batch, ``ServingEngine.forward_prefill``); a request that goes on by one token is one row of the engine's decode step
(``forward_decode``); one that goes on by several tokens is a continued prefill into its slot.  ``end`` gives slots
back.  After every step ``done <step>`` is printed.  Nothing here computes: model, cache and kernels are the engine's.
"""
from __future__ import annotations

import json
import os
import queue
import sys
import time

import torch

from .engine import SamplingParams, ServingEngine, _Request


class TraceRunner:
    def __init__(self, lm, max_tokens: int, use_graphs: bool = False):
        self.lm, self.max_len, self.use_graphs = lm, int(max_tokens) + 1, use_graphs
        self.engine: ServingEngine | None = None
        self.slot_of: dict[str, int] = {}
        self.length: dict[str, int] = {}

    def _engine(self, need: int) -> ServingEngine:
        e = self.engine
        if e is None or sum(s is None for s in e.slots) < need:
            if self.slot_of:
                raise RuntimeError("a batch may grow only while no request is live")
            slots = max(2 * need, 2 * e.max_batch if e is not None else 8)     # room for a later, larger batch
            self.engine = e = ServingEngine(self.lm, None, max_batch=slots, max_model_len=self.max_len,
                                            use_graphs=self.use_graphs, start=False)
        return e

    @torch.no_grad()
    def step(self, entries: list[dict], end: list[str]):
        """Run one step; returns float logits ``[wanted, vocab]`` on the host, or None when nothing is wanted."""
        new = [e for e in entries if e["id"] not in self.slot_of]
        out = None
        if new:
            if len(new) != len(entries):
                raise ValueError("a step either starts all its requests or continues all of them")
            eng = self._engine(len(new))
            free = [i for i, s in enumerate(eng.slots) if s is None]
            batch, rows, off = [], [], 0
            for e, slot in zip(new, free):
                batch.append((slot, _Request(list(e["tokens"]), SamplingParams(), False, queue.Queue(), time.time())))
                self.slot_of[e["id"]], self.length[e["id"]] = slot, len(e["tokens"])
                rows += [off + w for w in e["want"]]
                off += len(e["tokens"])
            h, _ = eng.forward_prefill(batch)
            if rows:
                out = eng._head(h[torch.tensor(rows, device=h.device)])
        elif entries:
            eng = self.engine
            if all(len(e["tokens"]) == 1 for e in entries):
                slots = [self.slot_of[e["id"]] for e in entries]
                eng.next_tok[torch.tensor(slots, device=eng.device)] = torch.tensor(
                    [e["tokens"][0] for e in entries], dtype=torch.long, device=eng.device)
                active = sorted(slots)
                logits = eng.forward_decode(active)
                rows = [active.index(s) for s, e in zip(slots, entries) if e["want"]]
                if rows:
                    out = logits[torch.tensor(rows, device=logits.device)]
                for e in entries:
                    self.length[e["id"]] += 1
            else:                                   # several tokens more: continued prefill, request by request
                parts = []
                for e in entries:
                    slot, P, n = self.slot_of[e["id"]], self.length[e["id"]], len(e["tokens"])
                    ids = torch.tensor([e["tokens"]], dtype=torch.long, device=eng.device)
                    h = eng.lm.model(ids, None, eng._slot_view(slot, P, n), None)
                    eng.cache.pos[slot] = P + n
                    self.length[e["id"]] = P + n
                    if e["want"]:
                        parts.append(eng._head(h[torch.tensor(e["want"], device=h.device)]))
                out = torch.cat(parts) if parts else None
        for rid in end:
            self.engine.release(self.slot_of.pop(rid))
            self.length.pop(rid, None)
        return None if out is None else out.float().cpu()


def run(model_dir: str, dtype: str, out_dir: str, max_tokens: int, stdin=None, stdout=None, device=None,
        use_graphs: bool = False) -> int:
    from ..models.registry import load_causal_lm
    stdin, stdout = stdin or sys.stdin, stdout or sys.stdout
    td = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    dev = torch.device(device or ("cuda" if torch.cuda.is_available() else "cpu"))
    if td == torch.float32:                 # true 32-bit products: no reduced-precision matrix mode
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    lm = load_causal_lm(model_dir, dtype=td, device=dev)
    runner = TraceRunner(lm, max_tokens, use_graphs)
    os.makedirs(out_dir, exist_ok=True)
    for line in stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        logits = runner.step(st.get("entries", []), st.get("end", []))
        if logits is not None:
            tmp = os.path.join(out_dir, f".{st['step']}.part")
            with open(tmp, "wb") as f:
                f.write(logits.contiguous().numpy().astype("<f4").tobytes())
            os.replace(tmp, os.path.join(out_dir, f"{st['step']}.f32"))
        stdout.write(f"done {st['step']}\n")
        stdout.flush()
    return 0
