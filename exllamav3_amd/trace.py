"""
Trace replay: feeds given token ids through a model step by step and writes the logits that are asked for.  Nothing is sampled.  It
drives the same objects as generation does -- registry.load_model, the model's `step`, its SlotStateCache -- and keeps no forward pass
or cache of its own.

Input (one JSON object per line):   {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["a"]}
Output: <out>/<step>.f32 = float32 little-endian [wanted, vocab] in the order of the entries and of "want" (only for steps that want
something), and the line "done <step>" on standard output after every step.
"""
from __future__ import annotations
import json
import os
import sys
import numpy as np


class TraceSession:
    def __init__(self, model, out_dir: str, max_tokens: int = 0):
        """max_tokens: the most tokens that live requests hold at once, if known: a model whose cache grows with its sequences sizes its pages from it."""
        self.model, self.out_dir = model, out_dir
        import inspect
        sized = max_tokens > 0 and "tokens" in inspect.signature(model.new_cache).parameters
        self.cache = model.new_cache(tokens=max_tokens) if sized else model.new_cache()
        self.slot_of: dict[str, int] = {}

    def run_step(self, rec: dict) -> int:
        entries, want = [], []
        for e in rec["entries"]:
            if e["id"] not in self.slot_of:
                self.slot_of[e["id"]] = self.cache.alloc()
            entries.append((self.slot_of[e["id"]], [int(t) for t in e["tokens"]]))
            want.append([int(p) for p in e.get("want", [])])
        wanted = sum(len(w) for w in want)
        if entries:
            sb = self.cache.begin_step(entries, want)
            logits = self.model.step(sb, self.cache)
            if wanted:
                a = logits.cpu().numpy().astype("<f4", copy=False)
                assert a.shape == (wanted, self.model.vocab)
                tmp = os.path.join(self.out_dir, f".{rec['step']}.f32.part")
                a.tofile(tmp)
                os.replace(tmp, os.path.join(self.out_dir, f"{rec['step']}.f32"))
        for i in rec.get("end", []):
            if i in self.slot_of:
                self.cache.release(self.slot_of.pop(i))
        return wanted

    def run(self, lines, out=sys.stdout):
        for line in lines:
            line = line.strip()
            if not line:
                continue
            rec = json.loads(line)
            self.run_step(rec)
            out.write(f"done {rec['step']}\n")
            out.flush()
