"""Trace replay: feed given token ids through an engine step by step and write logits.

A trace is a stream of JSON lines on standard input,
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["a"]}
Every step runs exactly the tokens it brings, all entries as one batch (portions of prompts beside
single decoded tokens), on the cache that earlier steps left: a request is admitted at its first
entry, may skip steps, and gives its pages back when it is listed in `end`.  For a step that wants
logits, `<out>/<step>.f32` gets them as little-endian fp32 [wanted, vocab], in the order of the
entries and of `want`; after every step `done <step>` is printed.  Nothing is sampled.

The replay drives the engine's own parts: `build_engine` (model registry, weight loading, cache
pool), the scheduler's `schedule_given` (pages from the block manager, decode rows first) and the
runner's `execute_logits` (the packing, cache and forward of `execute`).  A model with recurrent state gets
`max_requests` state slots, taken at a request's first entry and given back at its end like its pages.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Dict, List

import numpy as np


class TraceSession:
    def __init__(self, model_dir: str, dtype: str = "bfloat16", max_tokens: int = 4096, device: str = "",
                 max_requests: int = 4):
        import torch

        from .builder import EngineOptions, build_engine
        from .sequence import SamplingParams

        dev = device or ("cuda" if torch.cuda.is_available() else "cpu")
        bs = 16
        # the pool holds `max_tokens` tokens of live requests, each rounded up to whole pages
        tokens = (max_tokens + bs - 1) // bs * bs
        opts = EngineOptions(model=model_dir, weights=model_dir, device=dev, dtype=dtype, block_size=bs,
                             kv_cache_tokens=tokens, max_model_len=tokens, max_batch=max_requests,
                             graph_buckets=tuple(b for b in (1, 2, 4, 8, 16) if b <= max_requests) or (1,),
                             use_graphs=False, safe_decode=False, prefix_caching=False, ignore_eos=True,
                             state_slots=max_requests)
        self.engine = build_engine(opts)
        self.runner = self.engine.runner
        self.sched = self.engine.scheduler
        self.params = SamplingParams(max_new_tokens=0, ignore_eos=True, safe_decode=False)
        self.live: Dict[str, object] = {}

    def step(self, entries: List[dict], end: List[str]) -> np.ndarray:
        """Run one step; returns the wanted logits [n, vocab] (fp32, host)."""
        from .sequence import Sequence

        items = []
        for e in entries:
            seq = self.live.get(e["id"])
            if seq is None:
                seq = self.live[e["id"]] = Sequence(prompt_ids=[], params=self.params)
            seq.prompt_ids.extend(int(t) for t in e["tokens"])
            items.append((seq, len(e["tokens"]), e.get("want") or []))
        out = np.zeros((0, self.runner.cfg.vocab_size), dtype="<f4")
        if items:
            batch = self.sched.schedule_given([(s, n) for s, n, _ in items])
            want = {id(s): w for s, _, w in items}
            rows = [list(want[id(s)]) for s in batch.seqs]
            logits = self.runner.execute_logits(batch, rows).cpu().numpy()
            for s, n in zip(batch.seqs, batch.num_query):
                s.num_computed += n
            # batch order (decode rows first) -> the order of the entries
            at, o = {}, 0
            for s, r in zip(batch.seqs, rows):
                at[id(s)] = (o, o + len(r))
                o += len(r)
            parts = [logits[at[id(s)][0]:at[id(s)][1]] for s, _, _ in items]
            out = np.concatenate(parts, axis=0).astype("<f4") if parts else out
        for rid in end:
            seq = self.live.pop(rid, None)
            if seq is not None:
                self.sched.release(seq)
        return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description="replay a token trace through the engine and write logits")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    ap.add_argument("--out", required=True, help="folder for <step>.f32")
    ap.add_argument("--max-tokens", type=int, default=4096, help="tokens the cache pool holds at any time")
    ap.add_argument("--device", default="", help="cuda (default when present) or cpu")
    a = ap.parse_args(argv)
    os.makedirs(a.out, exist_ok=True)
    sess = TraceSession(a.model, a.dtype, a.max_tokens, a.device)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        logits = sess.step(st.get("entries") or [], st.get("end") or [])
        if logits.shape[0]:
            tmp = os.path.join(a.out, ".%s.part" % st["step"])
            with open(tmp, "wb") as f:
                f.write(logits.tobytes())
            os.replace(tmp, os.path.join(a.out, "%s.f32" % st["step"]))
        print("done %s" % st["step"], flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
