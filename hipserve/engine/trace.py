"""Teacher-forced trace replay: feed given token ids through the engine, step by step,
and write the logits at asked positions. Nothing is sampled.

The replay drives the engine's own parts: sequences (``engine/request.py``), the paged
cache's block manager and the recurrent-state slots, the runner's batch preparation and
its step function (``ModelRunner.prepare`` / ``execute``). Only the scheduling decision
itself — which requests run in a step and with how many tokens — comes from the trace
instead of the scheduler's policy: every step is one ``SchedulerOutput`` whose prompt
portions and single tokens run as one batch.

Input, one JSON object per line on stdin::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["a"]}

``entries`` lists, per request id, the tokens to append now and ``want``, offsets into
those tokens whose logits should be written; a request id seen for the first time starts
a new sequence. ``end`` names requests to drop once the step has run: their cache blocks
and their state slot return to the pools. If any row is wanted the step writes
``<out>/<step>.f32`` (little-endian float32 [rows, vocab], rows ordered by entry, then by
``want``); after every step a line ``done <step>`` goes to stdout.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np

from ..config import EngineConfig
from .request import SamplingParams, Sequence, Status
from .scheduler import ScheduledSeq, SchedulerOutput

MAX_LIVE = 4  # state slots / concurrently live requests of a replay


class TraceSession:
    def __init__(self, engine):
        self.engine = engine
        self.live: dict[str, Sequence] = {}

    def step(self, entries: list[dict], end: list[str]) -> np.ndarray:
        """Run one batch; returns the fp32 logits [wanted rows, vocab]."""
        eng = self.engine
        prefill, decode = [], []
        for e in entries:
            toks = [int(t) for t in e["tokens"]]
            if not toks:
                continue
            seq = self.live.get(e["id"])
            if seq is None:
                seq = Sequence(e["id"], [], SamplingParams(temperature=0.0, max_tokens=1))
                seq.status = Status.RUNNING
                self.live[e["id"]] = seq
                if eng.states is not None:
                    eng.states.allocate(seq)
            start = seq.num_computed_tokens
            seq.prompt_token_ids.extend(toks)
            target = start + len(toks)
            if target > eng.max_model_len:
                raise ValueError(f"request {e['id']!r} exceeds max_model_len {eng.max_model_len}")
            if not eng.blocks.can_grow(seq, target):
                raise RuntimeError("the cache pool is too small for the live requests")
            eng.blocks.grow(seq, target)
            ss = ScheduledSeq(seq, start, target)
            # a single token after the first step is a decode row, anything else a prompt portion
            (decode if len(toks) == 1 and start > 0 else prefill).append((ss, e.get("want") or []))
        so = SchedulerOutput(prefill=[p for p, _ in prefill], decode=[d for d, _ in decode])
        # batch rows: prefill portions in order, then one row per decode sequence
        row0, t = {}, 0
        for ss, _ in prefill:
            row0[id(ss)] = t
            t += ss.num_tokens
        for ss, _ in decode:
            row0[id(ss)] = t
            t += 1
        by_id = {ss.seq.request_id: (ss, want) for ss, want in prefill + decode}
        rows = []
        for e in entries:  # output order: the entries' order, then their want order
            if e["id"] in by_id and e["tokens"]:
                ss, want = by_id[e["id"]]
                rows += [row0[id(ss)] + int(w) for w in want]
        so.logits_rows = rows
        logits = np.zeros((0, eng.model_cfg.vocab_size), np.float32)
        if not so.empty:
            inp = eng.runner.prepare(so)
            logits = eng.runner.execute(inp, return_logits=True)
            for ss in so.prefill + so.decode:
                ss.seq.num_computed_tokens = ss.end
        for rid in end:
            seq = self.live.pop(rid, None)
            if seq is not None:
                eng.blocks.free(seq)
                if eng.states is not None:
                    eng.states.free(seq)
                eng.runner.release(seq)
        return logits


def build_engine(model: str, dtype: str, max_tokens: int, device: str | None = None, block_size: int = 16):
    import torch

    from ..parallel.comm import TPGroup
    from .llm_engine import LLMEngine

    device = device or ("cuda" if torch.cuda.is_available() else "cpu")
    blocks = -(-max_tokens // block_size) + 1   # the pool holds max_tokens; + the runner's scratch block
    cfg = EngineConfig(model=model, load_format="safetensors", dtype=dtype, device=device, block_size=block_size,
                       max_num_seqs=MAX_LIVE, max_num_batched_tokens=max(max_tokens, 64), num_kv_blocks=blocks,
                       max_model_len=max(max_tokens, 64), enable_prefix_caching=False, enforce_eager=True)
    tp = TPGroup(0, 1, None, torch.device("cuda", 0)) if device == "cuda" else TPGroup()
    return LLMEngine(cfg, tp=tp)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for the <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens the live requests hold at any time (sizes the cache pool)")
    ap.add_argument("--device", default=None, help="cuda (default when a GPU is visible) or cpu")
    a = ap.parse_args(argv)
    from ..config import resolve_model_config
    from ..models.registry import model_class

    import torch

    device = a.device or ("cuda" if torch.cuda.is_available() else "cpu")
    if a.dtype == "float32" and device == "cuda":
        if not getattr(model_class(resolve_model_config(a.model)), "supports_fp32", False):
            print("this model's kernels have no 32-bit build", file=sys.stderr)
            return 3
    os.makedirs(a.out, exist_ok=True)
    session = TraceSession(build_engine(a.model, a.dtype, a.max_tokens, device))
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        logits = session.step(st.get("entries") or [], st.get("end") or [])
        if logits.shape[0]:
            tmp = os.path.join(a.out, f".{st['step']}.f32.part")
            with open(tmp, "wb") as f:
                f.write(np.ascontiguousarray(logits, dtype="<f4").tobytes())
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        print(f"done {st['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
