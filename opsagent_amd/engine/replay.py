"""Token-id trace replay: feeds given tokens through the engine step by step
and returns logits; samples nothing.

A trace is a stream of steps. Each step names, per request, its next tokens
(a prompt portion or a single token) and the places among them whose logits
are wanted; all entries of a step run as ONE batch through the engine's own
flat multi-sequence forward (LLMEngine._forward_mixed — the function its
scheduler steps with), against the engine's paged cache and state-slot pool.
Requests are admitted at their first entry, may sit out steps, and give
their pages and slot back when the step that names them in `end` is done.
"""

from __future__ import annotations

import json
import os
import sys
from typing import Dict, List, Optional

import torch

from opsagent_amd.engine.engine import LLMEngine, Request, SamplingParams
from opsagent_amd.engine.kv_cache import SequenceState


class TraceReplayer:
    def __init__(self, engine: LLMEngine):
        if not engine.hybrid:
            raise NotImplementedError(
                "trace replay drives the flat multi-sequence step of hybrid models"
            )
        self.engine = engine
        self.live: Dict[str, Request] = {}

    def step(self, entries: List[dict], end: List[str]) -> Optional[torch.Tensor]:
        """Run one step; returns float32 logits [wanted, vocab] in entry and
        `want` order, or None if nothing is wanted."""
        eng = self.engine
        work, rows, off = [], [], 0
        for e in entries:
            toks = [int(t) for t in e["tokens"]]
            if not toks:
                continue
            req = self.live.get(e["id"])
            if req is None:
                req = Request(eng._next_id, [], SamplingParams())
                eng._next_id += 1
                req.seq = SequenceState(eng.kv, [], eng.state_pool)
                self.live[e["id"]] = req
            seq = req.seq
            start = seq.num_cached
            seq.token_ids.extend(toks)
            seq.ensure_capacity(start + len(toks))
            work.append((req, start, len(toks)))
            rows.extend(off + int(w) for w in e.get("want", []))
            off += len(toks)
        logits = None
        if work:
            hidden = eng._forward_mixed(work)
            if rows:
                idx = torch.tensor(rows, dtype=torch.int64).to(eng.device)
                logits = eng.model.compute_logits(hidden.index_select(0, idx)).float()
        for rid in end:
            req = self.live.pop(rid, None)
            if req is not None:
                req.seq.free()
        return logits


def main(argv: Optional[List[str]] = None) -> int:
    import argparse

    ap = argparse.ArgumentParser(
        prog="trace_run",
        description="Replay a token-id trace (JSON steps on stdin) through the engine "
                    "and write the wanted logits as <step>.f32 files.",
    )
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--out", required=True, help="folder for <step>.f32")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="tokens that live requests hold at most (each rounded up to a page multiple)")
    ap.add_argument("--slots", type=int, default=4, help="live requests at most")
    ap.add_argument("--block-size", type=int, default=32)
    ap.add_argument("--device", default=None, help="cpu forces the reference path")
    a = ap.parse_args(argv)

    if a.device == "cpu":
        os.environ["HIP_VISIBLE_DEVICES"] = os.environ["CUDA_VISIBLE_DEVICES"] = ""
    bs = a.block_size
    blocks = (a.max_tokens + bs - 1) // bs
    eng = LLMEngine({
        "model": a.model,
        "dtype": a.dtype,
        "kv_block_size": bs,
        "kv_num_blocks": blocks,
        "max_batch_size": a.slots,
        "state_slots": a.slots,
        "max_prefill_chunk": 1 << 30,
        "tokenizer_check": False,
        "max_seq_len": 1 << 30,
    })
    rp = TraceReplayer(eng)
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        logits = rp.step(st.get("entries", []), st.get("end", []))
        if logits is not None:
            data = logits.detach().to("cpu", torch.float32).contiguous().numpy()
            part = os.path.join(a.out, ".%d.part" % st["step"])
            with open(part, "wb") as f:
                f.write(data.astype("<f4").tobytes())
            os.replace(part, os.path.join(a.out, "%d.f32" % st["step"]))
        sys.stdout.write("done %d\n" % st["step"])
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
