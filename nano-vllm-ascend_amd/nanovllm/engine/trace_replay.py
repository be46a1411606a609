"""Replay of a recorded step trace: given token ids go through the engine's own step function, scheduler state, page and
state-slot managers and kernels, and the logits of the rows a step asks for are written out.  Nothing is sampled.

Input (one JSON object per line on standard input):

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["b"]}

`entries`: for each request its next tokens (a prompt's portion or a decoded token) and the places among them whose
logits are wanted; all entries of a step are ONE batch.  `end`: requests that are over after the step - their pages and
state slot go back to the pool.  Output: <out>/<step>.f32 = little-endian fp32 [wanted rows, vocab] in the order of the
entries, and a line `done <step>` on standard output after every step.

The page pool holds `max_tokens` tokens (pages of 64), there are four state slots: what a trace needs beyond that it gets
by finishing requests.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

PAGE = 64
LIVE_REQUESTS = 4


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="directory with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    ap.add_argument("--out", required=True, help="directory the logits files are written to")
    ap.add_argument("--max-tokens", type=int, required=True, help="tokens the page pool holds")
    a = ap.parse_args(argv)

    import torch

    from nanovllm.config import Config
    from nanovllm.engine.model_runner import ModelRunner
    from nanovllm.engine.scheduler import Scheduler
    from nanovllm.engine.sequence import Sequence

    pages = -(-max(a.max_tokens, PAGE) // PAGE)
    longest = pages * PAGE
    config = Config(a.model, dtype=a.dtype, kvcache_block_size=PAGE, num_kvcache_blocks=pages + 1,
                    max_num_seqs=LIVE_REQUESTS, num_state_slots=LIVE_REQUESTS, max_model_len=longest,
                    max_num_batched_tokens=longest, enforce_eager=True)
    if not config.hybrid_state:
        if a.dtype == "float32":
            print("this model family has no 32-bit serving mode", file=sys.stderr)
            return 3
        print("trace replay drives the row-step path (hybrid-state models); this model family steps through "
              "LLMEngine.step() only", file=sys.stderr)
        return 2
    runner = ModelRunner(config, 0)
    scheduler = Scheduler(config)
    os.makedirs(a.out, exist_ok=True)
    live: dict[str, Sequence] = {}
    try:
        for line in sys.stdin:
            line = line.strip()
            if not line:
                continue
            step = json.loads(line)
            runs, want, row0 = [], [], 0
            for e in step.get("entries", ()):
                toks = [int(t) for t in e["tokens"]]
                if not toks:
                    continue
                seq = live.get(e["id"])
                if seq is None:
                    seq = live[e["id"]] = Sequence(toks, request_id=e["id"], block_size=PAGE)
                    scheduler.admit_portion(seq, [])
                else:
                    scheduler.admit_portion(seq, toks)
                runs.append((seq, seq.num_computed_tokens, len(toks)))
                want += [row0 + int(w) for w in e.get("want", ())]
                row0 += len(toks)
            if runs:
                logits = runner.run_rows(runs, want)
                if want:
                    logits.to(torch.float32).cpu().numpy().astype("<f4").tofile(os.path.join(a.out, f"{step['step']}.f32"))
                else:
                    torch.cuda.current_stream().synchronize()
            for name in step.get("end", ()):
                seq = live.pop(name, None)
                if seq is not None:
                    scheduler.finish(seq)
            print(f"done {step['step']}", flush=True)
    finally:
        runner.exit()
    return 0


if __name__ == "__main__":
    sys.exit(main())
