"""Token-trace replay: feed given token ids through the engine step by
step and write the logits of chosen positions. Nothing is sampled.

    python -m gllm_amd.entrypoints.trace_replay --model DIR \\
        --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input carries one JSON object per line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3],
                             "want": [0, 2]}], "end": ["a"]}

* ``entries``: per request, its next tokens (a request is admitted at
  its first entry and may skip steps) and ``want``, the indices among
  these tokens whose logits are asked for.
* ``end``: requests that are over after this step; their KV pages and
  state slot go back to the pools.

All entries of a step form ONE batch through the engine's own path:
Scheduler.schedule_scripted (page allocation, in-flight records) ->
ModelRunner.step_logits (batch builder, paged KV / state pools, the
model's kernels) -> Scheduler.commit_scripted. A step that wants
logits writes ``<out>/<step>.f32`` (little-endian fp32 [wanted, vocab],
entries then ``want`` order); every step prints ``done <step>``.

The KV pool holds ``--max-tokens`` tokens (each live request rounded up
to whole pages) and there are ``--max-requests`` state slots, so pages
and slots are recycled across requests.
"""

import argparse
import json
import os
import sys

import numpy as np


def build_engine(model: str, dtype: str, max_tokens: int,
                 max_requests: int, device: str, page_size: int):
    from gllm_amd.config import EngineConfig
    from gllm_amd.engine.llm import LLM
    config = EngineConfig(
        model=model, dtype=dtype, device=device, page_size=page_size,
        enable_prefix_caching=False, use_graph=False, enable_overlap=False,
        maxd=max_requests, max_state_slots=max_requests,
        maxp=max(max_tokens, 1))
    # + 1: the runner keeps the last page as the graph scratch page
    pages = -(-max_tokens // page_size) + 1
    llm = LLM(config=config, num_pages_override=pages)
    llm.scheduler.log = False
    return llm


def replay(llm, lines, out_dir: str, emit=print) -> None:
    live = {}
    sched, runner = llm.scheduler, llm.runner
    for line in lines:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        chunks, rows, base = [], [], 0
        for ent in step.get("entries", []):
            toks = [int(t) for t in ent["tokens"]]
            seq = live.get(ent["id"])
            if seq is None:
                seq = llm.allocate_seq(toks)
                live[ent["id"]] = seq
            else:
                seq.extend_prompt(toks)
            chunks.append((seq, len(toks)))
            rows.extend(base + int(w) for w in ent.get("want", []))
            base += len(toks)
        if chunks:
            batch = sched.schedule_scripted(chunks)
            logits = runner.step_logits(batch, rows)
            sched.commit_scripted(batch)
            if rows:
                arr = logits.cpu().numpy().astype("<f4", copy=False)
                tmp = os.path.join(out_dir, ".%s.part" % step["step"])
                with open(tmp, "wb") as f:
                    f.write(np.ascontiguousarray(arr).tobytes())
                os.replace(tmp, os.path.join(out_dir,
                                             "%s.f32" % step["step"]))
        for rid in step.get("end", []):
            seq = live.pop(rid, None)
            if seq is not None:
                sched.release_scripted(seq)
                llm.seq_id_alloc.free(seq.seq_id)
        emit("done %s" % step["step"])


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16",
                    choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--max-requests", type=int, default=4)
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--device", default=None,
                    help="cuda (default when a GPU is present) or cpu")
    a = ap.parse_args(argv)
    os.makedirs(a.out, exist_ok=True)
    import torch
    device = a.device or ("cuda" if torch.cuda.is_available() else "cpu")
    llm = build_engine(a.model, a.dtype, a.max_tokens, a.max_requests,
                       device, a.page_size)

    def emit(text):
        sys.stdout.write(text + "\n")
        sys.stdout.flush()

    replay(llm, sys.stdin, a.out, emit)
    return 0


if __name__ == "__main__":
    sys.exit(main())
