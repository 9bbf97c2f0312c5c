"""Trace replay: feed given token ids through the engine step by step and write logits; nothing is sampled.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps arrive on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": ["a"]}

Every entry brings a request's next tokens (a request is admitted at its first entry and may sit out steps); ``want``
names the places among these tokens whose logits are written to <out>/<step>.f32 as little-endian fp32 [wanted, vocab],
in the order of the entries; ``end`` names the requests that are over after the step, whose pages and state slot go
back to the pools.  After each step the line ``done <step>`` is printed.

The replay drives the engine's own parts: ``Scheduler.commit`` admits requests and grows block tables (the same call
the engine's portion scheduler ends in), ``ModelRunner.run_portions`` runs the batch, ``Scheduler.finish`` releases.
The cache pool is sized for ``--max-tokens`` tokens (each request's share rounded up to whole blocks) and there are as
many state slots as ``--max-live`` (4), so blocks and slots are reused while a trace runs."""

import argparse
import json
import os
import sys

BLOCK = 64


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder the logits files are written to")
    ap.add_argument("--max-tokens", type=int, required=True, help="tokens the live requests hold at most")
    ap.add_argument("--max-live", type=int, default=4, help="requests live at once (state slots)")
    a = ap.parse_args(argv)

    from byox_vllm_amd.config import Config
    config = Config(a.model, dtype=a.dtype, kvcache_block_size=BLOCK, num_kvcache_blocks=-(-a.max_tokens // BLOCK),
                    max_num_seqs=a.max_live, num_state_slots=a.max_live, enforce_eager=True,
                    max_num_batched_tokens=1 << 30, max_model_len=1 << 30)
    if not config.portioned:
        print("trace replay needs a model that steps through portions", file=sys.stderr)
        return 3
    from byox_vllm_amd import build
    from byox_vllm_amd.models.registry import model_class
    build.ensure(model_class(config.hf_config).kernel_sources)     # a fresh checkout compiles what this model needs

    import numpy as np
    from byox_vllm_amd.engine.model_runner import ModelRunner
    from byox_vllm_amd.engine.scheduler import Scheduler
    from byox_vllm_amd.engine.sequence import Sequence
    runner = ModelRunner(config, 0, None)
    scheduler = Scheduler(config)
    os.makedirs(a.out, exist_ok=True)
    live: dict[str, Sequence] = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        plan, want = [], []
        for entry in step["entries"]:
            if not entry["tokens"]:
                continue                      # nothing to run for this request in this step
            seq = live.get(entry["id"])
            if seq is None:
                seq = live[entry["id"]] = Sequence(entry["tokens"], BLOCK)
                scheduler.add(seq)
            else:
                seq.extend_tokens(entry["tokens"])
            plan.append((seq, len(entry["tokens"])))
            want.append(list(entry.get("want") or []))
        if plan:
            scheduler.commit(plan)
            logits = runner.run_portions(plan, want=want)
            scheduler.advance(plan, [None] * len(plan))
            if logits is not None:
                tmp = os.path.join(a.out, f".{step['step']}.part")
                np.ascontiguousarray(logits.cpu().numpy().astype("<f4")).tofile(tmp)
                os.replace(tmp, os.path.join(a.out, f"{step['step']}.f32"))
        for name in step.get("end") or []:
            seq = live.pop(name, None)
            if seq is not None:
                scheduler.finish(seq)
        print(f"done {step['step']}", flush=True)
    runner.exit()
    return 0
