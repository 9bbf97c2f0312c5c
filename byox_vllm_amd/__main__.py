"""Command line of the engine.

    python -m byox_vllm_amd generate --model DIR [--dtype bfloat16|float32] --prompt-ids 5,17,3 [--prompt-ids ...]
                                     [--max-tokens 32] [--temperature 0] [--eager]
    python -m byox_vllm_amd trace --model DIR --dtype ... --out DIR --max-tokens N        (= bin/trace_run)

``generate`` builds the model the folder's config.json names (models/registry.py), compiles the kernels it needs when
no library is there yet, and prints one JSON line per prompt with the generated token ids (and text when the folder holds
a tokenizer)."""

import argparse
import json
import sys


def _generate(argv) -> int:
    ap = argparse.ArgumentParser(prog="python -m byox_vllm_amd generate")
    ap.add_argument("--model", required=True, help="folder with config.json and *.safetensors")
    ap.add_argument("--dtype", default=None, choices=["bfloat16", "float16", "float32"])
    ap.add_argument("--prompt-ids", action="append", default=[], help="comma-separated token ids; may be repeated")
    ap.add_argument("--prompt", action="append", default=[], help="text (needs a tokenizer in the model folder)")
    ap.add_argument("--max-tokens", type=int, default=32)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--eager", action="store_true", help="no hipGraph capture")
    ap.add_argument("--max-num-seqs", type=int, default=64)
    ap.add_argument("--block-size", type=int, default=256)
    a = ap.parse_args(argv)
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in a.prompt_ids] + list(a.prompt)
    if not prompts:
        ap.error("give at least one --prompt-ids or --prompt")
    from byox_vllm_amd import build
    from byox_vllm_amd.config import Config
    from byox_vllm_amd.models.registry import model_class
    probe = Config(a.model, dtype=a.dtype)
    sources = getattr(model_class(probe.hf_config), "kernel_sources", None)
    if sources is not None:
        build.ensure(sources)
    else:
        build.build_library()
    from byox_vllm_amd import LLM, SamplingParams
    llm = LLM(a.model, dtype=a.dtype, enforce_eager=a.eager, max_num_seqs=a.max_num_seqs, kvcache_block_size=a.block_size)
    outs = llm.generate(prompts, SamplingParams(temperature=a.temperature, max_tokens=a.max_tokens), use_tqdm=False)
    for prompt, out in zip(prompts, outs):
        print(json.dumps({"prompt": prompt, "token_ids": out["token_ids"], "text": out["text"]}), flush=True)
    llm._exit()
    return 0


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if not argv or argv[0] in ("-h", "--help"):
        print(__doc__)
        return 0
    command, rest = argv[0], argv[1:]
    if command == "generate":
        return _generate(rest)
    if command == "trace":
        from byox_vllm_amd.trace import main as trace_main
        return trace_main(rest)
    print(f"unknown command {command!r}\n{__doc__}", file=sys.stderr)
    return 2


if __name__ == "__main__":
    sys.exit(main())
