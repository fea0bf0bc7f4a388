"""``python -m nanospec_amd``: generate from token ids on the command line.

    python -m nanospec_amd --model DIR --prompt-ids 1,2,3 --prompt-ids 4,5 --max-tokens 16 --temperature 0

Option names are the reference's where it has them (SamplingParams: max_tokens, temperature, top_k, top_p,
seed; bench/run.py:162-172: --max-tokens, --temperature; EngineConfig: block_size, max_admit, max_running).
Token ids in, token ids out, one JSON line per prompt.
"""

from __future__ import annotations

import argparse
import json
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m nanospec_amd", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--prompt-ids", action="append", default=[], help="comma separated token ids; may be given several times")
    ap.add_argument("--prompts-file", help="file with one prompt per line (comma or space separated token ids)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--max-tokens", type=int, default=128)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=None)
    ap.add_argument("--logprobs", action="store_true")
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--num-blocks", type=int, default=None)
    ap.add_argument("--max-admit", type=int, default=32)
    ap.add_argument("--max-running", type=int, default=None)
    ap.add_argument("--max-step-tokens", type=int, default=None, help="token budget of a step (prompts are cut into portions)")
    ap.add_argument("--prefill-chunk", type=int, default=None)
    ap.add_argument("--no-graphs", action="store_true", help="do not replay captured graphs for decode steps")
    a = ap.parse_args(argv)

    prompts = [[int(t) for t in p.replace(",", " ").split()] for p in a.prompt_ids]
    if a.prompts_file:
        with open(a.prompts_file) as f:
            prompts += [[int(t) for t in line.replace(",", " ").split()] for line in f if line.strip()]
    if not prompts:
        ap.error("give --prompt-ids or --prompts-file")

    from . import SamplingParams
    from .engine import Engine, EngineConfig
    from .loader import load_model

    model = load_model(a.model, dtype=a.dtype)
    params = [SamplingParams(a.max_tokens, a.temperature, a.top_k, a.top_p, None if a.seed is None else a.seed + i, a.logprobs)
              for i in range(len(prompts))]
    blocks = a.num_blocks or sum(-(-(len(p) + a.max_tokens) // a.block_size) for p in prompts) + 1
    eng = Engine(model, EngineConfig(blocks, a.block_size, a.max_admit, a.max_running, cuda_graphs=not a.no_graphs,
                                     max_step_tokens=a.max_step_tokens, prefill_chunk=a.prefill_chunk))
    reqs = [eng.add(p, s) for p, s in zip(prompts, params)]
    while eng.sched.has_work:
        eng.step()
    for r in reqs:
        row = {"id": r.id, "prompt_ids": r.prompt_ids, "output_ids": r.out_tokens}
        if a.logprobs:
            row["logprobs"] = [t.logprob for t in r.logprobs]
        print(json.dumps(row), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
