"""Command line of the stand-alone engine.

    python -m mini_sglang_amd.cli generate --model DIR --prompt 5,17,3 [--prompt ...] --max-tokens 16 [--temperature 0.8 ...]
    python -m mini_sglang_amd.cli trace    --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N   < steps.jsonl

`generate` runs prompts (token ids) through the scheduler glue of offline.py -- chunked prefill, continuous decode from
captured graphs, the sampler -- and prints one JSON line per request.  `trace` replays recorded steps (`bin/trace_run` is this
subcommand): one JSON object a line, {"step": n, "entries": [{"id", "tokens", "want"}], "end": [ids]}; every step is one
batch of the engine's forward, the logits at the wanted places go to OUT/<step>.f32 (little-endian fp32 [wanted, vocab]),
and `done <step>` is printed once the step has run.  The model class comes from the folder's config.json (registry.py).
Shared objects a model needs are built on first use (hipcc, gfx950) when they are missing or older than their sources.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from pathlib import Path

_DTYPES = {"bfloat16": "bfloat16", "bf16": "bfloat16", "float32": "float32", "fp32": "float32"}


def ensure_built(only) -> None:
    import importlib.util

    here = Path(__file__).resolve().parent
    spec = importlib.util.spec_from_file_location("msgl_build", here / "build.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.build_all(force=False, verbose=False, only=only)


def _engine(args, *, max_running_req: int, num_tokens: int, graphs, page_size: int):
    import torch

    from .engine import Engine, EngineConfig
    from .hybrid import HybridConfig
    from .registry import load_model_dir, load_weights

    cfg, name = load_model_dir(args.model)
    hybrid = isinstance(cfg, HybridConfig)
    dtype = getattr(torch, _DTYPES[args.dtype])
    if dtype == torch.float32 and not hybrid:
        print("float32 is only available for the hybrid decoders", file=sys.stderr)
        raise SystemExit(3)
    # replaying a trace through a hybrid decoder touches its own kernels and the library GEMM only; drawing tokens and the
    # dense families need the rest
    ensure_built(("mix", "gemm") if hybrid and args.cmd == "trace" else ("hip", "mix", "gemm"))
    pages = -(-num_tokens // page_size)
    ecfg = EngineConfig(model=cfg, dtype=dtype, max_running_req=max_running_req, page_size=page_size, num_page_override=pages,
                        max_seq_len_override=pages * page_size, cuda_graph_bs=graphs, gemm_tune="off", refine_in_graph=False)
    eng = Engine(ecfg, torch.device("cuda:0"))
    load_weights(eng.model, args.model, name)
    return eng


def cmd_trace(args) -> int:
    import numpy as np
    import torch

    from .offline import StepReplayer

    out = Path(args.out)
    out.mkdir(parents=True, exist_ok=True)
    eng = _engine(args, max_running_req=args.max_requests, num_tokens=args.max_tokens, graphs=[], page_size=args.page_size)
    rep = StepReplayer(eng, seed=0)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        logits = rep.step(step.get("entries", ()), step.get("end", ()))
        if logits is not None:
            np.ascontiguousarray(logits.float().cpu().numpy().astype("<f4")).tofile(str(out / f"{step['step']}.f32"))
        else:
            torch.cuda.synchronize()
        print(f"done {step['step']}", flush=True)
    eng.shutdown()
    return 0


def cmd_generate(args) -> int:
    from .core import SamplingParams
    from .offline import OfflineRunner

    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in args.prompt]
    longest = max(len(p) for p in prompts) + args.max_tokens
    bs = [b for b in (1, 2, 4, 8, 16, 32) if b <= max(len(prompts), 1)] if not args.no_graphs else []
    eng = _engine(args, max_running_req=max(len(prompts), 1), num_tokens=len(prompts) * (longest + args.page_size),
                  graphs=bs, page_size=args.page_size)
    run = OfflineRunner(eng, max_extend_tokens=args.chunk, seed=0)
    sp = SamplingParams(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p, ignore_eos=True, max_tokens=args.max_tokens)
    stats = run.generate(prompts, [sp] * len(prompts))
    for p, st in zip(prompts, run.last_states):
        print(json.dumps({"prompt": p, "output": run.output_ids(st)}))
    print(json.dumps({"decode_steps": stats["decode_steps"], "wall_s": round(stats["wall_s"], 4)}), file=sys.stderr)
    eng.shutdown()
    return 0


def main(argv=None) -> int:
    os.environ.setdefault("HSA_ENABLE_IPC_MODE_LEGACY", "0")
    ap = argparse.ArgumentParser(prog="mini_sglang_amd")
    sub = ap.add_subparsers(dest="cmd", required=True)
    t = sub.add_parser("trace", help="replay recorded steps from standard input, write logits")
    t.add_argument("--model", required=True)
    t.add_argument("--dtype", default="bfloat16", choices=sorted(_DTYPES))
    t.add_argument("--out", required=True)
    t.add_argument("--max-tokens", type=int, required=True, help="tokens the cache pool holds")
    t.add_argument("--max-requests", type=int, default=4, help="request rows / recurrent-state slots")
    t.add_argument("--page-size", type=int, default=16)
    g = sub.add_parser("generate", help="generate from prompts given as comma-separated token ids")
    g.add_argument("--model", required=True)
    g.add_argument("--dtype", default="bfloat16", choices=sorted(_DTYPES))
    g.add_argument("--prompt", action="append", required=True)
    g.add_argument("--max-tokens", type=int, default=16)
    g.add_argument("--temperature", type=float, default=0.0)
    g.add_argument("--top-k", type=int, default=-1)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--chunk", type=int, default=8192, help="token budget of one prefill forward")
    g.add_argument("--page-size", type=int, default=16)
    g.add_argument("--no-graphs", action="store_true")
    args = ap.parse_args(argv)
    return cmd_trace(args) if args.cmd == "trace" else cmd_generate(args)


if __name__ == "__main__":
    sys.exit(main())
