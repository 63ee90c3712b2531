"""Command line:  python -m miniinfer_amd <generate | random-model | throughput | replay | bench> ...

`generate` takes the options of the reference's example (examples/minimal_engine.py:24-55: --model,
--max-tokens, --temperature, --max-num-seqs, --max-model-len); `throughput` those of its benchmark
(benchmark/bench_miniinfer.py:16-26: --num-seqs, --max-input-len, --max-output-len, --max-num-seqs,
--max-model-len, --page-size, --eager) with the same workload: seeded random token ids, random lengths,
temperature 0.6, ignore_eos, throughput = total output tokens / time after a warm-up.  `replay` feeds given token
ids through the model step by step and writes logits (the program `bin/trace_run`; `engine/replay.py`); `bench`
measures decode and prefill throughput and prints one JSON line (the program `bench.py`; `benchmark.py`).
"""

from __future__ import annotations

import argparse
import json
import sys
import time
from random import Random


def _engine_args(p):
  p.add_argument("--model", default=None, help="folder with config.json and *.safetensors")
  p.add_argument("--preset", default=None,
                 help="instead of --model: a named shape (see `random-model`) with random weights drawn on the device")
  p.add_argument("--num-hidden-layers", type=int, default=None, help="with --preset: fewer layers than the shape has")
  p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
  p.add_argument("--max-num-seqs", type=int, default=4, help="most sequences in a batch")
  p.add_argument("--max-model-len", type=int, default=512, help="most tokens of one sequence")
  p.add_argument("--page-size", type=int, default=16)
  p.add_argument("--num-pages", type=int, default=None, help="cache pages (default: from free device memory)")
  p.add_argument("--max-num-batched-tokens", type=int, default=8192, help="token budget of one step")
  p.add_argument("--no-chunked-prefill", action="store_true")
  p.add_argument("--eager", action="store_true", help="never replay decode steps from HIP graphs")
  p.add_argument("--no-overlap", action="store_true",
                 help="read each step's tokens back before the next step is launched")
  p.add_argument("--no-tune", action="store_true",
                 help="choose the kernels of small-batch products by rule instead of timing them at start")
  p.add_argument("--seed", type=int, default=0)
  p.add_argument("--load-format", default="safetensors", choices=["safetensors", "random"],
                 help="random: only the folder's config.json is read, the weights are drawn on the device from --seed")
  p.add_argument("--fixed-kernel-choices", action="store_true",
                 help="products of few rows go where a rule sends them, never where a timing at start-up did, so that "
                      "a run's kernels and roundings do not depend on timings")


def _engine(args):
  from miniinfer_amd import LLMEngine
  extra = {}
  if (args.model is None) == (args.preset is None):
    raise SystemExit("give exactly one of --model and --preset")
  if args.preset is not None:
    from miniinfer_amd.presets import preset
    extra = dict(model_config=preset(args.preset, args.num_hidden_layers), random_weights_seed=args.seed)
  return LLMEngine(model=args.model or "", **extra, dtype=args.dtype, max_num_seqs=args.max_num_seqs,
                   max_model_len=args.max_model_len, page_size=args.page_size, num_pages=args.num_pages,
                   max_num_batched_tokens=args.max_num_batched_tokens,
                   enable_chunked_prefill=not args.no_chunked_prefill, enforce_eager=args.eager, enable_overlap=not args.no_overlap,
                   tune_products=not args.no_tune, seed=args.seed, timed_kernel_choices=not args.fixed_kernel_choices,
                   **({} if args.preset is not None else {"load_format": args.load_format}))


def cmd_generate(args) -> int:
  from miniinfer_amd import SamplingParams
  prompts = []
  for s in args.prompt or []:
    prompts.append(s)
  for s in args.prompt_ids or []:
    prompts.append([int(x) for x in s.replace(",", " ").split()])
  with _engine(args) as engine:
    if args.num_prompts:
      rnd = Random(args.seed)
      V = engine.model.spec.vocab_size
      prompts += [[rnd.randrange(V) for _ in range(args.prompt_len)] for _ in range(args.num_prompts)]
    if not prompts:
      print("give --prompt, --prompt-ids or --num-prompts", file=sys.stderr)
      return 2
    sp = SamplingParams(max_tokens=args.max_tokens, temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                        ignore_eos=args.ignore_eos)
    outs = engine.generate(prompts=prompts, sampling_params=sp, use_tqdm=not args.quiet)
  for p, o in zip(prompts, outs):
    print(json.dumps({"prompt": p, "token_ids": o["token_ids"], "text": o["text"],
                      "finish_reason": o["finish_reason"]}))
  return 0


def cmd_random_model(args) -> int:
  import torch
  from miniinfer_amd.presets import preset
  from miniinfer_amd.config import Qwen3Config, resolve_architecture
  from miniinfer_amd.weights import write_random_model
  if args.config:
    with open(args.config) as f:
      raw = json.load(f)
    _, cls = resolve_architecture(raw)
    cfg = cls.from_dict(raw)
  else:
    cfg = preset(args.preset, args.num_hidden_layers)
  dt = {"bfloat16": torch.bfloat16, "float32": torch.float32}[args.dtype]
  write_random_model(cfg, args.out, seed=args.seed, dtype=dt)
  print(f"wrote {args.out}")
  return 0


def cmd_throughput(args) -> int:
  from miniinfer_amd import SamplingParams
  rnd = Random(0)
  with _engine(args) as engine:
    V = engine.model.spec.vocab_size
    hi = min(10000, V - 1)
    prompts = [[rnd.randint(0, hi) for _ in range(rnd.randint(min(100, args.max_input_len), args.max_input_len))]
               for _ in range(args.num_seqs)]
    sps = [SamplingParams(temperature=0.6, ignore_eos=True,
                          max_tokens=rnd.randint(min(100, args.max_output_len), args.max_output_len))
           for _ in range(args.num_seqs)]
    engine.generate(prompts=[prompts[0][:8]], sampling_params=SamplingParams(), use_tqdm=False)   # warm-up
    engine.warm_up(min(args.num_seqs, args.max_num_seqs), min(args.max_model_len, args.max_input_len + args.max_output_len))
    t0 = time.time()
    engine.generate(prompts=prompts, sampling_params=sps, use_tqdm=False)
    dt = time.time() - t0
  total = sum(sp.max_tokens for sp in sps)
  total_in = sum(len(p) for p in prompts)
  print(f"[miniinfer_amd] Total: {total}tok, Time: {dt:.2f}s, Throughput: {total / dt:.2f}tok/s "
        f"(input {total_in}tok, {total_in / dt:.2f}tok/s)")
  return 0


def cmd_replay(args) -> int:
  from miniinfer_amd.engine.replay import run
  return run(args.model, args.dtype, args.out, args.max_tokens, page_size=args.page_size)


def main(argv=None) -> int:
  argv = list(sys.argv[1:] if argv is None else argv)
  if argv and argv[0] == "bench":            # the benchmark parses its own options
    from miniinfer_amd.benchmark import main as bench_main
    return bench_main(argv[1:])
  ap = argparse.ArgumentParser(prog="python -m miniinfer_amd")
  sub = ap.add_subparsers(dest="cmd", required=True)

  g = sub.add_parser("generate", help="generate from prompts")
  _engine_args(g)
  g.add_argument("--max-tokens", type=int, default=64, help="most tokens to generate")
  g.add_argument("--temperature", type=float, default=0.7, help="sampling temperature (0 = greedy)")
  g.add_argument("--top-k", type=int, default=0)
  g.add_argument("--top-p", type=float, default=1.0)
  g.add_argument("--ignore-eos", action="store_true")
  g.add_argument("--prompt", action="append", help="text prompt (needs tokenizer.json in the model folder)")
  g.add_argument("--prompt-ids", action="append", help="token ids, comma or space separated")
  g.add_argument("--num-prompts", type=int, default=0, help="that many random prompts")
  g.add_argument("--prompt-len", type=int, default=16)
  g.add_argument("--quiet", action="store_true")
  g.set_defaults(fn=cmd_generate)

  r = sub.add_parser("random-model", help="write a model folder with random weights")
  r.add_argument("--preset", default="tiny-a")
  r.add_argument("--config", help="a config.json to take the sizes from instead of a preset")
  r.add_argument("--num-hidden-layers", type=int, default=None)
  r.add_argument("--seed", type=int, default=0)
  r.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
  r.add_argument("--out", required=True)
  r.set_defaults(fn=cmd_random_model)

  t = sub.add_parser("throughput", help="output tokens per second of a random workload")
  _engine_args(t)
  t.add_argument("--num-seqs", type=int, default=256)
  t.add_argument("--max-input-len", type=int, default=1024)
  t.add_argument("--max-output-len", type=int, default=1024)
  t.set_defaults(fn=cmd_throughput, max_num_seqs=256, max_model_len=4096)

  rp = sub.add_parser("replay", help="feed a trace of token ids (JSON lines on stdin) through the model, write logits")
  rp.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
  rp.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
  rp.add_argument("--out", required=True, help="folder for <step>.f32 files")
  rp.add_argument("--max-tokens", type=int, required=True, help="tokens the cache pool is made for")
  rp.add_argument("--page-size", type=int, default=16)
  rp.set_defaults(fn=cmd_replay)

  sub.add_parser("bench", add_help=False, help="decode and prefill throughput as one JSON line (`bench --help`)")

  args = ap.parse_args(argv)
  return args.fn(args)


if __name__ == "__main__":
  sys.exit(main())
