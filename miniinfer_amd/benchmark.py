"""Decode and prefill throughput of the engine on one MI355X, Qwen3-0.6B shape, random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 2048] [--preset qwen3-0.6b]
    python bench.py --mixed [--preset qwen3-8b] [--num-seqs 64] [--min-input 128] [--max-input 2048] [--output-len 256]
    python -m miniinfer_amd bench ...        (the same program)

A step is one decode step of the whole engine (schedule, batch building, model, sampling) with `batch`
requests that each hold `context` tokens in the cache.  Prints ONE JSON line: decoded tokens a second, the
2,048-token prefill, the decode step's HBM roofline, decode at batch 1 and 64, and (from a second engine with
longer sequences and more request slots, so that the first engine's figures do not depend on them) decode at batch
256 and at contexts of 32,768 tokens.  Fractions are given against the data sheet's peaks and against what two bare
kernels measure on this device when the run starts (one that only reads memory, one that only feeds the matrix
cores).

`--mixed` runs the serving workload instead: `num-seqs` requests with random prompts of `min-input` to `max-input`
tokens (uniform) and exactly `output-len` sampled tokens each, all added at once, so that the steps mix prompt
portions (token budget 8,192) with decoded tokens (the reference's benchmark/bench_miniinfer.py:28-58 with its
workload's numbers).  Prints one JSON line with output and input tokens a second, steps and preemptions.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}


def model_numbers(cfg, layers):
  H, I, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
  nq, nkv, d = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
  per_layer = (nq + 2 * nkv) * d * H + nq * d * H + 3 * H * I
  return dict(linear_params=per_layer * layers, head_params=V * H, kv_per_token=2 * layers * nkv * d)


def decode_bytes(cfg, layers, batch, context, esize):
  n = model_numbers(cfg, layers)
  return (n["linear_params"] + n["head_params"]) * esize + batch * context * n["kv_per_token"] * esize


def prefill_flops(cfg, layers, T):
  n = model_numbers(cfg, layers)
  attn = layers * 4 * cfg.num_attention_heads * cfg.head_dim * (T * (T + 1) // 2)
  return 2 * T * n["linear_params"] + attn + 2 * n["head_params"]


def decode_room(batch, context, steps, warmup, budget=8192):
  """Tokens a request of `time_decode` may come to hold: its context, the timed and untimed steps, and the steps it
  decodes while the other requests' prompts are still being run."""
  return context + steps + warmup + (-(-batch * context // budget) + 1) + 4


def time_decode(engine, batch, context, steps, warmup, seed):
  """`batch` requests with `context` random tokens each, prefilled through the engine; then `warmup` untimed and
  `steps` timed decode steps.  Returns seconds per step."""
  import torch
  from random import Random
  from miniinfer_amd import SamplingParams
  rnd = Random(seed)
  V = engine.model.spec.vocab_size
  # requests whose prompts go first decode while the others are still prefilled: leave room for that
  stagger = -(-batch * context // engine.config.max_num_batched_tokens) + 1
  sp = SamplingParams(temperature=0.0, max_tokens=warmup + steps + stagger + 2, ignore_eos=True)
  for _ in range(batch):
    engine.add_request([rnd.randrange(V) for _ in range(context)], sp)
  # prefill until every request is decoding
  while any(r.remaining != 1 or r.num_computed == 0 for r in engine.scheduler.running) or engine.scheduler.waiting:
    engine.step()
  for _ in range(warmup):
    engine.step()
  torch.cuda.synchronize()
  t0 = time.perf_counter()
  for _ in range(steps):
    so = engine.step()
    assert so.num_decode_tokens == batch and so.num_prefill_tokens == 0
  torch.cuda.synchronize()
  dt = (time.perf_counter() - t0) / steps
  while not engine.is_finished():
    engine.step()
  return dt


def time_prefill(engine, T, reps, seed):
  import torch
  from random import Random
  from miniinfer_amd import SamplingParams
  rnd = Random(seed)
  V = engine.model.spec.vocab_size
  sp = SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True)
  times = []
  for i in range(reps + 1):
    engine.add_request([rnd.randrange(V) for _ in range(T)], sp)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    tokens = done = 0
    while not engine.is_finished():     # one step runs the prompt; the engine may book it one call later
      so = engine.step()
      tokens += so.num_prefill_tokens
      done += len(so.finished)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert tokens == T and done == 1
    if i > 0:
      times.append(dt)
  return min(times)


def run_mixed(args) -> int:
  import torch
  from random import Random
  from miniinfer_amd import LLMEngine, SamplingParams
  from miniinfer_amd.kernels import ops
  from miniinfer_amd.presets import preset

  full = preset(args.preset)
  cfg = preset(args.preset, args.layers) if args.layers else full
  page_size = 16
  max_len = args.max_input + args.output_len + 16
  pages = args.mixed_pages or args.num_seqs * (-(-max_len // page_size)) + 16
  hbm_gbs, mfma_tflops = ops.measured_peaks()
  engine = LLMEngine(model="", model_config=cfg, random_weights_seed=0, dtype=args.dtype, page_size=page_size,
                     num_pages=pages, max_num_seqs=args.num_seqs, max_model_len=max_len, max_num_batched_tokens=8192,
                     enforce_eager=args.eager, tune_products=not args.no_tune, enable_overlap=not args.no_overlap)
  rnd = Random(0)
  V = cfg.vocab_size
  prompts = [[rnd.randrange(V) for _ in range(rnd.randint(args.min_input, args.max_input))] for _ in range(args.num_seqs)]
  sp = SamplingParams(temperature=0.6, ignore_eos=True, max_tokens=args.output_len)
  engine.generate([prompts[0][:8]], SamplingParams(temperature=0.6, max_tokens=2, ignore_eos=True), use_tqdm=False)
  engine.warm_up(args.num_seqs, max_len)
  torch.cuda.synchronize()
  steps0, pre0 = engine.num_steps, engine.scheduler.num_preemptions
  t0 = time.perf_counter()
  outs = engine.generate(prompts, sp, use_tqdm=False)
  torch.cuda.synchronize()
  dt = time.perf_counter() - t0
  n_out = sum(len(o["token_ids"]) for o in outs)
  n_in = sum(len(p) for p in prompts)
  assert n_out == args.num_seqs * args.output_len
  esize = 2 if args.dtype == "bfloat16" else 4
  n = model_numbers(cfg, cfg.num_hidden_layers)
  shape_name = {"qwen3-0.6b": "Qwen3-0.6B", "qwen3-8b": "Qwen3-8B", "qwen3-32b": "Qwen3-32B"}.get(args.preset, args.preset)
  steps = engine.num_steps - steps0
  # what the run must at least do: every weight once per step, and 2 flops per weight and token
  flops = 2.0 * (n_in + n_out) * n["linear_params"] + 2.0 * n_out * n["head_params"]
  rec = {
    "metric": f"output tok/s, {args.num_seqs} requests, prompts {args.min_input}-{args.max_input}, "
              f"{args.output_len} outputs each, mixed chunked-prefill/decode steps, {shape_name} shape",
    "value": round(n_out / dt, 1), "unit": "tok/s", "n_gpus": 1, "higher_is_better": True,
    "input_tok_s": round(n_in / dt, 1), "total_tok_s": round((n_in + n_out) / dt, 1), "seconds": round(dt, 3),
    "engine_steps": steps, "ms_per_step": round(dt / steps * 1e3, 3),
    "preemptions": engine.scheduler.num_preemptions - pre0, "input_tokens": n_in, "output_tokens": n_out,
    "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (seeded random token ids, random weights)",
    "config": {"model": args.preset, "layers": cfg.num_hidden_layers, "layers_full": full.num_hidden_layers,
               "hidden": cfg.hidden_size, "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
               "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
               "num_seqs": args.num_seqs, "min_input": args.min_input, "max_input": args.max_input,
               "output_len": args.output_len, "token_budget": 8192, "page_size": page_size, "pages": pages,
               "graphs": not args.eager, "overlap": not args.no_overlap, "temperature": 0.6},
    "weights_gbs": round(steps * (n["linear_params"] + n["head_params"]) * esize / dt / 1e9, 1),
    "frac_flops": round(flops / dt / PEAK_FLOPS[args.dtype], 4),
    "measured": {"hbm_gbs": round(hbm_gbs, 1), "mfma_bf16_tflops": round(mfma_tflops, 1)},
  }
  print(json.dumps(rec))
  return 0


def main(argv=None) -> int:
  ap = argparse.ArgumentParser(prog="bench")
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=64)
  ap.add_argument("--warmup", type=int, default=8)
  ap.add_argument("--batch", type=int, default=8)
  ap.add_argument("--context", type=int, default=2048)
  ap.add_argument("--preset", default=None, help="default: qwen3-0.6b, and qwen3-8b for --mixed")
  ap.add_argument("--layers", type=int, default=None, help="fewer layers than the preset (named in the record)")
  ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
  ap.add_argument("--eager", action="store_true")
  ap.add_argument("--no-tune", action="store_true", help="choose product kernels by rule instead of timing them at start")
  ap.add_argument("--no-points", action="store_true", help="skip batch 1 / 64 and the prefill")
  ap.add_argument("--only-prefill", action="store_true", help="run only the prefill (for profiling)")
  ap.add_argument("--prefill-tokens", type=int, default=2048,
                  help="with --only-prefill: tokens of the prompt (one step of that many tokens; default 2,048)")
  ap.add_argument("--no-overlap", action="store_true", help="read every step's tokens back before the next step is launched")
  ap.add_argument("--mixed", action="store_true", help="the serving workload: many requests, prompts and decodes mixed")
  ap.add_argument("--num-seqs", type=int, default=64)
  ap.add_argument("--min-input", type=int, default=128)
  ap.add_argument("--max-input", type=int, default=2048)
  ap.add_argument("--output-len", type=int, default=256)
  ap.add_argument("--mixed-pages", type=int, default=0, help="pages of the cache for --mixed (default: room for all)")
  ap.add_argument("--no-long-points", action="store_true",
                  help="skip the second engine's points (batch 256, contexts of 32,768 tokens)")
  args = ap.parse_args(argv)
  if args.gpus != 1:
    print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
    return 2
  if args.preset is None:
    args.preset = "qwen3-8b" if args.mixed else "qwen3-0.6b"
  if args.mixed:
    return run_mixed(args)

  import torch
  from miniinfer_amd import LLMEngine
  from miniinfer_amd.kernels import ops
  from miniinfer_amd.presets import preset

  full = preset(args.preset)
  cfg = preset(args.preset, args.layers) if args.layers else full
  layers = cfg.num_hidden_layers
  hbm_gbs, mfma_tflops = ops.measured_peaks()     # what a bare read loop and a bare matrix-core loop reach here
  mfma_flops = mfma_tflops * 1e12 if args.dtype == "bfloat16" else None
  if args.only_prefill:
    args.context, args.batch, args.no_points = max(args.context, args.prefill_tokens), 1, True
  max_batch = max(args.batch, 1 if args.no_points else 64)
  page_size = 16
  room = args.context + args.steps + args.warmup + (-(-max_batch * args.context // 8192)) + 16
  max_len = max(4096, room)
  pages = max_batch * (-(-room // page_size)) + 16
  engine = LLMEngine(model="", model_config=cfg, random_weights_seed=0, dtype=args.dtype, page_size=page_size,
                     num_pages=pages, max_num_seqs=max_batch, max_model_len=max_len,
                     max_num_batched_tokens=max(8192, args.prefill_tokens if args.only_prefill else 0),
                     enforce_eager=args.eager, tune_products=not args.no_tune, enable_overlap=not args.no_overlap)
  esize = 2 if args.dtype == "bfloat16" else 4
  if args.only_prefill:
    T = args.prefill_tokens
    psec = time_prefill(engine, T, reps=max(1, args.steps), seed=2)
    fl = prefill_flops(cfg, layers, T)
    print(json.dumps({"prefill": {"value": round(T / psec, 1), "tokens": T, "ms": round(psec * 1e3, 3),
                                  "frac": round(fl / psec / PEAK_FLOPS[args.dtype], 4),
                                  "frac_measured": round(fl / psec / mfma_flops, 4) if mfma_flops else None}}))
    return 0

  sec = time_decode(engine, args.batch, args.context, args.steps, args.warmup, seed=1)
  value = args.batch / sec
  mid_context = args.context + args.warmup + args.steps // 2
  bytes_step = decode_bytes(cfg, layers, args.batch, mid_context, esize)
  achieved = bytes_step / sec / 1e9
  shape_name = {"qwen3-0.6b": "Qwen3-0.6B", "qwen3-8b": "Qwen3-8B", "qwen3-32b": "Qwen3-32B"}.get(args.preset, args.preset)
  rec = {
    "metric": f"decode tok/s @ batch {args.batch}, {args.context:,}-token contexts, {shape_name} shape",
    "value": round(value, 2),
    "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(sec * 1e3, 4),
    "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
    "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (seeded random token ids, random weights)",
    "config": {
      "model": args.preset, "layers": layers, "layers_full": full.num_hidden_layers, "hidden": cfg.hidden_size,
      "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
      "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size, "tied_head": cfg.tie_word_embeddings,
      "global_batch": args.batch, "seq_len": args.context, "max_model_len": max_len, "page_size": page_size,
      "parallelism": "1 GPU", "graphs": not args.eager, "prefill_tokens": 2048,
    },
    "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                 "frac": round(achieved / PEAK_HBM_GBS, 4), "peak_measured": round(hbm_gbs, 1),
                 "frac_measured": round(achieved / hbm_gbs, 4)},
    "measured": {"hbm_gbs": round(hbm_gbs, 1), "mfma_bf16_tflops": round(mfma_tflops, 1)},
  }
  if not args.no_points:
    T = 2048
    psec = time_prefill(engine, T, reps=3, seed=2)
    fl = prefill_flops(cfg, layers, T)
    rec["prefill"] = {"value": round(T / psec, 1), "tokens": T, "ms": round(psec * 1e3, 3),
                      "frac": round(fl / psec / PEAK_FLOPS[args.dtype], 4),
                      "frac_measured": round(fl / psec / mfma_flops, 4) if mfma_flops else None}
    points, fracs = {}, {}

    def point(eng, name, b, ctx, steps, warm):
      s = time_decode(eng, b, ctx, steps, warm, seed=10 + b + ctx)
      points[name] = round(b / s, 2)
      fracs[name] = round(decode_bytes(cfg, layers, b, ctx + warm + steps // 2, esize) / s / 1e9 / PEAK_HBM_GBS, 4)

    for b in (1, 64):
      point(engine, f"decode_b{b}", b, args.context, max(8, args.steps // 2), max(2, args.warmup // 2))
    rec["startup_s"] = round(engine.startup_seconds, 2)
    if not args.no_long_points and args.preset == "qwen3-0.6b":
      # further sizes from an engine of their own: 256 request slots and sequences of 32,768 tokens and more
      del engine
      torch.cuda.empty_cache()
      long_ctx = 32768
      steps_l = max(8, args.steps // 4)
      room_l = decode_room(8, long_ctx, steps_l, 2)
      pages_l = max(256 * (-(-decode_room(256, args.context, steps_l, 2) // page_size)),
                    8 * (-(-room_l // page_size))) + 64
      eng2 = LLMEngine(model="", model_config=cfg, random_weights_seed=0, dtype=args.dtype, page_size=page_size,
                       num_pages=pages_l, max_num_seqs=256, max_model_len=room_l, max_num_batched_tokens=8192,
                       enforce_eager=args.eager, tune_products=not args.no_tune, enable_overlap=not args.no_overlap)
      point(eng2, "decode_b256", 256, args.context, steps_l, 2)
      point(eng2, f"decode_b1_ctx{long_ctx}", 1, long_ctx, steps_l, 2)
      point(eng2, f"decode_b8_ctx{long_ctx}", 8, long_ctx, steps_l, 2)
    rec["points"] = points
    rec["points_frac_hbm"] = fracs       # each point's bytes (weights once, the live requests' cache) / time / 8 TB/s
  print(json.dumps(rec))
  return 0


if __name__ == "__main__":
  sys.exit(main())
