"""Times single kernels of the library under HIP-graph replay, so that the figure is device time without launch gaps.

    python -m miniinfer_amd.kernels.microbench product --rows 8 --n 25600 --k 5120 --gate-up
    python -m miniinfer_amd.kernels.microbench prefill-attention --tokens 2048 --heads 16 --kv-heads 8 --head-dim 128
    python -m miniinfer_amd.kernels.microbench decode-attention --batch 8 --context 2048 --heads 16 --kv-heads 8
    python -m miniinfer_amd.kernels.microbench prompt-front --tokens 2048
    python -m miniinfer_amd.kernels.microbench choices --preset qwen3-8b

`product` times the weight-streaming product (`ops.gemm_skinny`) beside the library's product for the same operands;
the weights cycle through several copies so that they stream from memory, not from a cache.  `prefill-attention`
times `ops.attn_prefill` for one prompt in both of its variants; `decode-attention` times the split-key decode
kernel and its merge for a batch of requests, with and without the fused norm, rotation and cache write, over
several caches in turn; `prompt-front` times what precedes attention for a prompt's portion (head norms, rotation,
both cache writes: `ops.qk_norm_rope_cache`) beside a plain read and write of the same projection; `choices` builds a preset's model with random weights and prints what an engine measures
at its start: the time of the own and of the library kernel for each of the model's products at 1 to 64 rows.
All print one line per measurement; under
`rocprofv3 --pmc ...` the same commands give the kernels' counters.
"""

from __future__ import annotations

import argparse
import sys

import torch

from . import ops
from .tuning import graph_time_us

DEV = "cuda:0"


def cmd_product(args) -> int:
  rows_w = 2 * args.n if args.gate_up else args.n
  nbytes = rows_w * args.k * 2
  copies = args.copies or max(2, min(8, (1536 << 20) // nbytes))
  ws = [(torch.randn(rows_w, args.k, device=DEV) * 0.02).bfloat16() for _ in range(copies)]
  a = torch.randn(args.rows, args.k, device=DEV).bfloat16()
  out = torch.empty(args.rows, args.n, dtype=torch.bfloat16, device=DEV)
  turn = [0]

  def ours():
    ops.gemm_skinny(a, ws[turn[0] % copies], out, gate_up=args.gate_up, variant=0)
    turn[0] += 1

  def ours_ksplit():
    ops.gemm_skinny(a, ws[turn[0] % copies], out, gate_up=args.gate_up, variant=1)
    turn[0] += 1

  def ours_staged():
    ops.gemm_skinny(a, ws[turn[0] % copies], out, gate_up=args.gate_up, variant=2)
    turn[0] += 1

  def ours_staged_lines():
    ops.gemm_skinny(a, ws[turn[0] % copies], out, gate_up=args.gate_up, variant=4)
    turn[0] += 1

  def ours_both_staged():
    ops.gemm_skinny(a, ws[turn[0] % copies], out, gate_up=args.gate_up, variant=5)
    turn[0] += 1

  def ours_rows_shared_out():
    ops.gemm_skinny(a, ws[turn[0] % copies], out, gate_up=args.gate_up, variant=6)
    turn[0] += 1

  def library():
    torch.matmul(a, ws[turn[0] % copies].t())
    turn[0] += 1

  calls = copies * max(1, args.calls // copies)
  for name, fn in (("gemm_skinny", ours), ("gemm_skinny with the left operand staged", ours_staged),
                   ("gemm_skinny with the left operand staged and the weights in whole lines", ours_staged_lines),
                   ("gemm_skinny with both operands staged", ours_both_staged),
                   ("gemm_skinny with k split", ours_ksplit),
                   ("gemm_skinny with the rows of the left operand shared out", ours_rows_shared_out),
                   ("library", library)):
    t = graph_time_us(fn, calls)
    print(f"{name}: rows {args.rows}, weights [{rows_w}, {args.k}] {nbytes / 1e6:.1f} MB: {t:.1f} us, "
          f"{nbytes / t / 1e6:.2f} TB/s" + (" (without the activation)" if name == "library" and args.gate_up else ""))
  return 0


def cmd_prefill_attention(args) -> int:
  nq, nkv, d, P, L = args.heads, args.kv_heads, args.head_dim, args.page_size, args.tokens
  if not ops.mfma_attention_supported(torch.bfloat16, nq, nkv, d, P):
    print("these sizes go to the plain attention kernel, which this command does not time", file=sys.stderr)
    return 2
  pages = -(-L // P)
  g = torch.Generator(device=DEV).manual_seed(0)
  q = torch.randn(L, (nq + 2 * nkv) * d, device=DEV, generator=g).bfloat16()
  kp = torch.randn(pages + 1, nkv, P, d, device=DEV, generator=g).bfloat16()
  vp = torch.randn(pages + 1, nkv, d, P, device=DEV, generator=g).bfloat16()
  table = (torch.randperm(pages, device=DEV, generator=g) + 1).to(torch.int32).view(1, pages)
  cu = torch.tensor([0, L], dtype=torch.int32, device=DEV)
  kv = torch.tensor([L], dtype=torch.int32, device=DEV)
  out = torch.empty(L, nq * d, dtype=torch.bfloat16, device=DEV)
  tpb = ops.attn_prefill_tokens_per_block(nq, nkv, d)
  work = torch.tensor([(0, i) for i in reversed(range(-(-L // tpb)))], dtype=torch.int32, device=DEV)
  flops = 4 * nq * d * L * (L + 1) / 2
  tpb_wide = ops.attn_prefill_tokens_per_block(nq, nkv, d, wide=True)
  work_wide = torch.tensor([(0, i) for i in reversed(range(-(-L // tpb_wide)))], dtype=torch.int32, device=DEV) \
      if tpb_wide else None
  for variant in ("two_tiles", "dense") + (("wide",) if tpb_wide else ()):
    wk = work_wide if variant == "wide" else work
    t = graph_time_us(lambda: ops.attn_prefill(q, nq, nkv, d, out, kp, vp, table, wk, cu, kv, d ** -0.5, 0,
                                               variant=variant), args.calls)
    print(f"attn_prefill {variant}: {L} tokens, {nq}/{nkv} heads of {d}, {len(wk) * nkv} workgroups: {t:.1f} us, "
          f"{flops / t / 1e6:.0f} TFLOP/s")
  return 0


def cmd_decode_attention(args) -> int:
  from ..parts.attention import decode_launch, decode_splits
  nq, nkv, d, P, B, L = args.heads, args.kv_heads, args.head_dim, args.page_size, args.batch, args.context
  if not ops.mfma_attention_supported(torch.bfloat16, nq, nkv, d, P):
    print("these sizes go to the plain attention kernel, which this command does not time", file=sys.stderr)
    return 2
  per_req = -(-L // P)
  pages = B * per_req
  cache_bytes = 2 * pages * nkv * P * d * 2
  copies = args.copies or max(2, min(8, (1536 << 20) // cache_bytes))
  g = torch.Generator(device=DEV).manual_seed(0)
  caches = [(torch.randn(pages + 1, nkv, P, d, device=DEV, generator=g).bfloat16(),
             torch.randn(pages + 1, nkv, d, P, device=DEV, generator=g).bfloat16()) for _ in range(copies)]
  if args.pages == "ascending":        # request after request, as a free list in plain ascending order would hand them out
    table = (torch.arange(pages, device=DEV) + 1).to(torch.int32).view(B, per_req)
  elif args.pages == "pool":           # as the engine's page pool hands them out
    from ..cache.manager import PagePool
    pool = PagePool(pages)
    table = torch.tensor([pool.alloc(per_req) for _ in range(B)], dtype=torch.int32, device=DEV)
  else:
    table = (torch.randperm(pages, device=DEV, generator=g) + 1).to(torch.int32).view(B, per_req)
  qkv = torch.randn(B, (nq + 2 * nkv) * d, device=DEV, generator=g).bfloat16()
  cu = torch.arange(B + 1, dtype=torch.int32, device=DEV)
  kv = torch.full((B,), L, dtype=torch.int32, device=DEV)
  positions = torch.full((B,), L - 1, dtype=torch.int32, device=DEV)
  slots = (table[:, (L - 1) // P].to(torch.int64) * P + (L - 1) % P).to(torch.int32)
  weight = torch.ones(d, device=DEV)
  angles = torch.rand(L, d // 2, device=DEV, generator=g)
  cos_sin = torch.cat([angles.cos(), angles.sin()], dim=1).contiguous()
  out = torch.empty(B, nq * d, dtype=torch.bfloat16, device=DEV)
  tile_keys, waves = ops.attn_decode_geometry(d)
  splits, wide = decode_launch(B * nkv, L, tile_keys, waves, 2 * ops.compute_units())
  if args.wide != "auto":
    wide = args.wide == "on"
    splits = decode_splits(B * nkv, L, tile_keys, waves, 2 * ops.compute_units())
    splits = (splits + 1) // 2 if wide and splits >= 2 else splits
  splits = args.splits or splits
  part_o = torch.empty(B * nq * splits * d, device=DEV)
  part_ml = torch.empty(B * nq * splits * 2, device=DEV)
  turn = [0]

  streams = ops.decode_streams_keys(B, nkv, d, L) if args.stream_keys == "auto" else args.stream_keys == "on"

  def plain():
    k, v = caches[turn[0] % copies]
    turn[0] += 1
    ops.attn_decode(qkv, nq, nkv, d, out, k, v, table, cu, kv, 0, B, splits, part_o, part_ml, d ** -0.5, 0, streams, wide)

  def front():
    k, v = caches[turn[0] % copies]
    turn[0] += 1
    ops.attn_decode_front(qkv, nq, nkv, d, out, k, v, table, cu, kv, 0, B, splits, part_o, part_ml, d ** -0.5, 0,
                          weight, weight, 1e-6, cos_sin, positions, slots, streams, wide)

  calls = copies * max(1, args.calls // copies)
  for name, fn in (("attn_decode", plain), ("attn_decode_front", front)):
    t = graph_time_us(fn, calls)
    print(f"{name}: {B} requests of {L} tokens, {nq}/{nkv} heads of {d}, {splits} splits, "
          f"{ops.attn_decode_geometry(d, wide)[1]} waves a workgroup, "
          f"{'nontemporal' if streams else 'ordinary'} loads, cache {cache_bytes / 1e6:.1f} MB: "
          f"{t:.1f} us with the merge, {cache_bytes / t / 1e6:.2f} TB/s")
  return 0


def cmd_prompt_front(args) -> int:
  """What precedes attention for a prompt's portion: head norms, rotation, and both cache writes, one launch."""
  nq, nkv, d, P, T = args.heads, args.kv_heads, args.head_dim, args.page_size, args.tokens
  g = torch.Generator(device=DEV).manual_seed(0)
  copies = max(2, min(8, (1024 << 20) // max(1, T * (nq + 2 * nkv) * d * 2 * 2)))
  pages = -(-T // P) + 1
  qkvs = [torch.randn(T, (nq + 2 * nkv) * d, device=DEV, generator=g).bfloat16() for _ in range(copies)]
  kps = [torch.zeros(pages + 1, nkv, P, d, device=DEV, dtype=torch.bfloat16) for _ in range(copies)]
  vps = [torch.zeros(pages + 1, nkv, d, P, device=DEV, dtype=torch.bfloat16) for _ in range(copies)]
  weight = torch.ones(d, device=DEV)
  angles = torch.rand(T, d // 2, device=DEV, generator=g)
  cos_sin = torch.cat([angles.cos(), angles.sin()], dim=1).contiguous()
  positions = torch.arange(T, device=DEV, dtype=torch.int32)
  slots = torch.arange(T, device=DEV, dtype=torch.int32) + P         # a prompt's tokens fill pages one after the other
  turn = [0]

  def front():
    i = turn[0] % copies
    turn[0] += 1
    ops.qk_norm_rope_cache(qkvs[i], nq, nkv, d, weight, weight, 1e-6, cos_sin, positions, kps[i], vps[i], slots, P)

  def scale():
    i = turn[0] % copies
    turn[0] += 1
    qkvs[i].mul_(1.0)

  calls = copies * max(1, args.calls // copies)
  moved = T * ((nq + nkv) * d * 2 * 2 + nkv * d * 2 * 3)      # q, k read and written in place; k, v into the cache; v read
  t = graph_time_us(front, calls)
  print(f"qk_norm_rope_cache: {T} tokens, {nq}/{nkv} heads of {d}, pages of {P}: {t:.1f} us, "
        f"{moved / 1e6:.1f} MB moved, {moved / t / 1e6:.2f} TB/s")
  t = graph_time_us(scale, calls)
  print(f"for comparison, x *= 1 over the same projection (torch): {t:.1f} us, "
        f"{T * (nq + 2 * nkv) * d * 4 / t / 1e6:.2f} TB/s")
  return 0


def cmd_choices(args) -> int:
  from ..config import model_spec_of
  from ..presets import preset
  from ..weights import build_model, fill_random
  from .tuning import tune_products
  model = build_model(model_spec_of(preset(args.preset, args.num_hidden_layers)), torch.bfloat16, torch.device(DEV))
  fill_random(model, 0)
  tune_products(model.products(), log=print)
  return 0


def main(argv=None) -> int:
  ap = argparse.ArgumentParser(prog="python -m miniinfer_amd.kernels.microbench")
  sub = ap.add_subparsers(dest="cmd", required=True)
  p = sub.add_parser("product", help="the weight-streaming product beside the library's")
  p.add_argument("--rows", type=int, default=8)
  p.add_argument("--n", type=int, required=True, help="output columns (for --gate-up: of each half)")
  p.add_argument("--k", type=int, required=True)
  p.add_argument("--gate-up", action="store_true", help="a fused gate|up matrix [2 n, k] with the activation in the epilogue")
  p.add_argument("--calls", type=int, default=24)
  p.add_argument("--copies", type=int, default=0,
                 help="matrices the calls cycle through (default: up to 8, 1.5 GB at most); with many, the weights "
                      "come from memory and not from a cache that holds the few")
  p.set_defaults(fn=cmd_product)
  a = sub.add_parser("prefill-attention", help="the MFMA prefill attention for one prompt")
  a.add_argument("--tokens", type=int, default=2048)
  a.add_argument("--heads", type=int, default=16)
  a.add_argument("--kv-heads", type=int, default=8)
  a.add_argument("--head-dim", type=int, default=128)
  a.add_argument("--page-size", type=int, default=16)
  a.add_argument("--calls", type=int, default=20)
  a.set_defaults(fn=cmd_prefill_attention)
  d = sub.add_parser("decode-attention", help="the split-key decode attention and its merge")
  d.add_argument("--batch", type=int, default=8)
  d.add_argument("--context", type=int, default=2048)
  d.add_argument("--heads", type=int, default=16)
  d.add_argument("--kv-heads", type=int, default=8)
  d.add_argument("--head-dim", type=int, default=128)
  d.add_argument("--page-size", type=int, default=16)
  d.add_argument("--splits", type=int, default=0, help="key ranges per request (default: the engine's choice)")
  d.add_argument("--calls", type=int, default=24)
  d.add_argument("--pages", choices=["shuffled", "ascending", "pool"], default="shuffled",
                 help="which pages the requests hold: a random choice, request after request in ascending order, or "
                      "as the engine's page pool hands them out")
  d.add_argument("--wide", choices=["auto", "on", "off"], default="auto",
                 help="workgroups of twice the waves and half the key ranges (auto: the engine's rule, decode_launch)")
  d.add_argument("--stream-keys", choices=["auto", "on", "off"], default="auto",
                 help="nontemporal loads of the keys and values (auto: the engine's rule, ops.decode_streams_keys)")
  d.add_argument("--copies", type=int, default=0,
                 help="caches the calls cycle through, as a model's layers do (default: 2 to 8, 1.5 GB at most)")
  d.set_defaults(fn=cmd_decode_attention)
  f = sub.add_parser("prompt-front", help="head norms, rotation and cache writes of a prompt's portion")
  f.add_argument("--tokens", type=int, default=2048)
  f.add_argument("--heads", type=int, default=16)
  f.add_argument("--kv-heads", type=int, default=8)
  f.add_argument("--head-dim", type=int, default=128)
  f.add_argument("--page-size", type=int, default=16)
  f.add_argument("--calls", type=int, default=24)
  f.set_defaults(fn=cmd_prompt_front)
  c = sub.add_parser("choices", help="own against library kernel for each product of a preset's model")
  c.add_argument("--preset", default="qwen3-0.6b")
  c.add_argument("--num-hidden-layers", type=int, default=None)
  c.set_defaults(fn=cmd_choices)
  args = ap.parse_args(argv)
  if not torch.cuda.is_available():
    print("miniinfer_amd runs on the GPU only", file=sys.stderr)
    return 2
  return args.fn(args)


if __name__ == "__main__":
  sys.exit(main())
