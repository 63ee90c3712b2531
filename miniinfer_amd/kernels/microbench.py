"""Times single kernels of the library under HIP-graph replay, so that the figure is device time without launch gaps.

    python -m miniinfer_amd.kernels.microbench product --rows 8 --n 25600 --k 5120 --gate-up
    python -m miniinfer_amd.kernels.microbench prefill-attention --tokens 2048 --heads 16 --kv-heads 8 --head-dim 128

`product` times the weight-streaming product (`ops.gemm_skinny`) beside the library's product for the same operands;
the weights cycle through several copies so that they stream from memory, not from a cache.  `prefill-attention`
times `ops.attn_prefill` for one prompt in both of its variants.  Both print one line per measurement; under
`rocprofv3 --pmc ...` the same commands give the kernels' counters.
"""

from __future__ import annotations

import argparse
import sys

import torch

from . import ops

DEV = "cuda:0"


def graph_time_us(fn, calls: int) -> float:
  """Microseconds per call of `fn`, from one replay of a graph that holds `calls` calls."""
  fn()
  torch.cuda.synchronize()
  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):
    fn()
  torch.cuda.current_stream().wait_stream(side)
  torch.cuda.synchronize()
  g = torch.cuda.CUDAGraph()
  with torch.cuda.graph(g):
    for _ in range(calls):
      fn()
  g.replay()
  torch.cuda.synchronize()
  start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
  start.record()
  g.replay()
  end.record()
  torch.cuda.synchronize()
  return start.elapsed_time(end) / calls * 1e3


def cmd_product(args) -> int:
  rows_w = 2 * args.n if args.gate_up else args.n
  nbytes = rows_w * args.k * 2
  copies = max(2, min(8, (1536 << 20) // nbytes))
  ws = [(torch.randn(rows_w, args.k, device=DEV) * 0.02).bfloat16() for _ in range(copies)]
  a = torch.randn(args.rows, args.k, device=DEV).bfloat16()
  out = torch.empty(args.rows, args.n, dtype=torch.bfloat16, device=DEV)
  turn = [0]

  def ours():
    ops.gemm_skinny(a, ws[turn[0] % copies], out, gate_up=args.gate_up)
    turn[0] += 1

  def library():
    torch.matmul(a, ws[turn[0] % copies].t())
    turn[0] += 1

  calls = copies * max(1, args.calls // copies)
  for name, fn in (("gemm_skinny", ours), ("library", library)):
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
  for variant in ("two_tiles", "dense"):
    t = graph_time_us(lambda: ops.attn_prefill(q, nq, nkv, d, out, kp, vp, table, work, cu, kv, d ** -0.5, 0,
                                               variant=variant), args.calls)
    print(f"attn_prefill {variant}: {L} tokens, {nq}/{nkv} heads of {d}, {len(work) * nkv} workgroups: {t:.1f} us, "
          f"{flops / t / 1e6:.0f} TFLOP/s")
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
  p.set_defaults(fn=cmd_product)
  a = sub.add_parser("prefill-attention", help="the MFMA prefill attention for one prompt")
  a.add_argument("--tokens", type=int, default=2048)
  a.add_argument("--heads", type=int, default=16)
  a.add_argument("--kv-heads", type=int, default=8)
  a.add_argument("--head-dim", type=int, default=128)
  a.add_argument("--page-size", type=int, default=16)
  a.add_argument("--calls", type=int, default=20)
  a.set_defaults(fn=cmd_prefill_attention)
  args = ap.parse_args(argv)
  if not torch.cuda.is_available():
    print("miniinfer_amd runs on the GPU only", file=sys.stderr)
    return 2
  return args.fn(args)


if __name__ == "__main__":
  sys.exit(main())
