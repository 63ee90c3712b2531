"""Which kernel runs a product of few rows is measured, not guessed.

For a matrix of tens of MB and a handful of rows there are these candidates: this library's weight-streaming kernel
(`ops.gemm_skinny`, whose epilogue can take a norm's halves or the gated activation) in its forms (every
workgroup owns whole rows of the result, with the operands straight from memory, the left one or both staged through
LDS, the weights in half or whole memory lines; or k is split across workgroups and a second kernel adds the partial
results), and the library product
(hipBLASLt through `torch.matmul`, which splits k across workgroups and so reads the left operand less often, but
needs the norm and the activation as kernels of their own).  Which is quicker depends on the shape and the number
of rows in ways no short rule covers, so `tune_products` times them on the model's own matrices once, when an
engine is built, and `ops.skinny_preferred` then answers from the table.  Matrices below `MIN_ELEMENTS` are not
timed: there the weight-streaming kernel and its fusions win by the kernels they save.
"""

from __future__ import annotations

from typing import Callable, Dict, Iterable, List, Optional, Tuple

import torch

from . import ops

MIN_ELEMENTS = 2 << 20
UNFUSED_US = 4.5          # what a norm or activation kernel of its own costs inside a decode step (2.7 us + the gap before it)
LINES_MIN_ELEMENTS = 16 << 20   # matrices from this size up are also timed with their weights fetched in whole lines
KSPLIT_MARGIN = 0.9       # the k-split kernel replaces the library's product only if it takes at most this much of its time
LIBRARY_MARGIN = 0.92     # and the library's replaces a one-kernel product of this library only at this much of its time
RULE_MARGIN = 1.05        # what the rule would run stays unless the quickest candidate beats it by this factor


def graph_time_us(fn: Callable[[], None], calls: int, flush: Optional[torch.Tensor] = None) -> float:
  """Microseconds per call of `fn`, from one replay of a graph that holds `calls` calls (device time, no launch
  gaps).  `flush`: a large tensor that is overwritten before the timed replay, so that nothing read is cached."""
  fn()
  torch.cuda.synchronize()
  side = ops.side_stream()
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
  best = float("inf")
  start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
  for _ in range(2):
    if flush is not None:
      flush.zero_()
    start.record()
    g.replay()
    end.record()
    torch.cuda.synchronize()
    best = min(best, start.elapsed_time(end) / calls * 1e3)
  return best


def tune_products(products: Iterable[Tuple[torch.Tensor, bool]], log: Optional[Callable[[str], None]] = None) -> int:
  """products: (weight [N, K] or fused gate|up [2 I, K], is gate|up) of every product that decode steps run; the
  same shape usually comes once per layer, and the timing walks through all of them in turn so that the weights
  come from memory as they do in a step.  Fills the table behind `ops.skinny_preferred` for every shape of at
  least MIN_ELEMENTS and every row count in `ops.TUNE_ROWS`; returns the number of shapes timed."""
  groups: Dict[tuple, List[torch.Tensor]] = {}
  for w, gate_up in products:
    if w is None or w.dtype != torch.bfloat16 or not w.is_cuda or w.dim() != 2 or w.numel() < MIN_ELEMENTS:
      continue
    groups.setdefault((w.shape[0], w.shape[1], bool(gate_up)), []).append(w)
  timed = 0
  flush = None
  for (rows_w, K, gate_up), ws in groups.items():
    N = rows_w // 2 if gate_up else rows_w
    if ops.product_choice_known(rows_w, K, gate_up):
      continue
    probe = torch.zeros(1, K, dtype=torch.bfloat16, device=ws[0].device)
    if not ops.gemm_skinny_supported(probe, ws[0]):
      continue
    if flush is None:
      flush = torch.empty(512 << 20, dtype=torch.uint8, device=ws[0].device)
    calls = max(8, min(len(ws), 32))
    for M in ops.TUNE_ROWS:
      a = (torch.randn(M, K, device=ws[0].device) * 0.1).bfloat16()
      out = torch.empty(M, N, dtype=torch.bfloat16, device=a.device)
      turn = [0]

      def own(variant):
        def run():
          ops.gemm_skinny(a, ws[turn[0] % len(ws)], out, gate_up=gate_up, variant=variant)
          turn[0] += 1
        return run

      def library():
        torch.matmul(a, ws[turn[0] % len(ws)].t())
        turn[0] += 1

      # The kernel in which a workgroup owns whole rows of the result, in its forms: with the left operand staged
      # through LDS it is a few tenths of a microsecond slower when the operand is small and up to a quarter quicker
      # when it is not; with the weights fetched in whole memory lines, by loads into registers and an exchange
      # between lanes, large matrices stream up to a sixth faster and small ones slower; with both operands through
      # LDS (up to 16 rows) most shapes run a few percent quicker (small ones do not inside a step, and are not timed).
      # Which, depends on the shape.
      forms = {ops.OWN_ROWS: graph_time_us(own(0), calls, flush)}
      stage = M >= ops.STAGED_MIN_ROWS and K % 32 == 0
      if stage:
        forms[ops.OWN_ROWS_STAGED] = graph_time_us(own(2), calls, flush)
      if K % 64 == 0 and rows_w * K >= LINES_MIN_ELEMENTS:
        c = ops.OWN_ROWS_STAGED_LINES if stage else ops.OWN_ROWS_LINES
        forms[c] = graph_time_us(own(c - 1), calls, flush)
      if ops.both_staged_offered(M, rows_w, K, gate_up):
        forms[ops.OWN_ROWS_BOTH_STAGED] = graph_time_us(own(5), calls, flush)
      if M > 16 and K % 32 == 0 and not gate_up and -(-rows_w // 16) * -(-M // 16) <= 4 * ops.compute_units():
        forms[ops.OWN_ROWS_SHARED_OUT] = graph_time_us(own(6), calls, flush)
      rows_choice = min(forms, key=forms.get)
      t_rows = forms[rows_choice]
      # k is split from 16 rows up only: below, the left operand is too small for its re-reads to matter, and the
      # second kernel costs more than they do (at 16 rows it wins where k is long: 68 against 76 us for [5120, 25600])
      t_split = graph_time_us(own(1), calls, flush) if M >= 16 and not (gate_up and N % 4) else float("inf")
      t_lib = graph_time_us(library, calls, flush) + (2 if gate_up else 1) * UNFUSED_US
      # The own kernels end alike, so they are compared as timed.  Against the library the k-split kernel must
      # win by a tenth: inside a step of the 8B shape at 64 rows it lost 4 us a layer to the library's product for
      # the down projection although it had won this timing by 3 us (its partial results are 17 MB there).  And
      # the library must beat a one-kernel product by a twelfth: the 32B shape's gate|up product at 8 rows, 103 us
      # in the library against 121 here when timed alone, made the whole step 3% slower than this library's
      # kernel with the norm and the activation in it.
      if t_split < t_rows:
        choice = ops.OWN_KSPLIT if t_split <= KSPLIT_MARGIN * t_lib else ops.LIBRARY
      else:
        choice = rows_choice if LIBRARY_MARGIN * t_rows <= t_lib else ops.LIBRARY
      # Timings of candidates that lie close together change places from run to run, and with them the step's time
      # by a few percent: the rule's candidate is kept unless the winner is clearly quicker.
      timed_us = dict(forms)
      timed_us[ops.OWN_KSPLIT], timed_us[ops.LIBRARY] = t_split, t_lib
      rule = ops.rule_choice(M, rows_w, K, gate_up)
      if rule in timed_us and timed_us[rule] <= RULE_MARGIN * timed_us[choice]:
        choice = rule
      ops.set_product_choice(M, rows_w, K, gate_up, choice)
      if log is not None:
        names = {ops.LIBRARY: "library", ops.OWN_ROWS: "own", ops.OWN_KSPLIT: "own with k split",
                 ops.OWN_ROWS_STAGED: "own, left operand staged", ops.OWN_ROWS_LINES: "own, weights in whole lines",
                 ops.OWN_ROWS_STAGED_LINES: "own, left operand staged, weights in whole lines",
                 ops.OWN_ROWS_BOTH_STAGED: "own, both operands staged",
                 ops.OWN_ROWS_SHARED_OUT: "own, rows of the left operand shared out"}
        log(f"product [{rows_w}, {K}]{' gate|up' if gate_up else ''} x {M} rows: "
            + ", ".join(f"{names[c]} {t:.1f} us" for c, t in forms.items())
            + f", own with k split {t_split:.1f} us, library {t_lib:.1f} us with its extra kernels -> {names[choice]}")
    timed += 1
  if timed:
    # give the timing's buffers back to the driver: what is allocated next (the cache pools) then lies as it would
    # have without the timing (pools carved out of recycled blocks have streamed measurably slower)
    del flush
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
  return timed
