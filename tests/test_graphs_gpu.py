"""Decode steps replayed from HIP graphs give the logits of the same steps run eagerly: several replays of each
graph, with eager prompt steps and synchronisations between them, batches that change size (so padding entries
come and go), and block tables that grow past a width bucket."""

import numpy as np
import pytest
import torch

import tiny_models as tm

pytestmark = pytest.mark.gpu


def _runner(folder, dtype, graphs, pages=96):
  from miniinfer_amd.cache.manager import CacheManager
  from miniinfer_amd.engine.runner import ModelRunner
  from miniinfer_amd.weights import load_model
  dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
  model, _ = load_model(str(folder), dt, "cuda:0")
  cache = CacheManager(model.cache_needs(), page_size=16, num_pages=pages, max_requests=8,
                       max_model_len=model.spec.max_positions, dtype=dt, device="cuda:0")
  return ModelRunner(model, cache, use_graphs=graphs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_equal_eager_steps(tmp_path, dtype):
  from miniinfer_amd.engine.runner import StepEntry
  cfg, _ = tm.make_model(str(tmp_path / "m"), "C", seed=4, dtype=torch.bfloat16 if dtype == "bfloat16" else torch.float32,
                         std=0.05)
  runners = [_runner(tmp_path / "m", dtype, graphs=False), _runner(tmp_path / "m", dtype, graphs=True)]
  prompts = {r: tm.random_tokens(cfg, n, seed=n) for r, n in (("a", 250), ("b", 3), ("c", 40), ("d", 17), ("e", 9))}
  stream = {r: tm.random_tokens(cfg, 40, seed=100 + len(p)) for r, p in prompts.items()}
  outs = [[], []]
  for k, rn in enumerate(runners):
    live = []

    def start(r):
      rn.cache.admit(r)
      outs[k].append(rn.step([StepEntry(r, prompts[r], [len(prompts[r]) - 1])]).float().cpu())   # eager prompt step
      live.append(r)

    start("a"); start("b")
    for t in range(30):
      if t == 3: start("c")
      if t == 5: start("d"); start("e")
      if t == 12:
        rn.cache.release("b"); live.remove("b")
      if t == 20:
        rn.cache.release("d"); live.remove("d")
      lg = rn.step([StepEntry(r, [stream[r][t]], [0]) for r in live])       # single tokens only: graph path
      torch.cuda.synchronize()
      outs[k].append(lg.float().cpu())
    # request "a" crossed from 250 to 280 tokens: its table grew from 16 to 18 pages, past the 16-page bucket
    assert rn.cache.length("a") == 280
  assert len(runners[1]._graphs) >= 3 and not runners[0]._graphs
  tol = 1e-5 if dtype == "float32" else 2e-2
  for e, g in zip(*outs):
    assert e.shape == g.shape
    scale = float(e.abs().max())
    assert float((e - g).abs().max()) <= tol * max(scale, 1.0)


def test_engine_generates_the_same_with_and_without_graphs(tmp_path):
  from miniinfer_amd import LLMEngine, SamplingParams
  cfg, _ = tm.make_model(str(tmp_path / "m"), "B", seed=6, dtype=torch.float32, std=0.05)
  prompts = [tm.random_tokens(cfg, n, seed=n) for n in (4, 31, 18)]
  sps = [SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True),
         SamplingParams(temperature=0.9, max_tokens=25, ignore_eos=True, seed=3),
         SamplingParams(temperature=0.7, top_k=20, top_p=0.9, max_tokens=14, ignore_eos=True, seed=5)]
  res = []
  for eager in (True, False):
    with LLMEngine(model=str(tmp_path / "m"), dtype="float32", page_size=8, num_pages=64, max_num_seqs=4,
                   enforce_eager=eager) as eng:
      captured = eng.warm_up()            # every batch bucket up to max_num_seqs, every table width of the model
      assert (captured == 0) if eager else (captured >= 3 and all(g.ok for g in eng.runner._graphs.values()))
      res.append([o["token_ids"] for o in eng.generate(prompts, sps, use_tqdm=False)])
      assert len(eng.runner._graphs) == captured, "a step needed a graph that warm_up had not made"
  assert res[0] == res[1]


def test_graphs_of_many_requests_hold_library_products_and_still_equal_eager_steps(tmp_path):
  """Beyond 64 single tokens the products of a bfloat16 step are library calls, recorded into the graph with
  whatever the library adds to them.  Each graph checks itself against the eager step when it is made; here
  80 and then 100 requests decode for several steps through both paths, with eager work between the replays."""
  from miniinfer_amd.cache.manager import CacheManager
  from miniinfer_amd.engine.runner import ModelRunner, StepEntry
  from miniinfer_amd.weights import load_model
  cfg, _ = tm.make_model(str(tmp_path / "m"), "A", seed=8, dtype=torch.bfloat16, std=0.05)
  runners = []
  for graphs in (False, True):
    model, _ = load_model(str(tmp_path / "m"), torch.bfloat16, "cuda:0")
    cache = CacheManager(model.cache_needs(), page_size=16, num_pages=260, max_requests=128,
                         max_model_len=model.spec.max_positions, dtype=torch.bfloat16, device="cuda:0")
    runners.append(ModelRunner(model, cache, use_graphs=graphs))
  outs = [[], []]
  for k, rn in enumerate(runners):
    live = []
    for r in range(100):
      if r == 80:
        for t in range(4):
          outs[k].append(rn.step([StepEntry(q, [(7 * q + t) % cfg["vocab_size"]], [0]) for q in live]).float().cpu())
      rn.cache.admit(r)
      rn.step([StepEntry(r, tm.random_tokens(cfg, 3 + r % 9, seed=r), [])])      # eager prompt step
      live.append(r)
    for t in range(4, 9):
      outs[k].append(rn.step([StepEntry(q, [(7 * q + t) % cfg["vocab_size"]], [0]) for q in live]).float().cpu())
      torch.cuda.synchronize()
  assert {b for b, _ in runners[1]._graphs} == {96, 128}
  assert all(g.ok for g in runners[1]._graphs.values()), "a graph with library products did not reproduce the eager step"
  for e, g in zip(*outs):
    assert e.shape == g.shape
    assert float((e - g).abs().max()) <= 2e-2 * max(float(e.abs().max()), 1.0)


def test_a_step_whose_products_could_go_either_way_is_captured_both_ways(tmp_path, monkeypatch):
  """With 17 to 64 single tokens a product may go to the library or to this library's own kernel.  When the rule (or
  the measurement) says library, the runner captures the step both ways and keeps the quicker graph; whichever it
  keeps reproduces the eager steps."""
  from miniinfer_amd.cache.manager import CacheManager
  from miniinfer_amd.engine.runner import ModelRunner, StepEntry
  from miniinfer_amd.kernels import ops
  from miniinfer_amd.weights import load_model
  monkeypatch.setattr(ops, "SKINNY_OWN_ELEMENTS", 0)       # every matrix counts as large: library beyond 16 rows
  cfg, _ = tm.make_model(str(tmp_path / "m"), "B", seed=9, dtype=torch.bfloat16, std=0.05)
  runners = []
  for graphs in (False, True):
    model, _ = load_model(str(tmp_path / "m"), torch.bfloat16, "cuda:0")
    cache = CacheManager(model.cache_needs(), page_size=16, num_pages=120, max_requests=32,
                         max_model_len=model.spec.max_positions, dtype=torch.bfloat16, device="cuda:0")
    runners.append(ModelRunner(model, cache, use_graphs=graphs))
  outs = [[], []]
  counted = []
  for k, rn in enumerate(runners):
    live = []
    for r in range(24):
      rn.cache.admit(r)
      rn.step([StepEntry(r, tm.random_tokens(cfg, 2 + r % 11, seed=r), [])])
      live.append(r)
    before = tuple(rn.choices.library_products)
    for t in range(5):
      outs[k].append(rn.step([StepEntry(q, [(5 * q + t) % cfg["vocab_size"]], [0]) for q in live]).float().cpu())
      torch.cuda.synchronize()
    after = tuple(rn.choices.library_products)
    counted.append((after[0] - before[0], after[1] - before[1]))
  assert counted[0][1] > 0, "the eager steps of 24 rows sent no avoidable product to the library"
  assert {b for b, _ in runners[1]._graphs} == {24}
  assert all(g.ok for g in runners[1]._graphs.values())
  for e, g in zip(*outs):
    assert e.shape == g.shape
    assert float((e - g).abs().max()) <= 2e-2 * max(float(e.abs().max()), 1.0)
