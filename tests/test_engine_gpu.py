"""Generation through the entry point: greedy tokens equal the plain implementation's (which recomputes the
whole sequence for every token), under a small token budget, few pages, preemption, and with seeded sampling
that does not depend on batch mates."""

import pytest
import torch

import plain_qwen3 as plain
import tiny_models as tm

pytestmark = pytest.mark.gpu


def _model(tmp_path, name, dtype=torch.float32, seed=0):
  cfg, w = tm.make_model(str(tmp_path / "m"), name, seed=seed, dtype=dtype, std=0.05)
  return cfg, {k: v.float() for k, v in w.items()}


def test_greedy_config_a(tmp_path):
  """Tiny A: prompts 5/17/33, 16 new tokens each, greedy, page size 16."""
  from miniinfer_amd import LLMEngine, SamplingParams
  cfg, w = _model(tmp_path, "A")
  prompts = [tm.random_tokens(cfg, n, seed=n) for n in (5, 17, 33)]
  want = [plain.greedy_generate(p, 16, w, dict(cfg)) for p in prompts]
  with LLMEngine(model=str(tmp_path / "m"), dtype="float32", page_size=16, num_pages=32, max_num_seqs=4) as eng:
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=16, ignore_eos=True), use_tqdm=False)
  assert [o["token_ids"] for o in outs] == want
  assert all(o["finish_reason"] == "max_tokens" for o in outs)
  eng.cache.check()
  assert eng.cache.all_pages_free()


def test_greedy_config_b_chunked_budget_32(tmp_path):
  """Tiny B: prompts 1/9/40/64/100 under a step budget of 32 tokens, so prompts are cut and mixed with decodes."""
  from miniinfer_amd import LLMEngine, SamplingParams
  cfg, w = _model(tmp_path, "B")
  prompts = [tm.random_tokens(cfg, n, seed=10 + n) for n in (1, 9, 40, 64, 100)]
  want = [plain.greedy_generate(p, 12, w, dict(cfg)) for p in prompts]
  with LLMEngine(model=str(tmp_path / "m"), dtype="float32", page_size=8, num_pages=80, max_num_seqs=4,
                 max_num_batched_tokens=32) as eng:
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True), use_tqdm=False)
  assert [o["token_ids"] for o in outs] == want
  assert eng.cache.all_pages_free()


def test_greedy_survives_preemption(tmp_path):
  """So few pages that running requests are preempted and recomputed; the tokens do not change."""
  from miniinfer_amd import LLMEngine, SamplingParams
  cfg, w = _model(tmp_path, "B")
  prompts = [tm.random_tokens(cfg, n, seed=20 + n) for n in (30, 41, 25, 37)]
  want = [plain.greedy_generate(p, 40, w, dict(cfg)) for p in prompts]
  with LLMEngine(model=str(tmp_path / "m"), dtype="float32", page_size=8, num_pages=22, max_num_seqs=4,
                 max_num_batched_tokens=48) as eng:
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True), use_tqdm=False)
    assert eng.scheduler.num_preemptions > 0, "the test is meant to run out of pages"
  assert [o["token_ids"] for o in outs] == want
  assert eng.cache.all_pages_free()


def test_greedy_bfloat16_follows_plain(tmp_path):
  from miniinfer_amd import LLMEngine, SamplingParams
  cfg, w = _model(tmp_path, "C", dtype=torch.bfloat16)
  prompts = [tm.random_tokens(cfg, n, seed=30 + n) for n in (7, 60)]
  with LLMEngine(model=str(tmp_path / "m"), dtype="bfloat16", page_size=16, num_pages=32, max_num_seqs=4) as eng:
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True), use_tqdm=False)
  # each generated token is the plain argmax given the engine's own history, wherever the plain margin is clear
  for p, o in zip(prompts, outs):
    hist = list(p)
    for tok in o["token_ids"]:
      lg = plain.qwen3_logits(hist, w, dict(cfg))[-1]
      top2 = torch.topk(lg, 2).values
      if top2[0] - top2[1] > 0.05 * lg.abs().max():
        assert tok == int(lg.argmax())
      hist.append(tok)


def test_eos_and_seeded_sampling(tmp_path):
  from miniinfer_amd import LLMEngine, SamplingParams
  cfg, w = _model(tmp_path, "A")
  p0 = tm.random_tokens(cfg, 9, seed=1)
  first = plain.greedy_generate(p0, 3, w, dict(cfg))
  # eos = the third greedy token: generation stops there, unless ignore_eos
  with LLMEngine(model=str(tmp_path / "m"), dtype="float32", num_pages=32, max_num_seqs=4, eos=first[2]) as eng:
    out = eng.generate([p0], SamplingParams(temperature=0.0, max_tokens=10), use_tqdm=False)[0]
    stop = first.index(first[2]) + 1
    assert out["token_ids"] == first[:stop] and out["finish_reason"] == "eos"
    out = eng.generate([p0], SamplingParams(temperature=0.0, max_tokens=3, ignore_eos=True), use_tqdm=False)[0]
    assert out["token_ids"] == first and out["finish_reason"] == "max_tokens"
    # temperature sampling with a per-request seed: the same alone and among batch mates
    sp = SamplingParams(temperature=0.8, max_tokens=12, ignore_eos=True, seed=1234)
    alone = eng.generate([p0], sp, use_tqdm=False)[0]["token_ids"]
    others = [tm.random_tokens(cfg, n, seed=n) for n in (4, 20)]
    mixed = eng.generate([others[0], p0, others[1]],
                         [SamplingParams(temperature=1.0, max_tokens=5, ignore_eos=True), sp,
                          SamplingParams(temperature=0.0, max_tokens=7, ignore_eos=True)], use_tqdm=False)
    assert mixed[1]["token_ids"] == alone
    # the seed is what the draw depends on: the same seed repeats, another seed gives other tokens
    assert eng.generate([p0], sp, use_tqdm=False)[0]["token_ids"] == alone
    other = SamplingParams(temperature=0.8, max_tokens=12, ignore_eos=True, seed=4321)
    assert eng.generate([p0], other, use_tqdm=False)[0]["token_ids"] != alone
    # a request's own stop ids end it like the end-of-sequence id does, and are kept as its last token
    out = eng.generate([p0], SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True, stop_token_ids=[first[1]]),
                       use_tqdm=False)[0]
    assert out["token_ids"] == first[:first.index(first[1]) + 1] and out["finish_reason"] == "stop"


def test_unknown_option_is_an_error(tmp_path):
  from miniinfer_amd import LLMEngine
  _model(tmp_path, "A")
  with pytest.raises(TypeError, match="unknown engine option"):
    LLMEngine(model=str(tmp_path / "m"), max_modle_len=5)


def test_command_line_generate(tmp_path):
  import json
  import os
  import subprocess
  import sys
  cfg, w = _model(tmp_path, "A")
  prompt = tm.random_tokens(cfg, 6, seed=3)
  want = plain.greedy_generate(prompt, 5, w, dict(cfg))
  root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
  proc = subprocess.run([sys.executable, "-m", "miniinfer_amd", "generate", "--model", str(tmp_path / "m"),
                         "--dtype", "float32", "--max-tokens", "5", "--temperature", "0", "--ignore-eos",
                         "--max-model-len", "64", "--num-pages", "16", "--quiet",
                         "--prompt-ids", ",".join(map(str, prompt))],
                        capture_output=True, text=True, cwd=root, timeout=300)
  assert proc.returncode == 0, proc.stderr[-2000:]
  assert json.loads(proc.stdout.strip().splitlines()[-1])["token_ids"] == want


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_launching_ahead_of_the_tokens_changes_no_token(tmp_path, dtype):
  """With `enable_overlap` the engine launches a step before it has read the tokens of the one before (they stay
  on the device as placeholders' targets).  Same requests, same tokens and finish reasons as the synchronous
  loop: greedy and seeded sampling, an end-of-sequence token that is found one step late, so few pages that
  requests are preempted, prompts cut into portions."""
  from miniinfer_amd import LLMEngine, SamplingParams
  cfg, w = _model(tmp_path, "B", dtype=torch.bfloat16 if dtype == "bfloat16" else torch.float32)
  prompts = [tm.random_tokens(cfg, n, seed=50 + n) for n in (30, 41, 3, 25, 37, 12)]
  params = [SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True),
            SamplingParams(temperature=0.9, max_tokens=33, ignore_eos=True, seed=7),
            SamplingParams(temperature=0.0, max_tokens=30),
            SamplingParams(temperature=0.7, top_k=20, top_p=0.9, max_tokens=25, seed=11),
            SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True),
            SamplingParams(temperature=0.0, max_tokens=28)]
  results = {}
  for overlap in (False, True):
    # the end-of-sequence token is one that the third request produces early in greedy decoding
    with LLMEngine(model=str(tmp_path / "m"), dtype=dtype, page_size=8, num_pages=15, max_num_seqs=4,
                   max_num_batched_tokens=48, enable_overlap=overlap, eos=results.get("eos")) as eng:
      if "eos" not in results:
        probe = eng.generate([prompts[2]], SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True),
                             use_tqdm=False)[0]["token_ids"]
        results["eos"] = probe[3]
        eng.scheduler.eos_token_id = eng.eos_token_id = probe[3]
      outs = eng.generate(prompts, params, use_tqdm=False)
      results[overlap] = [(o["token_ids"], o["finish_reason"]) for o in outs]
      assert eng.cache.all_pages_free() and eng.is_finished()
      eng.cache.check()
      if overlap:
        assert eng.scheduler.num_preemptions > 0, "the test is meant to run out of pages"
  assert results[True] == results[False]
  assert results[True][2][1] == "eos" and len(results[True][2][0]) <= 4
  assert all(t >= 0 for toks, _ in results[True] for t in toks)


def test_stream_generate_yields_every_token_once_and_in_order(tmp_path):
  from miniinfer_amd import LLMEngine, SamplingParams
  cfg, w = _model(tmp_path, "A")
  prompts = [tm.random_tokens(cfg, n, seed=70 + n) for n in (5, 23, 11)]
  sps = [SamplingParams(temperature=0.0, max_tokens=9, ignore_eos=True),
         SamplingParams(temperature=0.8, max_tokens=14, ignore_eos=True, seed=2),
         SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True)]
  for overlap in (True, False):
    with LLMEngine(model=str(tmp_path / "m"), dtype="float32", num_pages=32, max_num_seqs=4, enable_overlap=overlap) as eng:
      whole = eng.generate(prompts, sps, use_tqdm=False)
      seen, ended = {}, {}
      for out in eng.stream_generate(prompts, sps):
        toks = seen.setdefault(out.request_id, [])
        toks.append(out.token_id)
        assert out.output_token_ids == toks and out.request_id not in ended
        if out.finished:
          ended[out.request_id] = out.finish_reason
      assert [seen[r] for r in sorted(seen, key=lambda r: int(r.split("-")[1]))] == [o["token_ids"] for o in whole]
      assert list(ended.values()) == ["max_tokens"] * 3 and eng.is_finished()
      assert eng.cache.all_pages_free()


def test_eos_comes_from_generation_config_json(tmp_path):
  import json
  from miniinfer_amd import LLMEngine, SamplingParams
  cfg, w = _model(tmp_path, "A")
  p0 = tm.random_tokens(cfg, 9, seed=1)
  first = plain.greedy_generate(p0, 4, w, dict(cfg))
  with open(tmp_path / "m" / "generation_config.json", "w") as f:
    json.dump({"eos_token_id": [first[3], 255]}, f)
  with LLMEngine(model=str(tmp_path / "m"), dtype="float32", num_pages=32, max_num_seqs=4) as eng:
    assert eng.eos_token_id == [first[3], 255]
    out = eng.generate([p0], SamplingParams(temperature=0.0, max_tokens=10), use_tqdm=False)[0]
  assert out["token_ids"] == first[:first.index(first[3]) + 1] and out["finish_reason"] == "eos"


def test_text_prompts_go_through_the_folder_s_tokenizer(tmp_path):
  """A tokenizer.json in the model folder (a word-level one, built here) turns text prompts into ids and the
  generated ids back into text; without one, a text prompt is an error that says what to do."""
  from tokenizers import Tokenizer
  from tokenizers.models import WordLevel
  from tokenizers.pre_tokenizers import Whitespace
  from miniinfer_amd import LLMEngine, SamplingParams
  cfg, w = _model(tmp_path, "A")
  with LLMEngine(model=str(tmp_path / "m"), dtype="float32", num_pages=32, max_num_seqs=4) as eng:
    with pytest.raises(ValueError, match="tokenizer.json"):
      eng.generate(["some words"], SamplingParams(max_tokens=2), use_tqdm=False)
  vocab = {f"w{i}": i for i in range(cfg["vocab_size"])}
  tok = Tokenizer(WordLevel(vocab, unk_token="w0"))
  tok.pre_tokenizer = Whitespace()
  tok.save(str(tmp_path / "m" / "tokenizer.json"))
  ids = tm.random_tokens(cfg, 11, seed=5)
  text = " ".join(f"w{i}" for i in ids)
  want = plain.greedy_generate(ids, 6, w, dict(cfg))
  with LLMEngine(model=str(tmp_path / "m"), dtype="float32", num_pages=32, max_num_seqs=4) as eng:
    sp = SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True)
    outs = eng.generate([text, ids], sp, use_tqdm=False)
    assert outs[0]["token_ids"] == want and outs[1]["token_ids"] == want
    assert outs[0]["text"].split() == [f"w{i}" for i in want]
    streamed = [o for o in eng.stream_generate(text, sp)]
    assert [o.token_id for o in streamed] == want and streamed[-1].full_text.split() == [f"w{i}" for i in want]
    assert "".join(o.delta_text for o in streamed) == streamed[-1].full_text


def test_cache_is_sized_from_device_memory_when_no_page_count_is_given(tmp_path):
  """Without `num_pages` the pool is what the device has left: bounded by the requests the engine may hold when
  memory is plenty, by memory when it is not; a step of the full token budget still runs beside it."""
  from miniinfer_amd import LLMEngine, SamplingParams
  from miniinfer_amd.cache import CacheManager
  cfg, w = _model(tmp_path, "B")
  prompts = [tm.random_tokens(cfg, n, seed=80 + n) for n in (100, 9, 64)]
  want = [plain.greedy_generate(p, 6, w, dict(cfg)) for p in prompts]
  sp = SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True)
  # plenty of memory: as many pages as max_num_seqs requests of max_model_len tokens can use
  with LLMEngine(model=str(tmp_path / "m"), dtype="float32", page_size=8, max_num_seqs=4, max_model_len=128) as eng:
    assert eng.num_pages == 4 * (128 // 8) == eng.cache.num_pages
    assert [o["token_ids"] for o in eng.generate(prompts, sp, use_tqdm=False)] == want
  del eng
  torch.cuda.empty_cache()
  # memory binds: leave the engine 64 MiB beyond what the largest step needs
  free, total = torch.cuda.mem_get_info()
  probe = LLMEngine(model=str(tmp_path / "m"), dtype="float32", page_size=8, max_num_seqs=256, num_pages=4)
  act = probe.activation_bytes()
  per_page = CacheManager.bytes_per_page(probe.model.cache_needs(), 8, torch.float32)
  del probe
  torch.cuda.empty_cache()
  free, total = torch.cuda.mem_get_info()
  room = 64 << 20
  util = 1.0 - (free - act - room) / total
  with LLMEngine(model=str(tmp_path / "m"), dtype="float32", page_size=8, max_num_seqs=256,
                 gpu_memory_utilization=util) as eng:
    pages = eng.num_pages
    assert pages < 256 * (256 // 8), "the test is meant to be bound by memory, not by the request limit"
    assert 0.8 * room <= (pages + 1) * per_page <= room, (pages, per_page, room)
    assert [o["token_ids"] for o in eng.generate(prompts, sp, use_tqdm=False)] == want
  with pytest.raises(RuntimeError, match="not enough device memory"):
    LLMEngine(model=str(tmp_path / "m"), dtype="float32", page_size=8, gpu_memory_utilization=1e-3)


@pytest.mark.parametrize("products", ["own", "own_ksplit", "own_staged", "own_staged_lines", "own_both_staged", "library",
                                      "library_gate_up"])
def test_bfloat16_tokens_follow_plain_with_either_product_kernel(tmp_path, products, monkeypatch):
  """The engine's choice between its own weight-streaming products (whole rows per workgroup, with or without the
  left operand staged through LDS and the weights fetched in whole lines, or k split across workgroups) and the library's is a matter of speed: with every
  small product forced to one of them, each generated token is one the plain implementation all but ties for."""
  from miniinfer_amd import LLMEngine, SamplingParams
  from miniinfer_amd.kernels import ops
  cfg, w = _model(tmp_path, "B", dtype=torch.bfloat16)
  prompts = [tm.random_tokens(cfg, n, seed=90 + n) for n in (7, 60, 33)]
  with LLMEngine(model=str(tmp_path / "m"), dtype="bfloat16", page_size=8, num_pages=64, max_num_seqs=4,
                 tune_products=False, max_num_batched_tokens=48) as eng:
    before = eng.choices.library_products[0]
    scaled_activations = []
    real = ops.silu_mul_scaled
    monkeypatch.setattr(ops, "silu_mul_scaled", lambda *a, **k: (scaled_activations.append(1), real(*a, **k))[1])
    if products == "own":
      eng.choices.own_only = True
      outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True), use_tqdm=False)
    else:
      choice = {"own_ksplit": ops.OWN_KSPLIT, "own_staged": ops.OWN_ROWS_STAGED,
                "own_staged_lines": ops.OWN_ROWS_STAGED_LINES, "own_both_staged": ops.OWN_ROWS_BOTH_STAGED,
                "library": ops.LIBRARY, "library_gate_up": ops.LIBRARY}[products]
      for rows in ops.TUNE_ROWS:
        for m in eng.model.products():
          # (library_gate_up: only the gate|up product goes to the library; the product before it keeps the norm's
          # first half in its ending, and the activation kernel applies the norm's row factor)
          mine = choice if products != "library_gate_up" or m[1] else ops.OWN_ROWS
          eng.choices.set(rows, m[0].shape[0], m[0].shape[1], m[1], mine)      # the engine's own table
      outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True), use_tqdm=False)
    assert not ops.current_choices().table                    # and nobody else's
    ran_library = eng.choices.library_products[0] - before
    assert (ran_library > 0) == (products in ("library", "library_gate_up"))
    assert (len(scaled_activations) > 0) == (products == "library_gate_up")
  for p, o in zip(prompts, outs):
    hist = list(p)
    for tok in o["token_ids"]:
      lg = plain.qwen3_logits(hist, w, dict(cfg))[-1]
      assert lg[tok] >= lg.max() - 0.03 * lg.abs().max(), f"token {tok} is not near the plain top"
      hist.append(tok)


def test_add_request_and_step_loop_hands_finished_requests_out_and_keeps_none(tmp_path):
  """The documented loop of `add_request` and `step` (no `generate`): every finished request comes out of exactly
  one `StepOutput.finished`, with its tokens, and the engine keeps no reference to it."""
  from miniinfer_amd import LLMEngine, SamplingParams
  cfg, w = _model(tmp_path, "A")
  prompts = [tm.random_tokens(cfg, n, seed=60 + n) for n in (5, 17, 33, 9)]
  want = {f"req-{i}": plain.greedy_generate(p, 6 + i, w, dict(cfg)) for i, p in enumerate(prompts)}
  with LLMEngine(model=str(tmp_path / "m"), dtype="float32", page_size=16, num_pages=32, max_num_seqs=4) as eng:
    for rounds in range(2):                     # the second round reuses the ids' numbers' successors
      ids = [eng.add_request(p, SamplingParams(temperature=0.0, max_tokens=6 + i, ignore_eos=True))
             for i, p in enumerate(prompts)]
      got = {}
      while not eng.is_finished():
        for r in eng.step().finished:
          assert r.request_id not in got
          got[r.request_id] = (list(r.outputs), r.finish_reason)
      assert sorted(got) == sorted(ids) and not eng._requests
      for i, rid in enumerate(ids):
        assert got[rid] == (want[f"req-{i}"], "max_tokens")
    assert eng.cache.all_pages_free()


@pytest.mark.parametrize("graphs", [False, True])
def test_overlapped_loop_lets_a_decode_sit_out_while_others_overwrite_the_device_tokens(tmp_path, graphs):
  """The overlapped loop with so few pages that a decode must wait: request a reaches max_tokens while its last
  token is still on the device, so its pages come back one call later; b's next token needs a new page and none is
  free, so b sits a step out (it is not preempted) while c decodes and its sampled token overwrites the device
  buffer from which b's own placeholder was to be read.  b must come back with its real token: every request's
  tokens are the plain implementation's."""
  from miniinfer_amd import LLMEngine, SamplingParams
  cfg, w = _model(tmp_path, "B")
  P = 8
  spec = [(8, 2), (15, 4), (24, 6)]             # (prompt tokens, max_tokens) of a, b, c
  prompts = [tm.random_tokens(cfg, n, seed=70 + n) for n, _ in spec]
  want = [plain.greedy_generate(p, m, w, dict(cfg)) for p, (_, m) in zip(prompts, spec)]
  with LLMEngine(model=str(tmp_path / "m"), dtype="float32", page_size=P, num_pages=8, max_num_seqs=3,
                 max_num_batched_tokens=64, enable_overlap=True, enforce_eager=not graphs) as eng:
    sat_out = []
    real = eng.scheduler.schedule

    def schedule():
      plan = real()
      decoding = [r for r in eng.scheduler.running if r.remaining == 1 and r.num_computed > 0]
      inside = {id(e.request) for e in plan.entries} if plan is not None else set()
      sat_out.extend(r.request_id for r in decoding if id(r) not in inside)
      return plan

    eng.scheduler.schedule = schedule
    outs = eng.generate(prompts, [SamplingParams(temperature=0.0, max_tokens=m, ignore_eos=True) for _, m in spec],
                        use_tqdm=False)
    assert eng.scheduler.num_preemptions == 0
    assert "req-1" in sat_out, "the test is meant to leave b's decode out of a step"
    assert eng.cache.all_pages_free()
  assert [o["token_ids"] for o in outs] == want
