"""Rules that size a launch or pick a kernel, as plain functions of sizes (no GPU)."""

import pytest


def test_decode_key_ranges_fill_one_round_and_stay_few():
  from miniinfer_amd.parts.attention import decode_splits
  for waves, tile in ((4, 64), (2, 32)):
    for entries in (1, 2, 4, 8, 12, 16, 24, 32, 48, 64, 96, 128, 256):
      for kv_heads in (1, 2, 8):
        for keys in (1, 63, 64, 300, 2048, 8192, 40000, 1 << 20):
          n = entries * kv_heads
          s = decode_splits(n, keys, tile, waves)
          tiles = -(-keys // tile)
          assert 1 <= s <= 64
          assert s == 1 or s * waves <= tiles                 # a wave of every range has a tile
          assert s <= 2 or n * s <= 512                        # more than two ranges only while they fit one round
  # the cases the rule was measured on
  assert decode_splits(8 * 8, 2048) == 8 and decode_splits(12 * 8, 2048) == 5 and decode_splits(24 * 8, 2048) == 2
  assert decode_splits(48 * 8, 2048) == 2 and decode_splits(64 * 8, 2048) == 1
  assert decode_splits(8, 8192) == 32 and decode_splits(8, 32768) == 64 and decode_splits(8, 2048) == 8
  # launches that fill a round of two workgroups a compute unit with two ranges or more take workgroups of twice the
  # waves and half the ranges; few workgroups and unsplit launches stay as they are
  from miniinfer_amd.parts.attention import decode_launch
  assert decode_launch(8 * 8, 2048) == (4, True) and decode_launch(16 * 8, 2048) == (2, True)
  assert decode_launch(32 * 8, 2048) == (1, True) and decode_launch(24 * 8, 2048) == (1, True)
  assert decode_launch(4 * 8, 2048) == (4, True) and decode_launch(8 * 8, 512) == (1, True)
  assert decode_launch(8, 2048) == (8, False) and decode_launch(2 * 8, 2048) == (8, False)       # too few workgroups
  assert decode_launch(12 * 8, 2048) == (5, False) and decode_launch(48 * 8, 2048) == (2, False)  # a second round
  assert decode_launch(64 * 8, 2048) == (1, False) and decode_launch(8, 32768) == (32, True)
  for n in (1, 8, 64, 100, 256, 384, 512):
    for keys in (100, 2048, 32768):
      s, wide = decode_launch(n, keys)
      assert s >= 1 and s * (8 if wide else 4) <= max(8 if wide else 4, -(-keys // 64)), (n, keys, s, wide)
  assert decode_splits(16, 32768) == 32 and decode_splits(1, 1 << 20) == 64
  assert decode_splits(8 * 4, 2048, 32, 2) == 16 and decode_splits(64 * 4, 2048, 32, 2) == 2


def test_product_kernel_choice_falls_back_to_the_rule_and_obeys_measurements():
  from miniinfer_amd.kernels import ops
  ops.clear_product_choices()
  try:
    assert ops.skinny_preferred(1, 4096, 4096) and ops.skinny_preferred(16, 51200, 5120, True)
    assert ops.skinny_preferred(64, 1024, 3072)                       # a small matrix
    assert not ops.skinny_preferred(17, 4096, 4096)                   # a large one with more than 16 rows
    assert not ops.skinny_preferred(65, 64, 64)                       # more rows than the kernel takes
    assert ops.rule_choice(64, 5120, 25600) == ops.OWN_KSPLIT and ops.rule_choice(32, 4096, 12288) == ops.LIBRARY
    assert ops.rule_choice(32, 6144, 4096) == ops.LIBRARY and ops.rule_choice(64, 24576, 4096, True) == ops.LIBRARY
    # which of the own kernels: k is split for more than 16 rows of 2,048 columns and more, and never for a
    # gate|up matrix whose halves are no multiple of 4 rows; from 4 rows up the weights come in whole lines, with the
    # left operand staged, when the matrix has 40 M elements in rows of 16,384 or more (a multiple of 64; not gate|up);
    # else up to 16 rows have both operands staged through LDS (k a multiple of 32) when the matrix has 16 M
    # elements, or rows of 2,048 columns and no activation behind it; what is left has the left operand staged from
    # 4 rows and 12 K elements
    assert ops.skinny_variant(64, 1024, 3072) == 6 and ops.skinny_variant(17, 1024, 2048) == 6   # few rows of the matrix
    assert ops.skinny_variant(64, 2048, 2048) == 1 and ops.skinny_variant(48, 2048, 2048) == 6 and ops.skinny_variant(16, 1024, 2048) == 5
    assert ops.skinny_variant(16, 1024, 3072) == 5 and ops.skinny_variant(64, 4096, 1024) == 2
    assert ops.skinny_variant(4, 1024, 2048) == 5 and ops.skinny_variant(8, 4096, 1024) == 0
    assert ops.skinny_variant(16, 4096, 1024) == 2 and ops.skinny_variant(8, 6144, 2048, True) == 2
    assert ops.skinny_variant(8, 4096, 4096) == 5 and ops.skinny_variant(16, 6144, 4096) == 5
    assert ops.skinny_variant(8, 4096, 12288) == 5 and ops.skinny_variant(32, 5120, 25600) == 1 and ops.skinny_variant(3, 4096, 25600) == 5
    assert ops.skinny_variant(8, 151936, 1024) == 5 and ops.skinny_variant(2, 151936, 1024) == 5
    assert ops.skinny_variant(8, 51200, 5120, True) == 5 and ops.skinny_variant(8, 5120, 25632) == 5
    assert ops.skinny_variant(8, 5120, 25600) == 4 and ops.skinny_variant(16, 24576, 4096, True) == 5
    assert ops.skinny_variant(1, 6144, 1024, True) == 0 and ops.skinny_variant(1, 4096, 1024) == 0
    assert ops.skinny_variant(1, 1024, 2048) == 5 and ops.skinny_variant(1, 4096, 4096) == 5
    assert ops.skinny_variant(3, 24576, 4096, True) == 5 and ops.skinny_variant(3, 6144, 2048, True) == 0
    assert ops.skinny_variant(8, 1024, 2000) == 2 and ops.skinny_variant(2, 1024, 2000) == 0
    assert ops.skinny_variant(20, 1024, 1024) == 6 and ops.skinny_variant(20, 4096, 1024) == 2 and ops.skinny_variant(4, 1024, 1000) == 0
    assert ops.skinny_variant(64, 2 * 1026, 4096, True) == 2 and ops.skinny_variant(64, 2 * 1028, 4096, True) == 1
    for p in ops.TUNE_ROWS:
      ops.set_product_choice(p, 4096, 4096, False, p > 8)
    assert not ops.skinny_preferred(3, 4096, 4096) and not ops.skinny_preferred(8, 4096, 4096)
    assert ops.skinny_preferred(9, 4096, 4096) and ops.skinny_preferred(64, 4096, 4096)
    assert ops.skinny_preferred(3, 4096, 4096, True)                  # another shape: not measured, the rule
    assert ops.skinny_variant(64, 4096, 4096) == 0                    # measured: the kernel that owns whole rows
    ops.set_product_choice(64, 4096, 4096, False, ops.OWN_KSPLIT)
    assert ops.skinny_preferred(64, 4096, 4096) and ops.skinny_variant(64, 4096, 4096) == 1
    assert ops.skinny_variant(48, 4096, 4096) == 0
    ops.set_product_choice(16, 4096, 4096, False, ops.OWN_ROWS_STAGED)
    assert ops.skinny_preferred(12, 4096, 4096) and ops.skinny_variant(12, 4096, 4096) == 2
    ops.set_product_choice(16, 4096, 4096, False, ops.OWN_ROWS_STAGED_LINES)
    assert ops.skinny_preferred(12, 4096, 4096) and ops.skinny_variant(12, 4096, 4096) == 4
    with ops.own_products_only():
      assert ops.skinny_preferred(3, 4096, 4096) and ops.skinny_preferred(40, 51200, 5120)
      assert not ops.skinny_preferred(65, 4096, 4096)
    assert not ops.skinny_preferred(3, 4096, 4096)
    # measurements can be set aside, and products that they send elsewhere than the rule would are counted
    count = ops.off_rule_products_run()
    assert not ops.skinny_preferred(3, 4096, 4096) and ops.off_rule_products_run() == count + 1
    with ops.rule_products_only():
      assert ops.skinny_preferred(3, 4096, 4096) and ops.skinny_variant(12, 4096, 4096) == 5
      assert ops.off_rule_products_run() == count + 1
    assert ops.skinny_variant(12, 4096, 4096) == 4
    assert ops.product_choice_known(4096, 4096, False) and not ops.product_choice_known(4096, 4096, True)
  finally:
    ops.clear_product_choices()


def test_what_a_decode_step_reads_past_the_caches():
  """Keys and values of a launch are streamed (nontemporal loads) from 512 MB on, counted with the upper bound of keys a
  decode graph is made for; matrices from 48 MB on go to the nontemporal build of the product kernels, and every matrix
  does while the table in use says so (the runner does, for steps whose keys and values fit the last-level cache)."""
  import torch
  from miniinfer_amd.kernels import ops
  # Qwen3-0.6B shape: 8 kv heads of 128, bfloat16: 4 KB a token and layer
  assert not ops.decode_streams_keys(8, 8, 128, 4096) and not ops.decode_streams_keys(24, 8, 128, 4096)
  assert ops.decode_streams_keys(32, 8, 128, 4096) and ops.decode_streams_keys(64, 8, 128, 2048)
  assert ops.decode_streams_keys(8, 8, 128, 32768) and not ops.decode_streams_keys(1, 8, 128, 32768)
  assert ops.decode_streams_keys(16, 8, 128, 4096, element_size=4)
  small = torch.empty(1024, 2048, dtype=torch.bfloat16, device="meta")
  head = torch.empty(151936, 1024, dtype=torch.bfloat16, device="meta")
  picked = []
  real = ops._lib
  ops._lib = lambda name, defines=(): picked.append(defines) or defines
  try:
    table = ops.ProductChoices()
    with table:
      assert ops._skinny_lib(small) == () and ops._skinny_lib(head) == (("SKINNY_NT", 1),)
      table.stream_weights = True
      assert ops._skinny_lib(small) == (("SKINNY_NT", 1),)
    assert ops._skinny_lib(small) == ()          # another table is in use again: its own switch counts
  finally:
    ops._lib = real
