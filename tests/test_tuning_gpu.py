"""The choice between this library's weight-streaming product and the library product is measured per shape; either
choice gives the right result, through `linear` and through the gated activation."""

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


@pytest.fixture
def clean_choices():
  from miniinfer_amd.kernels import ops
  ops.clear_product_choices()
  yield ops
  ops.clear_product_choices()


def test_products_are_timed_once_per_shape_and_small_ones_are_left_alone(clean_choices):
  ops = clean_choices
  from miniinfer_amd.kernels.tuning import MIN_ELEMENTS, tune_products
  g = torch.Generator(device=DEV).manual_seed(0)
  big = [(torch.randn(2048, 1024, device=DEV, generator=g) * 0.05).bfloat16() for _ in range(3)]
  gated = [(torch.randn(2 * 1024, 1024, device=DEV, generator=g) * 0.05).bfloat16() for _ in range(2)]
  small = (torch.randn(256, 512, device=DEV, generator=g) * 0.05).bfloat16()
  assert big[0].numel() >= MIN_ELEMENTS > small.numel()
  lines = []
  products = [(w, False) for w in big] + [(w, True) for w in gated] + [(small, False), (None, False)]
  assert tune_products(products, log=lines.append) == 2
  assert len(lines) == 2 * len(ops.TUNE_ROWS)
  assert ops.product_choice_known(2048, 1024, False) and ops.product_choice_known(2048, 1024, True)
  assert not ops.product_choice_known(256, 512, False)
  assert tune_products(products) == 0                      # nothing is timed twice
  # more rows than the kernel takes never go to it, whatever was measured
  assert not ops.skinny_preferred(65, 2048, 1024)


# the library / whole rows per workgroup / k split across workgroups / whole rows with the left operand staged /
# whole rows with the weights in whole lines / both / both operands staged
@pytest.mark.parametrize("choice", [0, 1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("M", [3, 16, 40])
def test_either_choice_gives_the_product(clean_choices, choice, M):
  ops = clean_choices
  own = choice != ops.LIBRARY
  from miniinfer_amd.parts.linear import gate_up_activation, linear
  g = torch.Generator().manual_seed(M)
  N, K, inter = 192, 160, 112
  w = (torch.randn(N, K, generator=g) * 0.1).bfloat16()
  wgu = (torch.randn(2 * inter, K, generator=g) * 0.1).bfloat16()
  x = torch.randn(M, K, generator=g).bfloat16()
  for p in ops.TUNE_ROWS:
    ops.set_product_choice(p, N, K, False, choice)
    ops.set_product_choice(p, 2 * inter, K, True, choice)
  assert ops.skinny_preferred(M, N, K) == own and ops.skinny_preferred(M, 2 * inter, K, True) == own
  if own:
    assert ops.skinny_variant(M, N, K) == choice - 1
  y = linear(x.to(DEV), w.to(DEV))
  torch.testing.assert_close(y.double().cpu(), x.double() @ w.double().T, rtol=2e-2, atol=2e-2)
  a = gate_up_activation(x.to(DEV), wgu.to(DEV))
  gu = x.double() @ wgu.double().T
  want = torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]
  torch.testing.assert_close(a.double().cpu(), want, rtol=3e-2, atol=3e-2)


@pytest.mark.parametrize("library", [True, False])
@pytest.mark.parametrize("M", [5, 40, 150])
def test_32_bit_results_from_bfloat16_operands_either_way(M, library, monkeypatch):
  """The logits' product: this library's kernel for up to 16 rows; beyond, the library's product with a 32-bit
  result, or (where a torch has none) the own kernel 64 rows at a time."""
  from miniinfer_amd.parts import linear as lin
  monkeypatch.setattr(lin, "_MM_TAKES_OUT_DTYPE", [library])
  g = torch.Generator().manual_seed(M)
  x = torch.randn(M, 96, generator=g).bfloat16()
  w = (torch.randn(333, 96, generator=g) * 0.1).bfloat16()
  y = lin.linear(x.to(DEV), w.to(DEV), out_dtype=torch.float32)
  assert y.dtype == torch.float32 and tuple(y.shape) == (M, 333)
  torch.testing.assert_close(y.double().cpu(), x.double() @ w.double().T, rtol=1e-4, atol=1e-3)
