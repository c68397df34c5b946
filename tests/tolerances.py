"""Floating-point acceptance rules shared by the GPU parity tests.

Two criteria, both required:
  * max|got - want| / max|want| <= 1e-2, the tolerance the path is specified to (bf16 outputs, f32 accumulation);
  * elementwise |got - want| <= 2e-2 * |want| + 1e-2 * rms(want) (3e-2 * rms for chained results, see below): the shape of the reference's own layer check
    (tests/unit/moe_test.py:78-83, rtol 2e-2 / atol 1e-2 on outputs of order one), with the absolute term tied to
    the tensor's own scale so that small-magnitude outputs cannot hide behind a large maximum.
"""

import torch

TOL = 1e-2
ELEM_RTOL = 2e-2
ELEM_ATOL_RMS = 1e-2
# For results that pass through values rounded to bf16 on the way (a chain of matmuls with bf16 intermediates, weights
# dequantised to bf16 before the product, gradients of such chains): the error of an element then scales with the
# magnitude of those intermediates, not with its own, and a handful of elements in 10^5 land between 1 and 3 % of the
# tensor's rms away from an f64 evaluation.
ELEM_ATOL_RMS_CHAINED = 3e-2


def relerr(got: torch.Tensor, want: torch.Tensor, elementwise: bool = True, atol_rms: float = ELEM_ATOL_RMS) -> float:
  """Max-norm relative error; raises if the elementwise criterion fails."""
  got, want = got.detach().float().cpu(), want.detach().float().cpu()
  assert got.shape == want.shape, (got.shape, want.shape)
  diff = (got - want).abs()
  if elementwise and want.numel():
    rms = float(want.double().pow(2).mean().sqrt())
    bound = ELEM_RTOL * want.abs() + atol_rms * rms
    bad = diff > bound
    if bool(bad.any()):
      i = int(torch.argmax((diff - bound).flatten()))
      raise AssertionError(
          f"elementwise tolerance: {int(bad.sum())} of {want.numel()} values off; worst at flat index {i}: "
          f"got {float(got.flatten()[i])}, want {float(want.flatten()[i])}, rms(want) {rms}")
  return float(diff.max() / want.abs().max().clamp_min(1e-30))
