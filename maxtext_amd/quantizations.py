"""Weight-side quantisers and storage formats (offline preparation, torch ops on any device).

Activations are quantised by the HIP kernels (kernels.gather_rows); the functions here prepare
expert weights once, at load time, in the layouts the grouped GEMM reads:

  int8   per-output-channel, per expert:  q [G, N, K] int8,  scale [G, N] f32
         (serve-mode layout gathered per row at src/maxtext/layers/moe.py:1450-1459;
          share_across_experts=True gives the [1,1,n] scale of kernels/megablox/ops.py:250-260)
  fp8    e4m3fn, 128x128 blocks:          q [G, N, K] fp8,   scale [G, ceil(N/128), ceil(K/128)] f32
         (storage format of checkpoint_conversion/standalone_scripts/deepseek_dequantize.py:42-68)
  int4   symmetric, groups of 128 along K: q [G, N, K/2] uint8 (two per byte, first value in the
         low nibble, stored +8 -- convert_deepseek_family_ckpt.py:56-84), scale [G, N, ceil(K/128)] bf16

Rounding: scale = absmax / qmax, q = round-half-even(x / scale) clipped; a zero absmax gives q = 0.
"""

from __future__ import annotations

import dataclasses
import math

import torch

FP8_E4M3_MAX = 448.0


@dataclasses.dataclass
class QArray:
  """Quantised tensor: values plus scales (the role qwix.pallas.QArray plays in ops.py:232-267).

  For expert weights `qvalue` is [G, N, K] (K contiguous; INT4: uint8 [G, N, K/2]) and `scale`
  has the layout described in the module docstring; `qtype` is "int8" | "fp8" | "int4" | "int4g32" | "mxfp4"
  (mxfp4: uint8 [G, N, K/2] e2m1 pairs and uint8 [G, N, K/32] e8m0 block scales).
  For activations `qvalue` is [M, K] and `scale` is [M] (int8) or [M, ceil(K/128)] (fp8).

  The optional fields override the layout a qtype implies (they mirror the scale arguments of moe_gmm):
  block_n / block_k: output channels / values of K per scale (block_n -1: one scale for all channels; block_k 0: all
  of K; for activations block_k -1: one scale for the tensor), kmajor: weight scales stored [G, K/block_k, N]
  (gmm_v2's [G, nb, 1, N]), shared: weight scales without the leading expert dimension.
  """

  qvalue: torch.Tensor
  scale: torch.Tensor
  qtype: str
  block_n: int | None = None
  block_k: int | None = None
  kmajor: bool = False
  shared: bool = False

  @property
  def shape(self):
    return self.qvalue.shape


@dataclasses.dataclass
class QtRule:
  """The fields of qwix.QtRule that gmm reads (ops.py:97-103, :241-266, :583-604)."""

  weight_qtype: object = None
  act_qtype: object = None
  bwd_qtype: object = None
  weight_calibration_method: str = "absmax"
  act_calibration_method: str = "absmax"
  bwd_calibration_method: str = "absmax"
  disable_channelwise_axes: bool = False


def get_static_scale(qmax: float, calibration_method: str) -> float:
  """Static symmetric scale from "fixed,max" / "fixed,-max,max" (layers/quantizations.py:928-958)."""
  if calibration_method is None or not calibration_method.lower().startswith("fixed"):
    raise ValueError(f"Only static scale quantization is supported, got {calibration_method}")
  args = [float(a) for a in calibration_method.split(",")[1:]]
  if len(args) == 1:
    args = [-args[0], args[0]]
  if len(args) != 2 or args[0] + args[1] != 0 or args[1] <= 0:
    raise ValueError(f"Expected format: 'fixed,max' or 'fixed,-max,max'. Got: {calibration_method}")
  scale = args[1] / qmax
  if scale < torch.finfo(torch.float32).tiny ** 0.5:
    scale = 1.0
  return scale


def _rint_div(x, scale):
  return torch.where(scale == 0, torch.zeros_like(x), torch.round(x / scale))


def quantize_weight_int8(w_gnk: torch.Tensor, share_across_experts: bool = False) -> QArray:
  """w [G, N, K] -> int8 per output channel."""
  w = w_gnk.to(torch.float32)
  if share_across_experts:
    absmax = w.abs().amax(dim=(0, 2), keepdim=True).expand(w.shape[0], w.shape[1], 1)
  else:
    absmax = w.abs().amax(dim=2, keepdim=True)
  scale = absmax / 127.0
  q = _rint_div(w, scale).clamp(-127, 127).to(torch.int8)
  return QArray(q.contiguous(), scale.squeeze(-1).contiguous(), "int8")


def quantize_weight_fp8_channel(w_gnk: torch.Tensor, share_across_experts: bool = True) -> QArray:
  """w [G, N, K] -> float8_e4m3fn with one f32 scale per output channel: shared by the experts ([1, 1, n], what
  qpl.quantize(rhs, channelwise_axes=[2]) yields, ops.py:250-260) or per expert.  The rounding of the third-party
  quantiser is not pinned; this uses scale = absmax / 448 and the round-to-nearest-even cast."""
  w = w_gnk.to(torch.float32)
  absmax = w.abs().amax(dim=(0, 2) if share_across_experts else 2, keepdim=True)
  scale = absmax / FP8_E4M3_MAX
  q = torch.where(scale == 0, torch.zeros_like(w), w / scale).clamp(-FP8_E4M3_MAX, FP8_E4M3_MAX).to(torch.float8_e4m3fn)
  sc = scale.reshape(1, -1) if share_across_experts else scale.squeeze(-1)
  return QArray(q.contiguous(), sc.contiguous(), "fp8", block_n=1, block_k=0, shared=share_across_experts)


def manual_quantize_weight(w_gnk: torch.Tensor, qtype: str, calibration_method: str) -> QArray:
  """Per-tensor static weight quantisation, layers/quantizations.py:961-991 (manual_quantize):
  q = clip(w / scale, -qmax, qmax).astype(qtype) with scale and bounds held as bf16 tensors (:923-925), so the
  division runs in promote(w.dtype, bf16); the QArray's scale is the python float in w's dtype.  int8 truncates
  toward zero, fp8 rounds to nearest even, as `.astype` does."""
  qmax = 127.0 if qtype == "int8" else FP8_E4M3_MAX
  scale = get_static_scale(qmax, calibration_method)
  s_bf = torch.tensor(scale, dtype=torch.float32).to(torch.bfloat16).float()
  y = w_gnk.float() / s_bf.to(w_gnk.device)
  if w_gnk.dtype == torch.bfloat16:
    y = y.to(torch.bfloat16).float()
  bound = float(torch.tensor(qmax).to(torch.bfloat16))
  y = y.clamp(-bound, bound)
  q = torch.trunc(y).clamp(-128, 127).to(torch.int8) if qtype == "int8" else y.to(torch.float8_e4m3fn)
  sc = torch.tensor([scale], dtype=torch.float32).to(w_gnk.dtype).float().to(w_gnk.device)
  return QArray(q.contiguous(), sc, qtype, block_n=-1, block_k=0, shared=True)


def quantize_weight_fp8_blocks(w_gnk: torch.Tensor, block: int = 128) -> QArray:
  """w [G, N, K] -> float8_e4m3fn with one f32 scale per block x block tile."""
  g, n, k = w_gnk.shape
  nb, kb = math.ceil(n / block), math.ceil(k / block)
  wp = torch.zeros((g, nb * block, kb * block), dtype=torch.float32, device=w_gnk.device)
  wp[:, :n, :k] = w_gnk
  wb = wp.view(g, nb, block, kb, block)
  scale = wb.abs().amax(dim=(2, 4), keepdim=True) / FP8_E4M3_MAX
  q = torch.where(scale == 0, torch.zeros_like(wb), wb / scale).clamp(-FP8_E4M3_MAX, FP8_E4M3_MAX)
  q = q.view(g, nb * block, kb * block)[:, :n, :k].to(torch.float8_e4m3fn)
  return QArray(q.contiguous(), scale.view(g, nb, kb).contiguous(), "fp8")


def quantize_weight_int4(w_gnk: torch.Tensor, group: int = 128) -> QArray:
  """w [G, N, K] -> packed int4 with bf16 scales per `group` values of K (ragged last group allowed)."""
  g, n, k = w_gnk.shape
  if k % 2:
    raise ValueError("K must be even to pack two int4 values per byte")
  ng = math.ceil(k / group)
  wp = torch.zeros((g, n, ng * group), dtype=torch.float32, device=w_gnk.device)
  wp[:, :, :k] = w_gnk
  wg = wp.view(g, n, ng, group)
  scale = (wg.abs().amax(-1, keepdim=True) / 7.0).clamp(min=1e-12).to(torch.bfloat16)
  q = torch.round(wg / scale.to(torch.float32)).clamp(-8, 7).to(torch.int16).view(g, n, ng * group)[:, :, :k]
  u = (q + 8).to(torch.uint8)
  packed = (u[..., 0::2] | (u[..., 1::2] << 4)).contiguous()
  return QArray(packed, scale.squeeze(-1).contiguous(), "int4" if group == 128 else f"int4g{group}")


def quantize_weight_mxfp4(w_gnk: torch.Tensor) -> QArray:
  """w [G, N, K] -> OCP MX fp4: e2m1 values (two per byte along K, first in the low nibble) with one e8m0 scale per
  32 values, the storage format of GPT-OSS checkpoints (dequantize_mxfp4.py:46-72).  Shared exponent =
  floor(log2(absmax of the block)) - 2, values rounded to the nearest e2m1 point, saturating at +-6."""
  g, n, k = w_gnk.shape
  if k % 32:
    raise ValueError("K must be a multiple of 32")
  x = w_gnk.float().reshape(g, n, k // 32, 32)
  amax = x.abs().amax(-1, keepdim=True)
  exp = torch.where(amax > 0, torch.floor(torch.log2(amax.clamp_min(1e-38))) - 2.0, torch.zeros_like(amax)).clamp(-127, 127)
  y = (x / torch.exp2(exp)).clamp(-6.0, 6.0)
  a = y.abs()
  # e2m1 magnitudes 0, .5, 1, 1.5, 2, 3, 4, 6 -> codes 0..7; thresholds are the midpoints (ties to the even code)
  code = ((a > 0.25).to(torch.uint8) + (a >= 0.75).to(torch.uint8) + (a > 1.25).to(torch.uint8) + (a >= 1.75).to(torch.uint8)
          + (a > 2.5).to(torch.uint8) + (a >= 3.5).to(torch.uint8) + (a > 5.0).to(torch.uint8))
  code = code | ((y < 0).to(torch.uint8) << 3)
  packed = (code[..., 0::2] | (code[..., 1::2] << 4)).reshape(g, n, k // 2).contiguous()
  scale = (exp.squeeze(-1) + 127.0).to(torch.uint8).contiguous()
  return QArray(packed, scale, "mxfp4")


def split_gate_kernel(kernel_de: torch.Tensor, terms: int = 3) -> torch.Tensor:
  """GateLogit kernel [d, E] (f32, moe.py:247-318) -> [terms, E, d] bf16 with sum(terms) == kernel to 24
  mantissa bits for terms == 3 (hi, mid, lo), the form moe_gate_route consumes; terms == 1 is the bf16 cast
  the reference applies when the gate runs in bf16 (moe.py:366)."""
  if terms not in (1, 3):
    raise ValueError("terms must be 1 or 3")
  w = kernel_de.detach().float().t().contiguous()
  out, rest = [], w
  for _ in range(terms):
    piece = rest.to(torch.bfloat16)
    out.append(piece)
    rest = rest - piece.float()
  return torch.stack(out).contiguous()
