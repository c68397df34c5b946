"""Checkpoint-shaped tensors -> formats adapters -> moe_gmm on the GPU, against the matmul of what the reference's
converters dequantise those tensors to (oracle restatements; the converters' own vectors pin them in
tests/test_formats.py and tests/test_oracle_golden.py)."""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tolerances import ELEM_ATOL_RMS_CHAINED, TOL, relerr

pytestmark = pytest.mark.gpu


def gmm_bf16(M, *args, **kwargs):
  """megablox.gmm with the layer dtype as preferred_element_type, as the reference's layer calls it (moe.py:1549)."""
  kwargs.setdefault("preferred_element_type", torch.bfloat16)
  return M.gmm(*args, **kwargs)


@pytest.fixture(scope="module")
def M():
  from maxtext_amd import _lib, megablox

  _lib.load()
  assert torch.cuda.is_available()
  return megablox


def dev(qa):
  from maxtext_amd.quantizations import QArray

  return QArray(qa.qvalue.cuda(), qa.scale.cuda(), qa.qtype, block_n=qa.block_n, block_k=qa.block_k, kmajor=qa.kmajor, shared=qa.shared)


def grouped(lhs, w_gnk, gs):
  """out[rows of group g] = lhs[rows] @ w[g]^T in f64; rows of no group are zero."""
  out = torch.zeros(lhs.shape[0], w_gnk.shape[1], dtype=torch.float64)
  start = 0
  for g_, sz in enumerate(gs):
    out[start : start + sz] = lhs[start : start + sz].double() @ w_gnk[g_].double().T
    start += sz
  return out


# rows per expert on both sides of the dispatch between the streaming kernels (decode) and the LDS-tiled ones (prefill)
GROUPS = [[3, 0, 7, 1], [300, 0, 180, 140]]


@pytest.mark.parametrize("gs", GROUPS)
def test_deepseek_fp8_state_dict_through_gmm(M, gs):
  """DeepSeek-V3 HF tensors (experts.{e}.*_proj.weight float8_e4m3fn + weight_scale_inv [N/128, K/128]) -> fp8 x fp8
  grouped matmul with 1 x 128 activation scales; expected: activations and weights dequantised per block
  (deepseek_dequantize.py:62-68), multiplied in f64."""
  from maxtext_amd import formats

  g = torch.Generator().manual_seed(3)
  e, n, k = len(gs), 384, 512
  m = sum(gs) + 5
  state = {}
  for i in range(e):
    for proj in ("gate_proj", "up_proj", "down_proj"):
      state[f"model.layers.7.mlp.experts.{i}.{proj}.weight"] = torch.randn(n, k, generator=g).to(torch.float8_e4m3fn)
      state[f"model.layers.7.mlp.experts.{i}.{proj}.weight_scale_inv"] = torch.rand(n // 128, k // 128, generator=g) * 0.02 + 1e-3
  w0, w1, _ = formats.deepseek_fp8_layer(state, 7, e)
  x = torch.randn(m, k, generator=g).to(torch.bfloat16)
  xq = M.quantize_lhs(x.cuda(), "fp8", blocks=128)
  gsz = np.array(gs, np.int32)
  got = gmm_bf16(M, xq, dev(w0), torch.from_numpy(gsz).cuda(), transpose_rhs=True)
  xs = xq.scale.cpu().reshape(m, k // 128)
  x_deq = (xq.qvalue.cpu().float().reshape(m, k // 128, 128) * xs[..., None]).reshape(m, k)
  w_deq = torch.stack([O.dequantize_fp8_blocks(w0.qvalue[i], w0.scale[i], 128).float() for i in range(e)])
  # (dequantize_fp8_blocks rounds to bf16; the kernel applies the block scales in f32: one bf16 ulp of the weights)
  want = grouped(x_deq, w_deq, gs)
  assert relerr(got, want) <= TOL
  # fused gate/up + SiLU as the layer runs it
  got_glu = gmm_bf16(M, xq, dev(w0), torch.from_numpy(gsz).cuda(), transpose_rhs=True, rhs_up=dev(w1), fuse_act="silu")
  w1_deq = torch.stack([O.dequantize_fp8_blocks(w1.qvalue[i], w1.scale[i], 128).float() for i in range(e)])
  h0, h1 = want, grouped(x_deq, w1_deq, gs)
  # a product of two matmul results: the error of either factor scales with the other, not with the product
  assert relerr(got_glu, torch.nn.functional.silu(h0) * h1, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2


@pytest.mark.parametrize("gs", GROUPS)
@pytest.mark.parametrize("group_size", [128, 32])
def test_compressed_int4_through_gmm(M, gs, group_size):
  """compressed-tensors pack-quantized int4 (int32 words, value + 8 per nibble, bf16 group scales;
  convert_deepseek_family_ckpt.py:56-84) -> bf16 x int4 grouped matmul; expected: the converter's dequantisation."""
  from maxtext_amd import formats

  rng = np.random.default_rng(5)
  e, n, k = len(gs), 192, 512
  m = sum(gs) + 3
  packed, scales, w_deq = [], [], []
  for _ in range(e):
    w = rng.integers(-8, 8, (n, k))
    words = np.zeros((n, k // 8), np.int64)
    for j in range(8):
      words |= ((w[:, j::8] + 8) & 0xF) << (4 * j)
    packed.append(torch.from_numpy(words.astype(np.uint32).view(np.int32).reshape(n, k // 8)))
    sc = torch.tensor(rng.random((n, k // group_size)) * 0.05 + 0.01, dtype=torch.bfloat16)
    scales.append(sc)
    w_deq.append((torch.from_numpy(w).float().reshape(n, k // group_size, group_size) * sc.float()[..., None]).reshape(n, k))
  qa = formats.compressed_int4_experts(packed, scales, [(n, k)] * e, group_size=group_size)
  x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).to(torch.bfloat16)
  got = gmm_bf16(M, x.cuda(), dev(qa), torch.tensor(gs, dtype=torch.int32).cuda(), transpose_rhs=True)
  assert relerr(got, grouped(x, torch.stack(w_deq), gs)) <= TOL


@pytest.mark.parametrize("gs", GROUPS)
def test_gpt_oss_mxfp4_through_gmm(M, gs):
  """GPT-OSS gate_up_proj_blocks / _scales / _bias with interleaved gate and up channels
  (convert_gpt_oss_ckpt.py:269-276) -> fused bf16 x mxfp4 matmul with biases and the clipped activation; expected:
  dequantize_mxfp4.py's values, split even / odd, through the oracle's activation."""
  from maxtext_amd import formats

  g = torch.Generator().manual_seed(6)
  e, f, d = len(gs), 160, 256
  m = sum(gs) + 2
  blocks = torch.randint(0, 256, (e, 2 * f, d // 32, 16), generator=g, dtype=torch.uint8)
  scales = torch.randint(118, 124, (e, 2 * f, d // 32), generator=g, dtype=torch.uint8)
  dblocks = torch.randint(0, 256, (e, d, f // 32, 16), generator=g, dtype=torch.uint8)
  dscales = torch.randint(118, 124, (e, d, f // 32), generator=g, dtype=torch.uint8)
  bias = torch.randn(e, 2 * f, generator=g) * 0.1
  dbias = torch.randn(e, d, generator=g) * 0.1
  wi_0, wi_1, wo, (b0, b1, bo) = formats.gpt_oss_mxfp4_layer(blocks, scales, dblocks, dscales, bias, dbias)
  x = (torch.randn(m, d, generator=g)).to(torch.bfloat16)
  gsz = torch.tensor(gs, dtype=torch.int32).cuda()
  inter = gmm_bf16(M, x.cuda(), dev(wi_0), gsz, transpose_rhs=True, rhs_up=dev(wi_1), fuse_act="swigluoai", act_limit=7.0,
                rhs_bias=b0.cuda(), rhs_up_bias=b1.cuda())
  full = O.dequantize_mxfp4(blocks, scales).float()  # [e, 2f, d]
  row_e = np.repeat(np.arange(e), gs)
  nrow = len(row_e)
  h0 = grouped(x, full[:, 0::2], gs)
  h1 = grouped(x, full[:, 1::2], gs)
  h0[:nrow] += bias[:, 0::2].double()[row_e]
  h1[:nrow] += bias[:, 1::2].double()[row_e]
  want_inter = O.apply_ffn_activation(h0.float(), h1.float(), "swigluoai", 7.0, out_dtype=torch.float32)
  want_inter[nrow:] = 0
  assert relerr(inter, want_inter, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2
  out = gmm_bf16(M, inter, dev(wo), gsz, transpose_rhs=True, rhs_bias=bo.cuda())
  want = grouped(inter.cpu(), O.dequantize_mxfp4(dblocks, dscales).float(), gs)
  want[:nrow] += dbias.double()[row_e]
  assert relerr(out, want) <= TOL


@pytest.mark.parametrize("gs", GROUPS)
def test_aqt_int8_serve_kernel_through_gmm(M, gs):
  """AQT serve-mode expert kernel (qvalue [E, K, N] int8, scale [E, 1, N]; moe.py:1450-1459: ragged_dot on the int8
  values, then times the row's expert scale) -> bf16 x int8 grouped matmul."""
  from maxtext_amd import formats

  g = torch.Generator().manual_seed(7)
  e, k, n = len(gs), 256, 320
  m = sum(gs)
  q = torch.randint(-127, 128, (e, k, n), generator=g, dtype=torch.int8)
  s = torch.rand(e, 1, n, generator=g) * 0.01 + 1e-3
  qa = formats.aqt_int8_experts(q, s)
  x = torch.randn(m, k, generator=g).to(torch.bfloat16)
  got = gmm_bf16(M, x.cuda(), dev(qa), torch.tensor(gs, dtype=torch.int32).cuda(), transpose_rhs=True)
  want = grouped(x, q.transpose(1, 2).float(), gs) * s[:, 0].double()[np.repeat(np.arange(e), gs)]
  assert relerr(got, want) <= TOL
