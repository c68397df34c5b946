"""GPU parity of the fp8_full recipe: e4m3 x e4m3 forward with per-row x per-channel (or static per-tensor) scales
(kernels/megablox/ops.py:232-267; rule of layers/quantizations.py:234-250, :798-855), its backward with quantised
residuals and float8_e5m2 gradients (ops.py:438-604), at sizes that reach the persistent 256 x 256 kernel and at sizes
that do not, against the CPU oracle on the oracle's own quantised operands.
"""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tolerances import ELEM_ATOL_RMS_CHAINED, relerr

pytestmark = pytest.mark.gpu


def gmm_bf16(*args, **kwargs):
  """megablox.gmm with the layer dtype as preferred_element_type, as the reference's layer calls it (moe.py:1549)."""
  from maxtext_amd import megablox

  kwargs.setdefault("preferred_element_type", torch.bfloat16)
  return megablox.gmm(*args, **kwargs)

TOL = 1e-2
E4M3 = torch.float8_e4m3fn


@pytest.fixture(scope="module")
def K():
  from maxtext_amd import kernels

  assert torch.cuda.is_available()
  return kernels


def cuda(x):
  if isinstance(x, np.ndarray):
    x = torch.from_numpy(x)
  return x.cuda().contiguous()


def _rows_fp8(x):
  """One scale per row: scale = absmax / 448, q = e4m3(x / scale) (the v1 rule this library adopts)."""
  s = x.abs().amax(1, keepdim=True) / 448.0
  q = torch.where(s == 0, torch.zeros_like(x), x / s).clamp(-448, 448).to(E4M3)
  return q, s[:, 0].contiguous()


def _channels_fp8(w_gnk, shared):
  """One scale per output channel, shared by the experts ([1, 1, n], ops.py:250-260) or per expert."""
  amax = w_gnk.abs().amax(dim=(0, 2) if shared else 2, keepdim=True)
  s = amax / 448.0
  q = torch.where(s == 0, torch.zeros_like(w_gnk), w_gnk / s).clamp(-448, 448).to(E4M3)
  return q, (s.reshape(1, -1) if shared else s.squeeze(-1)).contiguous()


def _problem(m, k, n, gs, seed):
  g = torch.Generator().manual_seed(seed)
  lhs = torch.randn(m, k, generator=g)
  w = torch.randn(len(gs), n, k, generator=g) * 0.05  # [G, N, K]
  return lhs, w, np.asarray(gs, np.int32)


# sizes the persistent stream kernel takes (128 rows per group on average, >= 128 tiles of 256 x 256) and sizes it does not
BIG = dict(m=4200, k=512, n=2048, gs=[1500, 0, 700, 1900])  # 100 trailing rows in no group; ragged tiles in every group
SMALL = dict(m=450, k=256, n=192, gs=[200, 0, 70, 150])


@pytest.mark.parametrize("shape", [BIG, SMALL], ids=["stream", "tiled"])
@pytest.mark.parametrize("shared", [True, False])
def test_gmm_fp8_row_by_channel_scales(K, shape, shared):
  """e4m3 x e4m3 with [m] x [n] scales applied to the finished sums: the oracle's dequantised product, and at the
  large shape the persistent kernel against the 128 x 128 kernel forced on the same operands."""
  lhs, w, gs = _problem(shape["m"], shape["k"], shape["n"], shape["gs"], 5)
  lq, ls = _rows_fp8(lhs)
  rq, rs = _channels_fp8(w, shared)
  want = O.gmm(lq, rq, gs, lhs_scale=ls, rhs_scale=rs, transpose_rhs=True)
  kw = dict(lhs_scale=cuda(ls), rhs_scale=cuda(rs), rhs_scale_block_n=1, rhs_scale_block_k=0, rhs_scale_shared=shared)
  got = K.gmm_raw(cuda(lq), cuda(rq), cuda(gs), **kw)
  assert relerr(got, want) <= TOL
  total = int(gs.sum())
  assert torch.all(got[total:] == 0)
  if shape is BIG:
    other = K.gmm_raw(cuda(lq), cuda(rq), cuda(gs), kernel="tiled", **kw)
    assert relerr(got, other.cpu()) <= 2e-3  # the same products in another order of summation, rounded to bf16


@pytest.mark.parametrize("shared", [True, False])
@pytest.mark.parametrize("m,k,n,gs", [(40, 1024, 128, [7, 0, 12, 1, 20]), (90, 3584, 328, [10, 25, 1, 16, 17, 9, 12]), (420, 512, 256, [1] * 300 + [100]),
                                      (45, 7680, 136, [7, 0, 12, 1, 20]), (70, 14336, 256, [5, 0, 9, 14, 3, 11, 2, 16, 1]),  # (rows past 7168 values)
                                      (100, 2048, 200, [32, 0, 17, 5, 31, 1]), (310, 1024, 128, [25] * 12),  # (32-row tiles)
                                      (160, 2048, 200, [64, 0, 17, 5, 63, 1]), (200, 512, 256, [40] * 5), (200, 8192, 264, [65, 30, 64, 1, 0, 30])])  # (64-row)
def test_gmm_fp8_row_by_channel_scales_at_decode_sizes(K, m, k, n, gs, shared):
  """e4m3 x e4m3 with [m] x [n] scales at a handful of rows per expert: the LDS-streamed persistent kernel (row and channel
  scales applied to the finished sums) against the oracle and against the register-staged kernel; both projections with
  an activation, biases, f32 output and rows read through an index."""
  lhs, w, gs = _problem(m, k, n, gs, 41)
  g = torch.Generator().manual_seed(42)
  w_up = torch.randn(len(gs), n, k, generator=g) * 0.05
  lq, ls = _rows_fp8(lhs)
  rq, rs = _channels_fp8(w, shared)
  uq, us = _channels_fp8(w_up, shared)
  kw = dict(lhs_scale=cuda(ls), rhs_scale=cuda(rs), rhs_scale_block_n=1, rhs_scale_block_k=0, rhs_scale_shared=shared)
  got = K.gmm_raw(cuda(lq), cuda(rq), cuda(gs), **kw)
  assert relerr(got, O.gmm(lq, rq, gs, lhs_scale=ls, rhs_scale=rs, transpose_rhs=True)) <= TOL
  assert torch.all(got[int(gs.sum()):] == 0)
  old = K.gmm_raw(cuda(lq), cuda(rq), cuda(gs), kernel="stream", **kw)
  assert relerr(got, old.cpu()) <= 8e-3  # the same products in another order of summation, rounded to bf16
  b0, b1 = torch.randn(len(gs), n, generator=g) * 0.1, torch.randn(len(gs), n, generator=g) * 0.1
  t_rows = max(m // 3, 1)
  idx = torch.randint(0, t_rows * 3, (m,), generator=g, dtype=torch.int32)
  rows = (idx // 3).long()
  got = K.gmm_raw(cuda(lq[:t_rows]), cuda(rq), cuda(gs), lhs_scale=cuda(ls[:t_rows]), rhs_scale=cuda(rs), rhs_up=cuda(uq), rhs_up_scale=cuda(us),
                  rhs_scale_block_n=1, rhs_scale_block_k=0, rhs_scale_shared=shared, act="swigluoai", act_limit=7.0, rhs_bias=cuda(b0),
                  rhs_up_bias=cuda(b1), lhs_row_idx=cuda(idx), lhs_row_idx_div=3, out_dtype=torch.float32)
  h0 = O.gmm(lq[rows], rq, gs, lhs_scale=ls[rows], rhs_scale=rs, transpose_rhs=True, rhs_bias=b0[:, None, :], out_dtype=torch.float32)
  h1 = O.gmm(lq[rows], uq, gs, lhs_scale=ls[rows], rhs_scale=us, transpose_rhs=True, rhs_bias=b1[:, None, :], out_dtype=torch.float32)
  want = O.apply_ffn_activation(h0, h1, "swigluoai", 7.0, out_dtype=torch.float32)
  assert got.dtype == torch.float32 and relerr(got, want) <= TOL


@pytest.mark.parametrize("act", ["silu", "swigluoai"])
def test_gmm_fp8_channel_scales_fused_glu_bias_and_row_index(K, act):
  """The persistent fp8 kernel with rhs_up + activation, per-expert biases, f32 output and activation rows read through
  an index (the fused permute): every epilogue variant of the int8 kernel carries over."""
  m, k, n, gs = 4096, 384, 2048, [1024, 1100, 900, 1072]
  t_rows = 1024
  g = torch.Generator().manual_seed(9)
  x = torch.randn(t_rows, k, generator=g)
  idx = torch.randint(0, t_rows * 4, (m,), generator=g, dtype=torch.int32)
  w0 = torch.randn(4, n, k, generator=g) * 0.05
  w1 = torch.randn(4, n, k, generator=g) * 0.05
  b0 = torch.randn(4, n, generator=g) * 0.1
  b1 = torch.randn(4, n, generator=g) * 0.1
  xq, xs = _rows_fp8(x)
  q0, s0 = _channels_fp8(w0, True)
  q1, s1 = _channels_fp8(w1, True)
  rows = (idx // 4).long()
  lq, ls = xq[rows], xs[rows]
  h0 = O.gmm(lq, q0, gs, lhs_scale=ls, rhs_scale=s0, transpose_rhs=True, rhs_bias=b0[:, None, :], out_dtype=torch.float32)
  h1 = O.gmm(lq, q1, gs, lhs_scale=ls, rhs_scale=s1, transpose_rhs=True, rhs_bias=b1[:, None, :], out_dtype=torch.float32)
  want = O.apply_ffn_activation(h0, h1, act, 7.0, out_dtype=torch.float32)
  got = K.gmm_raw(cuda(xq), cuda(q0), cuda(np.asarray(gs, np.int32)), lhs_scale=cuda(xs), rhs_scale=cuda(s0), rhs_up=cuda(q1),
                  rhs_up_scale=cuda(s1), rhs_scale_shared=True, act=act, act_limit=7.0, rhs_bias=cuda(b0), rhs_up_bias=cuda(b1),
                  lhs_row_idx=cuda(idx), lhs_row_idx_div=4, out_dtype=torch.float32)
  assert got.dtype == torch.float32 and relerr(got, want) <= TOL
  plain = K.gmm_raw(cuda(lq), cuda(q0), cuda(np.asarray(gs, np.int32)), lhs_scale=cuda(ls), rhs_scale=cuda(s0), rhs_up=cuda(q1),
                    rhs_up_scale=cuda(s1), rhs_scale_shared=True, act=act, act_limit=7.0)
  want_plain = O.apply_ffn_activation(
      O.gmm(lq, q0, gs, lhs_scale=ls, rhs_scale=s0, transpose_rhs=True, out_dtype=torch.float32),
      O.gmm(lq, q1, gs, lhs_scale=ls, rhs_scale=s1, transpose_rhs=True, out_dtype=torch.float32), act, 7.0)
  assert relerr(plain, want_plain) <= TOL


def test_gmm_fp8_static_per_tensor_scales(K):
  """The static scales of "fixed,-224,224" calibration (tests/integration/tokamax_test.py:53-114): one value for the
  activations, one for the weights, both 0.5."""
  lhs, w, gs = _problem(BIG["m"], BIG["k"], BIG["n"], BIG["gs"], 6)
  lq = (lhs / 0.5).clamp(-448, 448).to(E4M3)
  rq = (w / 0.5).clamp(-448, 448).to(E4M3)
  half = torch.tensor([0.5])
  want = O.gmm(lq, rq, gs, lhs_scale=half.reshape(1, 1), rhs_scale=half.reshape(1, 1).expand(1, BIG["n"]), transpose_rhs=True)
  got = K.gmm_raw(cuda(lq), cuda(rq), cuda(gs), lhs_scale=cuda(half), lhs_scale_block_k=-1, rhs_scale=cuda(half), rhs_scale_block_n=-1,
                  rhs_scale_shared=True)
  assert relerr(got, want) <= TOL


def test_gmm_e5m2_gradient_times_e4m3_weights(K):
  """float8_e5m2 activations (the quantised gradient, ops.py:583-604) x e4m3 weights on the fp8 MFMA: values drawn over
  the whole e5m2 range incl. subnormals, compared with the exact product of the same bytes."""
  m, k, n, gs = 4200, 640, 2048, np.asarray([1500, 0, 700, 1900], np.int32)
  assert K.gmm_lhs_e5m2_supported(m, k, n, 4)
  g = torch.Generator().manual_seed(21)
  d = (torch.randn(m, k, generator=g) * torch.exp2(torch.randint(-16, 12, (m, 1), generator=g).float())).to(torch.float8_e5m2)
  d[3, :8] = torch.tensor([57344.0, -57344.0, 2.0**-16, -(2.0**-16), 2.0**-14, 0.0, 1.5 * 2.0**-15, 49152.0]).to(torch.float8_e5m2)
  w = (torch.randn(4, n, k, generator=g) * 3).to(E4M3)
  s_row = torch.rand(m, generator=g) * 1e-3 + 1e-5
  want = O.gmm(d.float(), w.float(), gs, lhs_scale=s_row, transpose_rhs=True, out_dtype=torch.float32)
  one = torch.ones(1)
  got = K.gmm_raw(cuda(d), cuda(w), cuda(gs), lhs_scale=cuda(s_row), rhs_scale=cuda(one), rhs_scale_block_n=-1, rhs_scale_shared=True,
                  out_dtype=torch.float32)
  assert relerr(got, want) <= 1e-4  # exact products; what is left is the order of the f32 additions
  with pytest.raises(RuntimeError):  # shapes the persistent kernel does not take are refused, not mis-run
    K.gmm_raw(cuda(d[:450]), cuda(w), cuda(np.asarray([200, 0, 100, 150], np.int32)), lhs_scale=cuda(s_row[:450]), rhs_scale=cuda(one),
              rhs_scale_block_n=-1, rhs_scale_shared=True)


@pytest.mark.parametrize("lhs_dtype", [torch.float8_e5m2, E4M3], ids=["e5m2", "e4m3"])
def test_gmm_fp8_weights_read_as_gkn(K, lhs_dtype):
  """MOE_GMM_RHS_KN with fp8 operands (dlhs of the fp8_full backward from the forward's [G, N, K] weights, ops.py:470-485,
  without the re-layout): bit-equal to the same product on the transposed copy, ragged groups, an empty group, rows in no
  group, a group window, per-row scales and a row factor."""
  m, kc, n, gs = 4200, 640, 2048, np.asarray([1500, 0, 700, 1900], np.int32)  # contraction kc, n output channels
  assert K.gmm_fp8_rhs_kn_supported(m, kc, n, 4) and not K.gmm_fp8_rhs_kn_supported(m, kc, n + 128, 4)
  g = torch.Generator().manual_seed(23)
  d = (torch.randn(m, kc, generator=g) * torch.exp2(torch.randint(-10, 8, (m, 1), generator=g).float())).clamp(-448, 448).to(lhs_dtype)
  w_kn = (torch.randn(4, kc, n, generator=g) * 3).to(E4M3)  # [G, K, N]
  w_nk = w_kn.float().transpose(1, 2).contiguous().to(E4M3)  # the re-laid-out copy, [G, N, K]
  s_row = torch.rand(m, generator=g) * 1e-3 + 1e-5
  fac = torch.rand(m, generator=g) + 0.5
  one = torch.ones(1)
  kw = dict(lhs_scale=cuda(s_row), rhs_scale=cuda(one), rhs_scale_block_n=-1, rhs_scale_shared=True, out_dtype=torch.float32)
  for extra in (dict(), dict(out_row_scale=cuda(fac))):
    ref = K.gmm_raw(cuda(d), cuda(w_nk), cuda(gs), **kw, **extra)
    got = K.gmm_raw(cuda(d), cuda(w_kn), cuda(gs), rhs_kn=True, **kw, **extra)
    assert torch.equal(got, ref)
  want = O.gmm(d.float(), w_nk.float(), gs, lhs_scale=s_row, transpose_rhs=True, out_dtype=torch.float32)
  assert relerr(got / cuda(fac)[:, None], want) <= 1e-4
  # bf16 results (the paired 16-byte stores), as the backward asks for them
  kw16 = dict(kw, out_dtype=torch.bfloat16)
  assert torch.equal(K.gmm_raw(cuda(d), cuda(w_kn), cuda(gs), rhs_kn=True, **kw16), K.gmm_raw(cuda(d), cuda(w_nk), cuda(gs), **kw16))
  # a window of two local groups
  ref = K.gmm_raw(cuda(d), cuda(w_nk[2:4]), cuda(gs), group_offset=2, **kw)
  got = K.gmm_raw(cuda(d), cuda(w_kn[2:4]), cuda(gs), group_offset=2, rhs_kn=True, **kw)
  assert torch.equal(got, ref)
  with pytest.raises(RuntimeError):  # K-block scales do not run there
    K.gmm_raw(cuda(d.to(E4M3)), cuda(w_kn), cuda(gs), rhs_kn=True, lhs_scale=cuda(torch.ones(m, kc // 128)), lhs_scale_block_k=128,
              rhs_scale=cuda(torch.ones(4, n // 128, kc // 128)), rhs_scale_block_n=128, rhs_scale_block_k=128)


@pytest.mark.parametrize("dout_dtype", [torch.float8_e5m2, E4M3], ids=["e5m2", "e4m3"])
@pytest.mark.parametrize("offset,g_local", [(0, 4), (1, 2)])
def test_tgmm_on_fp8_operands_as_stored(K, dout_dtype, offset, g_local):
  """The drhs product of the fp8_full backward (ops.py:590-604) on 1-byte operands: e4m3 activations x e5m2 (or e4m3)
  gradient over the whole value range incl. subnormals, ragged groups (a group of 77 rows, an empty one, rows in no
  group), column scales, existing_out and f32 output, against the exact product of the same bytes; and equal, up to
  the order of the f32 additions, to the bf16 kernel on the widened operands."""
  m, k, n, gs = 4300, 2048, 2048, np.asarray([1500, 0, 77, 2600], np.int32)
  assert K.tgmm_fp8_supported(m, k, n, 4, g_local) and not K.tgmm_fp8_supported(m, 512, 1024, 4, g_local)
  g = torch.Generator().manual_seed(31 + offset)
  lhs = (torch.randn(m, k, generator=g) * torch.exp2(torch.randint(-8, 6, (m, 1), generator=g).float())).to(E4M3)
  spread = (-16, 12) if dout_dtype == torch.float8_e5m2 else (-8, 6)
  d = (torch.randn(m, n, generator=g) * torch.exp2(torch.randint(*spread, (1, n), generator=g).float())).to(dout_dtype)
  s_col = torch.rand(n, generator=g) * 1e-2 + 1e-4
  prev = (torch.randn(g_local, n, k, generator=g) * 4).to(torch.bfloat16)
  # oracle: [groups, k, n] from the dequantised bytes in f64, scaled per output row n, laid out [groups, n, k]
  want = O.tgmm(lhs.float(), d.float(), gs, num_actual_groups=g_local, group_offset=offset, out_dtype=torch.float64)
  want = want.transpose(1, 2) * s_col.double()[None, :, None]
  kw = dict(num_groups_local=g_local, group_offset=offset)
  got = K.tgmm_fp8(cuda(lhs), cuda(d), cuda(gs), out_row_scale=cuda(s_col), out_dtype=torch.float32, **kw)
  assert relerr(got, want.float()) <= 2e-4  # exact products; what is left is the order (and the MFMA's internal alignment) of the f32 additions
  wide = K.tgmm(cuda(lhs).to(torch.bfloat16), cuda(d).to(torch.bfloat16), cuda(gs), out_row_scale=cuda(s_col), out_dtype=torch.float32, **kw)
  assert relerr(got, wide) <= 2e-4
  # bf16 result (the paired-store epilogue), and existing_out joining the accumulator before the one rounding
  got16 = K.tgmm_fp8(cuda(lhs), cuda(d), cuda(gs), out_row_scale=cuda(s_col), **kw)
  assert torch.equal(got16, got.to(torch.bfloat16)) or relerr(got16, want.float()) <= 4e-3
  got_e = K.tgmm_fp8(cuda(lhs), cuda(d), cuda(gs), out_row_scale=cuda(s_col), existing_out=cuda(prev), **kw)
  assert relerr(got_e, (want + prev.double()).float()) <= 4e-3
  assert torch.all(got[1 - offset] == 0) if offset == 0 else True  # the empty group's gradient is zero
  with pytest.raises(RuntimeError):  # shapes without 256 x 256 tiles are refused, not mis-run
    K.tgmm_fp8(cuda(lhs[:, :384].contiguous()), cuda(d), cuda(gs), **kw)


@pytest.mark.parametrize("qdt", [torch.int8, E4M3], ids=["int8", "fp8"])
@pytest.mark.parametrize("shared", [True, False])
@pytest.mark.parametrize("G,N,Kd", [(3, 72, 264), (300, 16, 4096), (2, 24, 16384)], ids=["small", "two-pass", "long-rows"])
def test_quantize_rhs_bit_exact(K, qdt, shared, G, N, Kd):
  """The per-step weight quantiser (ops.py:250-260) against the host statement of the same rule: scale = absmax / qmax
  over each output channel (of all experts, or per expert), q = rint(w / scale) / the nearest-even float8 cast; values and
  scales bit for bit, incl. an all-zero channel and bf16 / bf16 quotients that are exact ties.  The shapes reach both
  routes: a channel that fits one block's registers (one pass) and, with 36 experts of 4096 values sharing a scale, one
  that does not (two passes)."""
  g = torch.Generator().manual_seed(41)
  w = (torch.randn(G, N, Kd, generator=g) * 0.05).to(torch.bfloat16)
  w[:, 5] = 0.0
  w[1, 9] = 0.0
  w[0, 7, :8] = torch.tensor([1.0, 0.5, 0.25, 0.75, -1.0, 0.375, 0.4375, 0.03125]).to(torch.bfloat16)
  w[:, 7, 8:] *= 0.1  # channel 7's absmax is the exact 1.0: its quotients are short binary fractions, many of them ties
  qmax = 127.0 if qdt == torch.int8 else 448.0
  wf = w.float()
  amax = wf.abs().amax(dim=(0, 2), keepdim=True) if shared else wf.abs().amax(dim=2, keepdim=True)
  sc = amax / qmax
  y = torch.where(sc == 0, torch.zeros_like(wf), wf / sc)
  want_q = torch.round(y).clamp(-qmax, qmax).to(qdt) if qdt == torch.int8 else y.clamp(-qmax, qmax).to(qdt)
  q, s = K.quantize_rhs(cuda(w), qdt, shared=shared)
  assert tuple(s.shape) == ((1, N) if shared else (G, N))
  assert torch.equal(s.cpu().reshape(-1), sc.reshape(-1))
  assert torch.equal(q.cpu().float(), want_q.float())
  assert float(s.cpu().reshape(-1, N)[0, 5]) == 0.0 and torch.all(q[:, 5].float() == 0)


@pytest.mark.parametrize("qdt,cal", [(torch.int8, "fixed,-4,4"), (E4M3, "fixed,-224,224"), (E4M3, "fixed,3")])
def test_quantize_rhs_static_equals_manual_quantize(K, qdt, cal):
  """The static per-tensor rule against the oracle's restatement of manual_quantize (layers/quantizations.py:961-991),
  pinned by exact rational arithmetic in the CPU tests: values bit for bit, out-of-range values clipped."""
  g = torch.Generator().manual_seed(42)
  w = (torch.randn(2, 40, 136, generator=g) * 2.0).to(torch.bfloat16)
  w[0, 0, :4] = torch.tensor([1000.0, -1000.0, 0.0, 3.0]).to(torch.bfloat16)
  qmax = 127.0 if qdt == torch.int8 else 448.0
  st = torch.tensor([O.get_static_scale(qmax, cal)], dtype=torch.float32)
  want_q, _ = O.manual_quantize(w, qdt, cal)
  q, s = K.quantize_rhs(cuda(w), qdt, static_scale=cuda(st))
  assert torch.equal(q.cpu().float(), want_q.float())


@pytest.mark.parametrize("n", [192, 2056])
def test_bwd_scale_grad_emits_e5m2_bytes(K, n):
  """quantize == 2 writes the float8_e5m2 bytes of exactly the values quantize == 1 writes as bf16, same scales."""
  g = torch.Generator().manual_seed(32)
  m = 333
  gs = np.array([40, 100, 0, 70, 93], np.int32)
  dout = (torch.randn(m, n, generator=g) * torch.rand(m, 1, generator=g) * 8).to(torch.bfloat16)
  dout[17] = 0.0
  dout[:, 11] = 0.0
  dout[5, 3] = float("inf")
  rs = torch.rand(3, n, generator=g) * 0.02 + 1e-4
  ls = torch.rand(m, generator=g) * 0.05 + 1e-4
  kw = dict(group_sizes=cuda(gs), num_groups_local=3, group_offset=1)
  b16, s16 = K.bwd_scale_grad(cuda(dout), cuda(rs), mode="dlhs", quantize=True, **kw)
  f8, s8 = K.bwd_scale_grad(cuda(dout), cuda(rs), mode="dlhs", quantize=True, as_fp8=True, **kw)
  assert f8.dtype == torch.float8_e5m2 and torch.equal(s16, s8)
  a, b = f8.float().cpu(), b16.float().cpu()
  assert torch.equal(torch.nan_to_num(a, nan=7.0), torch.nan_to_num(b, nan=7.0))
  b16, s16 = K.bwd_scale_grad(cuda(dout), cuda(ls), mode="drhs", quantize=True)
  f8, s8 = K.bwd_scale_grad(cuda(dout), cuda(ls), mode="drhs", quantize=True, as_fp8=True)
  assert torch.equal(torch.nan_to_num(s16, nan=7.0), torch.nan_to_num(s8, nan=7.0))
  assert torch.equal(torch.nan_to_num(f8.float(), nan=7.0), torch.nan_to_num(b16.float(), nan=7.0))


@pytest.mark.parametrize("shape", [BIG, SMALL], ids=["stream", "tiled"])
@pytest.mark.parametrize("calibration", ["absmax", "fixed,-224,224"])
@pytest.mark.parametrize("fwd", ["int8", "fp8"])
@pytest.mark.parametrize("bwd_q", [None, "float8_e5m2"])
def test_gmm_quantized_backward_fwd_dtypes_and_calibrations(shape, calibration, fwd, bwd_q):
  """The reference's quantised backward (ops.py:530-604) for int8 and fp8 (fp8_full) forwards, with dynamic and with
  static "fixed,-224,224" calibration of activations and weights (absmax for the gradient, tokamax_test.py:99-101),
  against the oracle on the quantised operands the forward produced."""
  from maxtext_amd import megablox
  from maxtext_amd.quantizations import QtRule

  if fwd == "int8" and calibration != "absmax":
    calibration = "fixed,-4,4"  # a range int8 activations of order one resolve
  m, k, n, gs = shape["m"], shape["k"], shape["n"], np.asarray(shape["gs"], np.int32)
  g = torch.Generator().manual_seed(12)
  lhs = torch.randn(m, k, generator=g).to(torch.bfloat16)
  w = (torch.randn(4, k, n, generator=g) * (0.05 if calibration == "absmax" else 1.0)).to(torch.bfloat16)  # [g, k, n]
  dout = torch.randn(m, n, generator=g).to(torch.bfloat16)
  rule = QtRule(weight_qtype=fwd, act_qtype=fwd, bwd_qtype=bwd_q, weight_calibration_method=calibration, act_calibration_method=calibration)

  lhs_g = cuda(lhs).requires_grad_()
  rhs_g = cuda(w).requires_grad_()
  out = gmm_bf16(lhs_g, rhs_g, cuda(gs), use_qwix_quantization=True, qwix_rule=rule)
  # the operands the forward quantised to, restated on the host and checked bit for bit against the library's quantisers
  qdt = torch.int8 if fwd == "int8" else E4M3
  qmax = 127.0 if fwd == "int8" else 448.0
  dev_l = megablox.quantize_lhs(cuda(lhs), fwd, calibration_method=calibration)
  dev_r = megablox.quantize_rhs(cuda(w.transpose(1, 2).contiguous()), fwd, calibration_method=calibration)  # [g, n, k]
  lq, rq = dev_l.qvalue.cpu(), dev_r.qvalue.cpu().transpose(1, 2)
  if calibration == "absmax":
    ls = lhs.float().abs().amax(1) / qmax
    y = torch.where(ls[:, None] == 0, torch.zeros_like(lhs.float()), lhs.float() / ls[:, None])
    want_lq = torch.round(y).clamp(-qmax, qmax).to(qdt) if fwd == "int8" else y.clamp(-qmax, qmax).to(qdt)
    assert torch.equal(dev_l.scale.cpu(), ls) and torch.equal(lq.float(), want_lq.float())
    rs = w.float().abs().amax(dim=(0, 1)) / qmax  # [n], shared by the experts
    y = torch.where(rs == 0, torch.zeros_like(w.float()), w.float() / rs)
    want_rq = torch.round(y).clamp(-qmax, qmax).to(qdt) if fwd == "int8" else y.clamp(-qmax, qmax).to(qdt)
    assert torch.equal(dev_r.scale.cpu().reshape(-1), rs) and torch.equal(rq.float(), want_rq.float())
  else:
    s = O.get_static_scale(qmax, calibration)
    ls = torch.full((m,), s)
    rs = torch.full((n,), s)
    # the static quantisers: x / scale clipped and cast (rint for int8 activations, nearest even for fp8; weights as
    # manual_quantize does)
    y = (lhs.float() / s).clamp(-qmax, qmax)
    want_lq = torch.round(y).to(qdt) if fwd == "int8" else y.to(qdt)
    assert torch.equal(lq.float(), want_lq.float())
    assert torch.equal(rq.float(), O.manual_quantize(w, qdt, calibration)[0].float())
  want_out = O.gmm(lq.float(), rq.float(), gs, lhs_scale=ls, rhs_scale=rs[None])
  assert relerr(out, want_out) <= TOL
  want_dl, want_dr = O.gmm_bwd_quantized(dout, lq.float(), ls, rq.float(), rs, gs, bwd_qtype=None if bwd_q is None else "e5m2")

  out.backward(cuda(dout))
  tol = TOL if bwd_q is None else 2e-2  # a gradient value next to an e5m2 rounding boundary may land on either side
  total = int(gs.sum())
  assert relerr(lhs_g.grad, want_dl, atol_rms=ELEM_ATOL_RMS_CHAINED) <= tol
  assert torch.all(lhs_g.grad[total:] == 0)
  assert rhs_g.grad.shape == want_dr.shape and relerr(rhs_g.grad, want_dr, atol_rms=ELEM_ATOL_RMS_CHAINED) <= tol
  assert torch.all(rhs_g.grad[1] == 0)


@pytest.mark.parametrize("bwd_q", [None, "float8_e5m2"], ids=["bf16grad", "e5m2grad"])
@pytest.mark.parametrize("fwd", ["int8", "float8_e4m3fn"], ids=["int8", "fp8"])
@pytest.mark.parametrize("shape", [dict(m=450, k=256, n=192, gs=[200, 0, 70, 150]), dict(m=1100, k=512, n=768, gs=[500, 0, 300, 260])],
                         ids=["small", "stream"])
def test_gmm_quantized_backward_per_tensor_scales(shape, fwd, bwd_q):
  """A rule with disable_channelwise_axes (channelwise_axes=[] at ops.py:245, :258, :568, :594, :601): one dynamic absmax
  scale for the activations, one for the weights and one for each of the two scaled gradients.  Forward operands bit for
  bit against the host statement of the rule, output and both gradients against the oracle's quantised backward."""
  from maxtext_amd import megablox
  from maxtext_amd.quantizations import QtRule

  m, k, n, gs = shape["m"], shape["k"], shape["n"], np.asarray(shape["gs"], np.int32)
  g = torch.Generator().manual_seed(13)
  lhs = torch.randn(m, k, generator=g).to(torch.bfloat16)
  w = (torch.randn(4, k, n, generator=g) * 0.05).to(torch.bfloat16)  # [g, k, n]
  dout = torch.randn(m, n, generator=g).to(torch.bfloat16)
  rule = QtRule(weight_qtype=fwd, act_qtype=fwd, bwd_qtype=bwd_q, disable_channelwise_axes=True)
  lhs_g = cuda(lhs).requires_grad_()
  rhs_g = cuda(w).requires_grad_()
  out = gmm_bf16(lhs_g, rhs_g, cuda(gs), use_qwix_quantization=True, qwix_rule=rule)
  qdt = torch.int8 if fwd == "int8" else E4M3
  qmax = 127.0 if fwd == "int8" else 448.0
  ls = lhs.float().abs().max() / qmax
  rs = w.float().abs().max() / qmax
  cast = (lambda y: torch.round(y).clamp(-qmax, qmax).to(qdt)) if fwd == "int8" else (lambda y: y.clamp(-qmax, qmax).to(qdt))
  lq, rq = cast(lhs.float() / ls), cast(w.float() / rs)
  dev_l = megablox.quantize_lhs(cuda(lhs), fwd, per_tensor=True)
  dev_r = megablox.quantize_rhs(cuda(w.transpose(1, 2).contiguous()), fwd, per_tensor=True)
  assert torch.equal(dev_l.scale.cpu().reshape(()), ls) and torch.equal(dev_l.qvalue.cpu().float(), lq.float())
  assert torch.equal(dev_r.scale.cpu().reshape(()), rs) and torch.equal(dev_r.qvalue.cpu().transpose(1, 2).float(), rq.float())
  ls_m, rs_n = ls.expand(m).contiguous(), rs.expand(n).contiguous()
  want_out = O.gmm(lq.float(), rq.float(), gs, lhs_scale=ls_m, rhs_scale=rs_n[None])
  assert relerr(out, want_out) <= TOL
  want_dl, want_dr = O.gmm_bwd_quantized(dout, lq.float(), ls_m, rq.float(), rs_n, gs, bwd_qtype=None if bwd_q is None else "e5m2",
                                         per_tensor=True)
  out.backward(cuda(dout))
  tol = TOL if bwd_q is None else 2e-2  # a gradient value next to an e5m2 rounding boundary may land on either side
  total = int(gs.sum())
  assert relerr(lhs_g.grad, want_dl, atol_rms=ELEM_ATOL_RMS_CHAINED) <= tol
  assert torch.all(lhs_g.grad[total:] == 0)
  assert rhs_g.grad.shape == want_dr.shape and relerr(rhs_g.grad, want_dr, atol_rms=ELEM_ATOL_RMS_CHAINED) <= tol
  assert torch.all(rhs_g.grad[1] == 0)


@pytest.mark.parametrize("calibration", ["absmax", "fixed,-224,224"], ids=["absmax", "static"])
@pytest.mark.parametrize("fwd", ["int8", "float8_e4m3fn"], ids=["int8", "fp8"])
def test_gmm_v2_forward_and_its_quantized_backward(fwd, calibration):
  """use_gmm_v2 on the differentiable path (ops.py:203-215, :241, :561-572, :636, :785): the forward leaves the bf16
  activations to the product, which quantises them by its own rule (per row and 512 values of K, or the static (1, 1)
  scale: the oracle's op-by-op restatement of pallas_mosaic_tpu_v2_gmm_kernel.py:489-542, bit-exact on the GPU in
  test_gpu_layouts); the backward quantises the kept bf16 activations per row by the v1 rule and then runs the
  reference's quantised backward with e5m2 gradients."""
  from maxtext_amd import megablox
  from maxtext_amd.quantizations import QtRule

  if fwd == "int8" and calibration != "absmax":
    calibration = "fixed,-4,4"
  m, k, n, gs = 450, 1024, 192, np.asarray([200, 0, 70, 150], np.int32)
  g = torch.Generator().manual_seed(14)
  lhs = torch.randn(m, k, generator=g).to(torch.bfloat16)
  lhs[:, 512:] *= 0.125  # the two K blocks of a row get different scales
  w = (torch.randn(4, k, n, generator=g) * (0.05 if calibration == "absmax" else 1.0)).to(torch.bfloat16)  # [g, k, n]
  dout = torch.randn(m, n, generator=g).to(torch.bfloat16)
  rule = QtRule(weight_qtype=fwd, act_qtype=fwd, bwd_qtype="float8_e5m2", weight_calibration_method=calibration,
                act_calibration_method=calibration)
  lhs_g = cuda(lhs).requires_grad_()
  rhs_g = cuda(w).requires_grad_()
  out = gmm_bf16(lhs_g, rhs_g, cuda(gs), use_qwix_quantization=True, qwix_rule=rule, use_gmm_v2=True)
  qdt = torch.int8 if fwd == "int8" else E4M3
  qmax = 127.0 if fwd == "int8" else 448.0
  static = None if calibration == "absmax" else O.get_static_scale(qmax, calibration)
  # weights: the library's quantiser (bit for bit against the host rule in the tests above)
  dev_r = megablox.quantize_rhs(cuda(w.transpose(1, 2).contiguous()), fwd, calibration_method=calibration)
  rq = dev_r.qvalue.cpu().transpose(1, 2)
  rs = dev_r.scale.cpu().reshape(-1).expand(n).contiguous() if dev_r.scale.numel() == 1 else dev_r.scale.cpu().reshape(-1)
  # forward: the product's own quantiser
  lq2, ls2 = O.quantize_lhs_v2(lhs, qdt, quant_block=512, static_scale=static)
  want_out = O.gmm(lq2, rq, gs, lhs_scale=ls2, rhs_scale=rs[None], quant_block=(512, k))
  assert relerr(out, want_out) <= TOL
  # backward: the v1 rule on the kept activations
  dev_l = megablox.quantize_lhs(cuda(lhs), fwd, calibration_method=calibration)
  lq = dev_l.qvalue.cpu()
  ls = dev_l.scale.cpu().reshape(-1)
  ls = ls.expand(m).contiguous() if ls.numel() == 1 else ls
  if static is None:
    assert torch.equal(ls, lhs.float().abs().amax(1) / qmax)
    assert not torch.equal(lq.float(), lq2.float())  # (the two rules differ on these rows: the test tells them apart)
  want_dl, want_dr = O.gmm_bwd_quantized(dout, lq.float(), ls, rq.float(), rs, gs, bwd_qtype="e5m2")
  out.backward(cuda(dout))
  total = int(gs.sum())
  assert relerr(lhs_g.grad, want_dl, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2
  assert torch.all(lhs_g.grad[total:] == 0)
  assert rhs_g.grad.shape == want_dr.shape and relerr(rhs_g.grad, want_dr, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2
  assert torch.all(rhs_g.grad[1] == 0)


def test_fp8_full_layer_gradients_tokamax_configuration():
  """The configuration of the reference's fp8_full training smoke test (tests/integration/tokamax_test.py:53-114:
  emb 256, moe_mlp 256, 2 experts + 1 shared, weights and activations "fixed,-224,224", gradients absmax e5m2): one
  expert MLP step gmm -> gmm -> SwiGLU -> gmm through megablox.gmm with the qwix rule, forward and all gradients
  against the oracle's quantised backward chained by hand."""
  from maxtext_amd import megablox
  from maxtext_amd.quantizations import QtRule

  cal = "fixed,-224,224"
  rule = QtRule(weight_qtype="float8_e4m3fn", act_qtype="float8_e4m3fn", bwd_qtype="float8_e5m2", weight_calibration_method=cal,
                act_calibration_method=cal, bwd_calibration_method="absmax")
  # (1024 rows: with the smoke test's 128 a single gradient value that falls on the other side of an e5m2 rounding
  # boundary, a 25 % step, moves a weight-gradient sum of 64 terms by 3 % of its rms)
  t, d, f, e = 1024, 256, 256, 2
  g = torch.Generator().manual_seed(3)
  gs = np.asarray([600, 424], np.int32)
  x = torch.randn(t, d, generator=g).to(torch.bfloat16)
  w0 = (torch.randn(e, d, f, generator=g) * 0.06).to(torch.bfloat16)
  w1 = (torch.randn(e, d, f, generator=g) * 0.06).to(torch.bfloat16)
  wo = (torch.randn(e, f, d, generator=g) * 0.06).to(torch.bfloat16)
  dy = torch.randn(t, d, generator=g).to(torch.bfloat16)
  xs, p0, p1, po = [cuda(v).requires_grad_() for v in (x, w0, w1, wo)]
  kw = dict(use_qwix_quantization=True, qwix_rule=rule)
  # the fused call's own composition, spelled out so that every stage's gradient can be read back
  g0 = gmm_bf16(xs, p0, cuda(gs), **kw)
  g1 = gmm_bf16(xs, p1, cuda(gs), **kw)
  h = megablox._GluFn.apply(g0, g1, "silu", 7.0)
  for v in (g0, g1, h):
    v.retain_grad()
  y = gmm_bf16(h, po, cuda(gs), **kw)
  y.backward(cuda(dy))
  fused = gmm_bf16(xs.detach().requires_grad_(), p0, cuda(gs), rhs_up=p1, fuse_act="silu", **kw)
  assert torch.equal(fused, h)

  # oracle: each stage on the operands the stage before it produced on the GPU (a bf16 rounding that differs between the
  # two sides would otherwise be quantised to fp8 / e5m2 on both and compared as a whole grid step, or move a column's
  # absmax scale)
  s = 0.5
  host = lambda v: v.detach().cpu()
  q = lambda v: (v.float() / s).clamp(-448, 448).to(E4M3).float()
  half_d, half_f, half_t = torch.full((d,), s), torch.full((f,), s), torch.full((t,), s)
  xq, q0, q1 = q(x), O.manual_quantize(w0, E4M3, cal)[0].float(), O.manual_quantize(w1, E4M3, cal)[0].float()
  assert relerr(g0, O.gmm(xq, q0, gs, lhs_scale=half_t, rhs_scale=half_f[None])) <= TOL
  assert relerr(g1, O.gmm(xq, q1, gs, lhs_scale=half_t, rhs_scale=half_f[None])) <= TOL
  assert relerr(h, O.apply_ffn_activation(host(g0), host(g1), "silu")) <= TOL
  hq, qo = q(host(h)), O.manual_quantize(wo, E4M3, cal)[0].float()
  assert relerr(y, O.gmm(hq, qo, gs, lhs_scale=half_t, rhs_scale=half_d[None]), atol_rms=ELEM_ATOL_RMS_CHAINED) <= TOL
  dh, dwo = O.gmm_bwd_quantized(dy, hq, half_t, qo, half_d, gs, bwd_qtype="e5m2")
  assert relerr(po.grad, dwo, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2
  assert relerr(h.grad, dh, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2
  # SwiGLU backward in f64
  a, b = host(g0).double().requires_grad_(), host(g1).double().requires_grad_()
  (torch.nn.functional.silu(a) * b).backward(host(h.grad).double())
  assert relerr(g0.grad, a.grad) <= TOL and relerr(g1.grad, b.grad) <= TOL
  dx0, dw0 = O.gmm_bwd_quantized(host(g0.grad), xq, half_t, q0, half_f, gs, bwd_qtype="e5m2")
  dx1, dw1 = O.gmm_bwd_quantized(host(g1.grad), xq, half_t, q1, half_f, gs, bwd_qtype="e5m2")
  assert relerr(p0.grad, dw0, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2
  assert relerr(p1.grad, dw1, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2
  assert relerr(xs.grad, dx0 + dx1, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2
