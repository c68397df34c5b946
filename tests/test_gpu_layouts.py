"""GPU parity of moe_gmm on the operand layouts the reference's own gmm produces and gmm_v2 consumes:

  * int8 and fp8 activations with one scale per row ([m, 1], ops.py:241-248) or one static scale for the tensor
    ((1, 1), ops.py:333-360), weights with one scale per output channel, per expert or shared by the experts
    ([1, 1, n], ops.py:250-260), or one scale for the tensor (manual_quantize, layers/quantizations.py:961-991);
  * gmm_v2's block scales: activations [m, K / 512] from the in-kernel quantiser
    (pallas_mosaic_tpu_v2_gmm_kernel.py:533-542), weights [g, nb, 1, n] (ops.py:310-331);
  * weight-only int8 / int4 with [g, nb, 1, n] scales;
  * f32 outputs (preferred_element_type, ops.py:50);
  * activation rows read through an index (permute fused into the matmul, kernels/ragged/ragged_gather.py:310-320)
    and a factor per result row (models/deepseek_batchsplit_fp8.py:1049),
each against oracle.gmm on the identical quantised operands.
"""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tolerances import ELEM_ATOL_RMS_CHAINED, TOL, relerr

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
  from maxtext_amd import kernels

  assert torch.cuda.is_available()
  return kernels


def cuda(x):
  if isinstance(x, np.ndarray):
    x = torch.from_numpy(x)
  return x.cuda().contiguous()


def native(w_gkn):
  return w_gkn.transpose(1, 2).contiguous()


def _q_operands(qdtype, m, k, n, g, seed):
  """Random already-quantised operands: lhs [m, k], rhs [g, k, n] of qdtype, and bf16 activations for the quantisers."""
  gen = torch.Generator().manual_seed(seed)
  x = torch.randn(m, k, generator=gen).to(torch.bfloat16)
  if qdtype == torch.int8:
    lq = torch.randint(-127, 128, (m, k), generator=gen).to(torch.int8)
    rq = torch.randint(-127, 128, (g, k, n), generator=gen).to(torch.int8)
  else:
    lq = (torch.randn(m, k, generator=gen) * 40).clamp(-448, 448).to(torch.float8_e4m3fn)
    rq = (torch.randn(g, k, n, generator=gen) * 40).clamp(-448, 448).to(torch.float8_e4m3fn)
  return x, lq, rq, gen


# (m, k, n, group_sizes): decode-sized, ragged mid-sized, prefill-sized (256 x 256 tiles), rows in no group at the end
LAYOUT_SHAPES = [
    (40, 256, 128, [3, 0, 17, 9, 1, 10]),
    (700, 384, 200, [130, 300, 0, 150, 100]),
    (4200, 512, 512, [1500, 0, 1400, 1196]),
]


@pytest.mark.parametrize("qdtype", [torch.int8, torch.float8_e4m3fn])
@pytest.mark.parametrize("m,k,n,gs", LAYOUT_SHAPES)
def test_gmm_row_and_channel_scale_layouts(K, qdtype, m, k, n, gs):
  """What _fwd_quantize_activation_and_weight hands the kernel (ops.py:232-267): lhs scale [m, 1] or per tensor, rhs
  scale per channel per expert, [1, 1, n] shared by the experts, or per tensor."""
  g = len(gs)
  gs = np.array(gs, np.int32)
  _, lq, rq, gen = _q_operands(qdtype, m, k, n, g, m + n)
  ls_row = torch.rand(m, generator=gen) * 0.02 + 0.005
  ls_one = torch.tensor([0.0123])
  rs_gn = torch.rand(g, n, generator=gen) * 0.01 + 0.002
  rs_n = rs_gn[:1].clone()
  rs_one = torch.tensor([0.0077])
  ru = torch.roll(rq, 1, dims=0)  # a second projection for the fused variant
  for ls, lbk in ((ls_row, 0), (ls_one, -1)):
    o_ls = ls[:, None] if lbk == 0 else ls.reshape(1, 1)
    for rs, bn, shared in ((rs_gn, 1, False), (rs_n, 1, True), (rs_one, -1, True)):
      o_rs = rs if bn == 1 else rs.reshape(1, 1).expand(1, n)
      kw = dict(lhs_scale=cuda(ls), lhs_scale_block_k=lbk, rhs_scale=cuda(rs), rhs_scale_block_n=bn, rhs_scale_shared=shared)
      got = K.gmm_raw(cuda(lq), cuda(native(rq)), cuda(gs), **kw)
      want = O.gmm(lq, rq, gs, lhs_scale=o_ls, rhs_scale=o_rs[:, None, None, :], out_dtype=torch.float32)
      assert relerr(got, want) <= TOL, (lbk, bn, shared)
      assert torch.all(got[int(gs.sum()):] == 0)
    # fused second projection + activation, per-channel scales
    got = K.gmm_raw(cuda(lq), cuda(native(rq)), cuda(gs), lhs_scale=cuda(ls), lhs_scale_block_k=lbk, rhs_scale=cuda(rs_gn),
                    rhs_up=cuda(native(ru)), rhs_up_scale=cuda(rs_gn), act="silu")
    h0 = O.gmm(lq, rq, gs, lhs_scale=o_ls, rhs_scale=rs_gn, out_dtype=torch.float32)
    h1 = O.gmm(lq, ru, gs, lhs_scale=o_ls, rhs_scale=rs_gn, out_dtype=torch.float32)
    # scale the pre-activations down so that silu is not saturated everywhere
    assert relerr(got, O.apply_ffn_activation(h0, h1, out_dtype=torch.float32)) <= TOL


@pytest.mark.parametrize("qdtype", [torch.int8, torch.float8_e4m3fn])
@pytest.mark.parametrize("m,k,n,gs,lhs_qb,rhs_qb", [
    (300, 1024, 256, [100, 0, 200], 512, 256),
    (300, 1024, 256, [100, 0, 200], 512, 1024),   # per-channel weights over all of K, block-scaled activations
    (900, 1536, 200, [130, 300, 0, 270, 150], 512, 128),
    (64, 512, 128, [3, 40, 0, 21], 128, 512),
    (2100, 512, 512, [700, 0, 800, 600], 0, 256),  # per-row activations, block-scaled weights
    (2100, 512, 512, [700, 0, 800, 600], -1, 128),  # static activation scale, block-scaled weights
])
def test_gmm_v2_block_scale_layouts(K, qdtype, m, k, n, gs, lhs_qb, rhs_qb):
  """gmm_v2's layouts: lhs scales [m, K / lhs_qb] from its in-kernel quantiser, rhs scales [g, K / rhs_qb, 1, n]."""
  g = len(gs)
  gs = np.array(gs, np.int32)
  x, lq, rq, gen = _q_operands(qdtype, m, k, n, g, m + k)
  if lhs_qb > 0:
    lq, ls = O.quantize_lhs_v2(x, qdtype, quant_block=lhs_qb)  # the reference's own quantiser
    kq, ks = K.gather_rows(cuda(x), out_dtype=qdtype, block_k=lhs_qb, rule="v2")
    assert torch.equal(kq.cpu().view(torch.uint8), lq.view(torch.uint8)) and torch.equal(ks.cpu(), ls)
    lbk, o_ls = lhs_qb, ls
  elif lhs_qb == 0:
    ls = torch.rand(m, generator=gen) * 0.02 + 0.005
    lbk, o_ls = 0, ls[:, None]
  else:
    ls = torch.tensor([0.0123])
    lbk, o_ls = -1, ls.reshape(1, 1)
  nb = k // rhs_qb
  rs = torch.rand(g, nb, 1, n, generator=gen) * 0.01 + 0.002
  kw = dict(lhs_scale=cuda(ls), lhs_scale_block_k=lbk, rhs_scale_block_k=0 if nb == 1 else rhs_qb, rhs_scale_kmajor=nb > 1)
  got = K.gmm_raw(cuda(lq), cuda(native(rq)), cuda(gs), rhs_scale=cuda(rs), **kw)
  want = O.gmm(lq, rq, gs, lhs_scale=o_ls, rhs_scale=rs, quant_block=(lhs_qb if lhs_qb > 0 else k, rhs_qb), out_dtype=torch.float32)
  assert relerr(got, want) <= TOL
  assert torch.all(got[int(gs.sum()):] == 0)
  # a shard of the experts, fused projections with biases, f32 output
  ru = torch.roll(rq, 1, dims=0)
  rsu = torch.roll(rs, 1, dims=0)
  b0 = torch.randn(g, n, generator=gen)
  b1 = torch.randn(g, n, generator=gen)
  got = K.gmm_raw(cuda(lq), cuda(native(rq[1:])), cuda(gs), rhs_scale=cuda(rs[1:]), rhs_up=cuda(native(ru[1:])), rhs_up_scale=cuda(rsu[1:]),
                  rhs_bias=cuda(b0[1:]), rhs_up_bias=cuda(b1[1:]), act="silu", group_offset=1, out_dtype=torch.float32, **kw)
  okw = dict(lhs_scale=o_ls, quant_block=(lhs_qb if lhs_qb > 0 else k, rhs_qb), out_dtype=torch.float32, group_offset=1)
  h0 = O.gmm(lq, rq[1:], gs, rhs_scale=rs[1:], rhs_bias=b0[1:, None, :], **okw)
  h1 = O.gmm(lq, ru[1:], gs, rhs_scale=rsu[1:], rhs_bias=b1[1:, None, :], **okw)
  assert got.dtype == torch.float32
  assert relerr(got, O.apply_ffn_activation(h0, h1, out_dtype=torch.float32)) <= TOL
  assert torch.all(got[: gs[0]] == 0)


@pytest.mark.parametrize("m,k,n,gs,qb", [(300, 512, 256, [100, 0, 200], 128), (40, 256, 128, [3, 0, 17, 20], 64), (1100, 1024, 512, [500, 600], 256)])
def test_gmm_weight_only_kmajor_scales(K, m, k, n, gs, qb):
  """Unquantised activations with gmm_v2's weight scales [g, nb, 1, n] (v2 kernel :448-454, :482-484): int8 and int4 weights."""
  g = len(gs)
  gs = np.array(gs, np.int32)
  gen = torch.Generator().manual_seed(k + qb)
  lhs = torch.randn(m, k, generator=gen).to(torch.bfloat16)
  nb = k // qb
  rs = torch.rand(g, nb, 1, n, generator=gen) * 0.01 + 0.002
  r8 = torch.randint(-127, 128, (g, k, n), generator=gen).to(torch.int8)
  got = K.gmm_raw(cuda(lhs), cuda(native(r8)), cuda(gs), rhs_scale=cuda(rs), rhs_scale_block_k=qb, rhs_scale_kmajor=True)
  want = O.gmm(lhs, r8, gs, rhs_scale=rs, quant_block=qb, out_dtype=torch.float32)
  assert relerr(got, want) <= TOL
  if qb % 32 == 0:
    r4 = torch.randint(-8, 8, (g, k, n), generator=gen).to(torch.int8)
    packed = O.pack_int4(native(r4))  # [g, n, k/2]
    from maxtext_amd._lib import MOE_INT4

    got = K.gmm_raw(cuda(lhs), cuda(packed), cuda(gs), rhs_scale=cuda(rs), rhs_dtype=MOE_INT4, rhs_scale_block_k=qb, rhs_scale_kmajor=True)
    want = O.gmm(lhs, r4, gs, rhs_scale=rs, quant_block=qb, out_dtype=torch.float32)
    assert relerr(got, want) <= TOL
  # per-tensor and shared per-channel scales on the per-channel path (streaming and tiled kernels)
  for kern in (None, "tiled"):
    got = K.gmm_raw(cuda(lhs), cuda(native(r8)), cuda(gs), rhs_scale=cuda(rs[0, 0, 0]), rhs_scale_shared=True, kernel=kern)
    assert relerr(got, O.gmm(lhs, r8, gs, rhs_scale=rs[:1, :1], out_dtype=torch.float32)) <= TOL
    got = K.gmm_raw(cuda(lhs), cuda(native(r8)), cuda(gs), rhs_scale=cuda(rs[0, 0, 0, :1]), rhs_scale_block_n=-1, rhs_scale_shared=True, kernel=kern)
    assert relerr(got, O.gmm(lhs, r8, gs, out_dtype=torch.float32).float() * float(rs[0, 0, 0, 0])) <= TOL


def _families():
  """(name, builder) pairs: one small problem per kernel family, each returning (gmm_raw kwargs, oracle callable)."""
  gen = torch.Generator().manual_seed(99)
  out = []

  def bf16(m, k, n, gs, kernel=None):
    lhs = torch.randn(m, k, generator=gen).to(torch.bfloat16)
    w = (torch.randn(len(gs), k, n, generator=gen) * 0.05).to(torch.bfloat16)
    return dict(lhs=lhs, rhs=native(w), kw=dict(kernel=kernel)), lambda l, **o: O.gmm(l, w, np.array(gs, np.int32), out_dtype=torch.float32, **o)

  def w8(m, k, n, gs, kernel=None):
    lhs = torch.randn(m, k, generator=gen).to(torch.bfloat16)
    q = torch.randint(-127, 128, (len(gs), k, n), generator=gen).to(torch.int8)
    s = torch.rand(len(gs), n, generator=gen) * 0.01 + 0.002
    return (dict(lhs=lhs, rhs=native(q), kw=dict(rhs_scale=s, kernel=kernel)),
            lambda l, **o: O.gmm(l, q, np.array(gs, np.int32), rhs_scale=s, out_dtype=torch.float32, **o))

  def i8(m, k, n, gs, kernel=None):
    lq = torch.randint(-127, 128, (m, k), generator=gen).to(torch.int8)
    ls = torch.rand(m, generator=gen) * 0.02 + 0.005
    q = torch.randint(-127, 128, (len(gs), k, n), generator=gen).to(torch.int8)
    s = torch.rand(len(gs), n, generator=gen) * 0.01 + 0.002
    return (dict(lhs=lq, lhs_scale=ls, rhs=native(q), kw=dict(rhs_scale=s, kernel=kernel)),
            lambda l, ls_, **o: O.gmm(l, q, np.array(gs, np.int32), lhs_scale=ls_[:, None], rhs_scale=s, out_dtype=torch.float32, **o))

  def f8(m, k, n, gs, kernel=None):
    x = torch.randn(m, k, generator=gen)
    w = torch.randn(len(gs), k, n, generator=gen) * 0.05
    aq, asc = O.quantize_fp8_blocks(x, 1, 128)
    wq, wsc = O.quantize_fp8_blocks(native(w), 128, 128)
    v2 = torch.repeat_interleave(wsc.permute(0, 2, 1), 128, dim=2)[:, :, None, :n]
    return (dict(lhs=aq, lhs_scale=asc, rhs=wq, kw=dict(rhs_scale=wsc, lhs_scale_block_k=128, rhs_scale_block_n=128, rhs_scale_block_k=128, kernel=kernel)),
            lambda l, ls_, **o: O.gmm(l, wq, np.array(gs, np.int32), lhs_scale=ls_, rhs_scale=v2, transpose_rhs=True, quant_block=128,
                                      out_dtype=torch.float32, **o))

  big = [700, 0, 800, 600]
  out.append(("bf16 tiled 64", bf16(90, 256, 128, [30, 0, 45, 15]), [30, 0, 45, 15]))
  out.append(("bf16 direct-to-LDS", bf16(2100, 512, 512, big), big))
  out.append(("bf16 direct-to-LDS 64-byte stages", bf16(2100, 512, 512, big, "dl64"), big))
  out.append(("int8 weights streaming", w8(40, 256, 128, [3, 0, 17, 20]), [3, 0, 17, 20]))
  out.append(("int8 weights tiled 128", w8(300, 256, 256, [100, 0, 200]), [100, 0, 200]))
  out.append(("int8 weights tiled 256", w8(2100, 512, 512, big), big))
  out.append(("int8 x int8 tiled 64", i8(90, 256, 128, [30, 0, 45, 15]), [30, 0, 45, 15]))
  out.append(("int8 x int8 direct-to-LDS", i8(2100, 512, 512, big), big))
  out.append(("fp8 blocks streaming", f8(40, 256, 128, [3, 0, 17, 20]), [3, 0, 17, 20]))
  out.append(("fp8 blocks streaming 64-row", f8(300, 256, 256, [100, 0, 200], "stream"), [100, 0, 200]))
  out.append(("fp8 blocks tiled", f8(300, 256, 256, [100, 0, 200]), [100, 0, 200]))
  out.append(("fp8 blocks 256 x 256", f8(2100, 512, 512, big, "big"), big))
  return out


@pytest.mark.parametrize("case", _families(), ids=lambda c: c[0])
def test_gmm_row_index_row_scale_and_f32_out_in_every_kernel_family(K, case):
  """The row index, the per-row factor and the f32 output are honoured by every kernel family, bit for bit equal to
  the same launch on explicitly gathered rows where that is expected (same operands, same order of accumulation)."""
  _, (args, oracle), gs = case
  gs = np.array(gs, np.int32)
  lhs, kw = args["lhs"], {k_: (cuda(v) if isinstance(v, torch.Tensor) else v) for k_, v in args["kw"].items()}
  ls = args.get("lhs_scale")
  m = lhs.shape[0]
  t, k = (m + 1) // 2, 2
  gen = torch.Generator().manual_seed(m)
  src = torch.randint(0, t * k, (m,), generator=gen).to(torch.int32)  # row i reads token src[i] // k
  tok = (src // k).long()
  rowf = torch.rand(m, generator=gen) + 0.5
  base_kw = dict(kw)
  if ls is not None:
    base_kw["lhs_scale"] = cuda(ls)
  plain = K.gmm_raw(cuda(lhs), cuda(args["rhs"]), cuda(gs), **base_kw)
  want = oracle(lhs) if ls is None else oracle(lhs, ls)
  assert relerr(plain, want) <= TOL
  f32 = K.gmm_raw(cuda(lhs), cuda(args["rhs"]), cuda(gs), out_dtype=torch.float32, **base_kw)
  assert f32.dtype == torch.float32 and torch.equal(f32.to(torch.bfloat16), plain)  # the same sums, rounded later
  assert relerr(f32, want) <= 2e-3
  # gathered explicitly against gathered inside the kernel: identical bits
  lhs_t = lhs[:t]
  idx_kw = dict(kw)
  gat_kw = dict(kw)
  if ls is not None:
    idx_kw["lhs_scale"] = cuda(ls[:t])
    gat_kw["lhs_scale"] = cuda(ls[:t][tok])
  via_idx = K.gmm_raw(cuda(lhs_t), cuda(args["rhs"]), cuda(gs), lhs_row_idx=cuda(src), lhs_row_idx_div=k, **idx_kw)
  gathered = K.gmm_raw(cuda(lhs_t[tok]), cuda(args["rhs"]), cuda(gs), **gat_kw)
  assert torch.equal(via_idx, gathered)
  want_g = oracle(lhs_t[tok]) if ls is None else oracle(lhs_t[tok], ls[:t][tok])
  assert relerr(via_idx, want_g) <= TOL
  scaled = K.gmm_raw(cuda(lhs_t), cuda(args["rhs"]), cuda(gs), lhs_row_idx=cuda(src), lhs_row_idx_div=k, out_row_scale=cuda(rowf), **idx_kw)
  assert relerr(scaled, want_g.float() * rowf[:, None]) <= TOL
  assert torch.all(scaled[int(gs.sum()):] == 0)
  # the factor multiplies the finished bf16 result (deepseek_batchsplit_fp8.py:1048-1049): two roundings, bit for bit
  assert torch.equal(scaled, (via_idx.float() * cuda(rowf)[:, None]).to(torch.bfloat16))
  scaled32 = K.gmm_raw(cuda(lhs_t), cuda(args["rhs"]), cuda(gs), lhs_row_idx=cuda(src), lhs_row_idx_div=k, out_row_scale=cuda(rowf),
                       out_dtype=torch.float32, **idx_kw)
  assert relerr(scaled32, want_g.float() * rowf[:, None]) <= 2e-3


@pytest.mark.parametrize("fmt", ["int8", "int4", "int4g32", "mxfp4"])
@pytest.mark.parametrize("glu", [False, True])
@pytest.mark.parametrize("regime", ["prefill", "mid"])
def test_weight_only_prefill_kernel_against_the_tiled_kernel_at_size(K, fmt, glu, regime):
  """The persistent weight-only kernel (raw weights through LDS, widened per wave, one request stream across tiles) on
  a shape with hundreds of tiles per block, ragged groups, a ragged last n-tile and an empty group, against the
  register-staged tiled kernel on the same operands (which the small-shape tests pin to the oracle), plus sampled rows
  against the oracle's dequantised matmul."""
  from maxtext_amd._lib import MOE_INT4, MOE_MXFP4

  g = torch.Generator(device="cuda").manual_seed(17)
  e, k, n = 16, 1088, 1984  # 17 stages of 64; 15.5 n-tiles of 128
  gs_h = np.array([700, 1031, 0, 512, 256, 1300, 90, 777, 640, 515, 513, 511, 1024, 300, 999, 1100], np.int32)
  if regime == "mid":  # 60 rows per expert on average: int8 / int4 run the same kernel on 128-row tiles (half of the row tiles multiplied)
    gs_h = np.array([70, 103, 0, 51, 25, 130, 9, 77, 64, 129, 128, 127, 1, 30, 99, 17], np.int32)
  m = int(gs_h.sum()) + 100  # 100 rows in no group
  gs = torch.from_numpy(gs_h).cuda()
  lhs = torch.randn(m, k, device="cuda", generator=g).to(torch.bfloat16)
  kw, ws = {}, []
  for _ in range(2 if glu else 1):
    if fmt == "int8":
      ws.append((torch.randint(-127, 128, (e, n, k), device="cuda", dtype=torch.int8, generator=g), torch.rand(e, n, device="cuda", generator=g) * 0.01 + 1e-3))
    elif fmt in ("int4", "int4g32"):
      grp = 128 if fmt == "int4" else 32
      ws.append((torch.randint(0, 256, (e, n, k // 2), device="cuda", dtype=torch.uint8, generator=g),
                 (torch.rand(e, n, (k + grp - 1) // grp, device="cuda", generator=g) * 0.01 + 1e-3).to(torch.bfloat16)))
      kw.update(rhs_dtype=MOE_INT4, rhs_scale_block_k=grp)
    else:
      ws.append((torch.randint(0, 256, (e, n, k // 2), device="cuda", dtype=torch.uint8, generator=g),
                 torch.randint(118, 126, (e, n, k // 32), device="cuda", dtype=torch.uint8, generator=g)))
      kw.update(rhs_dtype=MOE_MXFP4, rhs_scale_block_k=32)
  kw["rhs_scale"] = ws[0][1]
  if glu:
    kw.update(rhs_up=ws[1][0], rhs_up_scale=ws[1][1], act="silu")
  got = K.gmm_raw(lhs, ws[0][0], gs, **kw)
  ref = K.gmm_raw(lhs, ws[0][0], gs, kernel="tiled", **kw)
  # (group-128 int4 and MXFP4: the short last tiles of the groups run on the decode kernel, which sums over K in another
  # order and, for int4, keeps nibble * scale in f32 where the other two multiply weights rounded to bf16: up to one bf16
  # step of the result apart)
  # (for int4 the two arithmetic routes are compared in the max norm only: behind SwiGLU an element of small magnitude may
  # differ by a few per cent of the tensor's rms between them; the rows sampled below are held to the oracle elementwise)
  assert relerr(got, ref, elementwise=fmt != "int4") <= (8e-3 if fmt in ("int4", "mxfp4") else 1e-3)
  assert torch.all(got[int(gs_h.sum()):] == 0)
  # a few rows of three groups against the oracle (first / last row of a group, a row next to the empty group)
  off = np.concatenate([[0], np.cumsum(gs_h)])

  def deq(w, sc):
    w, sc = w.cpu(), sc.cpu()
    if fmt == "int8":
      return w.float() * sc[:, None]
    if fmt in ("int4", "int4g32"):
      return O.dequantize_int4(w, sc, 128 if fmt == "int4" else 32).float()
    return O.dequantize_mxfp4(w.reshape(n, k // 32, 16), sc).float()

  for gi in (0, 3, 15):
    rows = [int(off[gi]), int(off[gi + 1]) - 1]
    x = lhs[rows].cpu().double()
    h0 = x @ deq(ws[0][0][gi], ws[0][1][gi]).double().T
    want = torch.nn.functional.silu(h0) * (x @ deq(ws[1][0][gi], ws[1][1][gi]).double().T) if glu else h0
    assert relerr(got[rows], want, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2


@pytest.mark.parametrize("glu", [False, True])
@pytest.mark.parametrize("indexed", [False, True])
def test_fp8_prefill_stream_kernel_against_the_tiled_kernel_at_size(K, glu, indexed):
  """The persistent block-scaled fp8 kernel (256 x 256 tiles, scales staged through LDS four stages at a time, one
  request stream across tiles) on a shape with many tiles per block, ragged and empty groups, a ragged last n-tile and
  rows in no group, against the 128 x 128 kernel on the same operands (pinned to the oracle by the small-shape tests):
  both add scale * partial sum per 128-wide block in the same order, so the results agree bit for bit.  Sampled rows
  are checked against a float64 restatement of the block-scaled product."""
  g = torch.Generator(device="cuda").manual_seed(23)
  e, k, n = 12, 1536, 1664  # 12 stages (3 scale groups of 4); 6.5 n-tiles of 256
  gs_h = np.array([700, 1031, 0, 512, 256, 1300, 90, 777, 640, 515, 513, 260], np.int32)
  m = int(gs_h.sum()) + 60
  gs = torch.from_numpy(gs_h).cuda()
  lhs = (torch.randn(m, k, device="cuda", generator=g) * 2).to(torch.float8_e4m3fn)
  asc = torch.rand(m, k // 128, device="cuda", generator=g) * 0.02 + 1e-3
  ws = [((torch.randn(e, n, k, device="cuda", generator=g) * 2).to(torch.float8_e4m3fn),
         torch.rand(e, n // 128, k // 128, device="cuda", generator=g) * 0.02 + 1e-3) for _ in range(2)]
  kw = dict(lhs_scale=asc, rhs_scale=ws[0][1], lhs_scale_block_k=128, rhs_scale_block_n=128, rhs_scale_block_k=128)
  if glu:
    kw.update(rhs_up=ws[1][0], rhs_up_scale=ws[1][1], act="silu")
  src = torch.arange(m, device="cuda", dtype=torch.int32)
  if indexed:  # every activation row is read through an index, from half as many rows
    src = torch.randperm(m, device="cuda", generator=g).to(torch.int32)
    lhs, asc = lhs[: (m + 1) // 2].contiguous(), asc[: (m + 1) // 2].contiguous()
    kw.update(lhs_scale=asc, lhs_row_idx=src, lhs_row_idx_div=2, num_rows=m)
  got = K.gmm_raw(lhs, ws[0][0], gs, kernel="big", **kw)
  ref = K.gmm_raw(lhs, ws[0][0], gs, kernel="tiled", **kw)
  assert torch.equal(got, ref)
  assert torch.all(got[int(gs_h.sum()):] == 0)
  off = np.concatenate([[0], np.cumsum(gs_h)])

  def product(rows, w, sc):  # sum over the blocks of (a_scale * w_scale) * (a_block @ w_block^T)
    idx = (src[rows] // 2).long() if indexed else torch.tensor(rows)
    a = lhs[idx].cpu().double().reshape(len(rows), k // 128, 128) * asc[idx].cpu().double()[:, :, None]
    wd = w.cpu().double().reshape(n, k // 128, 128) * torch.repeat_interleave(sc.cpu().double(), 128, dim=0)[:, :, None]
    return torch.einsum("rbk,nbk->rn", a, wd)

  for gi in (0, 5, 11):
    rows = [int(off[gi]), int(off[gi + 1]) - 1]
    h0 = product(rows, ws[0][0][gi], ws[0][1][gi])
    want = torch.nn.functional.silu(h0) * product(rows, ws[1][0][gi], ws[1][1][gi]) if glu else h0
    assert relerr(got[rows], want, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2


def test_same_groups_flag_reuses_or_rebuilds_the_tile_list():
  # MOE_GMM_SAME_GROUPS: the second product of a layer runs on the first one's tile list when the tile height agrees and
  # rebuilds it when it does not; either way the result equals that of a call with a workspace of its own, bit for bit
  from maxtext_amd import kernels as K

  g = torch.Generator(device="cuda").manual_seed(21)
  e, d, f = 16, 256, 512
  w_up = (torch.randn((e, f, d), generator=g, device="cuda") * 0.05).to(torch.bfloat16)
  w_gate = (torch.randn((e, f, d), generator=g, device="cuda") * 0.05).to(torch.bfloat16)
  w_down = (torch.randn((e, d, f), generator=g, device="cuda") * 0.05).to(torch.bfloat16)
  w_down_q = torch.randint(-127, 128, (e, d, f), generator=g, device="cuda", dtype=torch.int8)
  w_down_s = torch.rand((e, d), generator=g, device="cuda") * 0.01
  for m, sizes in ((40, [7, 0, 12, 1, 20] + [0] * 11), (4096, [256] * 16), (1500, [100, 0, 300, 37, 63] + [100] * 10)):
    gs = torch.tensor(sizes, dtype=torch.int32, device="cuda")
    x = torch.randn((m, d), generator=g, device="cuda").to(torch.bfloat16)
    ws = K.gmm_workspace(m, e, "cuda")
    h = K.gmm_raw(x, w_gate, gs, rhs_up=w_up, act="silu", workspace=ws)
    # same tile height (bf16 x bf16 twice)
    y = K.gmm_raw(h, w_down, gs, workspace=ws, same_groups=True)
    assert torch.equal(y, K.gmm_raw(h, w_down, gs))
    # the weight-only format may take another tile height (streaming kernel below 16 rows per expert): list rebuilt
    yq = K.gmm_raw(h, w_down_q, gs, rhs_scale=w_down_s, workspace=ws, same_groups=True)
    assert torch.equal(yq, K.gmm_raw(h, w_down_q, gs, rhs_scale=w_down_s))
    # and back, still promising the same groups
    y2 = K.gmm_raw(h, w_down, gs, workspace=ws, same_groups=True)
    assert torch.equal(y2, y)
    # new group sizes in the same tensor: a call without the flag maps them, the flagged call behind it may reuse that
    gs.copy_(torch.tensor(list(reversed(sizes)), dtype=torch.int32))
    h2 = K.gmm_raw(x, w_gate, gs, rhs_up=w_up, act="silu", workspace=ws)
    y3 = K.gmm_raw(h2, w_down, gs, workspace=ws, same_groups=True)
    assert torch.equal(h2, K.gmm_raw(x, w_gate, gs, rhs_up=w_up, act="silu"))
    assert torch.equal(y3, K.gmm_raw(h2, w_down, gs))


@pytest.mark.parametrize("family", ["bf16", "int8w", "int4", "int4g32", "mxfp4", "int8", "fp8"])
def test_picked_kernel_against_the_tiled_kernel_on_random_large_shapes(K, family):
  """12 random shapes per operand family at sizes where the library picks among all of its kernels (2 to 48 groups, 20
  to 300 rows per group on average, uniform or Zipf-skewed with an empty group, rows in no group, K and N at the
  direct-to-LDS kernels' granularity and off it, with and without the fused activation, rows read through an index, a
  factor per result row, a window of the groups) against the register-staged tiled kernel on the same operands (which
  the small-shape tests pin to the oracle).  The kernels add in the same order and agree bit for bit, except the
  streaming kernel of the 4-bit formats, which sums per scale group first: there one bf16 step of the largest value."""
  from maxtext_amd._lib import MOE_INT4, MOE_MXFP4

  rng = np.random.default_rng(900 + sum(map(ord, family)))
  g = torch.Generator(device="cuda").manual_seed(5)
  rand = lambda *shape: torch.rand(*shape, device="cuda", generator=g)
  randn = lambda *shape: torch.randn(*shape, device="cuda", generator=g)
  bytes_ = lambda lo, hi, shape, dt: torch.randint(lo, hi, shape, device="cuda", dtype=dt, generator=g)
  for case in range(12):
    e = int(rng.integers(2, 49))
    k = int(rng.integers(2, 20)) * 128 if family == "fp8" else int(rng.integers(4, 40)) * 64
    n = int(rng.integers(2, 22)) * 128 if family == "fp8" else int(rng.integers(32, 360)) * 8
    avg = int(rng.choice([20, 40, 60, 100, 120, 140, 300]))
    if rng.random() < 0.4:
      p = 1.0 / np.arange(1, e + 1) ** 1.2
      gs = rng.multinomial(avg * e, p / p.sum())
      rng.shuffle(gs)
    else:
      gs = rng.integers(0, 2 * avg + 1, e)
    if e > 2:
      gs[rng.integers(0, e)] = 0
    m = max(int(gs.sum()) + int(rng.integers(0, 50)), 1)
    glu = bool(rng.integers(0, 2))
    kw = {}
    lhs = randn(m, k).to(torch.bfloat16)
    if family in ("int8w", "int8"):
      ws = [(bytes_(-127, 128, (e, n, k), torch.int8), rand(e, n) * 0.01 + 1e-3) for _ in range(2)]
      if family == "int8":
        lhs = bytes_(-127, 128, (m, k), torch.int8)
        kw["lhs_scale"] = rand(m) * 0.01 + 1e-3
    elif family in ("int4", "int4g32"):
      grp = 128 if family == "int4" else 32
      ws = [(bytes_(0, 256, (e, n, k // 2), torch.uint8), (rand(e, n, (k + grp - 1) // grp) * 0.01 + 1e-3).to(torch.bfloat16)) for _ in range(2)]
      kw.update(rhs_dtype=MOE_INT4, rhs_scale_block_k=grp)
    elif family == "mxfp4":
      ws = [(bytes_(0, 256, (e, n, k // 2), torch.uint8), bytes_(118, 126, (e, n, k // 32), torch.uint8)) for _ in range(2)]
      kw.update(rhs_dtype=MOE_MXFP4, rhs_scale_block_k=32)
    elif family == "fp8":
      lhs = (randn(m, k) * 2).to(torch.float8_e4m3fn)
      kw.update(lhs_scale=rand(m, k // 128) * 0.02 + 1e-3, lhs_scale_block_k=128, rhs_scale_block_n=128, rhs_scale_block_k=128)
      ws = [((randn(e, n, k) * 2).to(torch.float8_e4m3fn), rand(e, n // 128, k // 128) * 0.02 + 1e-3) for _ in range(2)]
    else:
      ws = [((randn(e, n, k) * 0.05).to(torch.bfloat16), None) for _ in range(2)]
    opts = []
    if rng.random() < 0.5:  # rows read through an index: a source with fewer rows, each read several times or never
      div = int(rng.integers(1, 4))
      src = torch.randperm(m, device="cuda", generator=g)[: m // div + 1]
      lhs = lhs[src].contiguous()
      if "lhs_scale" in kw:
        kw["lhs_scale"] = kw["lhs_scale"][src].contiguous()
      kw.update(lhs_row_idx=cuda(rng.integers(0, (m // div + 1) * div, m).astype(np.int32)), lhs_row_idx_div=div, num_rows=m)
      opts.append(f"index / {div}")
    if rng.random() < 0.5:
      kw["out_row_scale"] = rand(m) + 0.5
      opts.append("row factor")
    lo, hi = 0, int(gs.sum())
    if rng.random() < 0.4 and e > 3:
      off = int(rng.integers(0, e // 2))
      loc = int(rng.integers(1, e - off + 1))
      ws = [(w[off:off + loc].clone(), None if sc is None else sc[off:off + loc].clone()) for w, sc in ws]
      kw["group_offset"] = off
      lo, hi = int(gs[:off].sum()), int(gs[:off + loc].sum())
      opts.append(f"groups {off} .. {off + loc - 1}")
    if ws[0][1] is not None:
      kw["rhs_scale"] = ws[0][1]
    if glu:
      kw.update(rhs_up=ws[1][0], act="silu")
      if ws[1][1] is not None:
        kw["rhs_up_scale"] = ws[1][1]
    tag = f"{family} case {case}: m={m} k={k} n={n} glu={glu} {opts} group_sizes={gs.tolist()}"
    got = K.gmm_raw(lhs, ws[0][0], cuda(gs.astype(np.int32)), **kw)
    ref = K.gmm_raw(lhs, ws[0][0], cuda(gs.astype(np.int32)), kernel="tiled", **kw)
    assert torch.all(got[:lo] == 0) and torch.all(got[hi:] == 0), tag  # rows of no group and of groups outside the window
    if family in ("int4", "int4g32", "mxfp4"):
      worst, top = float((got.float() - ref.float()).abs().max()), float(ref.float().abs().max())
      # (a factor per row multiplies the rounded result and rounds again: one step before it can be two after it)
      assert worst <= 2.0 ** (-6 if "out_row_scale" in kw else -7) * top, f"{tag}: {worst} of {top}"
    else:
      assert torch.equal(got, ref), tag


@pytest.mark.parametrize("family", ["int4", "mxfp4", "fp8", "fp8c", "int8"])
def test_lds_streamed_decode_kernels_against_the_other_kernels_on_random_shapes(K, family):
  """10 random decode-sized shapes per operand family the persistent LDS-streamed kernels take (4 to 40 groups of 0 to 16
  rows, now and then a group of several tiles, for the row and channel scales also groups of up to 70 rows, or ~300 groups of a row or two with a last group of several tiles: the
  shape of a layer with a shared expert, whose tiles the fp8 kernel hands to blocks of their own; rows in no group; K over
  the kernels' whole range, N with a channel tail; with and without the fused activation, rows read through an index, a
  window of the groups) against another kernel of the library on the same operands: the register-staged streaming kernel
  (4-bit, fp8 with block scales) or the LDS-tiled one (fp8 / int8 with row and channel scales), which the small-shape
  tests pin to the oracle.  The sums over K are formed in another order: one bf16 step of the largest value."""
  from maxtext_amd._lib import MOE_INT4, MOE_MXFP4

  rng = np.random.default_rng(1700 + sum(map(ord, family)))
  g = torch.Generator(device="cuda").manual_seed(6)
  rand = lambda *shape: torch.rand(*shape, device="cuda", generator=g)
  randn = lambda *shape: torch.randn(*shape, device="cuda", generator=g)
  bytes_ = lambda lo, hi, shape, dt: torch.randint(lo, hi, shape, device="cuda", dtype=dt, generator=g)
  four_bit = family in ("int4", "mxfp4")
  for case in range(10):
    many = case % 5 == 4  # the shared-expert shape
    e = int(rng.integers(260, 330)) if many else int(rng.integers(4, 41))
    if four_bit:
      k = int(rng.integers(1, 25)) * 128 if family == "int4" else int(rng.integers(4, 97)) * 32
      if family == "int4" and rng.random() < 0.3:
        k = 2880
    else:
      # (fp8 with block scales: up to 7168; the per-row x per-channel kinds go on past that on their long-row variant)
      k = 512 if many else int(rng.integers(1, 15 if family == "fp8" else 22)) * 512
    n = int(rng.integers(16, 48)) * 8 if many else int(rng.integers(32, 80)) * 8
    gs = rng.integers(0, 3, e) if many else rng.integers(0, 17, e)
    if many:
      gs[-1] = int(rng.integers(20, 200))
    elif rng.random() < 0.5:
      gs[rng.integers(0, e)] = int(rng.integers(17, 60))
    if int(gs.sum()) > 13 * e:  # stay where the library takes the decode kernels
      gs = gs // 2
    if family in ("fp8c", "int8") and case % 3 == 1:  # 15 to 47 rows per group on average: the 32- and 64-row tiles of this kind's kernel
      gs = rng.integers(8, 72, e) if case % 2 else rng.integers(0, 40, e)
      while int(gs.sum()) > 47 * e:
        gs = gs * 3 // 4
    m = max(int(gs.sum()) + int(rng.integers(0, 20)), 1)
    glu = bool(rng.integers(0, 2))
    kw = {}
    lhs = randn(m, k).to(torch.bfloat16)
    if family == "int4":
      ws = [(bytes_(0, 256, (e, n, k // 2), torch.uint8), (rand(e, n, (k + 127) // 128) * 0.01 + 1e-3).to(torch.bfloat16)) for _ in range(2)]
      kw.update(rhs_dtype=MOE_INT4, rhs_scale_block_k=128)
    elif family == "mxfp4":
      ws = [(bytes_(0, 256, (e, n, k // 2), torch.uint8), bytes_(118, 126, (e, n, k // 32), torch.uint8)) for _ in range(2)]
      kw.update(rhs_dtype=MOE_MXFP4, rhs_scale_block_k=32)
    elif family == "fp8":
      lhs = (randn(m, k) * 2).to(torch.float8_e4m3fn)
      kw.update(lhs_scale=rand(m, k // 128) * 0.02 + 1e-3, lhs_scale_block_k=128, rhs_scale_block_n=128, rhs_scale_block_k=128)
      ws = [((randn(e, n, k) * 2).to(torch.float8_e4m3fn), rand(e, (n + 127) // 128, k // 128) * 0.02 + 1e-3) for _ in range(2)]
    elif family == "fp8c":
      lhs = (randn(m, k) * 2).to(torch.float8_e4m3fn)
      kw.update(lhs_scale=rand(m) * 0.02 + 1e-3, rhs_scale_block_n=1, rhs_scale_block_k=0)
      ws = [((randn(e, n, k) * 2).to(torch.float8_e4m3fn), rand(e, n) * 0.02 + 1e-3) for _ in range(2)]
    else:
      lhs = bytes_(-127, 128, (m, k), torch.int8)
      kw["lhs_scale"] = rand(m) * 0.01 + 1e-3
      ws = [(bytes_(-127, 128, (e, n, k), torch.int8), rand(e, n) * 0.01 + 1e-3) for _ in range(2)]
    opts = []
    if rng.random() < 0.5:
      div = int(rng.integers(1, 4))
      src = torch.randperm(m, device="cuda", generator=g)[: m // div + 1]
      lhs = lhs[src].contiguous()
      if "lhs_scale" in kw:
        kw["lhs_scale"] = kw["lhs_scale"][src].contiguous()
      kw.update(lhs_row_idx=cuda(rng.integers(0, (m // div + 1) * div, m).astype(np.int32)), lhs_row_idx_div=div, num_rows=m)
      opts.append(f"index / {div}")
    lo, hi = 0, int(gs.sum())
    if rng.random() < 0.3 and not many:
      off = int(rng.integers(0, e // 2))
      loc = int(rng.integers(1, e - off + 1))
      ws = [(w[off:off + loc].clone(), sc[off:off + loc].clone()) for w, sc in ws]
      kw["group_offset"] = off
      lo, hi = int(gs[:off].sum()), int(gs[:off + loc].sum())
      opts.append(f"groups {off} .. {off + loc - 1}")
    kw["rhs_scale"] = ws[0][1]
    if glu:
      kw.update(rhs_up=ws[1][0], rhs_up_scale=ws[1][1], act="silu")
    tag = f"{family} case {case}: m={m} k={k} n={n} glu={glu} {opts} group_sizes={gs.tolist()}"
    got = K.gmm_raw(lhs, ws[0][0], cuda(gs.astype(np.int32)), **kw)
    ref = K.gmm_raw(lhs, ws[0][0], cuda(gs.astype(np.int32)), kernel="stream" if four_bit or family == "fp8" else "tiled", **kw)
    assert torch.all(got[:lo] == 0) and torch.all(got[hi:] == 0), tag
    assert not torch.isnan(got.float()).any(), tag
    worst, top = float((got.float() - ref.float()).abs().max()), float(ref.float().abs().max())
    assert worst <= 2.0 ** -7 * top, f"{tag}: {worst} of {top}"
