"""`gmm(lhs, rhs, group_sizes, ...)` with the reference's signature, backed by moe_gmm.

Mirrors src/maxtext/kernels/megablox/ops.py:46-129 (exported as kernels/megablox/__init__.py:16):
same argument names, argument meaning and trace-time errors (backend.py:33-52, :335-345).
Arrays are torch CUDA tensors.  Quantised operands are passed as quantizations.QArray (the role
qpl.QArray plays in ops.py:232-267); plain bf16 operands are quantised on the fly when
lhs_quantize_dtype / rhs_quantize_dtype ask for it.

Extra keyword arguments the quantised expert path needs (they follow gmm_v2,
pallas_mosaic_tpu_v2_gmm_kernel.py:1297-1315): `rhs_up` (second projection, fused
act(lhs@rhs) * (lhs@rhs_up)), `fuse_act`, and `rhs_bias` / `rhs_up_bias` ([G, N] per-expert biases
added before the activation) and `partial_sum_up` (the partial sum of the second projection; `partial_sum` is the
reference's own argument).
"""

from __future__ import annotations

import torch

from maxtext_amd import kernels, quantizations
from maxtext_amd._lib import MOE_INT4, MOE_MXFP4
from maxtext_amd.quantizations import QArray

# When set to a list, the backward pass of gmm appends (stage, start_event, end_event) recorded on the launch stream.
PROFILE_EVENTS = None

_INT8_NAMES = ("int8", torch.int8)
_FP8_NAMES = ("fp8", "float8_e4m3fn", torch.float8_e4m3fn)
_INT4_NAMES = ("int4",)
_E5M2_NAMES = ("e5m2", "float8_e5m2", torch.float8_e5m2)


def _validate_args(lhs, rhs, group_sizes, expected_rhs_dims=3):
  """backend.py:33-52."""
  lq = lhs.qvalue if isinstance(lhs, QArray) else lhs
  rq = rhs.qvalue if isinstance(rhs, QArray) else rhs
  if lq.dim() != 2:
    raise ValueError(f"Expected 2-tensor for 'lhs' but got {lq.dim()}-tensor.")
  if rq.dim() != expected_rhs_dims:
    raise ValueError(f"Expected {expected_rhs_dims}-tensor for 'rhs' but got {rq.dim()}-tensor.")
  if group_sizes.dtype != torch.int32:
    raise ValueError(f"Expected 32-bit integer 'group_sizes' but got {group_sizes.dtype}.")


def _qname(qdtype):
  if qdtype in _INT8_NAMES:
    return "int8"
  if qdtype in _FP8_NAMES:
    return "fp8"
  if qdtype in _INT4_NAMES:
    return "int4"
  raise ValueError(f"unsupported quantisation dtype {qdtype}")


_TORCH_Q = {"int8": torch.int8, "fp8": torch.float8_e4m3fn}
_QMAX = {"int8": 127.0, "fp8": quantizations.FP8_E4M3_MAX}


def _static_scale_tensor(qname, calibration_method, device):
  return torch.tensor([quantizations.get_static_scale(_QMAX[qname], calibration_method)], dtype=torch.float32, device=device)


def quantize_lhs(lhs: torch.Tensor, qdtype, *, calibration_method="absmax", blocks=None, v2=False, per_tensor=False) -> QArray:
  """Activation quantiser.

  v2=False: the v1 path, qpl.quantize(lhs, act_qtype, channelwise_axes=[0], calibration_method) (ops.py:241-248):
  one scale per row, for int8 and for fp8; "fixed,..." gives one static scale for the tensor, per_tensor one dynamic
  scale for it (channelwise_axes=[]).  blocks=128 keeps the DeepSeek recipe's one scale per row and 128 values of K.
  v2=True: the quantiser inside gmm_v2 (pallas_mosaic_tpu_v2_gmm_kernel.py:528-542): one scale per row and 512 values
  of K (:1231), or the static (1, 1) scale of ops.py:333-360."""
  qname = _qname(qdtype)
  if qname not in _TORCH_Q:
    raise ValueError(f"unsupported lhs_quantize_dtype {qdtype}")
  rule = "v2" if v2 else "rint_div"
  if calibration_method is not None and calibration_method.lower().startswith("fixed"):
    st = _static_scale_tensor(qname, calibration_method, lhs.device)
    q, s = kernels.gather_rows(lhs, out_dtype=_TORCH_Q[qname], rule=rule, static_scale=st)
    return QArray(q, s, qname, block_k=-1)
  if per_tensor:
    # channelwise_axes=[] (disable_channelwise_axes, ops.py:245): one absmax scale for the tensor, found on the device and
    # then used like a static one
    st = kernels.tensor_scale(lhs, _QMAX[qname])
    q, s = kernels.gather_rows(lhs, out_dtype=_TORCH_Q[qname], rule=rule, static_scale=st)
    return QArray(q, s, qname, block_k=-1)
  block_k = 512 if v2 and blocks is None else (blocks or 0)
  q, s = kernels.gather_rows(lhs, out_dtype=_TORCH_Q[qname], block_k=block_k, rule=rule)
  return QArray(q, s, qname, block_k=block_k)


def quantize_rhs(rhs_gnk: torch.Tensor, qdtype, share_across_experts=True, *, calibration_method="absmax", manual=False,
                 fp8_blocks=False, per_tensor=False) -> QArray:
  """Weight quantiser for rhs in [G, N, K] layout: one scale per output channel shared by the experts, the [1, 1, n]
  scale of qpl.quantize(rhs, channelwise_axes=[2]) (ops.py:250-260), for int8 and fp8; manual=True is
  quantizations.manual_quantize (per tensor, static, ops.py:262-266); fp8_blocks=True the 128 x 128 blocks of DeepSeek
  checkpoints."""
  qname = _qname(qdtype)
  # a "fixed,-max,max" range gives qpl.quantize the same constant scale for every channel, i.e. the static per-tensor
  # quantiser; its exact arithmetic is third-party, manual_quantize's (layers/quantizations.py:961-991) is used for both
  static = manual or (calibration_method is not None and calibration_method.lower().startswith("fixed"))
  on_kernel = (qname in _TORCH_Q and not fp8_blocks and rhs_gnk.is_cuda and rhs_gnk.dtype == torch.bfloat16 and rhs_gnk.shape[2] % 8 == 0)
  if static:
    if on_kernel:
      st = _static_scale_tensor(qname, calibration_method, rhs_gnk.device)
      q, _ = kernels.quantize_rhs(rhs_gnk.contiguous(), _TORCH_Q[qname], static_scale=st)
      # (the QArray's scale is the python float in the weights' dtype, layers/quantizations.py:985-989)
      return QArray(q, st.to(rhs_gnk.dtype).float(), qname, block_n=-1, block_k=0, shared=True)
    return quantizations.manual_quantize_weight(rhs_gnk, qname, calibration_method)
  if per_tensor:
    if not on_kernel:
      raise NotImplementedError("per-tensor dynamic weight scales need bf16 weights on the GPU (K % 8 == 0)")
    q, sc = kernels.quantize_rhs(rhs_gnk.contiguous(), _TORCH_Q[qname], per_tensor=True)
    return QArray(q, sc, qname, block_n=-1, block_k=0, shared=True)
  if on_kernel:
    q, sc = kernels.quantize_rhs(rhs_gnk.contiguous(), _TORCH_Q[qname], shared=share_across_experts)
    return QArray(q, sc, qname, block_n=1, block_k=0, shared=share_across_experts)
  if qname == "int8":
    return quantizations.quantize_weight_int8(rhs_gnk, share_across_experts=share_across_experts)
  if qname == "fp8":
    if fp8_blocks:
      return quantizations.quantize_weight_fp8_blocks(rhs_gnk)
    return quantizations.quantize_weight_fp8_channel(rhs_gnk, share_across_experts=share_across_experts)
  return quantizations.quantize_weight_int4(rhs_gnk)


def _native_rhs(rhs, transpose_rhs):
  """-> rhs in [G, N, K] layout (zero copy when transpose_rhs=True)."""
  if isinstance(rhs, QArray):
    return rhs  # QArray weights are always stored [G, N, K]
  if transpose_rhs:
    return rhs if rhs.is_contiguous() else rhs.contiguous()
  return kernels.transpose_rhs(rhs.contiguous())


def _rhs_layout(q: QArray) -> dict:
  """moe_gmm's scale arguments for a weight QArray."""
  defaults = {"int8": (1, 0), "fp8": (128, 128), "int4": (1, 128), "int4g32": (1, 32), "mxfp4": (1, 32)}
  if q.qtype not in defaults:
    raise ValueError(f"unknown qtype {q.qtype}")
  bn, bk = defaults[q.qtype]
  kw = dict(rhs_scale_block_n=bn if q.block_n is None else q.block_n, rhs_scale_block_k=bk if q.block_k is None else q.block_k,
            rhs_scale_kmajor=q.kmajor, rhs_scale_shared=q.shared)
  if q.qtype.startswith("int4"):
    kw["rhs_dtype"] = MOE_INT4
  elif q.qtype == "mxfp4":
    kw["rhs_dtype"] = MOE_MXFP4
  return kw


def _lhs_layout(q: QArray) -> dict:
  bk = q.block_k if q.block_k is not None else (128 if q.qtype == "fp8" else 0)
  return dict(lhs_scale=q.scale, lhs_scale_block_k=bk)


def gmm(
    lhs,
    rhs,
    group_sizes,
    preferred_element_type=torch.float32,
    tiling=(128,) * 9,
    group_offset=None,
    existing_out=None,
    transpose_rhs=False,
    interpret=None,
    lhs_quantize_dtype=None,
    rhs_quantize_dtype=None,
    use_qwix_quantization=False,
    use_tokamax_backend=False,
    weight_gather_axes=None,
    lhs_vma_axes=(),
    rhs_vma_axes=(),
    qwix_rule=None,
    use_manual_quantization=False,
    use_gmm_v2=False,
    partial_sum=None,
    *,
    rhs_up=None,
    fuse_act=None,
    act_limit=7.0,
    rhs_bias=None,
    rhs_up_bias=None,
    partial_sum_up=None,
    bwd_quantize_dtype=None,
    lhs_row_idx=None,
    lhs_row_idx_div=1,
    workspace=None,
    same_groups=False,
    out_row_scale=None,
    lhs_row_inv=None,
):
  """Grouped matmul: out[rows of group g] = lhs[rows] @ rhs[g] (ops.py:46).

  bwd_quantize_dtype: the `bwd_qtype` of the reference's qwix rule (ops.py:97-103, :583-604): "float8_e5m2" quantises
  the incoming gradient of an int8 x int8 forward per row (for dlhs) and per column (for drhs); None leaves it as is.

  lhs: [m, k] bf16 tensor or QArray; rhs: [g, k, n] bf16 ([g, n, k] with transpose_rhs) or a
  QArray holding [G, N, K]; group_sizes: int32 [G_total] on the device.  `tiling`, `interpret`,
  the vma axes and `use_tokamax_backend` only select TPU code paths in the reference and are
  accepted and ignored; the tile shape is chosen from rows-per-expert inside moe_gmm.

  Quantisation follows ops.py:87-103 and _fwd_quantize_activation_and_weight (:232-267): with use_qwix_quantization
  the rule is `qwix_rule` (a quantizations.QtRule), otherwise one is made from lhs / rhs_quantize_dtype with "absmax"
  calibration.  Activations get one scale per row ([m, 1]), weights one per output channel shared by the experts
  ([1, 1, n]); use_manual_quantization quantises the weights per tensor with the rule's static range; "fixed,..."
  calibration gives static per-tensor scales.  With use_gmm_v2 the activations are quantised by gmm_v2's own rule
  (per row and 512 values of K, or the static (1, 1) scale, ops.py:333-360) to the type the weights ask for
  (pallas_mosaic_tpu_v2_gmm_kernel.py:1208-1223: int8 weights -> int8, fp8 weights -> fp8; int4 weights stay
  weight-only here).  preferred_element_type: float32 (the reference's default, ops.py:50) or bfloat16.
  lhs_row_idx / lhs_row_idx_div / out_row_scale: see kernels.gmm_raw (the permute and the routing weights fused in);
  lhs_row_inv: the inverse permutation of lhs_row_idx when it is one, used by the gradient of lhs (a deterministic sum over
  each token's copies).  Every argument is differentiable where the reference's is: lhs, rhs, rhs_up, the biases,
  partial_sum and existing_out (both receive the incoming gradient, ops.py:524-527), out_row_scale.
  """
  del tiling, interpret, lhs_vma_axes, rhs_vma_axes, use_tokamax_backend
  _validate_args(lhs, rhs, group_sizes)
  if preferred_element_type not in (torch.bfloat16, torch.float32):
    raise NotImplementedError("outputs are bfloat16 or float32")
  if existing_out is not None:
    # rows of local groups are written into the caller's buffer, all other rows keep their contents (backend.py:493-501)
    if existing_out.dtype != preferred_element_type or not existing_out.is_contiguous():
      raise ValueError("existing_out must be a contiguous tensor of preferred_element_type")
  if weight_gather_axes:
    raise NotImplementedError("weight all-gather belongs to the multi-device path")
  offset, offset_dev = 0, None
  needs_grad = torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad for t in (lhs, rhs, rhs_up, rhs_bias, rhs_up_bias))
  if group_offset is not None:
    if isinstance(group_offset, torch.Tensor):
      if group_offset.dim() != 0:
        raise ValueError(f"group_offset must be a ()-shaped array. Got: {tuple(group_offset.shape)}.")
      if group_offset.is_cuda and not needs_grad:
        # a device scalar (inside shard_map the reference derives it from jax.lax.axis_index, moe.py:2014-2019): handed to
        # the tile-map kernel as it is, the host never reads it
        offset_dev = group_offset.reshape(1).to(torch.int32)
      else:
        offset = int(group_offset.item())  # (the backward's kernels take the offset by value: one host read per call)
    else:
      offset = int(group_offset)

  # ops.py:87-103
  rule = None
  if use_qwix_quantization:
    rule = qwix_rule
    if not isinstance(rule, quantizations.QtRule):
      raise ValueError(f"Expect a QtRule for quantized training. But get quantization_rule={rule} for gmm.")
  elif lhs_quantize_dtype or rhs_quantize_dtype or bwd_quantize_dtype:
    rule = quantizations.QtRule(weight_qtype=rhs_quantize_dtype, act_qtype=lhs_quantize_dtype, bwd_qtype=bwd_quantize_dtype)

  needs_grad = needs_grad or (torch.is_grad_enabled() and any(
      isinstance(t, torch.Tensor) and t.requires_grad for t in (partial_sum, partial_sum_up, existing_out, out_row_scale)))
  if needs_grad:
    if rule is not None and (rule.bwd_calibration_method or "absmax") != "absmax":
      raise NotImplementedError("the gradient is quantised with absmax calibration")
    if existing_out is not None and existing_out.dtype != torch.bfloat16:
      raise NotImplementedError("existing_out is bfloat16 on the differentiable path")
    out = _gmm_with_grad(lhs, rhs, rhs_up, group_sizes, offset, transpose_rhs, rule, use_manual_quantization, fuse_act, act_limit,
                         rhs_bias, rhs_up_bias, partial_sum, partial_sum_up, existing_out, lhs_row_idx, lhs_row_idx_div, lhs_row_inv,
                         v2=bool(use_gmm_v2))
    if out_row_scale is not None:
      # the routing weights between the activation and wo (models/deepseek_batchsplit_fp8.py:1048-1049): the finished
      # bf16 result times the row's factor, rounded again; autograd gives both gradients
      out = (out.float() * out_row_scale.reshape(-1, 1).float()).to(torch.bfloat16)
    # (the differentiable kernels produce bf16; a float32 result is that value widened, and its gradient arrives rounded to bf16)
    return out if preferred_element_type == torch.bfloat16 else out.to(preferred_element_type)

  common = dict(group_offset=offset, group_offset_dev=offset_dev, out_dtype=preferred_element_type, lhs_row_idx=lhs_row_idx,
                lhs_row_idx_div=lhs_row_idx_div, out_row_scale=out_row_scale, workspace=workspace, same_groups=same_groups)
  if rhs_bias is not None:
    common["rhs_bias"] = rhs_bias.float().contiguous()  # [G, N] (rhs_bias [G, 1, N] of the v2 kernel, :573)
  if partial_sum is not None:  # [m, n], added to the product before the activation (ops.py:77)
    common["partial_sum"] = partial_sum.to(torch.bfloat16).contiguous()
  if existing_out is not None:
    common.update(out=existing_out, keep_other_rows=True)

  # [g, k, n] bf16 weights are read as they are where the kernel allows it (this is dlhs of a transpose_rhs=True layer:
  # ops.py:470-485), instead of being re-laid out for every call
  if (not transpose_rhs and rhs_up is None and rule is None and not isinstance(rhs, QArray) and not isinstance(lhs, QArray)
      and rhs.dtype == torch.bfloat16 and lhs.dtype == torch.bfloat16 and fuse_act is None and lhs_row_idx is None
      and kernels.gmm_rhs_kn_supported(lhs.shape[0], rhs.shape[1], rhs.shape[2], group_sizes.numel())):
    return kernels.gmm_raw(lhs.contiguous(), rhs.contiguous(), group_sizes, rhs_kn=True, **common)

  rhs_n = _native_rhs(rhs, transpose_rhs)
  up_n = _native_rhs(rhs_up, transpose_rhs) if rhs_up is not None else None
  if rule is not None and rule.weight_qtype and not isinstance(rhs_n, QArray):
    # disable_channelwise_axes: channelwise_axes=[] (ops.py:258), one dynamic scale for the whole tensor
    qkw = dict(calibration_method=rule.weight_calibration_method, manual=use_manual_quantization,
               per_tensor=bool(rule.disable_channelwise_axes))
    rhs_n = quantize_rhs(rhs_n, rule.weight_qtype, **qkw)
    if up_n is not None:
      up_n = quantize_rhs(up_n, rule.weight_qtype, **qkw)
  if rule is not None and rule.act_qtype and not isinstance(lhs, QArray):
    if not use_gmm_v2:
      lhs = quantize_lhs(lhs.contiguous(), rule.act_qtype, calibration_method=rule.act_calibration_method,
                         per_tensor=bool(rule.disable_channelwise_axes))
  if use_gmm_v2 and isinstance(rhs_n, QArray) and not isinstance(lhs, QArray) and rhs_n.qtype in ("int8", "fp8"):
    # gmm_v2 quantises the activations itself, to the type the weights ask for (:1208-1223), statically when the rule
    # carries a fixed range (ops.py:333-360)
    method = rule.act_calibration_method if rule is not None and rule.act_qtype else "absmax"
    lhs = quantize_lhs(lhs.contiguous(), rhs_n.qtype, calibration_method=method, v2=True)

  kw = dict(act=fuse_act, act_limit=act_limit, **common)
  if rhs_up_bias is not None:
    kw["rhs_up_bias"] = rhs_up_bias.float().contiguous()
  if partial_sum_up is not None:
    kw["partial_sum_up"] = partial_sum_up.to(torch.bfloat16).contiguous()
  if isinstance(lhs, QArray):
    kw.update(_lhs_layout(lhs))
    lhs_t = lhs.qvalue
  else:
    lhs_t = lhs.contiguous()
  if isinstance(rhs_n, QArray):
    kw["rhs_scale"] = rhs_n.scale
    kw.update(_rhs_layout(rhs_n))
    if up_n is not None:
      if not isinstance(up_n, QArray) or up_n.qtype != rhs_n.qtype:
        raise ValueError("rhs_up must be quantised like rhs")
      kw["rhs_up"], kw["rhs_up_scale"] = up_n.qvalue, up_n.scale
    rhs_t = rhs_n.qvalue
  else:
    rhs_t = rhs_n
    if up_n is not None:
      kw["rhs_up"] = up_n
  return kernels.gmm_raw(lhs_t, rhs_t, group_sizes, **kw)


def tgmm(
    lhs,
    rhs,
    group_sizes,
    preferred_element_type=torch.float32,
    tiling=(128, 128, 128),
    group_offset=None,
    num_actual_groups=None,
    existing_out=None,
    interpret=False,
    varying_axes=(),
):
  """Transposed grouped matmul out[g] = lhs[:, rows of g] @ rhs[rows of g, :] (backend.py:575-816).

  lhs: [k, m] bf16 (the reference passes the forward activation swapped, ops.py:889-899; a
  `.t()` view of a contiguous [m, k] tensor is consumed without a copy); rhs: [m, n] bf16 (the
  incoming gradient); returns [num_actual_groups, k, n] as a transposed view of the [G, N, K]
  buffer the kernel writes, which is the layout moe_gmm takes weights in.  existing_out
  ([num_actual_groups, k, n], float32 or bfloat16) is added in before the output is rounded.
  """
  del tiling, interpret, varying_axes
  if lhs.dim() != 2 or rhs.dim() != 2:
    raise ValueError("Expected 2-tensors for 'lhs' and 'rhs'.")
  if group_sizes.dtype != torch.int32:
    raise ValueError(f"Expected 32-bit integer 'group_sizes' but got {group_sizes.dtype}.")
  if lhs.shape[1] != rhs.shape[0]:
    raise ValueError(f"Expected lhs [k, m] and rhs [m, n] to share m, got {tuple(lhs.shape)} and {tuple(rhs.shape)}.")
  if preferred_element_type not in (torch.float32, torch.bfloat16):
    raise NotImplementedError("tgmm outputs are float32 or bfloat16")
  existing_nk = None
  if existing_out is not None:
    # added to the f32 accumulator before the one rounding to the output type (backend.py:733-734)
    g_local = group_sizes.numel() - (0 if group_offset is None else int(group_offset)) if num_actual_groups is None else int(num_actual_groups)
    if tuple(existing_out.shape) != (g_local, lhs.shape[0], rhs.shape[1]):
      raise ValueError(f"existing_out must be [{g_local}, {lhs.shape[0]}, {rhs.shape[1]}], got {tuple(existing_out.shape)}")
    if existing_out.dtype not in (torch.float32, torch.bfloat16):
      raise NotImplementedError("existing_out is float32 or bfloat16")
    existing_nk = existing_out.transpose(1, 2)  # the kernel's [G, N, K] layout; a view when the caller kept a result of tgmm
    if not existing_nk.is_contiguous():
      existing_nk = existing_nk.contiguous()
  offset = 0 if group_offset is None else int(group_offset)
  lhs_mk = lhs.t()
  if not lhs_mk.is_contiguous():
    lhs_mk = lhs_mk.contiguous()
  out = kernels.tgmm(
      lhs_mk, rhs.contiguous(), group_sizes, num_groups_local=num_actual_groups, group_offset=offset, out_dtype=preferred_element_type,
      existing_out=existing_nk,
  )
  return out.transpose(1, 2)


class _GmmFn(torch.autograd.Function):
  """Differentiable gmm for bf16 operands (custom VJP of ops.py:137-230 / :438-527).

  Unquantised forward, or a forward that quantises one side only: backward uses the bf16 residuals,
  dlhs = gmm(dout, rhs^T) (ops.py:612-642) and drhs = tgmm(lhs^T, dout) (ops.py:766-796).

  int8 x int8 and fp8 x fp8 forward (e4m3 both sides: the fp8_full recipe, layers/quantizations.py:234-250, :798-855;
  per-row x per-channel absmax scales, or the static per-tensor scales of "fixed,-max,max" calibration and of
  manual_quantize): the residuals are the quantised operands and the backward is the reference's (_bwd_prepare_inputs
  ops.py:530-580): the scale of the axis that disappears goes onto the gradient, dlhs = gmm(dout * rhs_scale[n], rhs_q^T),
  drhs = tgmm(lhs_q^T, dout * lhs_scale[m]); with bwd_q the two scaled gradients are first quantised to float8_e5m2 per
  row / per column (_bwd_quantize_gradient ops.py:583-604); scaling and quantisation are one kernel each
  (kernels.bwd_scale_grad).  Where the operands are exact in bf16 (int8, e4m3, e5m2 all are) the products run on the
  bf16 MFMA kernels; dlhs of an fp8 forward with a quantised gradient runs as e5m2 x e4m3 on the fp8 MFMA where the
  persistent kernel takes the shape (kernels.gmm_lhs_e5m2_supported).
  """

  @staticmethod
  def forward(ctx, lhs, rhs, group_sizes, offset, transpose_rhs, rule, manual, partial_sum=None, existing_out=None, row_idx=None, row_div=1,
              row_inv=None, v2=False):
    """partial_sum [m, n] is added to the product, existing_out [m, n] receives the rows of the local groups (both get
    the incoming gradient as theirs, ops.py:524-527); row_idx / row_div: row i of the product reads lhs row
    row_idx[i] // row_div (the fused permute: lhs holds the T token rows and no [m, k] copy is kept for the backward),
    row_inv: the inverse permutation of row_idx when it is one (the gradient of lhs is then a deterministic sum over each
    token's row_div copies instead of an atomic scatter).
    v2 (use_gmm_v2): the forward leaves the activations to the product, which quantises them itself per row and 512 values
    of K or with the static (1, 1) scale (ops.py:241, :333-360); the residual is the bf16 lhs, which the backward quantises
    per row by the v1 rule before it proceeds as above (_bwd_prepare_inputs, ops.py:561-572)."""
    lhs_q, rhs_q = (rule.act_qtype, rule.weight_qtype) if rule is not None else (None, None)
    bwd_q = rule.bwd_qtype if rule is not None else None
    ctx.offset, ctx.transpose_rhs, ctx.bwd_q = offset, transpose_rhs, bwd_q
    ctx.row_div, ctx.has_ps, ctx.has_eo = int(row_div), partial_sum is not None, existing_out is not None
    ctx.lhs_rows = lhs.shape[0]
    both_int8 = lhs_q in _INT8_NAMES and rhs_q in _INT8_NAMES
    both_fp8 = lhs_q in _FP8_NAMES and rhs_q in _FP8_NAMES
    ctx.quantized = both_int8 or both_fp8
    if bwd_q is not None and not ctx.quantized:
      raise NotImplementedError("bwd_quantize_dtype needs an int8 x int8 or fp8 x fp8 forward (channelwise or static scales)")
    if bwd_q is not None and bwd_q not in _E5M2_NAMES:
      raise ValueError(f"unsupported bwd_quantize_dtype {bwd_q}")
    extra = dict(partial_sum=partial_sum, existing_out=existing_out, lhs_row_idx=row_idx, lhs_row_idx_div=int(row_div))
    if existing_out is not None:
      ctx.mark_dirty(existing_out)
    none = torch.empty(0, device=lhs.device)
    idx_t = (row_idx if row_idx is not None else none, row_inv if row_inv is not None else none)
    ctx.has_idx, ctx.has_inv = row_idx is not None, row_inv is not None
    with torch.no_grad():
      if ctx.quantized:
        # disable_channelwise_axes: one dynamic scale per tensor (channelwise_axes=[], ops.py:245, :258), for the gradients too
        ctx.per_tensor = bool(rule.disable_channelwise_axes)
        rq = quantize_rhs(_native_rhs(rhs, transpose_rhs), rhs_q, calibration_method=rule.weight_calibration_method, manual=manual,
                          per_tensor=ctx.per_tensor)
        ctx.rhs_dtype = rhs.dtype
        ctx.v2_act = (lhs_q, rule.act_calibration_method) if v2 else None
        if v2:
          ctx.save_for_backward(lhs, none, rq.qvalue, rq.scale, group_sizes, *idx_t)
          return gmm(lhs, rq, group_sizes, torch.bfloat16, group_offset=offset, transpose_rhs=True, use_gmm_v2=True,
                     use_qwix_quantization=True, qwix_rule=rule, **extra)
        lq = quantize_lhs(lhs.contiguous(), lhs_q, calibration_method=rule.act_calibration_method, per_tensor=ctx.per_tensor)
        ctx.save_for_backward(lq.qvalue, lq.scale, rq.qvalue, rq.scale, group_sizes, *idx_t)
        return gmm(lq, rq, group_sizes, torch.bfloat16, group_offset=offset, transpose_rhs=True, **extra)
      ctx.save_for_backward(lhs, rhs, group_sizes, *idx_t)
      kw = {}
      if rule is not None:
        kw = dict(use_qwix_quantization=True, qwix_rule=rule, use_manual_quantization=manual, use_gmm_v2=v2)
      return gmm(lhs, rhs, group_sizes, torch.bfloat16, group_offset=offset, transpose_rhs=transpose_rhs, **kw, **extra)

  @staticmethod
  def _rows_to_tokens(ctx, d_rows, row_idx, row_inv):
    """Gradient of the rows read through the index -> gradient of the lhs rows themselves."""
    if not ctx.has_idx:
      return d_rows
    if ctx.has_inv:  # a permutation: token t's copies are the rows row_inv[t * div .. + div - 1], summed in f32 in that order
      return kernels.unpermute_combine(d_rows.contiguous(), None, k=ctx.row_div, inv_perm=row_inv)
    acc = torch.zeros((ctx.lhs_rows, d_rows.shape[1]), dtype=torch.float32, device=d_rows.device)
    acc.index_add_(0, torch.div(row_idx, ctx.row_div, rounding_mode="floor").long().clamp_(0, ctx.lhs_rows - 1), d_rows.float())
    return acc.to(d_rows.dtype)

  @staticmethod
  def _backward_quantized(ctx, dout):
    lq, ls, rq, rs, group_sizes, row_idx, row_inv = ctx.saved_tensors  # lq [m,k], ls [m] or [1]; rq [g,n,k], rs [g,n], [1,n] or [1]
    if getattr(ctx, "v2_act", None) is not None:
      # the residual is the bf16 activation: quantised here per row by the v1 rule (ops.py:561-572), not by the product's
      # own K-block rule
      q = quantize_lhs(lq.contiguous(), ctx.v2_act[0], calibration_method=ctx.v2_act[1], per_tensor=getattr(ctx, "per_tensor", False))
      lq, ls = q.qvalue, q.scale
    m, n = dout.shape
    k = lq.shape[1]
    g_local = rq.shape[0]
    fp8 = lq.dtype == torch.float8_e4m3fn
    dlhs = drhs = None
    quant = ctx.bwd_q is not None
    per_tensor = getattr(ctx, "per_tensor", False)
    ev = PROFILE_EVENTS
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(3)] if ev is not None else None
    if marks:
      marks[0].record()
    if ctx.needs_input_grad[0]:
      # dout times the weights' channel scales of each row's expert, e5m2 per row (one kernel)
      rs_gn = rs.reshape(-1, n) if rs.numel() % n == 0 else rs.reshape(1, 1).expand(1, n)
      rs_gn = (rs_gn if rs_gn.shape[0] == g_local else rs_gn[:1].expand(g_local, n)).contiguous()
      as_fp8 = fp8 and quant and kernels.gmm_lhs_e5m2_supported(m, n, k, group_sizes.numel())
      # the forward's [g, n, k] weights are the [G, K, N] layout of this product (n contracted, k the output axis): the fp8
      # stream kernel reads them as they are; the other routes take a re-laid-out copy [g, k, n]
      as_kn = as_fp8 and kernels.gmm_fp8_rhs_kn_supported(m, n, k, group_sizes.numel())
      w_t = None if as_kn else kernels.transpose_rhs(rq)
      if per_tensor:
        # one weight scale and ONE scale for the whole gradient (channelwise_axes=[], ops.py:594): it comes back as a
        # vector of equal entries, of which the products take the first (fp8 route) or one per row
        d, s_all = kernels.bwd_scale_grad(dout, rs.reshape(-1)[:1].contiguous(), mode="tensor", quantize=quant, as_fp8=as_fp8)
        s_row = None if s_all is None else s_all[:1].expand(m).contiguous()
      else:
        d, s_row = kernels.bwd_scale_grad(dout, rs_gn, mode="dlhs", quantize=quant, group_sizes=group_sizes, num_groups_local=g_local,
                                          group_offset=ctx.offset, as_fp8=as_fp8)
      one = torch.ones((1,), dtype=torch.float32, device=dout.device)
      if as_fp8:
        # e5m2 x e4m3 on the fp8 MFMA; the rows' scales are the activations' epilogue scales
        dlhs = kernels.gmm_raw(d, rq if as_kn else w_t, group_sizes, lhs_scale=s_row, rhs_scale=one, rhs_scale_block_n=_lib_per_tensor(),
                               rhs_scale_shared=True, group_offset=ctx.offset, rhs_kn=as_kn)
      else:
        # the row scales go back on in the product's epilogue (rounded bf16 result times scale, rounded again: what the
        # reference's two steps give)
        w_b = w_t if w_t.dtype == torch.int8 else w_t.to(torch.bfloat16)
        if w_b.dtype == torch.int8:
          dlhs = kernels.gmm_raw(d, w_b, group_sizes, rhs_scale=one, rhs_scale_block_n=_lib_per_tensor(), rhs_scale_shared=True,
                                 group_offset=ctx.offset, out_row_scale=s_row)
        else:
          dlhs = kernels.gmm_raw(d, w_b, group_sizes, group_offset=ctx.offset, out_row_scale=s_row)
      dlhs = _GmmFn._rows_to_tokens(ctx, dlhs, row_idx, row_inv)
    if marks:
      marks[1].record()
    if ctx.needs_input_grad[1]:
      # dout times the activations' row scales, e5m2 per column
      lq_rows = lq
      if ctx.has_idx:  # the quantised token rows, gathered for this product only (int8 / fp8 rows: half of a bf16 copy)
        tok = torch.div(row_idx, ctx.row_div, rounding_mode="floor").long().clamp_(0, lq.shape[0] - 1)
        lq_rows = lq[tok]
        ls = ls if ls.numel() == 1 else ls[tok].contiguous()
      ls_m = ls if ls.numel() == m else ls.reshape(1).expand(m).contiguous()
      # fp8 residuals and an e5m2 gradient multiply as they are stored on shapes the fp8 weight-gradient kernel takes
      bytes_in = fp8 and quant and kernels.tgmm_fp8_supported(m, k, n, group_sizes.numel(), g_local)
      if per_tensor:  # (ops.py:568, :601: one activation scale, one gradient scale; [n] equal entries serve as column scales)
        d, s_col = kernels.bwd_scale_grad(dout, ls.reshape(-1)[:1].contiguous(), mode="tensor", quantize=quant, as_fp8=bytes_in)
      else:
        d, s_col = kernels.bwd_scale_grad(dout, ls_m, mode="drhs", quantize=quant, as_fp8=bytes_in)
      # the column scales go back onto the f32 products in the kernel's epilogue, which rounds once to the weights' type
      direct = ctx.rhs_dtype in (torch.bfloat16, torch.float32)
      if marks:  # the weight-gradient launch alone, beside the stage that includes its quantiser passes
        marks += [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        marks[3].record()
      if bytes_in:
        w = kernels.tgmm_fp8(lq_rows.contiguous(), d, group_sizes, num_groups_local=g_local, group_offset=ctx.offset,
                             out_dtype=ctx.rhs_dtype if direct else torch.float32, out_row_scale=s_col)  # [g, n, k]
      else:
        w = kernels.tgmm(lq_rows.to(torch.bfloat16), d, group_sizes, num_groups_local=g_local, group_offset=ctx.offset,
                         out_dtype=ctx.rhs_dtype if direct else torch.float32, out_row_scale=s_col)  # [g, n, k]
      if marks:
        marks[4].record()
        ev.append((("tgmm_f8_kernel_" if bytes_in else "tgmm_kernel_") + f"k{k}_n{n}", marks[3], marks[4]))
      w = w.to(ctx.rhs_dtype)
      drhs = w if ctx.transpose_rhs else w.transpose(1, 2)
    if marks:
      marks[2].record()
      shape = f"k{k}_n{n}"
      ev.append(("dlhs_q_" + shape, marks[0], marks[1]))
      ev.append(("tgmm_q_" + shape, marks[1], marks[2]))
    return dlhs, drhs

  @staticmethod
  def backward(ctx, dout):
    g_in = dout
    dout = dout.to(torch.bfloat16).contiguous()
    # the gradients of partial_sum and existing_out are the incoming gradient itself (ops.py:524-527)
    tail = (None, None, None, None, None, g_in if ctx.has_ps else None, g_in if ctx.has_eo else None, None, None, None, None)
    if ctx.quantized:
      with torch.no_grad():
        dlhs, drhs = _GmmFn._backward_quantized(ctx, dout)
      return (dlhs, drhs) + tail
    lhs, rhs, group_sizes, row_idx, row_inv = ctx.saved_tensors
    dlhs = drhs = None
    ev = PROFILE_EVENTS
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(3)] if ev is not None else None
    with torch.no_grad():
      if marks:
        marks[0].record()
      if ctx.needs_input_grad[0]:
        # dout [m, n] @ rhs[g]^T: the kernel's weight layout [G, out, in] is here [G, k, n]
        dlhs = gmm(dout, rhs, group_sizes, torch.bfloat16, group_offset=ctx.offset, transpose_rhs=not ctx.transpose_rhs)
        # rows of groups outside [offset, offset + G_local) are zero in the forward output
        dlhs = _GmmFn._rows_to_tokens(ctx, dlhs, row_idx, row_inv)
      if marks:
        marks[1].record()
      if ctx.needs_input_grad[1]:
        # with a row index the gathered copy exists for this product only (it is not kept from the forward pass)
        rows = kernels.gather_rows(lhs.contiguous(), row_idx, ctx.row_div) if ctx.has_idx else lhs
        d = tgmm(rows.t(), dout, group_sizes, rhs.dtype, group_offset=ctx.offset, num_actual_groups=rhs.shape[0])
        drhs = d.transpose(1, 2) if ctx.transpose_rhs else d.contiguous()
      if marks:
        marks[2].record()
        shape = f"k{lhs.shape[1]}_n{dout.shape[1]}"
        ev.append(("dlhs_" + shape, marks[0], marks[1]))
        ev.append(("tgmm_" + shape, marks[1], marks[2]))
    return (dlhs, drhs) + tail


def _lib_per_tensor():
  from maxtext_amd import _lib

  return _lib.MOE_SCALE_PER_TENSOR


class _GluFn(torch.autograd.Function):
  """apply_ffn_activation of the expert MLP (moe.py:841-870) on kept projections, with its gradient."""

  @staticmethod
  def forward(ctx, h0, h1, kind, limit):
    ctx.save_for_backward(h0, h1)
    ctx.kind, ctx.limit = kind, limit
    return kernels.glu_act(h0, h1, kind, limit)

  @staticmethod
  def backward(ctx, dout):
    h0, h1 = ctx.saved_tensors
    dh0, dh1 = kernels.glu_act_bwd(h0, h1, dout.contiguous(), ctx.kind, ctx.limit)
    return dh0, dh1, None, None


class _BiasFn(torch.autograd.Function):
  """h + bias[expert of the row] for the differentiable path (the per-expert `mlp_bias` of moe.py:1952-1957, :2239-2242;
  the inference path adds it in the GEMM epilogue).  Rows of groups outside the local shard and rows past the last
  group stay as they are (zero).  The bias gradient is the per-group column sum of the incoming gradient."""

  @staticmethod
  def forward(ctx, h, bias, group_sizes, offset):
    g_local = bias.shape[0]
    ctx.save_for_backward(group_sizes)
    ctx.offset, ctx.g_local, ctx.bias_dtype = offset, g_local, bias.dtype
    return kernels.add_group_bias(h.contiguous(), bias.float().contiguous(), group_sizes, group_offset=offset)

  @staticmethod
  def backward(ctx, dout):
    (group_sizes,) = ctx.saved_tensors
    m, n = dout.shape
    # per-group column sums of dout = the weight gradient of a matmul with a column of ones: the transposed grouped
    # matmul clips group sizes that run past the last row exactly as the forward kernels do, in a fixed order
    if n % 8:
      raise NotImplementedError("the bias gradient needs a multiple of 8 output channels")
    ones = torch.ones((m, 8), dtype=torch.bfloat16, device=dout.device)
    sums = kernels.tgmm(ones, dout.to(torch.bfloat16).contiguous(), group_sizes, num_groups_local=ctx.g_local, group_offset=ctx.offset,
                        out_dtype=torch.float32)  # [G_local, N, 8], every one of the 8 columns holds the sum
    dbias = sums[:, :, 0].to(ctx.bias_dtype)
    return dout, dbias, None, None


def _gmm_with_grad(lhs, rhs, rhs_up, group_sizes, offset, transpose_rhs, rule, manual, fuse_act, act_limit, rhs_bias=None,
                   rhs_up_bias=None, partial_sum=None, partial_sum_up=None, existing_out=None, lhs_row_idx=None, lhs_row_idx_div=1,
                   lhs_row_inv=None, v2=False):
  for name, t in (("lhs", lhs), ("rhs", rhs), ("rhs_up", rhs_up)):
    if t is not None and not isinstance(t, torch.Tensor):
      raise NotImplementedError(f"gradients need bf16 tensors; {name} is already quantised")
  if existing_out is not None and (rhs_up is not None or rhs_bias is not None):
    raise NotImplementedError("existing_out takes the plain product (no rhs_up, no bias) on the differentiable path")
  ps = None if partial_sum is None else partial_sum.to(torch.bfloat16).contiguous()
  ps_up = None if partial_sum_up is None else partial_sum_up.to(torch.bfloat16).contiguous()
  idx = (lhs_row_idx, lhs_row_idx_div, lhs_row_inv)
  h0 = _GmmFn.apply(lhs, rhs, group_sizes, offset, transpose_rhs, rule, manual, ps, existing_out, *idx, v2)
  if rhs_bias is not None:
    h0 = _BiasFn.apply(h0, rhs_bias, group_sizes, offset)
  if rhs_up is None:
    if fuse_act is not None:
      raise ValueError("fuse_act needs rhs_up")
    return h0
  h1 = _GmmFn.apply(lhs, rhs_up, group_sizes, offset, transpose_rhs, rule, manual, ps_up, None, *idx, v2)
  if rhs_up_bias is not None:
    h1 = _BiasFn.apply(h1, rhs_up_bias, group_sizes, offset)
  if fuse_act is None:
    raise ValueError("rhs_up needs fuse_act")
  if fuse_act not in ("silu", "swigluoai", "silu_clip"):
    raise ValueError(f"unknown activation {fuse_act}")
  return _GluFn.apply(h0.contiguous(), h1.contiguous(), fuse_act, act_limit)
