"""Benchmark of the quantized MoE expert path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2]

One step = one pass of the hot path (top-k routing -> sort/permute with activation quantisation
-> fused wi_0/wi_1 grouped GEMM + SwiGLU -> activation quantisation -> wo grouped GEMM ->
unpermute + weighted combine) over one batch of synthetic input that is already resident in HBM.
The default workload is the Mixtral-8x7B-shape int8 prefill layer (8192 tokens, d 4096, f 14336,
8 experts, top-2).  Prints ONE JSON line.
"""

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"int8": 5000.0, "fp8": 5000.0, "bf16": 2500.0}  # dense MFMA, MI355X
PEAK_HBM_GBS = 8000.0

# HBM bytes per launch of the dominant kernel come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs that are made
# offline and summarised in profiles/*.md.  Each summary carries two machine-readable lines,
#   traffic_bytes_per_launch: <bytes>
#   kernel_source_sha256: <hash of the kernel's source files when the counters were read>
# and the figure is reported only while the sources still hash to that value: a kernel that changed since has no
# measured traffic until its profile is refreshed.
PROFILE_OF = {
    "c2": ("profiles/gmm_dls_kernel_int8_mixtral_prefill_c2.md", ["moe_gmm_dls.hip", "moe_gmm_common.h", "moe_common.h"]),
    "c2f8": ("profiles/gmm_dls_kernel_fp8_mixtral_shape_prefill_c2f8.md", ["moe_gmm_dls.hip", "moe_gmm_common.h", "moe_common.h"]),
    "c3": ("profiles/gmm_f8d_kernel_deepseek_decode_c3.md", ["moe_gmm_f8d.hip", "moe_gmm_f8d.h", "moe_gmm_common.h", "moe_common.h"]),
    "c4": ("profiles/gmm_dlw_kernel_int8w_qwen3_prefill_c4.md", ["moe_gmm_dlw.hip", "moe_gmm_common.h", "moe_common.h"]),
    "c5": ("profiles/gmm_dlw_kernel_int4w_gptoss_prefill_c5_t4096.md", ["moe_gmm_dlw.hip", "moe_gmm_common.h", "moe_common.h"]),
    "c2_t16": ("profiles/gmm_f8l_kernel_int8_mixtral_decode_c2_t16.md", ["moe_gmm_f8l.hip", "moe_gmm_f8d.h", "moe_gmm_common.h", "moe_common.h"]),
    "c2_t128": ("profiles/gmm_f8l_kernel_int8_mixtral_decode_c2_t128.md", ["moe_gmm_f8l.hip", "moe_gmm_f8d.h", "moe_gmm_common.h", "moe_common.h"]),
    "c2_train": ("profiles/tgmm_dl_kernel_bf16_mixtral_shape_train.md", ["moe_tgmm.hip", "moe_common.h"]),
    "c2_train_fp8_full": ("profiles/fp8_full_train_step_mixtral_shape.md", ["moe_tgmm.hip", "moe_common.h"]),
}


def kernel_source_hash(files):
  import hashlib

  h = hashlib.sha256()
  for name in files:
    with open(os.path.join(ROOT, "maxtext_amd", "csrc", name), "rb") as fh:
      h.update(name.encode() + b"\0" + fh.read())
  return h.hexdigest()


def measured_traffic(key):
  """(bytes or None, provenance) for the dominant kernel of workload `key` at its default size."""
  import re

  if key not in PROFILE_OF:
    return None, None
  rel, files = PROFILE_OF[key]
  now = kernel_source_hash(files)
  src = {"profile": rel, "kernel_sources": files, "source_sha256_now": now}
  try:
    with open(os.path.join(ROOT, rel)) as fh:
      text = fh.read()
  except OSError:
    return None, dict(src, status="no profile for this kernel")
  m_bytes = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", text, re.M)
  m_hash = re.search(r"^kernel_source_sha256:\s*([0-9a-f]{64})", text, re.M)
  if not m_bytes or not m_hash:
    return None, dict(src, status="profile carries no traffic figure")
  src["source_sha256_profiled"] = m_hash.group(1)
  if m_hash.group(1) != now:
    return None, dict(src, status="kernel source changed since the counters were read")
  return float(m_bytes.group(1)), dict(src, status="counters read on this kernel source")


def parse():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=20)
  ap.add_argument("--warmup", type=int, default=5)
  ap.add_argument("--workload", default=None, choices=["c1", "c2", "c3", "c4", "c5", "c5mx", "c2f8"],
                  help="one workload; by default c2 (the headline line), then c3 (reported under \"secondary\") and c1, c4, c5 (\"other_configs\")")
  ap.add_argument("--source-hash", action="store_true", help="print the kernel source hash that a profile summary of --workload records")
  ap.add_argument("--tokens", type=int, default=None, help="override the token count (c5 sweep)")
  ap.add_argument("--cpu-sample-tokens", type=int, default=None)
  ap.add_argument("--no-cpu-baseline", action="store_true")
  ap.add_argument("--gate", action="store_true",
                  help="include the router in the step: gate matmul + top-k from x (moe_gate_route) instead of given logits")
  ap.add_argument("--graph", action="store_true", help="replay the layer as one captured HIP graph (launch-bound shapes)")
  ap.add_argument("--cold", action="store_true",
                  help="overwrite 1 GiB between steps so that no weights survive in the last-level cache (decode sizes)")
  ap.add_argument("--train", action="store_true",
                  help="forward + backward of the layer with bf16 weights of the workload's shape (weight and input gradients)")
  ap.add_argument("--quant", default="none", choices=["none", "int8", "fp8_full"],
                  help="--train: quantisation of the grouped matmuls: int8 x int8 forward with the quantised backward, or the "
                       "reference's fp8_full recipe (e4m3 operands, e5m2 gradients, layers/quantizations.py:798-855)")
  ap.add_argument("--calibration", default="absmax", help="--train --quant fp8_full: calibration of weights and activations, "
                  "\"absmax\" or \"fixed,-max,max\" (tests/integration/tokamax_test.py:99-101 uses fixed,-224,224)")
  ap.add_argument("--calibrate-copy", action="store_true",
                  help="also run one plain 1 GiB device copy (reference dispatch for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE)")
  return ap.parse_args()


def dominant_kernel_model(wl, group_sizes):
  """Algorithmic work of one launch of the dominant kernel: the fused wi_0/wi_1 grouped GEMM."""
  cfg = wl.cfg
  d, f = cfg.emb_dim, cfg.moe_mlp_dim
  rows = int(group_sizes.sum())
  nonempty = int((group_sizes > 0).sum())
  flops = 4.0 * rows * d * f
  if wl.weight_quant == "fp8" and rows > 14 * len(group_sizes):
    # many rows per expert (prefill): the LDS kernels, bound by the fp8 MFMA rate (the persistent 256 x 256 stream from
    # 128 rows per expert on, the dispatch rule of moe_gmm; 128 x 128 tiles below)
    kernel = "gmm_f8s_kernel" if rows >= 128 * len(group_sizes) and d % 512 == 0 else "gmm_fp8_tiled_kernel"
    return dict(bound="mfma", work=flops, unit="TFLOP/s", peak=PEAK_TFLOPS["fp8"], scale=1e12,
                name=kernel + " (wi_0|wi_1 + SwiGLU)", dtype="fp8")
  if wl.weight_quant == "fp8":
    # HBM bound (decode): weights of the non-empty experts + block scales + activations in + out (the LDS-streamed persistent
    # kernel where moe_gmm gives it the shape: rows of a multiple of 512 values up to 7168)
    w_bytes = nonempty * 2.0 * d * f
    s_bytes = nonempty * 2.0 * (d / 128) * (f / 128) * 4 + rows * (d / 128) * 4
    io_bytes = rows * d * 1.0 + rows * f * 2.0
    return dict(bound="hbm", work=w_bytes + s_bytes + io_bytes, unit="GB/s", peak=PEAK_HBM_GBS, scale=1e9,
                name=("gmm_f8d_kernel" if d % 512 == 0 and d <= 7168 else "gmm_fp8_skinny_kernel") + " (wi_0|wi_1 + SwiGLU)", dtype="fp8")
  if wl.weight_quant in ("int4", "mxfp4") and rows <= 48 * cfg.num_experts:
    # weight-only 4-bit decode (the dispatch rule of moe_gmm for its streaming kernels: group-128 int4 and MXFP4 with rows of
    # up to 3072 values on the LDS-streamed persistent kernel, longer rows on the register-staged one): bound by streaming
    # the weights of the experts that were hit
    w_bytes = nonempty * 2.0 * d * f * 0.5
    s_bytes = nonempty * 2.0 * f * (math.ceil(d / 128) * 2 if wl.weight_quant == "int4" else d / 32)
    io_bytes = rows * d * 2.0 + rows * f * 2.0
    return dict(bound="hbm", work=w_bytes + s_bytes + io_bytes, unit="GB/s", peak=PEAK_HBM_GBS, scale=1e9,
                name=("gmm_wqs_kernel" if d <= 3072 and d % 32 == 0 else "gmm_wq_skinny_kernel") + " (wi_0|wi_1 + SwiGLU)", dtype="bf16")
  op = "int8" if cfg.act_quant == "int8" else "fp8" if cfg.act_quant == "fp8_row" else "bf16"
  if cfg.act_quant in ("int8", "fp8_row") and rows <= 48 * len(group_sizes) and d % 512 == 0:
    # 8-bit x 8-bit with per-row x per-channel scales up to 48 rows per expert (the dispatch rule of moe_gmm): the LDS-streamed
    # persistent kernel, bound by the weights
    w_bytes = nonempty * 2.0 * d * f
    return dict(bound="hbm", work=w_bytes + nonempty * 2.0 * f * 4 + rows * d * 1.0 + rows * f * 2.0, unit="GB/s", peak=PEAK_HBM_GBS, scale=1e9,
                name="gmm_f8l_kernel (wi_0|wi_1 + SwiGLU)", dtype=op)
  # the dispatch rule of moe_gmm for its persistent 256 x 256 kernels: 128 rows per expert on average (104 weight-only)
  if cfg.act_quant in ("int8", "fp8_row") or wl.weight_quant in (None, "bf16"):
    kernel = "gmm_dls_kernel" if rows >= 128 * len(group_sizes) else "gmm_tiled_kernel"
  else:
    # (from 16 rows per expert on: on 128-row tiles up to 112, on 256-row tiles above)
    kernel = "gmm_dlw_kernel" if rows >= 16 * len(group_sizes) and d % 64 == 0 else "gmm_tiled_kernel"
  return dict(bound="mfma", work=flops, unit="TFLOP/s", peak=PEAK_TFLOPS[op], scale=1e12,
              name=kernel + " (wi_0|wi_1 + SwiGLU)", dtype=op)


def cpu_baseline(wl, layer, sample_tokens):
  """The oracle's layer (torch CPU, f32 accumulation) on the first `sample_tokens` tokens of the same
  workload with the same quantised weights: a reported baseline, timed on this host's cores."""
  import torch

  from maxtext_amd import synthetic
  from oracle.layer import oracle_layer

  cfg = wl.cfg
  t = min(sample_tokens, wl.tokens)
  trip = lambda qa: tuple(v.cpu() if hasattr(v, "cpu") else v for v in synthetic.as_triple(qa))
  x = layer["x"][:, :t].cpu()
  logits = layer["gate_logits"][:, :t].cpu()
  pre = None if layer["pre_bias_logits"] is None else layer["pre_bias_logits"][:, :t].cpu()
  w0, w1, wo = trip(layer["wi_0"]), trip(layer["wi_1"]), trip(layer["wo"])
  torch.set_num_threads(max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))))
  t0 = time.perf_counter()
  oracle_layer(x, logits, pre, w0, w1, wo, num_experts=cfg.num_experts, k=cfg.num_experts_per_tok, emb_dim=cfg.emb_dim,
               mlp_dim=cfg.moe_mlp_dim, deepseek=cfg.is_deepseek, routed_scaling_factor=cfg.routed_scaling_factor,
               norm_topk_prob=cfg.norm_topk_prob, shared_experts=cfg.shared_experts, act_quant=cfg.act_quant,
               activation=cfg.activation, acc_dtype=torch.float32)
  dt = time.perf_counter() - t0
  import dataclasses

  flops = synthetic.layer_flops(dataclasses.replace(wl, tokens=t))
  return dict(value=flops / dt / 1e12, unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
              sample=f"first {t} of {wl.tokens} tokens, all experts, same d/f and quantised weights; {dt:.1f} s wall",
              seconds=dt)


def calibration(dtype_name, vendor_gemm_shape=None):
  """What this machine sustains on the two roofs, measured with the library's calibration kernels: a register-only
  MFMA loop (operands constant / changing every instruction: changing data draws more power and lowers the clock)
  and a plain streaming read of 2 GiB.  Reported beside the roofline, whose `peak` stays the published figure."""
  import torch

  import ctypes

  from maxtext_amd import _lib, build

  # the calibration loops live in a library of their own: they are a benchmark aid, not part of the MoE path's ABI
  if not os.path.exists(build.CALIB_LIB_PATH):
    raise RuntimeError(f"{build.CALIB_LIB_PATH} is missing: run `python -m maxtext_amd.build`")
  lib = ctypes.CDLL(build.CALIB_LIB_PATH)
  lib.calib_scratch_bytes.restype = ctypes.c_size_t
  lib.calib_mfma_ops.restype, lib.calib_mfma_ops.argtypes = ctypes.c_double, [ctypes.c_int, ctypes.c_int]
  lib.calib_mfma.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
  lib.calib_read.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p]

  def ok(status, what):
    if status != 0:
      raise RuntimeError(f"{what}: hip error {status}")

  stream = _lib.current_stream()
  scratch = torch.empty((lib.calib_scratch_bytes(),), dtype=torch.uint8, device="cuda")

  def best_ms(fn, reps=3):
    fn()
    torch.cuda.synchronize()
    out = []
    for _ in range(reps):
      a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
      a.record()
      fn()
      b.record()
      torch.cuda.synchronize()
      out.append(a.elapsed_time(b))
    return min(out)

  res = {}
  code = _lib.MOE_INT8 if dtype_name in ("int8", "fp8") else _lib.MOE_BF16
  iters = 4000
  ops = lib.calib_mfma_ops(code, iters)
  for key, rnd in (("mfma_constant_operands", 0), ("mfma_changing_operands", 1)):
    ms = best_ms(lambda: ok(lib.calib_mfma(code, rnd, iters, _lib.ptr(scratch), stream), "calib_mfma"))
    res[key] = ops / ms / 1e9
  res["mfma_unit"] = "TOP/s int8 (v_mfma_i32_16x16x64_i8)" if code == _lib.MOE_INT8 else "TFLOP/s bf16 (v_mfma_f32_16x16x32_bf16)"
  buf = torch.empty((1 << 31,), dtype=torch.uint8, device="cuda")
  buf.fill_(1)
  ms = best_ms(lambda: ok(lib.calib_read(_lib.ptr(buf), buf.numel(), _lib.ptr(scratch), stream), "calib_read"))
  res["hbm_read_gbs"] = buf.numel() / ms / 1e6
  del buf
  if vendor_gemm_shape is not None and code == _lib.MOE_INT8:
    # The vendor library's dense int8 GEMM (hipBLASLt behind torch._int_mm) at the shape of the dominant launch, with no
    # grouping, scales or activation: what a tuned kernel sustains on this box under the same power limit.
    m, k, n = vendor_gemm_shape
    gen = torch.Generator(device="cuda").manual_seed(1)
    a = torch.randint(-127, 128, (m, k), device="cuda", dtype=torch.int8, generator=gen)
    b = torch.randint(-127, 128, (n, k), device="cuda", dtype=torch.int8, generator=gen)
    try:
      ms = best_ms(lambda: torch._int_mm(a, b.t()))
      res["vendor_int8_gemm"] = {"tops": 2.0 * m * k * n / ms / 1e9, "shape_mkn": [m, k, n]}
    except Exception as exc:  # the library may lack a solution for a shape; the figure is only a reference point
      res["vendor_int8_gemm"] = {"error": str(exc)[:120]}
  return res


def train_cpu_baseline(wl, sample_tokens):
  """Forward + backward of the three grouped GEMMs with the oracle's gmm / tgmm (torch CPU, f32 results)
  on `sample_tokens` tokens spread evenly over the experts: a reported baseline."""
  import numpy as np
  import torch

  from oracle import moe_oracle as O

  cfg = wl.cfg
  e, d, f = cfg.num_experts, cfg.emb_dim, cfg.moe_mlp_dim
  m = sample_tokens * cfg.num_experts_per_tok
  gs = np.full((e,), m // e, np.int32)
  m = int(gs.sum())
  g = torch.Generator().manual_seed(0)
  x = torch.randn(m, d, generator=g).to(torch.bfloat16)
  w0, w1 = [(torch.randn(e, d, f, generator=g) * 0.02).to(torch.bfloat16) for _ in range(2)]
  wo = (torch.randn(e, f, d, generator=g) * 0.02).to(torch.bfloat16)
  dy = torch.randn(m, d, generator=g).to(torch.bfloat16)
  torch.set_num_threads(max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))))
  t0 = time.perf_counter()
  h0 = O.gmm(x, w0, gs, out_dtype=torch.float32, acc_dtype=torch.float32)
  h1 = O.gmm(x, w1, gs, out_dtype=torch.float32, acc_dtype=torch.float32)
  a = O.apply_ffn_activation(h0, h1, cfg.activation)
  O.gmm(a, wo, gs, out_dtype=torch.float32, acc_dtype=torch.float32)
  da = O.gmm(dy, wo.transpose(1, 2).contiguous(), gs, out_dtype=torch.bfloat16, acc_dtype=torch.float32)
  O.tgmm(a.float(), dy.float(), gs, out_dtype=torch.float32)
  for w in (w0, w1):
    O.gmm(da, w.transpose(1, 2).contiguous(), gs, out_dtype=torch.bfloat16, acc_dtype=torch.float32)
    O.tgmm(x.float(), da.float(), gs, out_dtype=torch.float32)
  dt = time.perf_counter() - t0
  return dict(value=18.0 * m * d * f / dt / 1e12, unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
              sample=f"{m} routed rows spread evenly over {e} experts, same d/f, bf16 weights, the nine grouped matmuls of "
                     f"forward + backward (activation derivative not included); {dt:.1f} s wall", seconds=dt)


def train_main(args):
  result = train_result(args, args.quant, args.calibration, args.steps, args.warmup)
  result["calibration"] = calibration("bf16")
  if not args.no_cpu_baseline:
    from maxtext_amd import synthetic

    result["cpu_baseline"] = train_cpu_baseline(synthetic.workload(args.workload, args.tokens), args.cpu_sample_tokens or 1024)
  print(json.dumps(result))


def train_result(args, quant, calibration_method, steps, warmup):
  """Forward + backward of the routed layer with bf16 weights: 3 forward GEMMs, 3 input-gradient GEMMs
  (moe_gmm on re-laid-out weights) and 3 weight-gradient launches (moe_tgmm) per step; quant "fp8_full" / "int8": the
  reference's quantised recipe for all nine products.  Returns the fields of the result line."""
  import torch

  from maxtext_amd import _lib, megablox, moe, synthetic

  _lib.load()
  torch.cuda.set_device(0)
  wl = synthetic.workload(args.workload, args.tokens)
  import dataclasses

  cfg = dataclasses.replace(wl.cfg, act_quant="int8" if quant == "int8" else None, shared_experts=0)
  if quant == "fp8_full":
    cfg = dataclasses.replace(cfg, quantization="fp8_full", use_qwix_quantization=True,
                              weight_quantization_calibration_method=calibration_method,
                              act_quantization_calibration_method=calibration_method)
  e, d, f, k, t = cfg.num_experts, cfg.emb_dim, cfg.moe_mlp_dim, cfg.num_experts_per_tok, wl.tokens
  g = torch.Generator(device="cuda").manual_seed(0)
  mk = lambda *shape: (torch.randn(*shape, device="cuda", generator=g) * 0.02).to(torch.bfloat16).requires_grad_()
  w0, w1, wo = mk(e, f, d), mk(e, f, d), mk(e, d, f)
  x = torch.randn(1, t, d, device="cuda", generator=g).to(torch.bfloat16).requires_grad_()
  dout = torch.randn(1, t, d, device="cuda", generator=g).to(torch.bfloat16)
  logits = torch.randn(1, t, e, device="cuda", generator=g)
  pre = torch.sigmoid(logits) if cfg.is_deepseek else None
  block = moe.RoutedMoE(cfg, w0, w1, wo)

  def step():
    for v in (x, w0, w1, wo):
      v.grad = None
    out = block.sparse_matmul(x, logits, pre, w0, w1, wo)[0]
    out.backward(dout)

  for _ in range(warmup):
    step()
  torch.cuda.synchronize()
  megablox.PROFILE_EVENTS = []
  t0 = time.perf_counter()
  for _ in range(steps):
    step()
  torch.cuda.synchronize()
  elapsed = time.perf_counter() - t0
  events, megablox.PROFILE_EVENTS = megablox.PROFILE_EVENTS, None
  stage_ms = {}
  for name in sorted({n for n, _, _ in events}):
    ts = [a.elapsed_time(b) for n, a, b in events if n == name]
    stage_ms[name] = sum(ts) / len(ts)
  m = t * k
  # weight gradient of wi_0 / wi_1: [E, f, d] from x [M, d] and d h [M, f]; of the quantised backward the launch alone (it
  # records its own names), on the MFMA rate of the operands it multiplies
  dom, dom_kernel, dom_peak = f"tgmm_k{d}_n{f}", "tgmm_dl_kernel", PEAK_TFLOPS["bf16"]
  if quant != "none":
    dom = f"tgmm_kernel_k{d}_n{f}"
    if f"tgmm_f8_kernel_k{d}_n{f}" in stage_ms:
      dom, dom_kernel, dom_peak = f"tgmm_f8_kernel_k{d}_n{f}", "tgmm_f8_kernel", PEAK_TFLOPS["fp8"]
  dom_ms = stage_ms[dom]
  achieved = 2.0 * m * d * f / (dom_ms * 1e-3) / 1e12
  flops = 18.0 * m * d * f
  traffic, traffic_source = measured_traffic(wl.name + "_train" + ("_fp8_full" if quant == "fp8_full" else "")) if args.tokens is None else (None, None)
  result = {
      "metric": "moe_bf16_layer_fwd_bwd_tflops", "value": flops / (elapsed / steps) / 1e12, "unit": "TFLOP/s",
      "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": elapsed * 1e3 / steps,
      "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
      "config": {"workload": f"{wl.name} shape, training: forward + backward of the MoE expert layer, {t} tokens, d_model {d}, "
                             f"d_ff {f}, {e} experts top-{k}, bf16 weights and activations, SwiGLU"
                             + ("" if quant == "none" else f", grouped matmuls quantised ({quant}, {calibration_method})"),
                 "tokens": t, "d_model": d, "d_ff": f, "experts": e, "top_k": k, "parallelism": "single GPU"},
      "roofline": dict(bound="mfma", achieved=achieved, peak=dom_peak, unit="TFLOP/s", frac=achieved / dom_peak,
                       traffic=traffic, traffic_source=traffic_source,
                       kernel=dom_kernel + " (weight gradient of wi_0 / wi_1)", kernel_ms=dom_ms),
      "stage_ms": stage_ms,
  }
  del block, w0, w1, wo, x
  torch.cuda.empty_cache()
  return result


def run_workload(args, name, tokens=None):
  """Builds workload `name`, times args.steps steps after args.warmup, returns the fields of its result line."""
  import torch

  from maxtext_amd import moe, synthetic

  wl = synthetic.workload(name, tokens)
  cfg = wl.cfg
  layer = synthetic.make_layer(wl, device="cuda")
  cls = moe.RoutedAndSharedMoE if cfg.shared_experts else moe.RoutedMoE
  block = cls(cfg, layer["wi_0"], layer["wi_1"], layer["wo"])
  routed = block.routed if cfg.shared_experts else block
  x, logits, pre = layer["x"], layer["gate_logits"], layer["pre_bias_logits"]

  if args.gate:
    gen = torch.Generator(device="cuda").manual_seed(5)
    routed.gate_kernel = torch.randn(cfg.emb_dim, cfg.num_experts, device="cuda", generator=gen) * 0.02
    if cfg.is_deepseek:
      routed.gate_bias = torch.randn(cfg.num_experts, device="cuda", generator=gen) * 0.01

  def step():
    if args.gate:
      return block(x)[0]
    if cfg.shared_experts:
      return block.sparse_matmul(x, logits, pre)[0]
    return block.sparse_matmul(x, logits, pre, layer["wi_0"], layer["wi_1"], layer["wo"])[0]

  if args.graph:
    from maxtext_amd import graph as graph_mod

    graphed = graph_mod.GraphedLayer(block, x, None if args.gate else logits, None if args.gate else pre)
    gx, gl, gp = graphed.inputs
    eager_step = step
    step = lambda: graphed(gx, gl, gp)

  for _ in range(args.warmup):
    step()
  torch.cuda.synchronize()

  routed.profile_events = []
  if args.cold:
    # decode-sized weights (C5: 0.4 GB) partly survive in the 256 MB last-level cache from one step to the next;
    # overwriting 1 GiB between steps makes every step start cold.  Steps are timed one by one with events.
    scratch = torch.zeros(1 << 30, dtype=torch.uint8, device="cuda")
    marks = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for a, b in marks:
      scratch.add_(1)
      a.record()
      out = step()
      b.record()
    torch.cuda.synchronize()
    elapsed = sum(a.elapsed_time(b) for a, b in marks) * 1e-3
  else:
    t0 = time.perf_counter()
    for _ in range(args.steps):
      out = step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
  if args.graph:  # per-kernel events cannot be recorded inside a replay: time the same kernels in a few eager steps
    for _ in range(3):
      if args.cold:
        scratch.add_(1)
      eager_step()
    torch.cuda.synchronize()
  events = routed.profile_events
  routed.profile_events = None
  ms_per_step = elapsed * 1e3 / args.steps

  # group sizes of this batch (read back after the timed region) for the algorithmic work model
  _, sel = routed.gate_and_route(x.reshape(-1, cfg.emb_dim)) if args.gate else routed.get_topk(logits, pre)
  gs = torch.bincount(sel.reshape(-1).long(), minlength=cfg.num_experts)
  if cfg.shared_experts:
    gs = torch.cat([gs, torch.tensor([wl.tokens], device=gs.device)])
  gs = gs.cpu().numpy()

  model = dominant_kernel_model(wl, gs)
  stage_ms = {}
  for stage in ("wi_glu", "wo"):
    ts = [a.elapsed_time(b) for (n, a, b) in events if n == stage]
    if ts:
      stage_ms[stage] = sum(ts) / len(ts)
  dom_ms = stage_ms.get("wi_glu")
  achieved = model["work"] / (dom_ms * 1e-3) / model["scale"] if dom_ms else None
  # (a token count other than the configuration's own has counters where a profile of that size is committed)
  traffic, traffic_source = measured_traffic(wl.name if tokens is None else f"{wl.name}_t{tokens}")
  roofline = dict(bound=model["bound"], achieved=achieved, peak=model["peak"], unit=model["unit"],
                  frac=(achieved / model["peak"]) if achieved else None, traffic=traffic, traffic_source=traffic_source,
                  kernel=model["name"], kernel_ms=dom_ms)

  # whole-layer minimum HBM traffic (weights of non-empty experts + activations in/out), for HBM-bound shapes
  nonempty = int((gs > 0).sum())
  min_bytes = nonempty * synthetic.weight_bytes_per_expert(wl) + wl.tokens * cfg.emb_dim * 2 * 2
  res = {
      "value": synthetic.layer_flops(wl) / (elapsed / args.steps) / 1e12,
      "unit": "TFLOP/s",
      "ms_per_step": ms_per_step,
      "dtype": model["dtype"],
      "config": {
          "workload": f"{wl.name}: MoE expert layer, {wl.tokens} tokens, d_model {cfg.emb_dim}, d_ff {cfg.moe_mlp_dim}, "
                      f"{cfg.num_experts} experts top-{cfg.num_experts_per_tok}"
                      f"{' + 1 shared' if cfg.shared_experts else ''}, {wl.weight_quant} weights, "
                      f"{cfg.act_quant or 'bf16'} activations, SwiGLU",
          "tokens": wl.tokens, "d_model": cfg.emb_dim, "d_ff": cfg.moe_mlp_dim, "experts": cfg.num_experts,
          "top_k": cfg.num_experts_per_tok, "parallelism": "single GPU",
      },
      "roofline": roofline,
      "stage_ms": stage_ms,
      "layer_gbps": min_bytes / (elapsed / args.steps) / 1e9,
  }
  vendor_shape = (int(gs.sum()), cfg.emb_dim, 2 * cfg.moe_mlp_dim) if model["dtype"] == "int8" and model["bound"] == "mfma" else None
  return res, wl, layer, model, vendor_shape


def main():
  args = parse()
  if args.source_hash:
    key = (args.workload or "c2") + ("_train" if args.train else "") + ("_fp8_full" if args.train and args.quant == "fp8_full" else "")
    print(kernel_source_hash(PROFILE_OF[key][1]))
    return
  if args.gpus != 1:
    print("bench.py measures one GPU: every box of this build has a single MI355X and the expert path has no "
          "multi-GPU code; run with --gpus 1", file=sys.stderr)
    sys.exit(2)

  import torch

  from maxtext_amd import _lib

  _lib.load()
  if not torch.cuda.is_available():
    print("bench.py needs a GPU", file=sys.stderr)
    sys.exit(2)
  torch.cuda.set_device(0)
  if args.train:
    args.workload = args.workload or "c2"
    return train_main(args)

  # BASELINE's metric names two workloads: the int8 prefill layer (its MFMA half, the headline value) and the fp8
  # decode layer (its HBM half).  With no --workload both run, one after the other, in this process.
  both = args.workload is None
  res, wl, layer, model, vendor_shape = run_workload(args, args.workload or "c2", args.tokens)
  result = {
      "metric": "moe_quant_gmm_layer_tflops",
      "value": res["value"],
      "unit": res["unit"],
      "n_gpus": 1,
      "steps": args.steps,
      "warmup": args.warmup,
      "ms_per_step": res["ms_per_step"],
      "higher_is_better": True,
      "scaling": "weak",
      "vs_baseline": None,
      "dtype": res["dtype"],
      "data": "synthetic",
      "config": res["config"],
      "roofline": res["roofline"],
      "stage_ms": res["stage_ms"],
      "graph": bool(args.graph),
      "cold_cache": bool(args.cold),
      "gate_in_step": bool(args.gate),
      "layer_gbps": res["layer_gbps"],
  }

  if args.calibrate_copy:
    src = torch.ones((1 << 28,), dtype=torch.int32, device="cuda")
    dst = torch.empty_like(src)
    torch.add(src, 1, out=dst)  # reads 1 GiB, writes 1 GiB
    torch.cuda.synchronize()
    del src, dst

  torch.cuda.empty_cache()
  result["calibration"] = calibration(model["dtype"], vendor_shape)
  if not args.no_cpu_baseline:
    sample = args.cpu_sample_tokens or {"c1": 2048, "c2": 8192, "c3": 64, "c4": 8192, "c5": 2048, "c5mx": 2048, "c2f8": 8192}[wl.name]
    result["cpu_baseline"] = cpu_baseline(wl, layer, sample)
  del layer
  torch.cuda.empty_cache()
  if both:
    sec, swl, slayer, smodel, _ = run_workload(args, "c3")
    sec_cpu = None if args.no_cpu_baseline else cpu_baseline(swl, slayer, args.cpu_sample_tokens or 64)
    del slayer
    result["secondary"] = {
        "workload": sec["config"]["workload"], "metric": "moe_quant_gmm_layer_tflops", "value": sec["value"], "unit": sec["unit"],
        "ms_per_step": sec["ms_per_step"], "steps": args.steps, "warmup": args.warmup, "dtype": sec["dtype"],
        "config": sec["config"], "roofline": sec["roofline"], "stage_ms": sec["stage_ms"], "layer_gbps": sec["layer_gbps"],
        "cpu_baseline": sec_cpu,
    }
    # the remaining configurations of the baseline (parity-test cases, not the headline), each timed the same way so
    # that one run records all five
    result["other_configs"] = []
    # (c2f8: the first configuration's shape with the fp8 operands of the fp8_full recipe, per row x per channel scales)
    for name in ("c1", "c4", "c5", "c2f8"):
      torch.cuda.empty_cache()
      o, _, olayer, _, _ = run_workload(args, name)
      del olayer
      result["other_configs"].append({
          "workload": o["config"]["workload"], "value": o["value"], "unit": o["unit"], "ms_per_step": o["ms_per_step"], "dtype": o["dtype"],
          "config": o["config"], "roofline": o["roofline"], "stage_ms": o["stage_ms"], "layer_gbps": o["layer_gbps"],
      })
      if name == "c1":
        # (a layer of 0.07 ms of kernels: issued call by call it is bound by the host's launches, so the same steps are also
        # timed as replays of one captured HIP graph)
        torch.cuda.empty_cache()
        sub = argparse.Namespace(**{**vars(args), "graph": True, "gate": False})
        o, _, olayer, _, _ = run_workload(sub, name)
        del olayer
        result["other_configs"][-1]["graph"] = {"ms_per_step": o["ms_per_step"], "value": o["value"], "unit": o["unit"], "roofline": o["roofline"]}
    # the decode half of the GPT-OSS token sweep (BASELINE's fifth configuration: 1, 16, 128, 1024 tokens; 4096 is the
    # line above): launch-bound sizes, so each is replayed as one captured HIP graph, once as it comes (the 0.4 GB of
    # weights partly live in the last-level cache from one replay to the next) and once with 1 GiB overwritten between
    # steps
    sweep = []
    for tokens in (1, 16, 128, 1024):
      entry = {"tokens": tokens}
      for key, cold in (("graph", False), ("graph_cold", True)):
        torch.cuda.empty_cache()
        sub = argparse.Namespace(**{**vars(args), "graph": True, "cold": cold, "gate": False})
        o, _, olayer, _, _ = run_workload(sub, "c5", tokens)
        del olayer
        entry[key] = {"ms_per_step": o["ms_per_step"], "layer_gbps": o["layer_gbps"], "value": o["value"], "unit": o["unit"],
                      "roofline": o["roofline"], "stage_ms": o["stage_ms"]}
        entry["workload"] = o["config"]["workload"]
      sweep.append(entry)
    result["c5_token_sweep"] = sweep
    # the first configuration at decode sizes (16 and 128 tokens: 4 and 32 rows per expert): 1.4 GB of int8 weights, bound by
    # reading them; issued call by call like the configurations above
    result["c2_decode"] = []
    for tokens in (16, 128):
      torch.cuda.empty_cache()
      o, _, olayer, _, _ = run_workload(args, "c2", tokens)
      del olayer
      result["c2_decode"].append({"tokens": tokens, "workload": o["config"]["workload"], "ms_per_step": o["ms_per_step"], "layer_gbps": o["layer_gbps"],
                                  "value": o["value"], "unit": o["unit"], "roofline": o["roofline"], "stage_ms": o["stage_ms"]})
    # forward + backward of the expert layer at the first configuration's shape, bf16 and the fp8_full recipe (a few steps
    # each; `python bench.py --train [--quant fp8_full]` is the full line with its calibration and CPU baseline)
    result["training"] = []
    for quant in ("none", "fp8_full"):
      torch.cuda.empty_cache()
      sub = argparse.Namespace(**{**vars(args), "workload": "c2", "tokens": None})
      tr = train_result(sub, quant, "absmax", min(args.steps, 5), min(args.warmup, 2))
      result["training"].append({k: tr[k] for k in ("metric", "value", "unit", "ms_per_step", "steps", "warmup", "config", "roofline", "stage_ms")})
  print(json.dumps(result))


if __name__ == "__main__":
  main()
