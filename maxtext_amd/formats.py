"""Checkpoint tensor layouts -> the weight layouts moe_gmm reads, without a dequantise / requantise round trip.

Each function takes tensors exactly as they sit in the checkpoint files (any device) and returns
quantizations.QArray objects in the kernels' [G, N, K] layout.  Where the stored bytes already have that
layout the result is a view (zero copy); otherwise the only work is a re-layout of the same bytes.

  DeepSeek-V3 HF fp8     weight [N, K] float8_e4m3fn + weight_scale_inv [N/128, K/128] f32
                         (checkpoint_conversion/standalone_scripts/deepseek_dequantize.py:42-68)
  compressed-tensors i4  weight_packed [N, K/8] int32 + weight_scale [N, K/group] (Kimi-K2 family,
                         convert_deepseek_family_ckpt.py:56-84)
  GPT-OSS HF mxfp4       *_blocks [E, N, K/32, 16] uint8 + *_scales [E, N, K/32] uint8
                         (dequantize_mxfp4.py:46-72; gate/up interleaved: convert_gpt_oss_ckpt.py:269-273)
  AQT serve-mode int8    qvalue [E, K, N] int8 + scale [E, 1, N] (layers/moe.py:1428-1431, :1450-1459)
"""

from __future__ import annotations

from typing import Mapping, Sequence

import torch

from maxtext_amd.quantizations import QArray


def deepseek_fp8_experts(weights: Sequence[torch.Tensor], scale_invs: Sequence[torch.Tensor]) -> QArray:
  """Per-expert `weight` / `weight_scale_inv` pairs -> one fp8 QArray [E, N, K] with [E, ceil(N/128), ceil(K/128)]
  scales.  `weight_scale_inv` is the multiplier of deepseek_dequantize.py:62-68 (w = q * s), i.e. the scale
  the kernel applies; e8m0 (uint8) scales are expanded as 2^(s - 127) (:51-52)."""
  if len(weights) != len(scale_invs) or not weights:
    raise ValueError("need one scale tensor per weight tensor")
  for w, s in zip(weights, scale_invs):
    if w.dtype != torch.float8_e4m3fn or w.dim() != 2 or s.dim() != 2:
      raise ValueError("expected float8_e4m3fn [N, K] weights with 2-D block scales")
    n, k = w.shape
    if tuple(s.shape) != ((n + 127) // 128, (k + 127) // 128):
      raise ValueError(f"scale shape {tuple(s.shape)} does not match 128x128 blocks of {tuple(w.shape)}")
  q = torch.stack(list(weights)).contiguous()
  s = torch.stack([torch.exp2(t.float() - 127.0) if t.dtype == torch.uint8 else t.float() for t in scale_invs]).contiguous()
  return QArray(q, s, "fp8")


def deepseek_fp8_layer(state: Mapping[str, torch.Tensor], layer: int, num_experts: int, prefix: str = "model.layers"):
  """(wi_0, wi_1, wo) of one MoE layer from a DeepSeek-V3 HF state dict: experts.{e}.gate_proj / up_proj / down_proj
  `.weight` + `.weight_scale_inv`."""
  out = []
  for proj in ("gate_proj", "up_proj", "down_proj"):
    names = [f"{prefix}.{layer}.mlp.experts.{e}.{proj}" for e in range(num_experts)]
    out.append(deepseek_fp8_experts([state[n + ".weight"] for n in names], [state[n + ".weight_scale_inv"] for n in names]))
  return tuple(out)


def compressed_int4_experts(packed: Sequence[torch.Tensor], scales: Sequence[torch.Tensor], shapes: Sequence[Sequence[int]],
                            group_size: int = 128) -> QArray:
  """compressed-tensors pack-quantized int4: int32 [N, K/8], weight k of a word in bits [4k, 4k+4), stored value + 8,
  symmetric group scales [N, K/group] (convert_deepseek_family_ckpt.py:56-84).  Read as little-endian bytes this is
  the kernels' packing (two values per byte, first in the low nibble), so the values are a view; the scales are
  cast to bf16.  group_size 128 or 32 (INT4_GROUP_SIZE of the Kimi-K2 variants, convert_deepseek_family_ckpt.py:51-53)."""
  if group_size not in (32, 128):
    raise NotImplementedError(f"int4 group size {group_size}: the kernels apply one scale per 32 or 128 values of K")
  qs, ss = [], []
  for p, s, shape in zip(packed, scales, shapes):
    n, k = int(shape[0]), int(shape[1])
    if p.dtype != torch.int32 or tuple(p.shape) != (n, (k + 7) // 8):
      raise ValueError(f"weight_packed must be int32 [{n}, {(k + 7) // 8}], got {p.dtype} {tuple(p.shape)}")
    if k % 32:
      raise ValueError("K must be a multiple of 32")
    if tuple(s.shape) != (n, (k + group_size - 1) // group_size):
      raise ValueError(f"weight_scale must be [{n}, {(k + group_size - 1) // group_size}]")
    qs.append(p.contiguous().view(torch.uint8)[:, : k // 2])
    ss.append(s.to(torch.bfloat16))
  return QArray(torch.stack(qs).contiguous(), torch.stack(ss).contiguous(), "int4" if group_size == 128 else "int4g32")


def mxfp4_experts(blocks: torch.Tensor, scales: torch.Tensor) -> QArray:
  """`*_blocks` [E, N, K/32, 16] uint8 + `*_scales` [E, N, K/32] uint8 -> mxfp4 QArray (a view: blocks of 16 bytes
  laid end to end are the rows [N, K/2] the kernel reads)."""
  if blocks.dtype != torch.uint8 or scales.dtype != torch.uint8 or blocks.dim() != 4 or blocks.shape[-1] != 16:
    raise ValueError("expected uint8 blocks [E, N, K/32, 16] and uint8 scales [E, N, K/32]")
  if tuple(scales.shape) != tuple(blocks.shape[:3]):
    raise ValueError("scales must have one byte per block")
  e, n, g, _ = blocks.shape
  return QArray(blocks.contiguous().reshape(e, n, g * 16), scales.contiguous(), "mxfp4")


def gpt_oss_mxfp4_layer(gate_up_blocks, gate_up_scales, down_blocks, down_scales, gate_up_bias=None, down_bias=None):
  """GPT-OSS expert tensors -> (wi_0, wi_1, wo[, (w0_bias, w1_bias, wo_bias)]).  Output channels of gate_up_proj are
  interleaved, even = gate (wi_0), odd = up (wi_1) (convert_gpt_oss_ckpt.py:269-276); splitting them is a row
  gather of the stored bytes."""
  wi_0 = mxfp4_experts(gate_up_blocks[:, 0::2], gate_up_scales[:, 0::2])
  wi_1 = mxfp4_experts(gate_up_blocks[:, 1::2], gate_up_scales[:, 1::2])
  wo = mxfp4_experts(down_blocks, down_scales)
  if gate_up_bias is None:
    return wi_0, wi_1, wo
  biases = (gate_up_bias[..., 0::2].float().contiguous(), gate_up_bias[..., 1::2].float().contiguous(),
            None if down_bias is None else down_bias.float().contiguous())
  return wi_0, wi_1, wo, biases


def aqt_int8_experts(qvalue: torch.Tensor, scale: torch.Tensor) -> QArray:
  """AQT serve-mode expert kernel: qvalue [E, K, N] int8 with per-expert, per-output-channel scale [E, 1, N]
  (applied per row in moe.py:1450-1459) -> int8 QArray [E, N, K] with scale [E, N]."""
  if qvalue.dtype != torch.int8 or qvalue.dim() != 3:
    raise ValueError("expected int8 qvalue [E, K, N]")
  e, k, n = qvalue.shape
  if scale.numel() != e * n:
    raise ValueError(f"scale must have E*N = {e * n} elements, got {tuple(scale.shape)}")
  return QArray(qvalue.transpose(1, 2).contiguous(), scale.reshape(e, n).float().contiguous(), "int8")


# ---- readers of checkpoint directories ------------------------------------------------------------------------------


class SafetensorsDir(Mapping):
  """The tensors of a Hugging Face checkpoint directory by name, read one at a time as they are asked for (`safe_open`:
  a memory-mapped read of the tensor's bytes, nothing is unpickled and no shard is loaded whole).  The name -> file map is
  `model.safetensors.index.json` when the directory has one (deepseek_dequantize.py:121-140, dequantize_mxfp4.py:84-100)
  and the key lists of every `*.safetensors` file otherwise (convert_deepseek_family_ckpt.py:315-331,
  convert_gpt_oss_ckpt.py:79-90).  `key_prefix` is stripped from the names (the text branch of a multimodal checkpoint,
  convert_deepseek_family_ckpt.py:320-327)."""

  INDEX = "model.safetensors.index.json"

  def __init__(self, path, key_prefix: str = "", device="cpu"):
    import glob
    import json
    import os

    self.path, self.device, self._prefix = path, str(device), key_prefix
    index = os.path.join(path, self.INDEX)
    if os.path.exists(index):
      with open(index, "r", encoding="utf8") as f:
        raw = json.load(f)["weight_map"]
    else:
      from safetensors import safe_open

      raw = {}
      for file in sorted(glob.glob(os.path.join(path, "[!.]*.safetensors"))):
        with safe_open(file, framework="pt", device="cpu") as f:
          for key in f.keys():
            raw[key] = os.path.basename(file)
      if not raw:
        raise FileNotFoundError(f"no {self.INDEX} and no *.safetensors file in {path}")
    self._files = {k[len(key_prefix):]: (k, v) for k, v in raw.items() if k.startswith(key_prefix)}

  def __getitem__(self, name):
    import os

    from safetensors import safe_open

    raw, file = self._files[name]
    with safe_open(os.path.join(self.path, file), framework="pt", device=self.device) as f:
      return f.get_tensor(raw)

  def __iter__(self):
    return iter(self._files)

  def __len__(self):
    return len(self._files)


def read_deepseek_fp8_layer(path, layer: int, num_experts: int, prefix: str = "model.layers", key_prefix: str = "", device="cpu"):
  """(wi_0, wi_1, wo) of one MoE layer straight from a DeepSeek fp8 checkpoint directory.  The block scales are looked up
  under both names the reference's reader tries: `<name>.weight_scale_inv` (V3) and `<name>.scale` (V4),
  deepseek_dequantize.py:155-175."""
  state = path if isinstance(path, Mapping) else SafetensorsDir(path, key_prefix, device)
  out = []
  for proj in ("gate_proj", "up_proj", "down_proj"):
    ws, ss = [], []
    for e in range(num_experts):
      name = f"{prefix}.{layer}.mlp.experts.{e}.{proj}"
      ws.append(state[name + ".weight"])
      ss.append(state[name + ".weight_scale_inv"] if name + ".weight_scale_inv" in state else state[name + ".scale"])
    out.append(deepseek_fp8_experts(ws, ss))
  return tuple(out)


def read_compressed_int4_layer(path, layer: int, num_experts: int, group_size: int = 32, prefix: str = "model.layers",
                               key_prefix: str = "", device="cpu"):
  """(wi_0, wi_1, wo) of one MoE layer from a compressed-tensors int4 checkpoint directory (Kimi-K2 family):
  `<name>.weight_packed`, `.weight_scale`, `.weight_shape` per expert and projection, the three tensors
  convert_deepseek_family_ckpt.py:343-361 hands to its dequantiser."""
  state = path if isinstance(path, Mapping) else SafetensorsDir(path, key_prefix, device)
  out = []
  for proj in ("gate_proj", "up_proj", "down_proj"):
    names = [f"{prefix}.{layer}.mlp.experts.{e}.{proj}" for e in range(num_experts)]
    out.append(compressed_int4_experts([state[n + ".weight_packed"] for n in names], [state[n + ".weight_scale"] for n in names],
                                       [state[n + ".weight_shape"].tolist() for n in names], group_size))
  return tuple(out)


def read_gpt_oss_mxfp4_layer(path, layer: int, experts: str = "model.layers.{layer}.mlp.experts", key_prefix: str = "", device="cpu"):
  """(wi_0, wi_1, wo, biases) of one GPT-OSS layer from its checkpoint directory: `gate_up_proj_blocks` / `_scales` /
  `_bias` and `down_proj_blocks` / `_scales` / `_bias` under `experts` (the `_blocks` / `_scales` pairs of
  dequantize_mxfp4.py:92-131)."""
  state = path if isinstance(path, Mapping) else SafetensorsDir(path, key_prefix, device)
  base = experts.format(layer=layer)
  get = lambda n: state[f"{base}.{n}"] if f"{base}.{n}" in state else None  # noqa: E731
  return gpt_oss_mxfp4_layer(state[f"{base}.gate_up_proj_blocks"], state[f"{base}.gate_up_proj_scales"], state[f"{base}.down_proj_blocks"],
                             state[f"{base}.down_proj_scales"], get("gate_up_proj_bias"), get("down_proj_bias"))
