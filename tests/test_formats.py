"""Checkpoint-format adapters (host logic, CPU): the bytes they hand to the kernels must dequantise, by the oracle's
restatement of the reference's converters, to what the reference's converters produce from the checkpoint tensors."""

import numpy as np
import pytest
import torch

from maxtext_amd import formats
from oracle import moe_oracle as O


def test_deepseek_fp8_is_zero_copy_and_matches_block_dequant():
  g = torch.Generator().manual_seed(0)
  n, k, e = 256, 384, 3
  ws = [(torch.randn(n, k, generator=g)).to(torch.float8_e4m3fn) for _ in range(e)]
  ss = [torch.rand(n // 128, k // 128, generator=g) * 0.01 + 1e-3 for _ in range(e)]
  qa = formats.deepseek_fp8_experts(ws, ss)
  assert qa.qtype == "fp8" and qa.qvalue.shape == (e, n, k) and qa.scale.shape == (e, 2, 3)
  for i in range(e):
    # deepseek_dequantize.py:62-68: q reshaped into 128x128 blocks times the block's scale
    want = (ws[i].float().reshape(2, 128, 3, 128) * ss[i].reshape(2, 1, 3, 1)).reshape(n, k)
    got = O.dequantize_fp8_blocks(qa.qvalue[i], qa.scale[i], 128)
    assert torch.equal(got, want.to(torch.bfloat16))
  state = {}
  for i in range(e):
    for proj in ("gate_proj", "up_proj", "down_proj"):
      state[f"model.layers.4.mlp.experts.{i}.{proj}.weight"] = ws[i]
      state[f"model.layers.4.mlp.experts.{i}.{proj}.weight_scale_inv"] = ss[i]
  w0, w1, wo = formats.deepseek_fp8_layer(state, 4, e)
  assert torch.equal(w0.qvalue.view(torch.uint8), qa.qvalue.view(torch.uint8)) and torch.equal(wo.scale, qa.scale)
  # e8m0 scales
  qa8 = formats.deepseek_fp8_experts(ws[:1], [torch.tensor([[127, 126, 128], [120, 127, 130]], dtype=torch.uint8)])
  assert qa8.scale[0].tolist() == [[1.0, 0.5, 2.0], [2.0**-7, 1.0, 8.0]]
  with pytest.raises(ValueError):
    formats.deepseek_fp8_experts(ws[:1], [torch.ones(3, 3)])


def test_compressed_int4_bytes_are_the_kernel_packing():
  """The reference's own vectors (tests/unit/dequantize_pack_quantized_int4_test.py:61-100): nibble k of the int32
  is weight k, value = nibble - 8; viewed as bytes that is low-nibble-first pairs."""
  n, k = 4, 256
  rng = np.random.default_rng(0)
  w = rng.integers(-8, 8, (n, k))
  words = np.zeros((n, k // 8), np.int64)
  for j in range(8):
    words |= ((w[:, j::8] + 8) & 0xF) << (4 * j)
  packed = torch.from_numpy(words.astype(np.uint32).view(np.int32).reshape(n, k // 8))
  scale = torch.tensor(rng.random((n, k // 128)) + 0.5, dtype=torch.bfloat16)
  qa = formats.compressed_int4_experts([packed], [scale], [(n, k)])
  assert qa.qtype == "int4" and qa.qvalue.shape == (1, n, k // 2)
  assert np.array_equal(O.unpack_int4(qa.qvalue[0]).numpy(), w)
  want = torch.from_numpy(w).float().reshape(n, k // 128, 128) * scale.float()[..., None]
  assert torch.equal(O.dequantize_int4(qa.qvalue[0], qa.scale[0], 128), want.reshape(n, k).to(torch.bfloat16))
  # the all-ones word of the reference test: nibbles 0xF -> +7 everywhere; zero word -> -8
  ones = torch.full((1, 4), -1, dtype=torch.int32)
  assert torch.all(O.unpack_int4(formats.compressed_int4_experts([ones], [torch.ones(1, 1)], [(1, 32)]).qvalue[0]) == 7)
  with pytest.raises(NotImplementedError):
    formats.compressed_int4_experts([packed], [scale], [(n, k)], group_size=64)
  # group 32 (INT4_GROUP_SIZE of the Kimi-K2 variants, convert_deepseek_family_ckpt.py:51-53)
  scale32 = torch.tensor(rng.random((n, k // 32)) + 0.5, dtype=torch.bfloat16)
  qa32 = formats.compressed_int4_experts([packed], [scale32], [(n, k)], group_size=32)
  assert qa32.qtype == "int4g32" and qa32.scale.shape == (1, n, k // 32)
  want32 = torch.from_numpy(w).float().reshape(n, k // 32, 32) * scale32.float()[..., None]
  assert torch.equal(O.dequantize_int4(qa32.qvalue[0], qa32.scale[0], 32), want32.reshape(n, k).to(torch.bfloat16))


def test_gpt_oss_mxfp4_deinterleave_matches_dequantised_split():
  g = torch.Generator().manual_seed(1)
  e, f, d = 2, 24, 64
  blocks = torch.randint(0, 256, (e, 2 * f, d // 32, 16), generator=g, dtype=torch.uint8)
  scales = torch.randint(120, 132, (e, 2 * f, d // 32), generator=g, dtype=torch.uint8)
  dblocks = torch.randint(0, 256, (e, d, f * 2 // 32 + 1, 16), generator=g, dtype=torch.uint8)
  dscales = torch.randint(120, 132, (e, d, f * 2 // 32 + 1), generator=g, dtype=torch.uint8)
  bias = torch.randn(e, 2 * f, generator=g)
  wi_0, wi_1, wo, (b0, b1, bo) = formats.gpt_oss_mxfp4_layer(blocks, scales, dblocks, dscales, bias, None)
  full = O.dequantize_mxfp4(blocks, scales)  # [e, 2f, d]: what dequantize_mxfp4.py produces before the split
  deq = lambda qa: O.dequantize_mxfp4(qa.qvalue.reshape(qa.qvalue.shape[0], qa.qvalue.shape[1], -1, 16), qa.scale)
  assert torch.equal(deq(wi_0), full[:, 0::2]) and torch.equal(deq(wi_1), full[:, 1::2])  # convert_gpt_oss_ckpt.py:270-271
  assert torch.equal(deq(wo), O.dequantize_mxfp4(dblocks, dscales))
  assert torch.equal(b0, bias[:, 0::2]) and torch.equal(b1, bias[:, 1::2]) and bo is None
  assert wi_0.qtype == "mxfp4" and wi_0.qvalue.shape == (e, f, d // 2) and wi_0.scale.shape == (e, f, d // 32)


def test_aqt_int8_relayout():
  g = torch.Generator().manual_seed(2)
  q = torch.randint(-127, 128, (3, 16, 8), generator=g, dtype=torch.int8)
  s = torch.rand(3, 1, 8, generator=g)
  qa = formats.aqt_int8_experts(q, s)
  assert qa.qvalue.shape == (3, 8, 16) and qa.scale.shape == (3, 8)
  # moe.py:1450-1459: out = ragged_dot(x, qvalue) * scale[expert] per output channel
  x = torch.randn(5, 16, generator=g)
  for ex in range(3):
    want = (x @ q[ex].float()) * s[ex, 0]
    got = (x @ qa.qvalue[ex].float().T) * qa.scale[ex]
    assert torch.allclose(got, want)


def _write_shards(tmp_path, tensors, shards, with_index):
  """Splits `tensors` over `shards` safetensors files the way a Hugging Face checkpoint directory does."""
  import json

  from safetensors.torch import save_file

  names = sorted(tensors)
  weight_map = {}
  for i in range(shards):
    part = {n: tensors[n].contiguous() for n in names[i::shards]}
    file = f"model-{i + 1:05d}-of-{shards:05d}.safetensors"
    save_file(part, str(tmp_path / file))
    weight_map.update({n: file for n in part})
  if with_index:
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"metadata": {}, "weight_map": weight_map}))


@pytest.mark.parametrize("with_index", [True, False])
@pytest.mark.parametrize("v4_names", [False, True])
def test_read_deepseek_fp8_layer_from_a_checkpoint_directory(tmp_path, with_index, v4_names):
  """A sharded fp8 checkpoint directory (index file or bare shards; `weight_scale_inv` or the V4 `scale` name,
  deepseek_dequantize.py:155-175) read tensor by tensor gives the operands the in-memory adapter gives, and they
  dequantise to what deepseek_dequantize.py:42-68 computes."""
  g = torch.Generator().manual_seed(3)
  n, k, e, layer = 256, 128, 4, 5
  tensors, per_proj = {"model.embed_tokens.weight": torch.zeros(8, 4, dtype=torch.bfloat16)}, {}
  for proj in ("gate_proj", "up_proj", "down_proj"):
    for i in range(e):
      w = torch.randn(n, k, generator=g).to(torch.float8_e4m3fn)
      s = torch.rand(n // 128, k // 128, generator=g) * 0.01 + 1e-3
      base = f"model.layers.{layer}.mlp.experts.{i}.{proj}"
      tensors[base + ".weight"] = w
      tensors[base + (".scale" if v4_names else ".weight_scale_inv")] = s
      per_proj.setdefault(proj, []).append((w, s))
  _write_shards(tmp_path, tensors, 3, with_index)
  got = formats.read_deepseek_fp8_layer(str(tmp_path), layer, e)
  for qa, proj in zip(got, ("gate_proj", "up_proj", "down_proj")):
    want = formats.deepseek_fp8_experts([w for w, _ in per_proj[proj]], [s for _, s in per_proj[proj]])
    assert torch.equal(qa.qvalue.view(torch.uint8), want.qvalue.view(torch.uint8)) and torch.equal(qa.scale, want.scale)
    w, s = per_proj[proj][2]
    dense = (w.float().reshape(n // 128, 128, k // 128, 128) * s.reshape(n // 128, 1, k // 128, 1)).reshape(n, k).to(torch.bfloat16)
    assert torch.equal(O.dequantize_fp8_blocks(qa.qvalue[2], qa.scale[2], 128), dense)
  d = formats.SafetensorsDir(str(tmp_path))
  assert len(d) == len(tensors) and "model.embed_tokens.weight" in d and "nope" not in d
  with pytest.raises(KeyError):
    formats.read_deepseek_fp8_layer(str(tmp_path), layer + 1, e)


def test_read_compressed_int4_and_gpt_oss_layers_from_checkpoint_directories(tmp_path):
  """compressed-tensors int4 (weight_packed / weight_scale / weight_shape, convert_deepseek_family_ckpt.py:343-361, under a
  multimodal key prefix) and GPT-OSS blocks / scales / biases (dequantize_mxfp4.py:92-131) read from files equal the
  in-memory adapters on the same tensors."""
  rng = np.random.default_rng(1)
  n, k, e, layer = 8, 64, 2, 3
  i4, packed, scales = {}, {}, {}
  for proj in ("gate_proj", "up_proj", "down_proj"):
    for i in range(e):
      base = f"language_model.model.layers.{layer}.mlp.experts.{i}.{proj}"
      p = torch.from_numpy(rng.integers(-2**31, 2**31, (n, k // 8), dtype=np.int64).astype(np.int32))
      s = torch.tensor(rng.random((n, k // 32)) + 0.5, dtype=torch.bfloat16)
      i4[base + ".weight_packed"], i4[base + ".weight_scale"] = p, s
      i4[base + ".weight_shape"] = torch.tensor([n, k], dtype=torch.int32)
      packed.setdefault(proj, []).append(p)
      scales.setdefault(proj, []).append(s)
  i4["vision_tower.patch_embed.weight"] = torch.zeros(2, 2)
  d4 = tmp_path / "int4"
  d4.mkdir()
  _write_shards(d4, i4, 2, with_index=False)
  got = formats.read_compressed_int4_layer(str(d4), layer, e, group_size=32, key_prefix="language_model.")
  for qa, proj in zip(got, ("gate_proj", "up_proj", "down_proj")):
    want = formats.compressed_int4_experts(packed[proj], scales[proj], [(n, k)] * e, 32)
    assert qa.qtype == "int4g32" and torch.equal(qa.qvalue, want.qvalue) and torch.equal(qa.scale, want.scale)

  ne, f2, d = 3, 16, 64
  oss = {
      f"model.layers.{layer}.mlp.experts.gate_up_proj_blocks": torch.from_numpy(rng.integers(0, 256, (ne, 2 * f2, d // 32, 16), dtype=np.uint8)),
      f"model.layers.{layer}.mlp.experts.gate_up_proj_scales": torch.from_numpy(rng.integers(120, 130, (ne, 2 * f2, d // 32), dtype=np.uint8)),
      f"model.layers.{layer}.mlp.experts.gate_up_proj_bias": torch.randn(ne, 2 * f2).to(torch.bfloat16),
      f"model.layers.{layer}.mlp.experts.down_proj_blocks": torch.from_numpy(rng.integers(0, 256, (ne, d, f2 * 2 // 32, 16), dtype=np.uint8)),
      f"model.layers.{layer}.mlp.experts.down_proj_scales": torch.from_numpy(rng.integers(120, 130, (ne, d, f2 * 2 // 32), dtype=np.uint8)),
      f"model.layers.{layer}.mlp.experts.down_proj_bias": torch.randn(ne, d).to(torch.bfloat16),
  }
  do = tmp_path / "oss"
  do.mkdir()
  _write_shards(do, oss, 2, with_index=True)
  w0, w1, wo, biases = formats.read_gpt_oss_mxfp4_layer(str(do), layer)
  base = f"model.layers.{layer}.mlp.experts."
  x0, x1, xo, xb = formats.gpt_oss_mxfp4_layer(oss[base + "gate_up_proj_blocks"], oss[base + "gate_up_proj_scales"], oss[base + "down_proj_blocks"],
                                               oss[base + "down_proj_scales"], oss[base + "gate_up_proj_bias"], oss[base + "down_proj_bias"])
  for a, b in ((w0, x0), (w1, x1), (wo, xo)):
    assert torch.equal(a.qvalue, b.qvalue) and torch.equal(a.scale, b.scale)
  assert all(torch.equal(a, b) for a, b in zip(biases, xb))
