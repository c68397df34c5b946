"""HIP-graph replay of one MoE layer call for launch-bound shapes (decode, small prefill).

The C ABI neither allocates nor synchronises and never reads `group_sizes` on the host, so a whole
layer call (about a dozen kernels) can be captured once and replayed as a single graph launch.  The
captured call reads its inputs from fixed buffers; `GraphedLayer.__call__` copies the new inputs into
them, replays, and returns the fixed output buffer (valid until the next call).
"""

from __future__ import annotations

import torch


class GraphedLayer:
  """Captures `block.sparse_matmul` for fixed input shapes.

  block: moe.RoutedMoE or moe.RoutedAndSharedMoE (weights are captured by reference: updating them in
  place is seen by later replays).  x: [B, S, d] bf16; gate_logits / pre_bias_logits: [B, S, E] f32, or
  gate_logits=None to capture `block(x)` with the router (gate matmul + top-k) inside the graph.
  """

  def __init__(self, block, x, gate_logits=None, pre_bias_logits=None, warmup: int = 2):
    self.block = block
    self._x = x.clone()
    self._logits = None if gate_logits is None else gate_logits.clone()
    self._pre = None if pre_bias_logits is None else pre_bias_logits.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.no_grad():
      for _ in range(warmup):  # first calls load code objects and size the allocator's pools
        self._run()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    self.graph = torch.cuda.CUDAGraph()
    with torch.no_grad(), torch.cuda.graph(self.graph):
      self._out = self._run()

  def _run(self):
    b = self.block
    if self._logits is None:
      return b(self._x)[0]
    if getattr(b, "routed", None) is not None:
      return b.sparse_matmul(self._x, self._logits, self._pre)[0]
    return b.sparse_matmul(self._x, self._logits, self._pre, b.wi_0, b.wi_1, b.wo)[0]

  def __call__(self, x, gate_logits=None, pre_bias_logits=None):
    if x.shape != self._x.shape:
      raise ValueError(f"captured for x {tuple(self._x.shape)}")
    if (gate_logits is None) != (self._logits is None) or (pre_bias_logits is None) != (self._pre is None):
      raise ValueError("gate_logits / pre_bias_logits must be given exactly when they were given at capture")
    if gate_logits is not None and gate_logits.shape != self._logits.shape:
      raise ValueError(f"captured for logits {tuple(self._logits.shape)}")
    if x.data_ptr() != self._x.data_ptr():
      self._x.copy_(x)
    if gate_logits is not None and gate_logits.data_ptr() != self._logits.data_ptr():
      self._logits.copy_(gate_logits)
    if self._pre is not None and pre_bias_logits.data_ptr() != self._pre.data_ptr():
      self._pre.copy_(pre_bias_logits)
    self.graph.replay()
    return self._out

  @property
  def inputs(self):
    """The fixed input buffers (write into them directly to skip the copies)."""
    return self._x, self._logits, self._pre
