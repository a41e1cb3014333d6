"""Whole decoder layers with the constructor and ``forward`` of the reference's
benchmark layers, for like-for-like whole-layer throughput runs.

``BlockTopkDecoderLayer`` mirrors benchmark/blocktopk_decoder.py:96-240 and
``DenseDecoderLayer`` mirrors benchmark/dense_decoder.py: RMSNorm -> fused
``wqkv`` -> q/k RMSNorm -> [append, page scoring, top-k, attention] -> ``wo`` ->
residual -> RMSNorm -> SwiGLU MLP -> residual, for one tensor-parallel shard
(head counts and MLP width divided by ``world_size``, as the reference does at
:101-106).  Everything except the GEMMs runs on the HIP kernels of this
package: the RMSNorms (the reference calls flashinfer's through its layer_norm
and qk_norm ops, benchmark/model_utils.py:4-25) with the first residual add
folded in, the q/k norm + split of the fused projection, the attention path,
and the gated activation.  The GEMMs are hipBLASLt through PyTorch; the gate and
up projections run as one GEMM over their stacked weights, and the last
residual add rides on the down projection (``addmm``).

The reference reads the model shape from the Hugging Face hub
(benchmark/blocktopk.py:65); ``qwen3_config`` provides the same fields offline.
"""
from __future__ import annotations

import math
from types import SimpleNamespace

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops
from .blocktopk_decoder import BlockTopkPagedAttention, DensePagedAttention

# Published Qwen3 shapes (general knowledge; the reference fetches them from the hub).
_QWEN3 = {
    "Qwen3-0.6B": dict(hidden_size=1024, intermediate_size=3072, num_attention_heads=16, num_key_value_heads=8, num_hidden_layers=28),
    "Qwen3-1.7B": dict(hidden_size=2048, intermediate_size=6144, num_attention_heads=16, num_key_value_heads=8, num_hidden_layers=28),
    "Qwen3-4B": dict(hidden_size=2560, intermediate_size=9728, num_attention_heads=32, num_key_value_heads=8, num_hidden_layers=36),
    "Qwen3-8B": dict(hidden_size=4096, intermediate_size=12288, num_attention_heads=32, num_key_value_heads=8, num_hidden_layers=36),
    "Qwen3-14B": dict(hidden_size=5120, intermediate_size=17408, num_attention_heads=40, num_key_value_heads=8, num_hidden_layers=40),
    "Qwen3-32B": dict(hidden_size=5120, intermediate_size=25600, num_attention_heads=64, num_key_value_heads=8, num_hidden_layers=64),
}

_ACT = ("silu", "gelu", "relu")


def qwen3_config(name: str) -> SimpleNamespace:
    """The config fields the layers read (benchmark/blocktopk_decoder.py:101-121)."""
    key = name.split("/")[-1]
    if key not in _QWEN3:
        raise KeyError(f"unknown model {name!r}; known: {sorted(_QWEN3)}")
    return SimpleNamespace(head_dim=128, rms_norm_eps=1e-6, hidden_act="silu", max_position_embeddings=40960,
                           rope_theta=1000000.0, eos_token_id=151645, **_QWEN3[key])


def rms_norm(x: torch.Tensor, eps: float, weight: torch.Tensor) -> torch.Tensor:
    """RMSNorm over the last dimension with fp32 statistics, argument order of the
    reference's layer_norm / qk_norm (benchmark/model_utils.py:4-25)."""
    return ops.rms_norm(x, weight, eps)


def init_weights(m):
    """benchmark/blocktopk_decoder.py:88-94."""
    if isinstance(m, nn.Linear):
        nn.init.kaiming_uniform_(m.weight, a=math.sqrt(5))
        if m.bias is not None:
            fan_in, _ = nn.init._calculate_fan_in_and_fan_out(m.weight)
            bound = 1 / math.sqrt(fan_in)
            nn.init.uniform_(m.bias, -bound, bound)


class _LayerBase(nn.Module):
    def __init__(self, config, world_size, batch_size, device, dtype):
        super().__init__()
        self.num_heads = config.num_attention_heads // world_size
        self.num_kv_heads = config.num_key_value_heads // world_size
        if self.num_heads < 1 or self.num_kv_heads < 1:
            raise ValueError("world_size exceeds the number of heads")
        self.num_key_value_groups = self.num_heads // self.num_kv_heads
        self.head_dim = config.head_dim
        self.dim = config.hidden_size
        self.intermediate_size = config.intermediate_size // world_size
        self.eps = config.rms_norm_eps
        if config.hidden_act not in _ACT:
            raise ValueError(f"hidden_act {config.hidden_act!r} is not one of {_ACT}")
        self.activation = config.hidden_act
        self.batch_size = batch_size

        self.qnorm_weight = nn.Parameter(torch.ones(self.head_dim))
        self.knorm_weight = nn.Parameter(torch.ones(self.head_dim))
        self.input_layernorm_weight = nn.Parameter(torch.ones(self.dim))
        self.post_attention_layernorm_weight = nn.Parameter(torch.ones(self.dim))
        total_head_dim = (self.num_heads + 2 * self.num_kv_heads) * self.head_dim
        self.wqkv = nn.Linear(self.dim, total_head_dim, bias=True)
        self.wo = nn.Linear(self.head_dim * self.num_heads, self.dim, bias=False)
        self.up_proj = nn.Linear(self.dim, self.intermediate_size, bias=False)
        self.gate_proj = nn.Linear(self.dim, self.intermediate_size, bias=False)
        self.down_proj = nn.Linear(self.intermediate_size, self.dim, bias=False)
        self._gate_up = None

    def _gate_up_weight(self) -> torch.Tensor:
        """[2 * intermediate, hidden]: gate_proj over up_proj.  Built on first use
        (``prepare_wrapper`` or the first forward; again after the module moved or
        changed dtype); the two parameters then become views of it, so no weight
        is held twice and loading a state dict into them keeps filling the stacked
        tensor."""
        w = self._gate_up
        if w is None:
            g, u = self.gate_proj.weight, self.up_proj.weight
            n = self.intermediate_size
            w = torch.cat([g.data, u.data], dim=0)
            g.data, u.data = w[:n], w[n:]
            self._gate_up = w
        return w

    def _apply(self, fn, recurse=True):
        # .to() / .cuda() / .half() replace the parameters: the stacked weight is rebuilt on next use
        self._gate_up = None
        return super()._apply(fn, recurse)

    def graphed(self, example_hidden_states: torch.Tensor) -> GraphedLayer:
        """This layer's forward as one replayable HIP graph (see GraphedLayer)."""
        return GraphedLayer(self, example_hidden_states)

    def _qkv(self, hidden_states):
        """benchmark/blocktopk_decoder.py:192-207: norm, fused projection, split, q/k norm."""
        bsz, q_len, _ = hidden_states.size()
        if q_len != 1:
            raise ValueError("decode layers take one token per sequence")
        x = torch.ops.kinetics.layer_norm(hidden_states, self.eps, self.input_layernorm_weight)
        qkv = self.wqkv(x).view(bsz, -1)
        return torch.ops.kinetics.qkv_norm_split(qkv, self.qnorm_weight, self.knorm_weight, self.eps, self.num_heads,
                                                 self.num_kv_heads)

    def _finish(self, residual, o):
        """benchmark/blocktopk_decoder.py:226-240: wo, residual, norm, SwiGLU MLP, residual."""
        bsz = o.shape[0]
        # h = residual + wo(o), written over the projection's own output (the layer
        # input stays untouched), and x = norm(h) in the same pass
        h = self.wo(o.reshape(bsz, self.head_dim * self.num_heads))
        x = torch.ops.kinetics.fused_layer_norm(residual.reshape(bsz, self.dim), h, self.eps,
                                                self.post_attention_layernorm_weight)
        n = self.intermediate_size
        gate_up = F.linear(x, self._gate_up_weight())
        y = torch.ops.kinetics.gated_act(gate_up[:, :n], gate_up[:, n:], self.activation)
        return torch.addmm(h, y, self.down_proj.weight.t()).view(bsz, 1, self.dim)


class GraphedLayer:
    """A layer's ``forward`` recorded once as a HIP graph and replayed per step:
    one submission instead of a dozen launches.  This is the launch-overhead half
    of what the reference gets from ``torch.compile(mode="max-autotune")``
    (benchmark/blocktopk.py:41-43); the kernels are the same as in eager mode.
    Input and output live in fixed buffers: ``__call__`` copies ``hidden_states``
    in and returns the graph's own output tensor, which the next call overwrites."""

    def __init__(self, layer, example: torch.Tensor, warmup: int = 3):
        self.layer = layer
        self.static_in = example.clone()
        side = torch.cuda.Stream(device=example.device)
        side.wait_stream(torch.cuda.current_stream(example.device))
        with torch.cuda.stream(side):
            for _ in range(warmup):  # first-use work (stacked weights, GEMM plans) stays outside the graph
                layer(self.static_in)
        torch.cuda.current_stream(example.device).wait_stream(side)
        torch.cuda.synchronize(example.device)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.static_out = layer(self.static_in)

    def __call__(self, hidden_states: torch.Tensor) -> torch.Tensor:
        self.static_in.copy_(hidden_states)
        self.graph.replay()
        return self.static_out


class BlockTopkDecoderLayer(_LayerBase):
    """Constructor arguments as benchmark/blocktopk_decoder.py:97-99."""

    def __init__(self, config, world_size, batch_size, prefix_len, max_len, page_size, topk_page, device, dtype, seed: int = 0):
        super().__init__(config, world_size, batch_size, device, dtype)
        self.attn = BlockTopkPagedAttention(self.num_heads, self.num_kv_heads, self.head_dim, batch_size, prefix_len, max_len,
                                            page_size, topk_page, device=device, dtype=dtype, seed=seed)

    def prepare_wrapper(self, prefix_len=None, topk_page_indices=None):
        """Present for call compatibility (benchmark/blocktopk_decoder.py:243-265): the
        HIP kernels need no planning step.  Stacks the gate/up weights, so that a
        compiled forward finds them in place."""
        self._gate_up_weight()
        return None

    # no_grad where the reference has inference_mode (benchmark/blocktopk_decoder.py:186): with
    # inference mode on, AOT functionalisation cannot wrap an op result that is a view of an
    # intermediate it never saw (nn.Linear on a 3-D input returns one), so the layer would not
    # compile beyond Dynamo's tracing.
    @torch.no_grad()
    def forward(self, hidden_states):
        q, k, v = self._qkv(hidden_states)
        o = self.attn(q, k, v)
        return self._finish(hidden_states, o)


class DenseDecoderLayer(_LayerBase):
    """The dense baseline layer (benchmark/dense_decoder.py)."""

    def __init__(self, config, world_size, batch_size, prefix_len, max_len, page_size, device, dtype, seed: int = 0):
        super().__init__(config, world_size, batch_size, device, dtype)
        self.attn = DensePagedAttention(self.num_heads, self.num_kv_heads, self.head_dim, batch_size, prefix_len, max_len,
                                        page_size, device=device, dtype=dtype, seed=seed)

    def prepare_wrapper(self):
        self._gate_up_weight()
        return None

    @torch.no_grad()  # see BlockTopkDecoderLayer.forward
    def forward(self, hidden_states):
        q, k, v = self._qkv(hidden_states)
        o = self.attn(q, k, v)
        return self._finish(hidden_states, o)
