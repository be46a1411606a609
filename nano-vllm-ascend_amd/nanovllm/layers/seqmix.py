"""Layer classes of the 32-bit-residual model families (kernels: csrc/gemm_any.hip, csrc/seqmix.hip).

Each class is one mechanism with its constants as constructor arguments, so that a model file only wires them by its
configuration:

  OutputLayerNorm           LayerNorm (weight + bias) applied to a sublayer's OUTPUT and added to the residual
  SlidingWindowAttention    paged sliding-window attention, linear distance bias per head, whole-projection q / k RMS norm,
                            optional value mixing with an earlier layer's values, sigmoid output gate
  ChannelDeltaMixer         gated delta rule with a decay per head and key channel behind short causal convolutions;
                            recurrent state and convolution tail live in per-sequence state slots
  GroupedSparseMLP          sparse mixture of SwiGLU experts, group-limited top-k routing with a choice correction,
                            un-renormalised weights, identity experts

Activations are fp32 tensors [rows, features]; matrices are stored in the serving dtype (bf16, or fp32 for the exact
mode), vectors always in fp32.  A step's rows come with the metadata of utils/context.py: cu_seqlens_q, kv_lens (the
sequences' lengths INCLUDING this step's rows), slot_mapping, block_tables, state_slots.  Prompt portions and single
decoded tokens are the same thing to every kernel here: a run of rows that continues a sequence.
"""
from __future__ import annotations

import torch
from torch import nn

from nanovllm import ops
from nanovllm.utils.context import get_context


def _vector(n: int, fill: float = 0.0) -> nn.Parameter:
    return nn.Parameter(torch.full((n,), fill, dtype=torch.float32), requires_grad=False)


def _matrix(*shape) -> nn.Parameter:
    return nn.Parameter(torch.empty(*shape), requires_grad=False)  # (the default dtype = the serving dtype)


class MergedRows(nn.Module):
    """Several projections of the same input stacked along their output features (one GEMM instead of several); a
    checkpoint's separate tensors land in their row ranges through `weight_loader(param, tensor, shard_name)`."""

    def __init__(self, in_features: int, parts: dict[str, int], dtype=None):
        super().__init__()
        self.offsets, off = {}, 0
        for name, n in parts.items():
            self.offsets[name] = (off, n)
            off += n
        self.weight = nn.Parameter(torch.empty(off, in_features, dtype=dtype), requires_grad=False)
        self.weight.weight_loader = self._load

    def _load(self, param, tensor, shard):
        off, n = self.offsets[shard]
        assert tensor.shape[0] == n, (shard, tuple(tensor.shape), n)
        param.data[off:off + n].copy_(tensor)

    def cols(self, y: torch.Tensor, name: str) -> torch.Tensor:
        off, n = self.offsets[name]
        return y[:, off:off + n]

    def forward(self, x: torch.Tensor, exact: bool = False) -> torch.Tensor:
        return ops.gemm_any(x, self.weight, exact=exact)


class OutputLayerNorm(nn.Module):
    def __init__(self, width: int, eps: float):
        super().__init__()
        self.eps = eps
        self.weight, self.bias = _vector(width, 1.0), _vector(width)

    def add_to(self, residual: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
        """residual += LN(y), in place."""
        return ops.layernorm_f32(y, self.weight, self.bias, self.eps, add_to=residual)

    def forward(self, y: torch.Tensor) -> torch.Tensor:
        return ops.layernorm_f32(y, self.weight, self.bias, self.eps)


class SlidingWindowAttention(nn.Module):
    """mixes_values: "first" (this layer's values are what later layers mix in), "later" (mixes them in with its
    own coefficient) or None."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, window: int, scale: float, eps: float,
                 mixes_values: str | None = None):
        super().__init__()
        assert heads % kv_heads == 0
        self.H, self.G, self.D, self.Dv, self.window, self.scale, self.eps = heads, kv_heads, dim, vdim, window, scale, eps
        self.mixes_values = mixes_values
        self.qkvg = MergedRows(width, {"q": heads * dim, "k": kv_heads * dim, "v": kv_heads * vdim, "g": heads * vdim})
        self.q_norm, self.k_norm = _vector(heads * dim, 1.0), _vector(kv_heads * dim, 1.0)
        self.vmix = _vector(1)
        self.o = _matrix(width, heads * vdim)
        self.k_cache = self.v_cache = torch.tensor([])

    def cache_shapes(self, num_blocks: int, block_size: int):
        return (num_blocks, self.G, block_size, self.D), (num_blocks, self.G, block_size, self.Dv)

    def forward(self, x: torch.Tensor, v_first: torch.Tensor | None):
        ctx, m = get_context(), self.qkvg
        y = m(x)
        (qo, _), (ko, _), (vo, nv), (go, _) = m.offsets["q"], m.offsets["k"], m.offsets["v"], m.offsets["g"]
        mix_in = v_first if self.mixes_values == "later" else None
        ops.swa_prepare(y, qo, ko, vo, self.q_norm, self.k_norm, self.eps, mix_in, self.vmix if mix_in is not None else None,
                        self.k_cache, self.v_cache, ctx.slot_mapping, self.H, self.G, self.D, self.Dv, ctx.block_size)
        o = ops.swa_attention(m.cols(y, "q"), self.k_cache, self.v_cache, ctx.block_tables, ctx.cu_seqlens_q, ctx.kv_lens,
                              self.H, self.G, self.D, self.Dv, ctx.block_size, self.window, self.scale,
                              gate=m.cols(y, "g"))
        return ops.gemm_any(o, self.o), (y[:, vo:vo + nv] if self.mixes_values == "first" else v_first)


class ChannelDeltaMixer(nn.Module):
    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, taps: int, decay_rank: int,
                 gate_rank: int, eps: float):
        super().__init__()
        assert heads % kv_heads == 0
        self.H, self.G, self.D, self.Dv, self.taps, self.eps = heads, kv_heads, dim, vdim, taps, eps
        parts = {"q": kv_heads * dim, "k": kv_heads * dim, "v": heads * vdim}
        self.qkv = MergedRows(width, parts)
        self.conv = MergedRows(taps, parts, dtype=torch.float32)  # [channels, taps]: per-channel filters, same row ranges
        self.low = MergedRows(width, {"a1": decay_rank, "g1": gate_rank, "b": heads})
        self.a2, self.g2 = _matrix(heads * dim, decay_rank), _matrix(heads * vdim, gate_rank)
        self.dt_bias, self.A_log, self.norm = _vector(heads * dim), _vector(heads), _vector(vdim, 1.0)
        self.o = _matrix(width, heads * vdim)
        self.state = self.conv_state = torch.tensor([])

    def state_shapes(self, n_slots: int):
        return ((n_slots, ops.channel_delta_state_elems(self.H, self.D, self.Dv)),
                (n_slots, max(self.taps - 1, 1), self.qkv.weight.shape[0]))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        cu, kv, slots = ctx.cu_seqlens_q, ctx.kv_lens, ctx.state_slots
        pre = self.qkv(x)
        qkv = ops.causal_conv_silu(pre, self.conv.weight, self.conv_state, cu, kv, slots)
        ops.causal_conv_state(pre, self.taps, self.conv_state, cu, kv, slots)
        low = self.low(x)
        decay_pre = ops.gemm_any(self.low.cols(low, "a1"), self.a2)
        gate_pre = ops.gemm_any(self.low.cols(low, "g1"), self.g2)
        off = self.qkv.offsets
        o = ops.channel_delta(qkv, off["q"][0], off["k"][0], off["v"][0], self.low.cols(low, "b"), decay_pre, self.dt_bias,
                              self.A_log, gate_pre, self.norm, self.state, cu, kv, slots, self.H, self.G, self.D, self.Dv,
                              self.eps)
        return ops.gemm_any(o, self.o)


class GroupedSparseMLP(nn.Module):
    def __init__(self, width: int, ff: int, experts: int, identity: int, top_k: int, groups: int, keep: int):
        super().__init__()
        self.E, self.n_out, self.top_k, self.groups, self.keep = experts, experts + identity, top_k, groups, keep
        assert self.n_out % groups == 0 and 1 <= keep <= groups and top_k <= keep * (self.n_out // groups)
        self.router = _matrix(self.n_out, width)
        self.correction = _vector(self.n_out)
        self.gate, self.up, self.down = _matrix(experts, ff, width), _matrix(experts, ff, width), _matrix(experts, width, ff)
        for p in (self.gate, self.up, self.down):
            p.weight_loader = lambda param, tensor, expert: param.data[expert].copy_(tensor)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        z = ops.gemm_any(x, self.router, exact=True)  # router logits in true 32-bit in every serving mode
        ids, wts = ops.route_grouped(z, self.correction, self.top_k, self.groups, self.keep)
        offsets, pair_token, pair_index = ops.moe_sort(ids, self.n_out)
        P = ids.numel()
        act = ops.gemm_any_grouped(x, pair_token, self.gate, self.up, offsets, P, None, P)
        y = ops.gemm_any_grouped(act, None, self.down, None, offsets, P, pair_index, P)
        return ops.moe_combine_f32(y, x, ids, wts, self.E)
