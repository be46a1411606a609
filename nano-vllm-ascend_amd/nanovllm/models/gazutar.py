"""Gazutar: a decoder whose layers alternate, in an order its configuration lists, between sliding-window attention
with a linear distance bias and a channel-wise gated delta rule, each followed by a group-routed sparse feed-forward;
LayerNorm sits on every sublayer's OUTPUT (x <- x + LN(f(x))), the residual stream is fp32.

The mechanisms are the classes of layers/seqmix.py; this file reads the configuration, wires the layers, names the
checkpoint's tensors and says what cache and state a sequence needs:

  config.json   {"architecture": "Gazutar", "vocab", "width", "logit_scale", "norm": {"eps"}, "layers": [{"type":
                "attention" | "channel_delta", "mixer": {...}, "mlp": {...} | null}, ...]}
  checkpoint    embed, head, final.norm(.b), l<i>.norm1(.b), l<i>.norm2(.b), l<i>.mix.<name>, l<i>.mlp.<name>;
                sizes that the configuration does not give (the ranks of the low-rank decay and gate projections)
                are read from the checkpoint's header
  per sequence  K / V pages of every attention layer (key and value head sizes differ) and, for every channel_delta
                layer, one state slot: the fp32 state [heads, dim, vdim] and the convolution's last taps - 1 inputs
"""
from __future__ import annotations

import json
import os
import struct

import torch
from torch import nn

from nanovllm import ops
from nanovllm.layers.seqmix import ChannelDeltaMixer, GroupedSparseMLP, OutputLayerNorm, SlidingWindowAttention


def safetensors_shapes(path: str) -> dict[str, tuple]:
    """name -> shape from a safetensors header (8-byte little-endian length, then that many bytes of JSON)."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
    return {k: tuple(v["shape"]) for k, v in header.items() if k != "__metadata__"}


class GazutarConfig:
    """config.json of this design with the attribute names the engine reads from a configuration object."""
    architectures = ["Gazutar"]
    model_type = "gazutar"
    max_position_embeddings = None   # no position table: positions enter through distances only
    eos_token_id = None
    native = True                    # not a transformers configuration

    def __init__(self, raw: dict, tensor_shapes: dict | None = None, dtype: str = "bfloat16"):
        self.raw = raw
        self.vocab_size, self.hidden_size = int(raw["vocab"]), int(raw["width"])
        self.layers = raw["layers"]
        self.num_hidden_layers = len(self.layers)
        self.norm_eps = float(raw["norm"]["eps"])
        self.logit_scale = float(raw.get("logit_scale", 1.0))
        self.tensor_shapes = tensor_shapes or {}
        self.torch_dtype = dtype

    @classmethod
    def from_dir(cls, path: str, dtype: str = "bfloat16") -> "GazutarConfig":
        with open(os.path.join(path, "config.json")) as f:
            raw = json.load(f)
        ckpt = os.path.join(path, "model.safetensors")
        return cls(raw, safetensors_shapes(ckpt) if os.path.exists(ckpt) else None, dtype)

    def rank_of(self, layer: int, name: str, mixer: dict) -> int:
        shape = self.tensor_shapes.get(f"l{layer}.mix.{name}")
        if shape is not None:
            return int(shape[0])
        return int(mixer.get("rank", max(8, self.hidden_size // 8)))  # synthetic weights only


class GazutarLayer(nn.Module):
    def __init__(self, cfg: GazutarConfig, index: int, value_mixing: str | None):
        super().__init__()
        spec, W, eps = cfg.layers[index], cfg.hidden_size, cfg.norm_eps
        m = spec["mixer"]
        self.kind = spec["type"]
        if self.kind == "attention":
            self.mix = SlidingWindowAttention(W, m["heads"], m["kv_heads"], m["dim"], m["vdim"], int(m["mask"]["size"]),
                                              float(m["scale"]), eps, value_mixing)
        elif self.kind == "channel_delta":
            self.mix = ChannelDeltaMixer(W, m["heads"], m["kv_heads"], m["dim"], m["vdim"], int(m["conv"]),
                                         cfg.rank_of(index, "a1", m), cfg.rank_of(index, "g1", m), eps)
        else:
            raise NotImplementedError(f"layer {index}: mixer type {self.kind!r}")
        self.norm1 = OutputLayerNorm(W, eps)
        ml = spec.get("mlp")
        self.mlp = self.norm2 = None
        if ml is not None:
            if ml.get("kind", "moe") != "moe":
                raise NotImplementedError(f"layer {index}: feed-forward kind {ml.get('kind')!r}")
            r = ml["router"]
            g = r.get("groups") or {"count": 1, "keep": 1}
            self.mlp = GroupedSparseMLP(W, int(ml["expert"]["ff"]), int(r["experts"]), int(r.get("identity", 0)),
                                        int(r["top"]), int(g["count"]), int(g["keep"]))
            self.norm2 = OutputLayerNorm(W, eps)


class GazutarForCausalLM(nn.Module):
    hybrid_state = True   # sequences own recurrent-state slots beside their K/V pages: ModelRunner takes the row-step path
    fp32_residual = True

    def __init__(self, config: GazutarConfig):
        super().__init__()
        self.config = config
        W, V = config.hidden_size, config.vocab_size
        self.embed = nn.Parameter(torch.empty(V, W), requires_grad=False)
        seen_mixing, layers = False, []
        for i, spec in enumerate(config.layers):
            mixing = None
            if spec["type"] == "attention" and spec["mixer"].get("v_mix"):
                mixing = "later" if seen_mixing else "first"
                seen_mixing = True
            layers.append(GazutarLayer(config, i, mixing))
        self.layers = nn.ModuleList(layers)
        self.final_norm = OutputLayerNorm(W, config.norm_eps)
        self.head = nn.Parameter(torch.empty(V, W), requires_grad=False)
        self.trace_layers: list | None = None  # bring-up hook: receives a copy of the residual stream after every layer

    # ---- checkpoint names -> parameters (utils/loader.py) ------------------------------------------------------
    def map_checkpoint_name(self, name: str):
        """-> parameter path, (parameter path, shard) for tensors that land inside a merged / stacked parameter, or None
        for a tensor this configuration has no use for."""
        if name in ("embed", "head"):
            return name
        if name.startswith("final.norm"):
            return "final_norm.bias" if name.endswith(".b") else "final_norm.weight"
        layer, rest = name.split(".", 1)
        i = int(layer[1:])
        pre = f"layers.{i}."
        if rest.startswith("norm"):
            if rest.startswith("norm2") and self.layers[i].mlp is None:
                return None  # (a layer without feed-forward has no second norm: a tensor of that name is ignored)
            return pre + (rest[:-2] + ".bias" if rest.endswith(".b") else rest + ".weight")
        part, leaf = rest.split(".", 1)
        if part == "mlp":
            if leaf in ("router", "correction"):
                return pre + "mlp." + leaf
            expert, proj = leaf.split(".")
            return pre + "mlp." + proj, int(expert[1:])
        if self.layers[i].kind == "attention":
            if leaf in ("q", "k", "v", "g"):
                return pre + "mix.qkvg.weight", leaf
            return pre + "mix." + {"q.norm": "q_norm", "k.norm": "k_norm", "vmix": "vmix", "o": "o"}[leaf]
        if leaf in ("q", "k", "v"):
            return pre + "mix.qkv.weight", leaf
        if leaf.endswith(".conv"):
            return pre + "mix.conv.weight", leaf[0]
        if leaf in ("a1", "g1", "b"):
            return pre + "mix.low.weight", leaf
        return pre + "mix." + leaf  # a2, g2, dt_bias, A_log, norm, o

    def synthetic_state(self, seed: int = 0):
        """Random tensors under the checkpoint's names (no-checkpoint mode: benchmarks)."""
        g = torch.Generator().manual_seed(seed)
        cfg, W = self.config, self.config.hidden_size
        def mat(*shape, std=None):
            return torch.randn(*shape, generator=g) * (std if std is not None else shape[-1] ** -0.5)
        yield "embed", mat(cfg.vocab_size, W, std=1.0)
        yield "head", mat(cfg.vocab_size, W)
        for i, layer in enumerate(self.layers):
            mx = layer.mix
            if layer.kind == "attention":
                for n, (_, rows) in mx.qkvg.offsets.items():
                    yield f"l{i}.mix.{n}", mat(rows, W)
                yield f"l{i}.mix.vmix", torch.tensor(0.3)
                yield f"l{i}.mix.o", mat(W, mx.H * mx.Dv)
            else:
                for n, (_, rows) in mx.qkv.offsets.items():
                    yield f"l{i}.mix.{n}", mat(rows, W)
                    yield f"l{i}.mix.{n}.conv", mat(rows, mx.taps, std=0.5)
                for n, (_, rows) in mx.low.offsets.items():
                    yield f"l{i}.mix.{n}", mat(rows, W)
                yield f"l{i}.mix.a2", mat(*mx.a2.shape)
                yield f"l{i}.mix.g2", mat(*mx.g2.shape)
                yield f"l{i}.mix.A_log", torch.randn(mx.H, generator=g) * 0.5 - 1.0
                yield f"l{i}.mix.dt_bias", torch.randn(mx.H * mx.D, generator=g) - 1.0
                yield f"l{i}.mix.o", mat(W, mx.H * mx.Dv)
            if layer.mlp is not None:
                ml = layer.mlp
                yield f"l{i}.mlp.router", mat(ml.n_out, W)
                ff = ml.gate.shape[1]
                for e in range(ml.E):
                    yield f"l{i}.mlp.e{e}.gate", mat(ff, W)
                    yield f"l{i}.mlp.e{e}.up", mat(ff, W)
                    yield f"l{i}.mlp.e{e}.down", mat(W, ff)

    # ---- cache and state ------------------------------------------------------------------------------------------
    def cache_bytes_per_block(self, block_size: int, itemsize: int) -> int:
        return sum(block_size * l.mix.G * (l.mix.D + l.mix.Dv) * itemsize for l in self.layers if l.kind == "attention")

    def state_bytes_per_slot(self) -> int:
        n = 0
        for l in self.layers:
            if l.kind == "channel_delta":
                s, c = l.mix.state_shapes(1)
                n += 4 * (s[1] + c[1] * c[2])
        return n

    def bind_cache(self, num_blocks: int, block_size: int, n_slots: int, dtype: torch.dtype, device) -> None:
        """Pages for the attention layers (serving dtype), state slots for the recurrent ones (fp32).  Nothing has to be
        cleared when a page or a slot changes hands: a sequence's first row starts every state from zero and no kernel
        reads a cache row its own sequence has not written."""
        for l in self.layers:
            if l.kind == "attention":
                ks, vs = l.mix.cache_shapes(num_blocks, block_size)
                l.mix.k_cache = torch.zeros(ks, dtype=dtype, device=device)
                l.mix.v_cache = torch.zeros(vs, dtype=dtype, device=device)
            else:
                ss, cs = l.mix.state_shapes(n_slots)
                l.mix.state = torch.zeros(ss, dtype=torch.float32, device=device)
                l.mix.conv_state = torch.zeros(cs, dtype=torch.float32, device=device)

    # ---- one step over the rows the context describes ----------------------------------------------------------------
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor | None = None) -> torch.Tensor:
        x = ops.embedding_f32(input_ids, self.embed)
        v_first = None
        for layer in self.layers:
            if layer.kind == "attention":
                y, v_first = layer.mix(x, v_first)
            else:
                y = layer.mix(x)
            layer.norm1.add_to(x, y)
            if layer.mlp is not None:
                layer.norm2.add_to(x, layer.mlp(x))
            if self.trace_layers is not None:
                self.trace_layers.append(x.clone())
        return x

    def compute_logits(self, hidden: torch.Tensor, rows: torch.Tensor | None = None) -> torch.Tensor:
        """fp32 logits of the given rows (default: all)."""
        if rows is not None:
            hidden = hidden.index_select(0, rows)
        return ops.gemm_any(self.final_norm(hidden), self.head, alpha=self.config.logit_scale)
