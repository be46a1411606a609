"""Zedirax: a pre-norm decoder whose layers - in an order its configuration lists - mix the sequence with a minimal gated
recurrence, a latent (low-rank key/value) attention or a log-distance-biased grouped attention, each followed by a dense
gated or a sparse feed-forward (or none); every layer reads a learned weighted sum of the embedding and of all earlier
layers' results, the residual stream is fp32.

The mechanisms are the classes of layers/seqmix.py; this file reads the configuration, wires the layers, names the
checkpoint's tensors and says what cache and state a sequence needs:

  config.json   {"architecture": "Zedirax", "vocab", "width", "residual_mult", "norm": {"eps"}, "layers": [{"type":
                "mingru" | "latent_attention" | "attention", "mixer": {...}, "mlp": {"kind": "dense" | "moe", ...} | null}]}
  checkpoint    embed, head, final.norm, l<i>.norm1, l<i>.norm2, l<i>.dwa, l<i>.mix.<name>, l<i>.mlp.<name>
  per sequence  pages: K / V rows of every attention layer, one [latent | rotated key] row per latent-attention layer;
                a state slot: one fp32 vector per mingru layer
"""
from __future__ import annotations

import json
import os

import torch
from torch import nn

from nanovllm import ops
from nanovllm.layers.seqmix import (BiasedAttention, DepthMixedResidual, GatedDenseMLP, LatentAttention, MinGRUMixer,
                                    SharedSparseMLP, _vector)


class ZediraxConfig:
    """config.json of this design with the attribute names the engine reads from a configuration object."""
    architectures = ["Zedirax"]
    model_type = "zedirax"
    max_position_embeddings = None   # positions enter through distances, temperatures and rotations computed on the fly
    eos_token_id = None
    native = True                    # not a transformers configuration

    def __init__(self, raw: dict, dtype: str = "bfloat16"):
        self.raw = raw
        self.vocab_size, self.hidden_size = int(raw["vocab"]), int(raw["width"])
        self.layers = raw["layers"]
        self.num_hidden_layers = len(self.layers)
        self.norm_eps = float(raw["norm"]["eps"])
        self.residual_mult = float(raw.get("residual_mult", 1.0))
        self.torch_dtype = dtype

    @classmethod
    def from_dir(cls, path: str, dtype: str = "bfloat16") -> "ZediraxConfig":
        with open(os.path.join(path, "config.json")) as f:
            return cls(json.load(f), dtype)


class ZediraxLayer(nn.Module):
    def __init__(self, cfg: ZediraxConfig, index: int):
        super().__init__()
        spec, W, eps = cfg.layers[index], cfg.hidden_size, cfg.norm_eps
        m = spec["mixer"]
        self.kind = spec["type"]
        if self.kind == "mingru":
            self.mix = MinGRUMixer(W, int(m["width"]))
        elif self.kind == "latent_attention":
            rot = m.get("rot") or {}
            self.mix = LatentAttention(W, int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"]),
                                       int(rot.get("dims", m["rot_dim"])), float(rot.get("base", 10000.0)),
                                       float(m["scale"]), eps)
        elif self.kind == "attention":
            qt = m.get("q_temp") or {}
            self.mix = BiasedAttention(W, int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"]),
                                       float(m["scale"]), float(qt.get("coef", 0.0)), int(qt.get("every", 0)))
        else:
            raise NotImplementedError(f"layer {index}: mixer type {self.kind!r}")
        self.norm1 = _vector(W)           # RMS-norm weights stored around zero: the factor is 1 + w
        self.dwa = _vector(index + 2)     # weights of the embedding and the results of the layers 0..index
        ml = spec.get("mlp")
        self.mlp = self.norm2 = None
        if ml is not None:
            kind = ml.get("kind")
            if kind == "dense":
                self.mlp = GatedDenseMLP(W, int(ml["ff"]), "gelu_tanh")
            elif kind == "moe":
                sh = ml.get("shared") or {}
                self.mlp = SharedSparseMLP(W, int(ml["expert"]["ff"]), int(ml["router"]["experts"]), int(ml["router"]["top"]),
                                           int(sh.get("ff", 0)), "gelu")
            else:
                raise NotImplementedError(f"layer {index}: feed-forward kind {kind!r}")
            self.norm2 = _vector(W)


class ZediraxForCausalLM(nn.Module):
    hybrid_state = True   # sequences own recurrent-state slots beside their pages: ModelRunner takes the row-step path
    fp32_residual = True

    def __init__(self, config: ZediraxConfig):
        super().__init__()
        self.config = config
        W, V = config.hidden_size, config.vocab_size
        self.embed = nn.Parameter(torch.empty(V, W), requires_grad=False)
        self.layers = nn.ModuleList([ZediraxLayer(config, i) for i in range(len(config.layers))])
        self.final_norm = _vector(W)
        self.register_buffer("unit", torch.ones(1, dtype=torch.float32), persistent=False)
        self.head = nn.Parameter(torch.empty(V, W), requires_grad=False)
        self.trace_layers: list | None = None  # bring-up hook: receives a copy of what every layer hands on

    # ---- checkpoint names -> parameters (utils/loader.py) ------------------------------------------------------
    def map_checkpoint_name(self, name: str):
        """-> parameter path, (parameter path, shard) for tensors that land inside a merged / stacked parameter, or None
        for a tensor this configuration has no use for."""
        if name in ("embed", "head"):
            return name
        if name == "final.norm":
            return "final_norm"
        layer, rest = name.split(".", 1)
        i = int(layer[1:])
        pre, L = f"layers.{i}.", self.layers[i]
        if rest in ("norm1", "dwa"):
            return pre + rest
        if rest == "norm2":
            return pre + rest if L.mlp is not None else None
        part, leaf = rest.split(".", 1)
        if part == "mlp":
            if isinstance(L.mlp, GatedDenseMLP):
                return pre + "mlp." + {"gate": "gate", "up": "up", "down": "down", "gate.b": "gate_b", "up.b": "up_b",
                                       "down.b": "down_b"}[leaf]
            if leaf == "router":
                return pre + "mlp.router.weight", "router"
            if leaf.startswith("shared."):
                if leaf == "shared.sg":
                    return pre + "mlp.router.weight", "sg"
                return pre + "mlp.shared_" + leaf.split(".")[1]
            expert, proj = leaf.split(".")
            return pre + "mlp." + proj, int(expert[1:])
        if L.kind == "mingru":
            if leaf in ("z", "x", "g"):
                return pre + "mix.zxg.weight", leaf
            if leaf in ("z.b", "x.b"):
                return pre + "mix.zxg.bias", leaf[0]
            return pre + "mix." + leaf  # o
        if L.kind == "latent_attention":
            if leaf in ("q", "dkv", "g"):
                return pre + "mix.qcg.weight", leaf
            return pre + "mix." + {"dkv.norm": "c_norm", "uk": "uk_t", "uv": "uv", "o": "o"}[leaf]
        if leaf in ("q", "k", "v"):
            return pre + "mix.qkv.weight", leaf
        return pre + "mix." + leaf  # r1, r2, o

    def synthetic_state(self, seed: int = 0):
        """Random tensors under the checkpoint's names (no-checkpoint mode: benchmarks)."""
        g = torch.Generator().manual_seed(seed)
        cfg, W = self.config, self.config.hidden_size

        def mat(*shape, std=None):
            return torch.randn(*shape, generator=g) * (std if std is not None else shape[-1] ** -0.5)

        yield "embed", mat(cfg.vocab_size, W, std=1.0)
        yield "head", mat(cfg.vocab_size, W)
        yield "final.norm", mat(W, std=0.05)
        for i, layer in enumerate(self.layers):
            mx, p = layer.mix, f"l{i}."
            yield p + "norm1", mat(W, std=0.05)
            d = mat(i + 2, std=0.1)
            d[-1] += 1.0
            yield p + "dwa", d
            if layer.kind == "mingru":
                for n in ("z", "x", "g"):
                    yield p + "mix." + n, mat(mx.n, W)
                yield p + "mix.z.b", mat(mx.n, std=0.3)
                yield p + "mix.x.b", mat(mx.n, std=0.3)
                yield p + "mix.o", mat(W, mx.n)
            elif layer.kind == "latent_attention":
                for n, (_, rows) in mx.qcg.offsets.items():
                    yield p + "mix." + n, mat(rows, W)
                yield p + "mix.dkv.norm", 1 + mat(mx.C, std=0.05)
                yield p + "mix.uk", mat(mx.H * mx.D, mx.C)
                yield p + "mix.uv", mat(mx.H * mx.Dv, mx.C)
                yield p + "mix.o", mat(W, mx.H * mx.Dv)
            else:
                for n, (_, rows) in mx.qkv.offsets.items():
                    yield p + "mix." + n, mat(rows, W)
                yield p + "mix.r1", torch.rand(mx.H, generator=g) + 0.1
                yield p + "mix.r2", torch.rand(mx.H, generator=g) + 0.1
                yield p + "mix.o", mat(W, mx.H * mx.Dv)
            ml = layer.mlp
            if ml is None:
                continue
            yield p + "norm2", mat(W, std=0.05)
            if isinstance(ml, GatedDenseMLP):
                ff = ml.gate.shape[0]
                yield p + "mlp.gate", mat(ff, W)
                yield p + "mlp.gate.b", mat(ff, std=0.1)
                yield p + "mlp.up", mat(ff, W)
                yield p + "mlp.up.b", mat(ff, std=0.1)
                yield p + "mlp.down", mat(W, ff)
                yield p + "mlp.down.b", mat(W, std=0.1)
            else:
                ff = ml.up.shape[1]
                yield p + "mlp.router", mat(ml.E, W)
                for e in range(ml.E):
                    yield p + f"mlp.e{e}.up", mat(ff, W)
                    yield p + f"mlp.e{e}.down", mat(W, ff)
                if ml.shared:
                    fs = ml.shared_up.shape[0]
                    yield p + "mlp.shared.up", mat(fs, W)
                    yield p + "mlp.shared.down", mat(W, fs)
                    yield p + "mlp.shared.sg", mat(1, W)

    # ---- cache and state ------------------------------------------------------------------------------------------
    def cache_bytes_per_block(self, block_size: int, itemsize: int) -> int:
        n = 0
        for l in self.layers:
            if l.kind == "attention":
                n += l.mix.G * (l.mix.D + l.mix.Dv)
            elif l.kind == "latent_attention":
                n += l.mix.C + l.mix.R
        return block_size * n * itemsize

    def state_bytes_per_slot(self) -> int:
        return sum(4 * l.mix.n for l in self.layers if l.kind == "mingru")

    def bind_cache(self, num_blocks: int, block_size: int, n_slots: int, dtype: torch.dtype, device) -> None:
        """Pages for the attention layers (serving dtype), state slots for the recurrent ones (fp32).  Nothing has to be
        cleared when a page or a slot changes hands: a sequence's first row starts its state from zero and no kernel reads
        a cache row its own sequence has not written."""
        for l in self.layers:
            if l.kind == "attention":
                ks, vs = l.mix.cache_shapes(num_blocks, block_size)
                l.mix.k_cache = torch.zeros(ks, dtype=dtype, device=device)
                l.mix.v_cache = torch.zeros(vs, dtype=dtype, device=device)
            elif l.kind == "latent_attention":
                l.mix.cache = torch.zeros(l.mix.cache_shape(num_blocks, block_size), dtype=dtype, device=device)
            else:
                l.mix.state = torch.zeros((n_slots, l.mix.n), dtype=torch.float32, device=device)

    # ---- one step over the rows the context describes ----------------------------------------------------------------
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor | None = None) -> torch.Tensor:
        cfg, n = self.config, len(self.layers)
        res = DepthMixedResidual(input_ids.numel(), cfg.hidden_size, n, cfg.residual_mult, cfg.norm_eps, self.unit)
        ops.embedding_f32(input_ids, self.embed, out=res.stack[0])
        h = res.begin(self.layers[0].norm1)
        for i, layer in enumerate(self.layers):
            y = layer.mix(h)
            if layer.mlp is not None:
                y = layer.mlp(res.add_and_norm(y, layer.norm2))
            h = res.next_layer(y, layer.dwa, self.layers[i + 1].norm1 if i + 1 < n else None)
            if self.trace_layers is not None:
                self.trace_layers.append(res.current.clone())
        return res.current

    def compute_logits(self, hidden: torch.Tensor, rows: torch.Tensor | None = None) -> torch.Tensor:
        """fp32 logits of the given rows (default: all)."""
        if rows is not None:
            hidden = hidden.index_select(0, rows)
        return ops.gemm_any(ops.add_rmsnorm_f32(hidden, None, 0.0, self.final_norm, self.config.norm_eps, 1.0), self.head)
