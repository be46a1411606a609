"""Shared pieces of the Gazutar tests: small configurations of the design (none of them a shipped model's), random
checkpoints written as a model directory, and a replay helper that feeds sequences to the engine's row-step path in a given
cut (portions, batches) and collects the logits of every position."""
import json
import os
import tempfile

import numpy as np
import torch


def attention(heads=6, kv_heads=3, dim=40, vdim=24, window=17, scale=0.2, v_mix=False):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window}, "scale": scale}
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention", "mixer": m}


def delta(heads=4, kv_heads=2, dim=48, vdim=32, conv=4):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def moe(ff=56, experts=6, identity=2, top=3, count=4, keep=2):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "identity": identity, "top": top, "groups": {"count": count, "keep": keep}}}


def config(layers, width=80, vocab=97, logit_scale=1.5, eps=1e-5):
    return {"architecture": "Gazutar", "vocab": vocab, "width": width, "logit_scale": logit_scale, "norm": {"eps": eps},
            "layers": layers}


def with_mlp(layer, mlp):
    return dict(layer, mlp=mlp)


# attention first, unequal head sizes, a width that is no multiple of 32, a layer without feed-forward, two value-mixing
# layers, identity experts in one router and none (and a single group) in the other
MIXED = config([
    with_mlp(attention(v_mix=True), moe()),
    with_mlp(delta(), None),
    with_mlp(attention(window=9, v_mix=True), moe(ff=40, experts=5, identity=0, top=2, count=1, keep=1)),
    with_mlp(delta(heads=2, kv_heads=2, dim=32, vdim=64, conv=2), moe()),
])


def write_model_dir(cfg: dict, weights: dict) -> str:
    from safetensors.torch import save_file

    d = tempfile.mkdtemp(prefix="gazutar_")
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in weights.items()}, os.path.join(d, "model.safetensors"))
    return d


def row_errs(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Row-wise rms difference relative to the rms of the expected row."""
    got, want = got.double(), want.double()
    return (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-9)


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    return float(row_errs(got, want).max())


F32_BAR, BF16_BAR = 5e-5, 3e-2


def assert_close(got: torch.Tensor, want: torch.Tensor, dtype: str, what="") -> None:
    """float32 mode: every row within F32_BAR.  bfloat16 mode: rounding noise of a few 1e-3 per row - but a router's
    near-tie that falls the other way under bf16 rounding replaces an expert for that token and moves its row (and,
    through the recurrent state, every later row of the sequence) by tens of percent, so up to a quarter of the rows may be
    off; position-exact faults are the float32 runs' business."""
    e = row_errs(got, want)
    if dtype == "float32":
        assert float(e.max()) <= F32_BAR, (what, float(e.max()), int(e.argmax()))
    else:
        off = int((e > BF16_BAR).sum())
        assert float(e.median()) <= BF16_BAR / 2 and off <= max(1, e.numel() // 4), (what, float(e.median()), off, e.numel())


class Replay:
    """ModelRunner + Scheduler of one model directory, driven like a trace replay."""

    def __init__(self, model_dir: str, dtype: str, pages: int = 24, page: int = 16, slots: int = 4):
        from nanovllm.config import Config
        from nanovllm.engine.model_runner import ModelRunner
        from nanovllm.engine.scheduler import Scheduler

        self.page = page
        self.config = Config(model_dir, dtype=dtype, kvcache_block_size=page, num_kvcache_blocks=pages + 1,
                             max_num_seqs=slots, num_state_slots=slots, max_model_len=pages * page,
                             max_num_batched_tokens=pages * page, enforce_eager=True)
        self.runner = ModelRunner(self.config, 0)
        self.scheduler = Scheduler(self.config)
        self.live = {}

    def step(self, entries, end=()):
        """entries: [(name, tokens)] -> {name: logits [len(tokens), vocab]} (every row is asked for)."""
        from nanovllm.engine.sequence import Sequence

        runs, names = [], []
        for name, toks in entries:
            seq = self.live.get(name)
            if seq is None:
                seq = self.live[name] = Sequence(list(toks), request_id=name, block_size=self.page)
                self.scheduler.admit_portion(seq, [])
            else:
                self.scheduler.admit_portion(seq, list(toks))
            runs.append((seq, seq.num_computed_tokens, len(toks)))
            names.append(name)
        total = sum(c for _, _, c in runs)
        logits = self.runner.run_rows(runs, list(range(total))).cpu()
        out, a = {}, 0
        for name, (_, _, c) in zip(names, runs):
            out[name] = logits[a:a + c]
            a += c
        for name in end:
            self.scheduler.finish(self.live.pop(name))
        return out

    def feed(self, name, tokens, cuts, end=True):
        """One sequence alone, cut into portions of the given sizes (the rest token by token)."""
        rows, a = [], 0
        sizes = list(cuts)
        while a < len(tokens):
            n = sizes.pop(0) if sizes else 1
            n = min(n, len(tokens) - a)
            last = a + n == len(tokens)
            rows.append(self.step([(name, tokens[a:a + n])], end=[name] if (last and end) else [])[name])
            a += n
        return torch.cat(rows)

    def close(self):
        self.runner.exit()


def tokens_of(n: int, vocab: int, seed: int) -> list[int]:
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()
