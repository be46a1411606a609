"""Shared pieces of the Zedirax tests: small configurations of the design (sizes of the tests' own making: widths that are
no multiple of 32, key / value / latent sizes that are not whole 16-byte pieces next to ones that are), random checkpoints
written as a model directory.  The replay helper that feeds sequences to the engine's row-step path in a given cut is the
one of gazutar_harness (it is not specific to a model)."""
import json
import os
import tempfile

import torch

from gazutar_harness import F32_BAR, Replay, rel_err, row_errs, tokens_of  # noqa: F401 (re-exported)

BF16_MEDIAN, BF16_ROW = 2e-2, 6e-2


def assert_close(got: torch.Tensor, want: torch.Tensor, dtype: str, what="") -> None:
    """float32 mode: every row within F32_BAR (row-wise rms difference / rms of the expected row).  bfloat16 mode: the
    rounding of activations on their way into the matrix cores gives these six-layer stacks about 1e-2 per row, and a sharp
    softmax or a router's near-tie that falls the other way moves single rows (and, through the recurrent state, later
    ones) by tens of percent: the median row within BF16_MEDIAN, at most a quarter of the rows over BF16_ROW.
    Position-exact faults are the float32 runs' business."""
    e = row_errs(got, want)
    if dtype == "float32":
        assert float(e.max()) <= F32_BAR, (what, float(e.max()), int(e.argmax()))
    else:
        off = int((e > BF16_ROW).sum())
        assert float(e.median()) <= BF16_MEDIAN and off <= max(1, e.numel() // 4), (what, float(e.median()), off, e.numel())


def mingru(width=56):
    return {"type": "mingru", "mixer": {"width": width}}


def latent(heads=3, dim=24, rot_dim=8, vdim=20, kv_rank=40, dims=None, base=10000.0, scale=0.15):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
                      "rot": {"base": base, "dims": rot_dim if dims is None else dims}}}


def attention(heads=6, kv_heads=3, dim=40, vdim=24, scale=0.2, coef=0.3, every=7):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if every:
        m["q_temp"] = {"coef": coef, "every": every}
    return {"type": "attention", "mixer": m}


def dense(ff=88):
    return {"kind": "dense", "ff": ff}


def moe(ff=40, experts=7, top=3, shared=24):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def with_mlp(layer, mlp):
    return dict(layer, mlp=mlp)


def config(layers, width=80, vocab=97, mult=0.6, eps=1e-5):
    return {"architecture": "Zedirax", "vocab": vocab, "width": width, "residual_mult": mult, "norm": {"eps": eps},
            "layers": layers}


# recurrence first, every mixer and every feed-forward form, a layer without feed-forward, a router without a shared expert,
# an attention without temperature and with one key/value head per query head, a rotation over part of the rotated entries
MIXED = config([
    with_mlp(mingru(), moe()),
    with_mlp(attention(), dense()),
    with_mlp(latent(), moe(ff=24, experts=5, top=2, shared=0)),
    with_mlp(mingru(width=96), None),
    with_mlp(attention(heads=4, kv_heads=4, dim=16, vdim=32, every=0), dense(ff=40)),
    with_mlp(latent(heads=2, dim=16, rot_dim=12, vdim=36, kv_rank=36, dims=4, base=50.0), dense(ff=64)),
])


def write_model_dir(cfg: dict, weights: dict) -> str:
    from safetensors.torch import save_file

    d = tempfile.mkdtemp(prefix="zedirax_")
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in weights.items()}, os.path.join(d, "model.safetensors"))
    return d
