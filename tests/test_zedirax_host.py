"""Host-side pieces of the Zedirax integration (no GPU): the configuration reader, the checkpoint name map through the
framework's loader, what a sequence needs in pages and state slots, and the plain statement's own consistency."""
import os

import pytest
import torch

from zedirax_harness import MIXED, attention, config, dense, latent, mingru, moe, with_mlp, write_model_dir
from oracle import zedirax as Z


@pytest.fixture(scope="module")
def model_dir():
    return write_model_dir(MIXED, Z.random_model(MIXED, seed=1))


def test_config_is_read_from_the_directory(model_dir):
    from nanovllm.config import Config

    c = Config(model_dir, dtype="float32", max_model_len=128, max_num_batched_tokens=128)
    hf = c.hf_config
    assert c.hybrid_state and hf.architectures == ["Zedirax"]
    assert (hf.vocab_size, hf.hidden_size, hf.num_hidden_layers) == (MIXED["vocab"], MIXED["width"], 6)
    assert hf.residual_mult == 0.6 and hf.norm_eps == 1e-5 and c.eos == -1 and c.max_model_len == 128


def test_every_tensor_lands_in_a_parameter(model_dir):
    """Load through the framework's loader on the CPU: every parameter is written, merged and stacked ones in the right
    row ranges, the per-head up-projections in their batched layouts, and nothing of the checkpoint is left over."""
    from nanovllm.models.zedirax import ZediraxConfig, ZediraxForCausalLM
    from nanovllm.utils.loader import load_model
    from safetensors.torch import load_file

    model = ZediraxForCausalLM(ZediraxConfig.from_dir(model_dir))
    for p in model.parameters():
        p.data.fill_(float("nan"))
    load_model(model, model_dir)
    w = {k: v.float() for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    for name, p in model.named_parameters():
        if name.endswith("zxg.bias"):
            continue  # (checked below: the g part has no bias in the checkpoint and must stay zero)
        assert not torch.isnan(p).any(), name
    gru, att, lat = model.layers[0].mix, model.layers[1].mix, model.layers[2].mix
    o = gru.zxg.offsets
    assert torch.equal(gru.zxg.weight[o["x"][0]:o["x"][0] + o["x"][1]], w["l0.mix.x"])
    assert torch.equal(gru.zxg.bias[o["z"][0]:o["z"][0] + o["z"][1]], w["l0.mix.z.b"])
    assert torch.equal(gru.zxg.bias[o["x"][0]:o["x"][0] + o["x"][1]], w["l0.mix.x.b"])
    o = att.qkv.offsets
    assert torch.equal(att.qkv.weight[o["v"][0]:], w["l1.mix.v"]) and torch.equal(att.r2, w["l1.mix.r2"])
    H, D, C, Dv = lat.H, lat.D, lat.C, lat.Dv
    assert torch.equal(lat.uk_t[1], w["l2.mix.uk"][D:2 * D].T) and lat.uk_t.shape == (H, C, D)
    assert torch.equal(lat.uv[2], w["l2.mix.uv"][2 * Dv:3 * Dv]) and torch.equal(lat.c_norm, w["l2.mix.dkv.norm"])
    o = lat.qcg.offsets
    assert torch.equal(lat.qcg.weight[o["dkv"][0]:o["dkv"][0] + o["dkv"][1]], w["l2.mix.dkv"])
    ml = model.layers[0].mlp
    assert torch.equal(ml.router.weight[:ml.E], w["l0.mlp.router"]) and torch.equal(ml.router.weight[ml.E:], w["l0.mlp.shared.sg"])
    assert torch.equal(ml.up[4], w["l0.mlp.e4.up"]) and torch.equal(ml.shared_down, w["l0.mlp.shared.down"])
    assert not model.layers[2].mlp.shared and model.layers[2].mlp.router.weight.shape[0] == 5
    assert torch.equal(model.layers[1].mlp.up_b, w["l1.mlp.up.b"]) and torch.equal(model.layers[4].dwa, w["l4.dwa"])
    assert model.layers[3].mlp is None and model.layers[3].norm2 is None
    assert model.layers[1].mix.temp_every == 7 and model.layers[4].mix.temp_every == 0 and model.layers[5].mix.rot_dims == 4
    assert set(w) == set(Z.tensor_shapes(MIXED))
    # the g rows of the merged recurrent projection have no bias tensor
    og = gru.zxg.offsets["g"]
    gru.zxg.bias.data[og[0]:og[0] + og[1]].zero_()
    assert not torch.isnan(gru.zxg.bias).any()


def test_a_fresh_model_has_zero_gate_bias():
    from nanovllm.models.zedirax import ZediraxConfig, ZediraxForCausalLM

    model = ZediraxForCausalLM(ZediraxConfig(config([with_mlp(mingru(8), None)], width=16, vocab=11)))
    assert float(model.layers[0].mix.zxg.bias.abs().sum()) == 0.0


def test_pages_and_state_of_a_sequence(model_dir):
    from nanovllm.models.zedirax import ZediraxConfig, ZediraxForCausalLM

    model = ZediraxForCausalLM(ZediraxConfig.from_dir(model_dir))
    # attention layers: G (D + Dv) per token; latent layers: kv_rank + rot_dim per token - not heads * (dim + vdim)
    per_token = 3 * (40 + 24) + (40 + 8) + 4 * (16 + 32) + (36 + 12)
    assert model.cache_bytes_per_block(16, 2) == 16 * per_token * 2
    assert model.state_bytes_per_slot() == 4 * (56 + 96)
    only_attention = ZediraxForCausalLM(ZediraxConfig(config([with_mlp(attention(), None)])))
    assert only_attention.state_bytes_per_slot() == 0
    only_recurrent = ZediraxForCausalLM(ZediraxConfig(config([with_mlp(mingru(), None)])))
    assert only_recurrent.cache_bytes_per_block(16, 2) == 0


def test_synthetic_checkpoint_names_match_the_design(model_dir):
    from nanovllm.models.zedirax import ZediraxConfig, ZediraxForCausalLM

    model = ZediraxForCausalLM(ZediraxConfig.from_dir(model_dir))
    got = {name: tuple(t.shape) for name, t in model.synthetic_state(0)}
    assert got == {k: tuple(v) for k, v in Z.tensor_shapes(MIXED).items()}


def test_unknown_parts_are_refused():
    from nanovllm.models.zedirax import ZediraxConfig, ZediraxForCausalLM

    with pytest.raises(NotImplementedError):
        ZediraxForCausalLM(ZediraxConfig(config([{"type": "convolution", "mixer": {}, "mlp": None}])))
    with pytest.raises(NotImplementedError):
        ZediraxForCausalLM(ZediraxConfig(config([with_mlp(mingru(), {"kind": "maxout", "ff": 8})])))


# ---- the plain statement against itself -------------------------------------------------------------------------------
def test_plain_recurrence_is_causal_and_carries():
    cfg = config([with_mlp(mingru(24), None), with_mlp(latent(), None), with_mlp(attention(), moe())], width=48, vocab=31)
    w = Z.random_model(cfg, seed=2)
    toks = list(range(30))
    full = Z.forward(cfg, w, toks)
    assert torch.allclose(Z.forward(cfg, w, toks[:17]), full[:17], atol=1e-10)


def test_plain_latent_attention_equals_explicit_heads():
    """The latent form written out with explicit per-head keys and values (no shared parts) gives the same numbers."""
    torch.manual_seed(0)
    m = latent(heads=2, dim=6, rot_dim=4, vdim=5, kv_rank=7)["mixer"]
    T, W = 9, 12
    p = {"q": torch.randn(2 * 10, W), "dkv": torch.randn(11, W), "dkv.norm": torch.rand(7) + 0.5, "uk": torch.randn(12, 7),
         "uv": torch.randn(10, 7), "g": torch.randn(10, W), "o": torch.randn(W, 10)}
    p = {k: v.double() for k, v in p.items()}
    h = torch.randn(T, W).double()
    got = Z.latent_attention_mixer(h, p, m, 1e-6)
    pos = torch.arange(T)
    dkv = h @ p["dkv"].T
    c = dkv[:, :7] / torch.sqrt((dkv[:, :7] ** 2).mean(-1, keepdim=True) + 1e-6) * p["dkv.norm"]
    outs = []
    for hd in range(2):
        q = (h @ p["q"].T)[:, hd * 10:(hd + 1) * 10]
        k = torch.cat([c @ p["uk"][hd * 6:(hd + 1) * 6].T, Z.rotate(dkv[:, 7:], pos, 4, 10000.0)], -1)
        qq = torch.cat([q[:, :6], Z.rotate(q[:, 6:], pos, 4, 10000.0)], -1)
        v = c @ p["uv"][hd * 5:(hd + 1) * 5].T
        s = (qq @ k.T) * m["scale"]
        s = s.masked_fill(pos.view(1, T) > pos.view(T, 1), float("-inf"))
        outs.append(torch.softmax(s, -1) @ v)
    want = (torch.cat(outs, -1) * torch.sigmoid(h @ p["g"].T)) @ p["o"].T
    assert torch.allclose(got, want, atol=1e-10)
