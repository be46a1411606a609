"""Host-side pieces of the Gazutar integration (no GPU): the configuration reader, the checkpoint name map and loader,
page and state-slot bookkeeping of sequences that carry recurrent state, the scheduler's portion-wise admission."""
import json
import os

import pytest
import torch

from gazutar_harness import MIXED, write_model_dir
from oracle import gazutar as G


@pytest.fixture(scope="module")
def model_dir():
    return write_model_dir(MIXED, G.random_model(MIXED, seed=1))


def test_config_is_read_from_the_directory(model_dir):
    from nanovllm.config import Config

    c = Config(model_dir, dtype="float32", max_model_len=128, max_num_batched_tokens=128)
    hf = c.hf_config
    assert c.hybrid_state and hf.architectures == ["Gazutar"]
    assert (hf.vocab_size, hf.hidden_size, hf.num_hidden_layers) == (MIXED["vocab"], MIXED["width"], 4)
    assert hf.tensor_shapes["l1.mix.a1"] == (10, 80)          # a size only the checkpoint's header gives
    assert c.max_model_len == 128 and c.eos == -1


def test_every_tensor_lands_in_a_parameter(model_dir):
    """Load through the framework's loader on the CPU: every parameter is written, merged and stacked ones in the right
    row ranges, and nothing of the checkpoint is left over."""
    from nanovllm.models.gazutar import GazutarConfig, GazutarForCausalLM
    from nanovllm.utils.loader import load_model
    from safetensors.torch import load_file

    model = GazutarForCausalLM(GazutarConfig.from_dir(model_dir))
    for p in model.parameters():
        p.data.fill_(float("nan"))
    load_model(model, model_dir)
    assert not any(torch.isnan(p).any() for p in model.parameters())
    w = load_file(os.path.join(model_dir, "model.safetensors"))
    att, dl = model.layers[0].mix, model.layers[1].mix
    o = att.qkvg.offsets
    assert torch.equal(att.qkvg.weight[o["k"][0]:o["k"][0] + o["k"][1]], w["l0.mix.k"].float())
    assert torch.equal(att.qkvg.weight[o["g"][0]:], w["l0.mix.g"].float())
    assert torch.equal(dl.conv.weight[dl.conv.offsets["v"][0]:], w["l1.mix.v.conv"].float())
    assert torch.equal(dl.low.weight[dl.low.offsets["b"][0]:], w["l1.mix.b"].float())
    assert torch.equal(model.layers[0].mlp.down[4], w["l0.mlp.e4.down"].float())
    assert torch.equal(model.layers[3].norm2.bias, w["l3.norm2.b"].float())
    assert model.layers[1].mlp is None and model.layers[0].mix.mixes_values == "first" and model.layers[2].mix.mixes_values == "later"
    assert float(model.layers[2].mix.vmix) == float(w["l2.mix.vmix"].float())


def test_unknown_mixer_is_refused(tmp_path):
    from nanovllm.models.gazutar import GazutarConfig, GazutarForCausalLM

    raw = json.loads(json.dumps(MIXED))
    raw["layers"][0]["type"] = "something_else"
    with pytest.raises(NotImplementedError):
        GazutarForCausalLM(GazutarConfig(raw))


def _sched(pages=6, slots=2, page=16):
    from nanovllm.engine.scheduler import Scheduler

    class C:
        max_num_seqs, max_num_batched_tokens, max_model_len, eos = slots, 256, 256, -1
        num_kvcache_blocks, kvcache_block_size, hybrid_state, num_state_slots = pages + 1, page, True, slots
    return Scheduler(C)


def test_pages_are_private_and_come_back():
    from nanovllm.engine.block_manager import PlainBlockManager
    from nanovllm.engine.sequence import Sequence

    s = _sched()
    bm = s.block_manager
    assert isinstance(bm, PlainBlockManager)
    a, b = Sequence([1] * 20, block_size=16), Sequence([1] * 20, block_size=16)   # equal tokens: nothing may be shared
    s.admit_portion(a, [])
    s.admit_portion(b, [])
    assert a.block_table == [0, 1] and b.block_table == [2, 3] and (a.state_slot, b.state_slot) == (0, 1)
    s.admit_portion(a, [5] * 12)            # 32 tokens: still two pages
    assert a.block_table == [0, 1] and len(a) == 32
    s.admit_portion(a, [5])                 # 33: a third page
    assert a.block_table == [0, 1, 4]
    with pytest.raises(RuntimeError):
        s.admit_portion(b, [7] * 40)        # 60 tokens = 4 pages, one free
    s.finish(a)
    assert list(bm.free_block_ids) == [5, 4, 1, 0] and a.state_slot == -1 and s.state_slots.free == [0]
    c = Sequence([2] * 5, block_size=16)
    s.admit_portion(c, [])
    assert c.state_slot == 0 and c.block_table == [5]
    with pytest.raises(RuntimeError):
        s.admit_portion(Sequence([3], block_size=16), [])   # a third live sequence


def test_scheduler_steps_take_and_release_slots():
    """schedule(): admission stops at the last free slot; a preempted sequence gives its slot and pages back and is
    prefilled again from position 0."""
    from nanovllm.engine.sequence import Sequence

    s = _sched(pages=4, slots=2)
    seqs = [Sequence([1] * 30, block_size=16), Sequence([2] * 30, block_size=16), Sequence([3] * 4, block_size=16)]
    for q in seqs:
        q.max_tokens, q.ignore_eos = 8, True
        s.add(q)
    picked, is_prefill = s.schedule()
    assert is_prefill and picked == seqs[:2] and [q.state_slot for q in seqs] == [0, 1, -1]
    s.postprocess(picked, [9, 9])
    picked, is_prefill = s.schedule()       # the third request has pages but no slot: decode goes on
    assert not is_prefill and picked == seqs[:2]
    s.postprocess(picked, [9, 9])           # both now hold 32 tokens = 2 pages each: the pool is empty
    picked, is_prefill = s.schedule()
    assert not is_prefill and picked == seqs[:2]
    s.postprocess(picked, [9, 9])
    picked, is_prefill = s.schedule()       # 33rd token: a page is needed - the last sequence is preempted
    assert not is_prefill and picked == [seqs[0]] and seqs[1].state_slot == -1 and not seqs[1].block_table
    assert s.waiting[0] is seqs[1] and seqs[0].state_slot == 0


def test_row_scheduling_cuts_prompts_and_batches_decodes():
    """schedule_rows(): a token budget of 32 rows per step - a long prompt goes in portions, the next prompt joins the step
    that has budget left, a decoded token rides beside a portion, the third request waits for a slot."""
    from nanovllm.engine.sequence import Sequence

    s = _sched(pages=12, slots=2)
    s.max_num_batched_tokens = 32
    a, b, c = (Sequence([7] * n, block_size=16) for n in (50, 10, 5))
    for q in (a, b, c):
        q.max_tokens, q.ignore_eos = 3, True
        s.add(q)

    def step():
        runs = s.schedule_rows()
        done = [q for q, start, count in runs if start + count == len(q)]
        for q, start, count in runs:
            q.num_computed_tokens = start + count        # what the runner does
        s.postprocess(done, [9] * len(done))
        return [(q.seq_id - a.seq_id, start, count) for q, start, count in runs]

    assert step() == [(0, 0, 32)]
    assert step() == [(0, 32, 18), (1, 0, 10)] and (a.state_slot, b.state_slot, c.state_slot) == (0, 1, -1)
    assert step() == [(0, 50, 1), (1, 10, 1)]
    assert step() == [(0, 51, 1), (1, 11, 1)]            # both reach max_tokens = 3 and leave
    assert a.is_finished and b.is_finished and s.state_slots.free == [1, 0]
    assert step() == [(2, 0, 5)] and c.state_slot == 0
    assert len(a.block_table) == 0 and len(c.block_table) == 1


def test_row_scheduling_preempts_from_the_right_when_pages_run_out():
    from nanovllm.engine.sequence import Sequence

    s = _sched(pages=4, slots=2)
    s.max_num_batched_tokens = 64
    a, b = Sequence([1] * 31, block_size=16), Sequence([2] * 30, block_size=16)
    for q in (a, b):
        q.max_tokens, q.ignore_eos = 8, True
        s.add(q)
    runs = s.schedule_rows()
    assert [(start, count) for _, start, count in runs] == [(0, 31), (0, 30)]
    for q, start, count in runs:
        q.num_computed_tokens = start + count
    s.postprocess([a, b], [9, 9])                        # 32 and 31 tokens: the four pages are full
    runs = s.schedule_rows()                             # a's 33rd token needs a fifth page: b goes
    assert [(q is a, start, count) for q, start, count in runs] == [(True, 31, 1)] or \
        [(q is a, start, count) for q, start, count in runs] == [(True, 31, 1), (False, 30, 1)]
    for q, start, count in runs:
        q.num_computed_tokens = start + count
    s.postprocess([q for q, _, _ in runs], [9] * len(runs))
    runs = s.schedule_rows()
    assert runs[0][0] is a and b.state_slot == -1 and s.waiting[0] is b and not b.block_table
