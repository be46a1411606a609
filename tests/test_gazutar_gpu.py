"""Gazutar on the GPU against the plain statement of its mechanisms in oracle/gazutar.py (float64, one sequence at a time,
dense scores, a Python loop over time).  Small configurations of the tests' own making, random bf16-representable weights;
where random weights would hide a fault the weights or inputs are shaped so that it shows.

Bars (gazutar_harness.assert_close): float32 serving mode 5e-5 on every row (row-wise rms difference / rms of the expected
logits), bfloat16 mode 3e-2 on all but a few rows; two runs of the engine that differ only in the cut (portions, batch,
pages, slots) 2e-5 in float32."""

import pytest
import torch

from gazutar_harness import BF16_BAR, F32_BAR, MIXED, Replay, assert_close, attention, config, delta, moe, rel_err, tokens_of, with_mlp, write_model_dir
from oracle import gazutar as G

pytestmark = pytest.mark.gpu

CUT_BAR = 2e-5


def expected(cfg, weights, tokens):
    return G.forward(cfg, weights, tokens, dtype=torch.float64)


@pytest.fixture(scope="module")
def mixed_model():
    w = G.random_model(MIXED, seed=3)
    return MIXED, w, write_model_dir(MIXED, w)


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def mixed_replay(request, mixed_model):
    r = Replay(mixed_model[2], request.param)
    yield request.param, r
    r.close()


# ------------------------------------------------------------------------------------------------ each mechanism alone
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,layers", [
    ("attention", [with_mlp(attention(), None)]),
    ("attention_one_group", [with_mlp(attention(heads=4, kv_heads=4, dim=24, vdim=72, window=5), None)]),
    ("attention_gqa_all", [with_mlp(attention(heads=8, kv_heads=1, dim=16, vdim=8, window=64), None)]),
    ("attention_odd_sizes", [with_mlp(attention(heads=2, kv_heads=1, dim=10, vdim=6, window=8), None)]),  # element-wise loads
    ("value_mixing", [with_mlp(attention(v_mix=True), None), with_mlp(attention(v_mix=True, window=30), None),
                      with_mlp(attention(v_mix=True, window=3), None)]),
    ("delta", [with_mlp(delta(), None)]),
    ("delta_wide_value", [with_mlp(delta(heads=3, kv_heads=1, dim=20, vdim=100, conv=2), None)]),
    ("delta_wide_key", [with_mlp(delta(heads=2, kv_heads=2, dim=130, vdim=24, conv=7), None)]),
    ("delta_128", [with_mlp(delta(heads=2, kv_heads=1, dim=128, vdim=128, conv=4), None)]),
    ("delta_no_conv_memory", [with_mlp(delta(conv=1), None)]),
    ("sparse_ff", [with_mlp(attention(), moe())]),
    ("sparse_ff_no_identity_one_group", [with_mlp(delta(), moe(experts=7, identity=0, top=7, count=1, keep=1))]),
    ("sparse_ff_all_groups_top1", [with_mlp(delta(), moe(experts=9, identity=3, top=1, count=6, keep=6))]),
])
def test_mechanism_alone(name, layers, dtype):
    cfg = config(layers, width=72 if "wide" in name else 80)
    w = G.random_model(cfg, seed=11)
    toks = tokens_of(45, cfg["vocab"], 5)
    r = Replay(write_model_dir(cfg, w), dtype)
    try:
        r.runner.model.trace_layers = []
        got = r.feed("a", toks, [45])
        want_layers = []
        want = G.forward(cfg, w, toks, collect=want_layers)
        for i, (a, b) in enumerate(zip(r.runner.model.trace_layers, want_layers)):
            assert_close(a.cpu(), b, dtype, f"residual after layer {i}")
        assert_close(got, want, dtype)
    finally:
        r.close()


def test_router_choices_and_weights():
    """Group limits, the correction entering the choice but not the weight, negative choice scores, identity experts."""
    from nanovllm import ops

    torch.manual_seed(0)
    T, n, top, count, keep = 64, 12, 3, 4, 2
    z = torch.randn(T, n) * 2
    corr = torch.randn(n) * 0.3 - 0.5        # choice scores mostly NEGATIVE: a masked expert must lose against them
    cfg = {"router": {"experts": 10, "identity": 2, "top": top, "groups": {"count": count, "keep": keep}}}
    ids, wts = G.route(z.double(), {"router": torch.eye(n, dtype=torch.float64), "correction": corr.double()}, cfg)
    got_ids, got_w = ops.route_grouped(z.cuda(), corr.cuda(), top, count, keep)
    assert torch.equal(got_ids.cpu().long(), ids)
    assert torch.allclose(got_w.cpu().double(), wts, atol=1e-6)
    assert (wts.sum(-1) < 0.999).any()       # not renormalised


@pytest.mark.parametrize("H,G,D,Dv,window,T,start", [(4, 2, 64, 48, 70, 200, 0), (2, 2, 128, 128, 33, 90, 57), (8, 1, 32, 16, 300, 150, 0),
                                                     (2, 1, 256, 160, 40, 70, 5)])
def test_window_attention_on_the_matrix_cores(H, G, D, Dv, window, T, start):
    """The MFMA form of the window attention (prompt portions over a bf16 cache) at the operator level: q and the softmax
    weights enter the matrix cores as bf16 hi + lo pairs, so the result stays at fp32 quality (1e-4 of the output's size;
    a plain bf16 q or p would show as 4e-3).  Scattered pages; a portion that continues `start` cached tokens."""
    from nanovllm import ops

    g = torch.Generator().manual_seed(D + T)
    bs, n = 16, start + T
    k = torch.randn(n, G, D, generator=g).bfloat16()
    v = torch.randn(n, G, Dv, generator=g).bfloat16()
    q = torch.randn(n, H, D, generator=g)
    n_blocks = -(-n // bs)
    table = torch.randperm(n_blocks + 3, generator=g)[:n_blocks].to(torch.int32)
    kc = torch.zeros(n_blocks + 3, G, bs, D, dtype=torch.bfloat16)
    vc = torch.zeros(n_blocks + 3, G, bs, Dv, dtype=torch.bfloat16)
    for p in range(n):
        kc[table[p // bs], :, p % bs] = k[p]
        vc[table[p // bs], :, p % bs] = v[p]
    want = G_windowed(q, k, v, 0.17, window)[start:]
    got = ops.swa_attention(q[start:].reshape(T, H * D).contiguous().cuda(), kc.cuda(), vc.cuda(), table.view(1, -1).cuda(),
                            torch.tensor([0, T], dtype=torch.int32).cuda(), torch.tensor([n], dtype=torch.int32).cuda(),
                            H, G, D, Dv, bs, window, 0.17).cpu().double().view(T, H, Dv)
    assert (got - want).abs().max() <= 1e-4 * want.abs().max(), float((got - want).abs().max() / want.abs().max())


def G_windowed(q, k, v, scale, window):
    return G.windowed_attention(q.double(), k.double(), v.double(), scale, window)


@pytest.mark.parametrize("n,experts,top,count,keep", [(130, 128, 6, 10, 3), (130, 126, 9, 65, 7), (512, 500, 8, 8, 2)])
def test_router_many_outputs(n, experts, top, count, keep):
    """More router outputs than lanes (several per lane), more groups than lanes."""
    from nanovllm import ops

    g = torch.Generator().manual_seed(n + count)
    z = torch.randn(40, n, generator=g) * 3
    corr = torch.randn(n, generator=g) * 0.02
    cfg = {"router": {"experts": experts, "identity": n - experts, "top": top, "groups": {"count": count, "keep": keep}}}
    ids, wts = G.route(z.double(), {"router": torch.eye(n, dtype=torch.float64), "correction": corr.double()}, cfg)
    got_ids, got_w = ops.route_grouped(z.cuda(), corr.cuda(), top, count, keep)
    assert torch.equal(got_ids.cpu().long(), ids)
    assert torch.allclose(got_w.cpu().double(), wts, atol=1e-6)


@pytest.mark.parametrize("M,N,K", [(1, 70, 33), (3, 5, 129), (8, 64, 64), (9, 65, 31), (200, 130, 200), (64, 64, 32),
                                   (600, 200, 100), (513, 128, 64), (40, 300, 264), (4, 50, 1100), (70, 33, 1100), (1100, 40, 70)])
@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float32])
def test_gemm_any_shapes(M, N, K, wdtype):
    from nanovllm import ops

    g = torch.Generator().manual_seed(M * 1000 + N)
    x = torch.randn(M, K + 3, generator=g)[:, 1:K + 1]           # a column slice: unaligned rows, ldx != K
    w = torch.randn(N, K, generator=g).to(wdtype)
    want = x.double() @ w.double().T * 0.5
    for exact in (False, True):
        got = ops.gemm_any(x.cuda(), w.cuda(), alpha=0.5, exact=exact).cpu().double()
        rounds_x = wdtype == torch.bfloat16 and not exact and M > 8
        tol = 2e-2 if rounds_x else 1e-5
        assert (got - want).abs().max() <= tol * K ** 0.5, (exact, float((got - want).abs().max()))


@pytest.mark.parametrize("rows,counts", [(700, [300, 0, 131, 269, 0]), (24, [3, 0, 9, 12, 0]), (6, [0, 6, 0, 0, 0]),
                                          (130, [1, 128, 0, 1, 0])])
@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("dual", [False, True])
def test_grouped_gemm_against_a_loop(rows, counts, wdtype, dual):
    """The experts' grouped GEMM in each of its kernels (prefill-sized tiles, decode-sized tiles, row kernel): gathered input
    rows, scattered output rows, empty groups, SwiGLU epilogue."""
    from nanovllm import ops

    g = torch.Generator().manual_seed(rows)
    E, N, K, T = len(counts), 88, 72, 50
    x = torch.randn(T, K, generator=g)
    w = (torch.randn(E, N, K, generator=g) * K ** -0.5).to(wdtype)
    w2 = (torch.randn(E, N, K, generator=g) * K ** -0.5).to(wdtype) if dual else None
    offsets = torch.tensor([0] + list(torch.tensor(counts).cumsum(0)), dtype=torch.int32)
    x_rows = torch.randint(0, T, (rows,), generator=g, dtype=torch.int32)
    y_rows = torch.randperm(rows, generator=g).to(torch.int32)
    got = ops.gemm_any_grouped(x.cuda(), x_rows.cuda(), w.cuda(), None if w2 is None else w2.cuda(), offsets.cuda(), rows,
                               y_rows.cuda(), rows).cpu().double()
    xr = x.bfloat16().double() if (wdtype == torch.bfloat16 and rows > 8) else x.double()
    for e in range(E):
        for p in range(int(offsets[e]), int(offsets[e + 1])):
            h = xr[x_rows[p]]
            want = h @ w[e].double().T
            if dual:
                want = torch.nn.functional.silu(want) * (h @ w2[e].double().T)
            assert (got[y_rows[p]] - want).abs().max() <= 2e-4, (e, p)


# ------------------------------------------------------------------------------------------------ cuts of one sequence
def test_whole_prompt(mixed_model, mixed_replay):
    cfg, w, _ = mixed_model
    dtype, r = mixed_replay
    toks = tokens_of(70, cfg["vocab"], 1)
    assert_close(r.feed("p", toks, [70]), expected(cfg, w, toks), dtype)


def test_prefill_then_token_by_token(mixed_model, mixed_replay):
    """Decoding through pages and state slots: 20 prompt tokens, then 60 single tokens (across page borders at 32, 48, 64,
    over both layers' windows, far beyond the convolutions' taps)."""
    cfg, w, _ = mixed_model
    dtype, r = mixed_replay
    toks = tokens_of(80, cfg["vocab"], 2)
    got = r.feed("d", toks, [20])
    assert_close(got, expected(cfg, w, toks), dtype)


def test_first_tokens_one_by_one(mixed_model, mixed_replay):
    """A sequence that starts with single tokens: zero state, zero-padded convolution, windows shorter than their size."""
    cfg, w, _ = mixed_model
    dtype, r = mixed_replay
    toks = tokens_of(12, cfg["vocab"], 3)
    assert_close(r.feed("f", toks, []), expected(cfg, w, toks), dtype)


@pytest.mark.parametrize("cuts", [[2, 2, 2, 3, 5, 2, 16, 15, 17, 2], [31, 2, 33], [16, 16, 16, 16], [1, 2, 1, 2, 40],
                                  [8, 9, 9, 9, 9]])
def test_portions(mixed_model, mixed_replay, cuts):
    """Portions down to two tokens, ending on and off page borders (16), window edges (9, 17) and taps."""
    cfg, w, _ = mixed_model
    dtype, r = mixed_replay
    toks = tokens_of(75, cfg["vocab"], 4)
    got = r.feed("c", toks, cuts)
    assert_close(got, expected(cfg, w, toks), dtype)
    if dtype == "float32":
        assert rel_err(got, r.feed("w", toks, [75])) <= CUT_BAR


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_windows_wider_than_a_chunk_of_keys(dtype):
    """Windows of 70, 150 and 400 keys (the kernels take keys 64 at a time: several rounds of the running softmax, the
    window's lower edge inside a round), head sizes 64 / 96 and 256 / 8, 330 tokens: whole, in portions, decoded."""
    cfg = config([with_mlp(attention(heads=4, kv_heads=2, dim=64, vdim=96, window=150, scale=0.3, v_mix=True), None),
                  with_mlp(attention(heads=2, kv_heads=2, dim=256, vdim=8, window=70, scale=0.2), None),
                  with_mlp(attention(heads=4, kv_heads=2, dim=64, vdim=96, window=400, scale=0.3, v_mix=True), None)],
                 width=96, vocab=61)
    w = G.random_model(cfg, seed=21)
    toks = tokens_of(330, 61, 8)
    want = expected(cfg, w, toks)
    r = Replay(write_model_dir(cfg, w), dtype, pages=48)
    try:
        assert_close(r.feed("a", toks, [330]), want, dtype)
        assert_close(r.feed("b", toks, [100, 3, 64, 65, 2, 70]), want, dtype)     # then 26 single tokens
        assert_close(r.feed("c", toks, [140] + [1] * 100 + [90]), want, dtype)
    finally:
        r.close()


def test_wide_window_with_odd_head_sizes():
    """The element-wise attention kernel (head sizes that are not whole 16-byte pieces) over several rounds of keys."""
    cfg = config([with_mlp(attention(heads=3, kv_heads=1, dim=10, vdim=6, window=100, scale=0.4), None)], width=40, vocab=29)
    w = G.random_model(cfg, seed=23)
    toks = tokens_of(230, 29, 9)
    want = expected(cfg, w, toks)
    r = Replay(write_model_dir(cfg, w), "float32", pages=32)
    try:
        assert_close(r.feed("a", toks, [230]), want, "float32")
        assert_close(r.feed("b", toks, [101, 2, 99] + [1] * 20 + [8]), want, "float32")
    finally:
        r.close()


def test_long_decoding(mixed_model, mixed_replay):
    cfg, w, _ = mixed_model
    dtype, r = mixed_replay
    toks = tokens_of(300, cfg["vocab"], 6)
    got = r.feed("l", toks, [3])
    assert_close(got, expected(cfg, w, toks), dtype)


# ------------------------------------------------------------------------------------------------ batches, pages, slots
def test_unequal_batch_equals_alone(mixed_model, mixed_replay):
    """Four requests of unequal length in mixed steps (portions beside single tokens, a request left out of a step, one that
    ends and whose pages and slot the next one takes) against each request alone."""
    cfg, w, _ = mixed_model
    dtype, r = mixed_replay
    V = cfg["vocab"]
    seqs = {"a": tokens_of(50, V, 10), "b": tokens_of(7, V, 11), "c": tokens_of(33, V, 12), "d": tokens_of(21, V, 13),
            "e": tokens_of(40, V, 14)}
    plan = [
        ([("a", 17), ("b", 2)], []),
        ([("a", 1), ("b", 3), ("c", 30)], []),
        ([("a", 1), ("c", 1), ("d", 21)], ["d"]),          # b left out
        ([("a", 16), ("b", 2), ("c", 1), ("e", 2)], ["b"]),  # e takes d's slot and pages
        ([("e", 30), ("c", 1), ("a", 15)], ["a", "c"]),
        ([("e", 8)], ["e"]),
    ]
    at = {k: 0 for k in seqs}
    got = {k: [] for k in seqs}
    slots_seen = {}
    for entries, end in plan:
        step = [(k, seqs[k][at[k]:at[k] + n]) for k, n in entries]
        out = r.step(step, end=[])
        for k, n in entries:
            got[k].append(out[k])
            at[k] += n
            slots_seen[k] = r.live[k].state_slot
        for k in end:
            assert at[k] == len(seqs[k])
            r.scheduler.finish(r.live.pop(k))
    assert slots_seen["e"] == slots_seen["d"], "the freed slot was not used again"
    for k, toks in seqs.items():
        both = torch.cat(got[k])
        assert_close(both, expected(cfg, w, toks), dtype)
        if dtype == "float32":
            assert rel_err(both, r.feed(k + "_alone", toks, [len(toks)])) <= CUT_BAR, k


def test_pages_and_slots_reused_without_clearing(mixed_model):
    """A pool of exactly one request's pages and ONE state slot: every request runs in what the previous one left behind."""
    cfg, w, d = mixed_model
    r = Replay(d, "float32", pages=5, slots=1)
    try:
        for seed, cuts in ((20, [80]), (21, [40, 2, 30]), (22, [])):
            toks = tokens_of(80 if cuts != [] else 20, cfg["vocab"], seed)
            assert rel_err(r.feed("x", toks, cuts), expected(cfg, w, toks)) <= F32_BAR
            assert len(r.scheduler.block_manager.free_block_ids) == 5 and r.scheduler.state_slots.free == [0]
    finally:
        r.close()


# ------------------------------------------------------------------------------------------------ faults that random weights hide
def _spiky_attention_model(window):
    """One attention layer whose keys and queries are (almost) a function of the token alone, so that token 1 is what every
    query looks for: its score stands out by e^12 wherever it is visible; the values separate token 1 from the rest."""
    cfg = config([with_mlp(attention(heads=2, kv_heads=1, dim=16, vdim=16, window=window, scale=1.0), None)], width=32,
                 vocab=8, logit_scale=1.0)
    w = G.random_model(cfg, seed=5)
    w["embed"] = torch.zeros(8, 32)
    w["embed"][:, 0] = 1.0
    w["embed"][1, 1] = 6.0                        # token 1 carries a large feature 1
    for t in range(2, 8):
        w["embed"][t, 2 + t % 4] = 1.0
    wq, wk, wv = torch.zeros(32, 32), torch.zeros(16, 32), torch.zeros(16, 32)
    wq[0, 0] = wq[16, 0] = 4.0                    # every query: channel 0 of both heads
    wk[0, 1] = 1.0                                # key channel 0 = feature 1: large for token 1 only
    wk[1, 0] = 1.0
    wv[:, 1] = 1.0
    wv[3, 2:6] = 1.0
    w["l0.mix.q"], w["l0.mix.k"], w["l0.mix.v"] = wq, wk, wv
    w["l0.mix.q.norm"], w["l0.mix.k.norm"] = torch.ones(32), torch.ones(16) * 3.0
    w["l0.mix.g"] = torch.zeros(32, 32)
    return cfg, {k: v.bfloat16().float() for k, v in w.items()}


@pytest.mark.parametrize("window", [5, 16, 17, 40])
def test_window_edges_with_a_dominant_key(window):
    """The dominant key sits at position p; the rows at p + window - 1 (last one that sees it) and p + window (first one that
    does not) differ by the whole output.  In a prompt, in portions whose edges fall on those rows, and decoded alone; the key
    is also placed at a page border."""
    cfg, w = _spiky_attention_model(window)
    d = write_model_dir(cfg, w)
    r = Replay(d, "float32", pages=12)
    try:
        for p in (0, 3, 15, 16, 31):
            n = p + window + 6
            toks = [2 + (i % 6) for i in range(n)]
            toks[p] = 1
            want = expected(cfg, w, toks)
            inside, outside = p + window - 1, p + window
            assert (want[inside] - want[outside]).abs().max() > 0.5, "the test's weights do not separate the two rows"
            for cuts in ([n], [inside, 1, 1], [outside, 2], [p + 1], [inside + 1, 2, 2], [2, 2, 2]):
                got = r.feed("s", toks, cuts)
                assert rel_err(got, want) <= F32_BAR, (p, cuts)
    finally:
        r.close()


def test_far_write_survives_in_the_state():
    """A delta layer with almost no decay: what position 2 wrote decides the outputs 150 tokens later; a state lost or cleared
    at a portion's start, or a slot mixed up in a batch, shows at full size."""
    cfg = config([with_mlp(delta(heads=2, kv_heads=1, dim=24, vdim=16, conv=3), None)], width=48, vocab=31)
    w = G.random_model(cfg, seed=9)
    w["l0.mix.A_log"] = torch.full((2,), -9.0)
    w = {k: v.bfloat16().float() for k, v in w.items()}
    toks = tokens_of(160, 31, 7)
    other = list(toks)
    other[2] = (toks[2] + 1) % 31
    want, want_other = expected(cfg, w, toks), expected(cfg, w, other)
    assert rel_err(want_other[150:], want[150:]) > 1e-2, "the early token has no influence: the test's weights are wrong"
    r = Replay(write_model_dir(cfg, w), "float32", pages=24)
    try:
        assert rel_err(r.feed("a", toks, [160]), want) <= F32_BAR
        assert rel_err(r.feed("b", toks, [5, 70, 2, 2, 60]), want) <= F32_BAR
        # two sequences that differ in the early token only, side by side in every step, in swapped slots
        for cut in (40, 1):
            at, got = 0, {"x": [], "y": []}
            while at < 160:
                n = min(cut, 160 - at)
                out = r.step([("y", other[at:at + n]), ("x", toks[at:at + n])])
                got["x"].append(out["x"])
                got["y"].append(out["y"])
                at += n
            for k in ("x", "y"):
                r.scheduler.finish(r.live.pop(k))
            assert rel_err(torch.cat(got["x"]), want) <= F32_BAR and rel_err(torch.cat(got["y"]), want_other) <= F32_BAR
    finally:
        r.close()


# ------------------------------------------------------------------------------------------------ the engine's own entry point
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_llm(mixed_model, dtype):
    """LLM.generate: the scheduler's prefill and decode steps, its page and slot managers, the sampler.  Every generated token
    must be the plain model's best token given the same history (or within the serving dtype's noise of it)."""
    from nanovllm import LLM, SamplingParams

    cfg, w, d = mixed_model
    llm = LLM(d, dtype=dtype, kvcache_block_size=16, num_kvcache_blocks=40, max_num_seqs=3, max_model_len=256,
              max_num_batched_tokens=256, warmup=False)
    try:
        prompts = [tokens_of(n, cfg["vocab"], 30 + n) for n in (5, 40, 17, 33, 2)]   # five requests over three slots
        outs = llm.generate(prompts, SamplingParams(max_tokens=12, greedy=True, ignore_eos=True), use_tqdm=False)
        assert len(outs) == 5
        for prompt, out in zip(prompts, outs):
            gen = out["token_ids"]
            assert len(gen) == 12
            logits = expected(cfg, w, prompt + gen)
            for i, tok in enumerate(gen):
                row = logits[len(prompt) - 1 + i]
                assert row.max() - row[tok] <= 0.06, (i, tok, int(row.argmax()))  # (the sampler reads bf16 logits)
    finally:
        llm.exit()


def test_engine_with_default_start_up(mixed_model):
    """LLM(model_dir) as a user calls it: warm-up generations, pages sized from free memory, captured decode steps."""
    from nanovllm import LLM, SamplingParams

    cfg, w, d = mixed_model
    llm = LLM(d, kvcache_block_size=16, max_num_seqs=4, max_model_len=64, max_num_batched_tokens=256,
              gpu_memory_utilization=0.05)
    try:
        assert llm.model_runner.row_graphs and llm.config.num_kvcache_blocks > 100
        prompt = tokens_of(20, cfg["vocab"], 5)
        out = llm.generate([prompt], SamplingParams(max_tokens=6, greedy=True, ignore_eos=True), use_tqdm=False)[0]
        logits = expected(cfg, w, prompt + out["token_ids"])
        for i, tok in enumerate(out["token_ids"]):
            row = logits[len(prompt) - 1 + i]
            assert row.max() - row[tok] <= 0.06
        assert llm.ttft
    finally:
        llm.exit()


def test_captured_decode_steps_equal_eager(mixed_model):
    """The engine's decode steps replay hipGraphs padded to a batch bucket (here 3 live requests in the bucket of 4, the
    padded row writing the spare state slot): same tokens and, for the real rows, the same logits as eager launches -
    over several replays with the engine's own eager prefill steps between them."""
    from nanovllm import LLM, SamplingParams

    cfg, w, d = mixed_model
    prompts = [tokens_of(n, cfg["vocab"], 70 + n) for n in (9, 31, 16, 5, 22)]
    sp = SamplingParams(max_tokens=10, greedy=True, ignore_eos=True)
    runs, logits = [], []
    for eager in (True, False):
        llm = LLM(d, dtype="float32", kvcache_block_size=16, num_kvcache_blocks=40, max_num_seqs=4, max_model_len=128,
                  max_num_batched_tokens=128, warmup=False, enforce_eager=eager)
        try:
            assert bool(llm.model_runner.row_graphs) == (not eager)
            runs.append([o["token_ids"] for o in llm.generate(prompts[:3], sp, use_tqdm=False)])
            runs[-1] += [o["token_ids"] for o in llm.generate(prompts[3:], sp, use_tqdm=False)]
            logits.append(llm.model_runner.last_logits.float().cpu().clone())
        finally:
            llm.exit()
    assert runs[0] == runs[1]
    assert rel_err(logits[1], logits[0]) <= CUT_BAR


def test_engine_chunked_prefill_equals_whole_prompts(mixed_model):
    """Config.chunked_prefill: the engine's own scheduler cuts prompts into portions (24 rows per step here) and batches
    them with the other requests' decoded tokens; the generated tokens are those of whole-prompt prefill steps."""
    from nanovllm import LLM, SamplingParams

    cfg, w, d = mixed_model
    prompts = [tokens_of(n, cfg["vocab"], 90 + n) for n in (70, 9, 41, 3, 26)]
    sp = SamplingParams(max_tokens=9, greedy=True, ignore_eos=True)
    runs = []
    for kw in (dict(max_num_batched_tokens=128), dict(max_num_batched_tokens=24, chunked_prefill=True)):
        llm = LLM(d, dtype="float32", kvcache_block_size=16, num_kvcache_blocks=40, max_num_seqs=3, max_model_len=128,
                  warmup=False, **kw)
        try:
            runs.append([o["token_ids"] for o in llm.generate(prompts, sp, use_tqdm=False)])
        finally:
            llm.exit()
    assert runs[0] == runs[1]
    for prompt, gen in zip(prompts, runs[1]):
        logits = expected(cfg, w, prompt + gen)
        for i, tok in enumerate(gen):
            row = logits[len(prompt) - 1 + i]
            assert row.max() - row[tok] <= 0.06, (i, tok, int(row.argmax()))


def test_preempted_request_is_recomputed(mixed_model):
    """So few pages that a running request is preempted: it gives its pages and slot back, comes back with its completion
    tokens and is recomputed from position 0 - the tokens are the ones it gets with room for everybody."""
    from nanovllm import LLM, SamplingParams

    cfg, w, d = mixed_model
    prompts = [tokens_of(30, cfg["vocab"], 50), tokens_of(28, cfg["vocab"], 51)]
    sp = SamplingParams(max_tokens=24, greedy=True, ignore_eos=True)
    runs = []
    for blocks in (40, 7):   # 7 - 1 reserved = 6 pages of 16: two requests of ~54 tokens do not fit side by side
        llm = LLM(d, dtype="float32", kvcache_block_size=16, num_kvcache_blocks=blocks, max_num_seqs=2, max_model_len=96,
                  max_num_batched_tokens=96, warmup=False)
        try:
            runs.append([o["token_ids"] for o in llm.generate(prompts, sp, use_tqdm=False)])
        finally:
            llm.exit()
    assert runs[0] == runs[1]


def test_trace_replay_program(mixed_model, tmp_path):
    """bin/trace_run end to end: steps on standard input, logits files and `done` lines out."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    cfg, w, d = mixed_model
    toks = tokens_of(30, cfg["vocab"], 60)
    steps = [{"step": 0, "entries": [{"id": "q", "tokens": toks[:20], "want": [0, 19]}], "end": []},
             {"step": 1, "entries": [{"id": "q", "tokens": toks[20:29], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "q", "tokens": toks[29:], "want": [0]}], "end": ["q"]}]
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(repo, "bin", "trace_run"), "--model", d, "--dtype", "float32",
                        "--out", str(tmp_path), "--max-tokens", "128"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    want = expected(cfg, w, toks)
    got0 = torch.from_numpy(np.fromfile(tmp_path / "0.f32", dtype="<f4").reshape(2, -1))
    got2 = torch.from_numpy(np.fromfile(tmp_path / "2.f32", dtype="<f4").reshape(1, -1))
    assert not (tmp_path / "1.f32").exists()
    assert rel_err(got0, want[[0, 19]]) <= F32_BAR and rel_err(got2, want[[29]]) <= F32_BAR
