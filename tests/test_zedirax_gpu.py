"""Zedirax on the GPU against the plain statement of its mechanisms in oracle/zedirax.py (float64, one sequence at a time,
dense scores, a Python loop over time).  Small configurations of the tests' own making, random bf16-representable weights;
where random weights would hide a fault the weights or inputs are shaped so that it shows.

Bars (zedirax_harness.assert_close): float32 serving mode 5e-5 on every row (row-wise rms difference / rms of the expected
logits), bfloat16 mode 2e-2 on the median row and 6e-2 on all but a few rows; two runs of the engine that differ only in the
cut (portions, batch, pages, slots) 2e-5 in float32."""
import pytest
import torch

from zedirax_harness import (F32_BAR, MIXED, Replay, assert_close, attention, config, dense, latent, mingru, moe, rel_err,
                             tokens_of, with_mlp, write_model_dir)
from oracle import zedirax as Z

pytestmark = pytest.mark.gpu

CUT_BAR = 2e-5


def expected(cfg, weights, tokens):
    return Z.forward(cfg, weights, tokens, dtype=torch.float64)


@pytest.fixture(scope="module")
def mixed_model():
    w = Z.random_model(MIXED, seed=3)
    return MIXED, w, write_model_dir(MIXED, w)


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def mixed_replay(request, mixed_model):
    r = Replay(mixed_model[2], request.param)
    yield request.param, r
    r.close()


# ------------------------------------------------------------------------------------------------ each mechanism alone
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,layers", [
    ("mingru", [with_mlp(mingru(), None)]),
    ("mingru_wider_than_the_model", [with_mlp(mingru(300), None)]),
    ("latent", [with_mlp(latent(), None)]),
    ("latent_part_rotation", [with_mlp(latent(heads=2, dim=16, rot_dim=12, vdim=36, kv_rank=36, dims=4, base=50.0), None)]),
    ("latent_odd_sizes", [with_mlp(latent(heads=5, dim=10, rot_dim=6, vdim=7, kv_rank=13, dims=6), None)]),   # element-wise loads
    ("latent_matrix_core_sizes", [with_mlp(latent(heads=4, dim=32, rot_dim=16, vdim=32, kv_rank=48, scale=0.1), None)]),
    ("latent_wide", [with_mlp(latent(heads=2, dim=40, rot_dim=32, vdim=24, kv_rank=288, scale=0.05), None)]),
    ("latent_one_head_no_rotation", [with_mlp(latent(heads=1, dim=24, rot_dim=8, vdim=16, kv_rank=24, dims=0), None)]),
    ("attention", [with_mlp(attention(), None)]),
    ("attention_no_temperature", [with_mlp(attention(heads=4, kv_heads=4, dim=24, vdim=72, every=0), None)]),
    ("attention_one_kv_head", [with_mlp(attention(heads=8, kv_heads=1, dim=16, vdim=8, every=1, coef=0.2), None)]),
    ("attention_odd_sizes", [with_mlp(attention(heads=2, kv_heads=1, dim=10, vdim=6, every=3), None)]),
    ("attention_matrix_core_sizes", [with_mlp(attention(heads=4, kv_heads=2, dim=64, vdim=96, every=16, scale=0.1), None)]),
    ("dense_ff", [with_mlp(mingru(), dense())]),
    ("dense_ff_odd", [with_mlp(attention(), dense(ff=37))]),
    ("sparse_ff", [with_mlp(attention(), moe())]),
    ("sparse_ff_no_shared", [with_mlp(mingru(), moe(ff=24, experts=5, top=2, shared=0))]),
    ("sparse_ff_all_experts", [with_mlp(latent(), moe(ff=16, experts=4, top=4, shared=8))]),
    ("sparse_ff_top1_many_experts", [with_mlp(mingru(), moe(ff=8, experts=70, top=1, shared=40))]),
    ("depth_mix_of_five", [with_mlp(mingru(), None)] * 5),
])
def test_mechanism_alone(name, layers, dtype):
    cfg = config(layers, width=72 if "wide" in name else 80, mult=1.0 if "top1" in name else 0.6)
    w = Z.random_model(cfg, seed=11)
    toks = tokens_of(45, cfg["vocab"], 5)
    r = Replay(write_model_dir(cfg, w), dtype)
    try:
        r.runner.model.trace_layers = []
        got = r.feed("a", toks, [45])
        want_layers = []
        want = Z.forward(cfg, w, toks, collect=want_layers)
        for i, (a, b) in enumerate(zip(r.runner.model.trace_layers, want_layers)):
            assert_close(a.cpu(), b, dtype, f"what layer {i} hands on")
        assert_close(got, want, dtype)
        # the same tokens again, one by one, through the cache / the state
        assert_close(r.feed("b", toks, [3]), want, dtype)
    finally:
        r.close()


# ------------------------------------------------------------------------------------------------ operators
@pytest.mark.parametrize("T,n,top", [(64, 12, 3), (40, 130, 6), (33, 512, 8), (5, 7, 7), (9, 65, 1)])
def test_router_choices_and_weights(T, n, top):
    from nanovllm import ops

    g = torch.Generator().manual_seed(n + top)
    z = torch.randn(T, n + 2, generator=g) * 2          # two more columns than outputs: they must not be chosen
    z[:, n:] = 50.0
    val, idx = torch.topk(z[:, :n].double(), top, dim=-1)
    ids, wts = ops.route_topk(z.cuda(), n, top)
    assert torch.equal(ids.cpu().long(), idx)
    assert torch.allclose(wts.cpu().double(), torch.softmax(val, -1), atol=1e-6)


@pytest.mark.parametrize("M", [1, 4, 8, 40, 200, 600])
@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float32])
def test_projection_epilogues(M, wdtype):
    """Bias, each activation, the gated pair with two biases, in every kernel of the general projection."""
    from nanovllm import _C, ops

    g = torch.Generator().manual_seed(M)
    N, K = 70, 52
    x = torch.randn(M, K, generator=g)
    w = (torch.randn(N, K, generator=g) * K ** -0.5).to(wdtype)
    w2 = (torch.randn(N, K, generator=g) * K ** -0.5).to(wdtype)
    b, b2 = torch.randn(N, generator=g), torch.randn(N, generator=g)
    xr = x.bfloat16().double() if (wdtype == torch.bfloat16 and M > 8) else x.double()
    a, a2 = xr @ w.double().T + b.double(), xr @ w2.double().T + b2.double()
    acts = {_C.ACT_NONE: lambda z: z, _C.ACT_SILU: lambda z: z * torch.sigmoid(z), _C.ACT_GELU_TANH: Z.gelu_tanh,
            _C.ACT_GELU_ERF: Z.gelu_erf, _C.ACT_SIGMOID: torch.sigmoid}
    for act, f in acts.items():
        got = ops.gemm_any_act(x.cuda(), w.cuda(), bias=b.cuda(), act=act).cpu().double()
        assert (got - f(a)).abs().max() <= 2e-5, act
        got = ops.gemm_any_act(x.cuda(), w.cuda(), bias=b.cuda(), act=act, w2=w2.cuda(), bias2=b2.cuda(), alpha=0.5).cpu().double()
        assert (got - 0.5 * f(a) * a2).abs().max() <= 4e-5, act
    got = ops.gemm_any_act(x.cuda(), w.cuda(), act=_C.ACT_GELU_ERF, w2=w2.cuda()).cpu().double()
    assert (got - Z.gelu_erf(a - b.double()) * (a2 - b2.double())).abs().max() <= 4e-5


@pytest.mark.parametrize("M", [1, 7, 33, 130, 520])
@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float32])
def test_projection_per_head(M, wdtype):
    """The batched form: head-major rows inside wider buffers, one weight per head, optional sigmoid gate."""
    from nanovllm import ops

    g = torch.Generator().manual_seed(M + 1)
    B, N, K, xs, ys = 5, 22, 20, 27, 30
    xbuf = torch.randn(M, 3 + B * xs, generator=g)
    w = (torch.randn(B, N, K, generator=g) * K ** -0.5).to(wdtype)
    gate = torch.randn(M, B * N + 1, generator=g)
    for use_gate in (False, True):
        out = torch.full((M, B * ys), 7.0).cuda()
        ops.gemm_any_batched(xbuf.cuda()[:, 3:], xs, w.cuda(), out, ys, gate=gate.cuda()[:, 1:] if use_gate else None, gate_batch=N)
        out = out.cpu().double()
        for b in range(B):
            x = xbuf[:, 3 + b * xs:3 + b * xs + K]
            xr = x.bfloat16().double() if (wdtype == torch.bfloat16 and M > 8) else x.double()
            want = xr @ w[b].double().T
            if use_gate:
                want = want * torch.sigmoid(gate[:, 1 + b * N:1 + (b + 1) * N].double())
            assert (out[:, b * ys:b * ys + N] - want).abs().max() <= 2e-5, (b, use_gate)
            assert (out[:, b * ys + N:(b + 1) * ys] == 7.0).all(), "wrote outside its columns"


@pytest.mark.parametrize("lens,starts", [([300], [0]), ([1, 1, 1], [5, 0, 9]), ([64, 65, 2, 130], [0, 3, 0, 64]), ([700, 3], [1, 0])])
def test_gated_scan_in_segments(lens, starts):
    """The recurrence's segmented walk against a loop over time: sequences longer than a segment, exactly one segment, one
    row; states carried in from slots (start > 0) or zero (start 0) whatever the slot holds; the new state written back."""
    from nanovllm import ops

    g = torch.Generator().manual_seed(sum(lens))
    n, T = 37, sum(lens)
    proj = torch.randn(T, 3 * n + 5, generator=g)
    proj[:, 2:2 + n] -= 2.0                       # gates mostly closed: long memory
    state = torch.randn(len(lens) + 2, n, generator=g)
    slots = torch.randperm(len(lens) + 2, generator=g)[:len(lens)].to(torch.int32)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    kv = torch.tensor([s + c for s, c in zip(starts, lens)], dtype=torch.int32)
    st = state.clone().cuda()
    out = ops.mingru_scan(proj.cuda(), 2, 2 + n, 5 + 2 * n, n, st, cu.cuda(), kv.cuda(), slots.cuda(), max(lens)).cpu().double()
    p = proj.double()
    for i, (c, s0) in enumerate(zip(lens, starts)):
        S = state[slots[i]].double() if s0 > 0 else torch.zeros(n, dtype=torch.float64)
        for r in range(int(cu[i]), int(cu[i]) + c):
            z, u, gt = torch.sigmoid(p[r, 2:2 + n]), p[r, 2 + n:2 + 2 * n], p[r, 5 + 2 * n:5 + 3 * n]
            S = (1 - z) * S + z * torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
            assert (out[r] - S * gt * torch.sigmoid(gt)).abs().max() <= 1e-5, (i, r)
        assert (st[slots[i]].cpu().double() - S).abs().max() <= 1e-5
    untouched = [j for j in range(len(lens) + 2) if j not in slots.tolist()]
    assert torch.equal(st.cpu()[untouched], state[untouched])


@pytest.mark.parametrize("H,G,D,Dv,T,start,alias", [(4, 2, 64, 48, 200, 0, False), (2, 2, 128, 128, 90, 57, False), (8, 1, 32, 16, 150, 0, False),
                                                     (6, 1, 64, 48, 170, 30, True), (3, 1, 256, 224, 80, 5, True)])
def test_log_biased_attention_on_the_matrix_cores(H, G, D, Dv, T, start, alias):
    """The MFMA form of the paged attention (prompt portions over a bf16 cache) with the log-distance bias, plain causal
    (no window), at the operator level; `alias`: the values are the leading channels of the key rows (one cache)."""
    from nanovllm import _C, ops

    g = torch.Generator().manual_seed(D + T)
    bs, n = 16, start + T
    k = torch.randn(n, G, D, generator=g).bfloat16()
    v = k[..., :Dv] if alias else torch.randn(n, G, Dv, generator=g).bfloat16()
    q = torch.randn(n, H, D, generator=g)
    r1, r2 = torch.rand(H, generator=g) + 0.2, torch.rand(H, generator=g) * 3
    n_blocks = -(-n // bs)
    table = torch.randperm(n_blocks + 3, generator=g)[:n_blocks].to(torch.int32)
    kc = torch.zeros(n_blocks + 3, G, bs, D, dtype=torch.bfloat16)
    vc = torch.zeros(n_blocks + 3, G, bs, Dv, dtype=torch.bfloat16)
    for p in range(n):
        kc[table[p // bs], :, p % bs] = k[p]
        vc[table[p // bs], :, p % bs] = v[p]
    pos = torch.arange(n)
    dist = (pos.view(n, 1) - pos.view(1, n)).clamp(min=0).double()
    s = torch.einsum("ihd,jhd->hij", q.double(), k.double().repeat_interleave(H // G, 1)) * 0.17
    s = s - r1.double().view(H, 1, 1) * torch.log(1 + r2.double().view(H, 1, 1) * dist)
    want = Z.causal_softmax_attention(s, v.double().repeat_interleave(H // G, 1))[start:]
    kc_d = kc.cuda()
    vc_d = kc_d if alias else vc.cuda()
    got = ops.paged_attention_f32(q[start:].reshape(T, H * D).contiguous().cuda(), kc_d, vc_d, D if alias else Dv,
                                  table.view(1, -1).cuda(), torch.tensor([0, T], dtype=torch.int32).cuda(),
                                  torch.tensor([n], dtype=torch.int32).cuda(), H, G, D, Dv, bs, 2 ** 31 - 1, 0.17,
                                  _C.BIAS_LOG, r1.cuda(), r2.cuda()).cpu().double().view(T, H, Dv)
    assert (got - want).abs().max() <= 1e-4 * want.abs().max(), float((got - want).abs().max() / want.abs().max())


@pytest.mark.parametrize("H,G,D,Dv,alias,window", [(4, 2, 64, 48, False, None), (8, 1, 128, 128, False, 70), (20, 1, 64, 48, True, None),
                                                    (6, 6, 32, 16, False, None), (16, 1, 256, 192, True, None), (3, 1, 256, 224, True, 33)])
def test_decode_attention_with_the_heads_as_columns(H, G, D, Dv, alias, window):
    """Decode steps over a bf16 cache: a kv head's query heads are the columns of one matrix-core tile (more than 16 heads:
    several tiles), four waves split the keys.  Sequences of 1 to 300 cached tokens (fewer keys than waves, a partial last
    round), scattered pages, log-distance bias, with and without a window, values inside the key rows or apart."""
    from nanovllm import _C, ops

    g = torch.Generator().manual_seed(H * D + Dv)
    bs, lens = 16, [1, 2, 31, 32, 33, 129, 300]
    n_blocks = sum(-(-n // bs) for n in lens)
    perm = torch.randperm(n_blocks + 2, generator=g)
    kc = torch.zeros(n_blocks + 2, G, bs, D, dtype=torch.bfloat16)
    vc = torch.zeros(n_blocks + 2, G, bs, Dv, dtype=torch.bfloat16)
    tables = torch.full((len(lens), -(-max(lens) // bs)), -1, dtype=torch.int32)
    r1, r2 = torch.rand(H, generator=g) + 0.2, torch.rand(H, generator=g) * 3
    q = torch.randn(len(lens), H, D, generator=g)
    want, used = [], 0
    for i, n in enumerate(lens):
        k = torch.randn(n, G, D, generator=g).bfloat16()
        v = k[..., :Dv] if alias else torch.randn(n, G, Dv, generator=g).bfloat16()
        nb = -(-n // bs)
        tables[i, :nb] = perm[used:used + nb].to(torch.int32)
        used += nb
        for p in range(n):
            kc[tables[i, p // bs], :, p % bs] = k[p]
            vc[tables[i, p // bs], :, p % bs] = v[p]
        dist = (n - 1 - torch.arange(n)).double()
        s = torch.einsum("hd,jhd->hj", q[i].double(), k.double().repeat_interleave(H // G, 1)) * 0.11
        s = s - r1.double().view(H, 1) * torch.log(1 + r2.double().view(H, 1) * dist)
        if window is not None:
            s = s.masked_fill(dist.view(1, n) >= window, float("-inf"))
        want.append(torch.einsum("hj,jhd->hd", torch.softmax(s, -1), v.double().repeat_interleave(H // G, 1)))
    want = torch.stack(want)
    kc_d = kc.cuda()
    got = ops.paged_attention_f32(q.reshape(len(lens), H * D).cuda(), kc_d, kc_d if alias else vc.cuda(), D if alias else Dv,
                                  tables.cuda(), torch.arange(len(lens) + 1, dtype=torch.int32).cuda(),
                                  torch.tensor(lens, dtype=torch.int32).cuda(), H, G, D, Dv, bs, window or 2 ** 31 - 1, 0.11,
                                  _C.BIAS_LOG, r1.cuda(), r2.cuda()).cpu().double().view(len(lens), H, Dv)
    assert (got - want).abs().max() <= 1e-4 * want.abs().max(), float((got - want).abs().max() / want.abs().max())


# ------------------------------------------------------------------------------------------------ cuts of one sequence
def test_whole_prompt(mixed_model, mixed_replay):
    cfg, w, _ = mixed_model
    dtype, r = mixed_replay
    toks = tokens_of(70, cfg["vocab"], 1)
    assert_close(r.feed("p", toks, [70]), expected(cfg, w, toks), dtype)


def test_prefill_then_token_by_token(mixed_model, mixed_replay):
    """Decoding through pages and state slots: 20 prompt tokens, then 60 single tokens (across page borders at 32, 48, 64 and
    the temperature steps at multiples of 7)."""
    cfg, w, _ = mixed_model
    dtype, r = mixed_replay
    toks = tokens_of(80, cfg["vocab"], 2)
    assert_close(r.feed("d", toks, [20]), expected(cfg, w, toks), dtype)


def test_first_tokens_one_by_one(mixed_model, mixed_replay):
    """A sequence that starts with single tokens: zero state, position 0 unrotated, temperature 1 before the first step."""
    cfg, w, _ = mixed_model
    dtype, r = mixed_replay
    toks = tokens_of(12, cfg["vocab"], 3)
    assert_close(r.feed("f", toks, []), expected(cfg, w, toks), dtype)


@pytest.mark.parametrize("cuts", [[2, 2, 2, 3, 5, 2, 16, 15, 17, 2], [31, 2, 33], [16, 16, 16, 16], [1, 2, 1, 2, 40],
                                  [6, 1, 7, 7, 6, 2, 14]])
def test_portions(mixed_model, mixed_replay, cuts):
    """Portions down to two tokens, ending on and off page borders (16) and temperature steps (position + 1 = 7 k)."""
    cfg, w, _ = mixed_model
    dtype, r = mixed_replay
    toks = tokens_of(75, cfg["vocab"], 4)
    got = r.feed("c", toks, cuts)
    assert_close(got, expected(cfg, w, toks), dtype)
    if dtype == "float32":
        assert rel_err(got, r.feed("w", toks, [75])) <= CUT_BAR


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_hundreds_of_keys(dtype):
    """330 tokens (the kernels take keys 64 at a time: several rounds of the running softmax; the recurrence walks in
    segments of 64 rows) with head sizes of every attention kernel: whole, in portions, decoded."""
    cfg = config([with_mlp(attention(heads=4, kv_heads=2, dim=64, vdim=96, scale=0.1, every=50), None),
                  with_mlp(latent(heads=4, dim=32, rot_dim=16, vdim=32, kv_rank=48, scale=0.1), None),
                  with_mlp(mingru(), None),
                  with_mlp(attention(heads=2, kv_heads=1, dim=10, vdim=6, every=64), None),
                  with_mlp(latent(heads=2, dim=12, rot_dim=6, vdim=10, kv_rank=22, dims=6), dense(ff=32))],
                 width=96, vocab=61)
    w = Z.random_model(cfg, seed=21)
    toks = tokens_of(330, 61, 8)
    want = expected(cfg, w, toks)
    r = Replay(write_model_dir(cfg, w), dtype, pages=48)
    try:
        assert_close(r.feed("a", toks, [330]), want, dtype)
        assert_close(r.feed("b", toks, [100, 3, 64, 65, 2, 70]), want, dtype)     # then 26 single tokens
        assert_close(r.feed("c", toks, [140] + [1] * 100 + [90]), want, dtype)
    finally:
        r.close()


def test_long_decoding(mixed_model, mixed_replay):
    cfg, w, _ = mixed_model
    dtype, r = mixed_replay
    toks = tokens_of(300, cfg["vocab"], 6)
    assert_close(r.feed("l", toks, [3]), expected(cfg, w, toks), dtype)


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
def _one_hot_embedding(vocab, width):
    e = torch.zeros(vocab, width)
    e[:, 0] = 1.0
    e[1, 1] = 6.0                                 # token 1 carries a large feature 1
    for t in range(2, vocab):
        e[t, 2 + t % 4] = 1.0
    return e


def _spiky_attention_model():
    """A biased attention whose keys and queries are a function of the token alone: token 1 is what every query looks for
    (its score stands out by far more than the distance bias takes off over hundreds of positions), and only token 1
    carries the value that reaches the logits."""
    cfg = config([with_mlp(attention(heads=2, kv_heads=1, dim=16, vdim=16, scale=1.0, every=0), None)], width=32, vocab=8, mult=1.0)
    w = Z.random_model(cfg, seed=5)
    w["embed"] = _one_hot_embedding(8, 32)
    wq, wk, wv = torch.zeros(32, 32), torch.zeros(16, 32), torch.zeros(16, 32)
    wq[0, 0] = wq[16, 0] = 6.0                    # every query: channel 0 of both heads
    wk[0, 1] = 1.0                                # key channel 0 = feature 1: large for token 1 only
    wv[:, 1] = 1.0
    w["l0.mix.q"], w["l0.mix.k"], w["l0.mix.v"] = wq, wk, wv
    w["l0.norm1"] = torch.zeros(32)
    w["l0.mix.r1"], w["l0.mix.r2"] = torch.tensor([0.5, 1.0]), torch.tensor([1.0, 0.3])
    return cfg, {k: v.bfloat16().float() for k, v in w.items()}


def _spiky_latent_model():
    """The same idea through the latent: the latent's channel 0 is large for token 1 only and every query looks for it."""
    cfg = config([with_mlp(latent(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=16, scale=1.0), None)], width=32, vocab=8, mult=1.0)
    w = Z.random_model(cfg, seed=6)
    w["embed"] = _one_hot_embedding(8, 32)
    wq, wd, uk, uv = torch.zeros(24, 32), torch.zeros(20, 32), torch.zeros(16, 16), torch.zeros(16, 16)
    wq[0, 0] = wq[12, 0] = 8.0                    # unrotated channel 0 of both heads
    wd[0, 1] = 1.0                                # latent channel 0 = feature 1
    wd[1, 0] = 1.0
    wd[16, 0] = wd[17, 0] = 0.3                   # a little of the rotated key part, the same for every token
    wq[8, 0] = wq[20, 0] = 0.3
    uk[0, 0] = uk[8, 0] = 1.0
    uv[:, 0] = 1.0
    w["l0.mix.q"], w["l0.mix.dkv"], w["l0.mix.uk"], w["l0.mix.uv"] = wq, wd, uk, uv
    w["l0.mix.dkv.norm"] = torch.ones(16)
    w["l0.mix.g"] = torch.zeros(16, 32)
    w["l0.norm1"] = torch.zeros(32)
    return cfg, {k: v.bfloat16().float() for k, v in w.items()}


@pytest.mark.parametrize("maker", [_spiky_attention_model, _spiky_latent_model])
def test_a_far_key_among_hundreds(maker):
    """One dominant key at position p; every later row's output is that key's value, hundreds of positions on, across many
    pages: a page of the block table that is skipped, a chunk of keys that is dropped, or a first key that is lost shows at
    full size.  In a prompt, in portions, decoded; the key at position 0, at a page's last and first slot."""
    cfg, w = maker()
    r = Replay(write_model_dir(cfg, w), "float32", pages=30)
    try:
        for p in (0, 15, 16, 130):
            n = 400
            toks = [2 + (i % 6) for i in range(n)]
            toks[p] = 1
            plain = [2 + (i % 6) for i in range(n)]
            want, without = expected(cfg, w, toks), expected(cfg, w, plain)
            assert rel_err(without[n - 1:], want[n - 1:]) > 0.05, "the far key has no influence: the test's weights are wrong"
            for cuts in ([n], [p + 1, 2, 200, 2], [300] + [1] * 60 + [40], [129, 129, 129]):
                assert rel_err(r.feed("s", toks, cuts), want) <= F32_BAR, (p, cuts)
    finally:
        r.close()


def test_temperature_steps_at_the_right_row():
    """Query temperature with a large coefficient: the row at position every - 1 is the first with factor 1 + coef ln 2; an
    off-by-one in the position (or a portion that restarts the count) moves that row by tens of percent."""
    cfg = config([with_mlp(attention(heads=2, kv_heads=2, dim=8, vdim=8, scale=0.5, coef=3.0, every=5), None)], width=24, vocab=19)
    w = Z.random_model(cfg, seed=8)
    flat = dict(cfg["layers"][0]["mixer"])
    toks = tokens_of(23, 19, 2)
    want = expected(cfg, w, toks)
    cfg_off = config([dict(cfg["layers"][0], mixer=dict(flat, q_temp={"coef": 3.0, "every": 6}))], width=24, vocab=19)
    assert rel_err(expected(cfg_off, w, toks)[4:5], want[4:5]) > 0.02, "the step does not show in this row"
    r = Replay(write_model_dir(cfg, w), "float32")
    try:
        for cuts in ([23], [4, 1, 1, 4, 5], [5, 5, 5], [2, 2] + [1] * 19):
            assert rel_err(r.feed("t", toks, cuts), want) <= F32_BAR, cuts
    finally:
        r.close()


def test_far_write_survives_in_the_state():
    """A recurrence whose gates are almost closed: what position 2 wrote decides the outputs 150 tokens later; a state lost or
    cleared at a portion's start, or a slot mixed up in a batch, shows at full size."""
    cfg = config([with_mlp(mingru(40), None)], width=48, vocab=31)
    w = Z.random_model(cfg, seed=9)
    w["l0.mix.z.b"] = torch.full((40,), -7.0)
    w["l0.mix.z"] = w["l0.mix.z"] * 0.1
    w = {k: v.bfloat16().float() for k, v in w.items()}
    toks = tokens_of(160, 31, 7)
    other = list(toks)
    other[2] = (toks[2] + 1) % 31
    want, want_other = expected(cfg, w, toks), expected(cfg, w, other)
    assert rel_err(want_other[150:], want[150:]) > 1e-3, "the early token has no influence: the test's weights are wrong"
    r = Replay(write_model_dir(cfg, w), "float32", pages=24)
    try:
        assert rel_err(r.feed("a", toks, [160]), want) <= F32_BAR
        assert rel_err(r.feed("b", toks, [5, 70, 2, 2, 60]), want) <= F32_BAR
        for cut in (40, 1):   # two sequences that differ in the early token only, side by side in every step
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


def test_rotation_follows_the_position():
    """A latent attention whose scores come from the rotated parts only, with a small base (fast rotation): the same tokens
    at other positions give other outputs, so a portion or a decoded token rotated with the wrong position shows."""
    cfg = config([with_mlp(latent(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=16, base=3.0, scale=1.0), None)], width=32, vocab=23)
    w = Z.random_model(cfg, seed=10)
    w["l0.mix.uk"] = torch.zeros_like(w["l0.mix.uk"])
    toks = tokens_of(20, 23, 1) * 3
    want = expected(cfg, w, toks)
    assert rel_err(want[40:], want[20:40]) > 1e-2, "the position does not show"
    r = Replay(write_model_dir(cfg, w), "float32")
    try:
        for cuts in ([60], [20, 20, 20], [19, 2, 2, 17], [33]):
            assert rel_err(r.feed("r", toks, cuts), want) <= F32_BAR, cuts
    finally:
        r.close()


# ------------------------------------------------------------------------------------------------ the engine's own entry point
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_llm(mixed_model, dtype):
    """LLM.generate: the scheduler's prefill and decode steps, its page and slot managers, captured decode steps, the sampler.
    Every generated token must be the plain model's best token given the same history (or within the sampler's bf16 logits
    of it); in the bfloat16 mode a sharp softmax now and then moves a row by more than that: two of the sixty may differ."""
    from nanovllm import LLM, SamplingParams

    cfg, w, d = mixed_model
    llm = LLM(d, dtype=dtype, kvcache_block_size=16, num_kvcache_blocks=40, max_num_seqs=3, max_model_len=256,
              max_num_batched_tokens=256, warmup=False)
    try:
        assert llm.model_runner.row_graphs
        prompts = [tokens_of(n, cfg["vocab"], 30 + n) for n in (5, 40, 17, 33, 2)]   # five requests over three slots
        outs = llm.generate(prompts, SamplingParams(max_tokens=12, greedy=True, ignore_eos=True), use_tqdm=False)
        assert len(outs) == 5
        off = []
        for prompt, out in zip(prompts, outs):
            gen = out["token_ids"]
            assert len(gen) == 12
            logits = expected(cfg, w, prompt + gen)
            for i, tok in enumerate(gen):
                row = logits[len(prompt) - 1 + i]
                if row.max() - row[tok] > 0.06:
                    off.append((len(prompt), i, tok, int(row.argmax()), float(row.max() - row[tok])))
        assert len(off) <= (0 if dtype == "float32" else 2), off
    finally:
        llm.exit()


def test_captured_decode_steps_equal_eager(mixed_model):
    """Decode steps replay hipGraphs padded to a batch bucket (3 live requests in the bucket of 4, the padded row writing the
    spare state slot): same tokens and the same logits as eager launches, over several replays with eager prefill steps
    between them."""
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
    """Config.chunked_prefill: the engine's own scheduler cuts prompts into portions (24 rows per step) and batches them
    with the other requests' decoded tokens; the generated tokens are those of whole-prompt prefill steps."""
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


def test_trace_replay_program(mixed_model, tmp_path):
    """bin/trace_run end to end: steps on standard input, logits files and `done` lines out; two requests in one step."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    cfg, w, d = mixed_model
    toks, other = tokens_of(30, cfg["vocab"], 60), tokens_of(9, cfg["vocab"], 61)
    steps = [{"step": 0, "entries": [{"id": "q", "tokens": toks[:20], "want": [0, 19]}], "end": []},
             {"step": 1, "entries": [{"id": "q", "tokens": toks[20:29], "want": []}, {"id": "o", "tokens": other[:8], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "o", "tokens": other[8:], "want": [0]}, {"id": "q", "tokens": toks[29:], "want": [0]}],
              "end": ["q", "o"]}]
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(repo, "bin", "trace_run"), "--model", d, "--dtype", "float32",
                        "--out", str(tmp_path), "--max-tokens", "128"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    want, want_o = expected(cfg, w, toks), expected(cfg, w, other)
    got0 = torch.from_numpy(np.fromfile(tmp_path / "0.f32", dtype="<f4").reshape(2, -1))
    got2 = torch.from_numpy(np.fromfile(tmp_path / "2.f32", dtype="<f4").reshape(2, -1))
    assert not (tmp_path / "1.f32").exists()
    assert rel_err(got0, want[[0, 19]]) <= F32_BAR
    assert rel_err(got2[:1], want_o[[8]]) <= F32_BAR and rel_err(got2[1:], want[[29]]) <= F32_BAR
