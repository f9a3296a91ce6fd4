"""The Nurasun design through the engine against the plain implementation (``plain_nurasun``): whole prompts layer
by layer, prefill against token-by-token decoding, portions down to two tokens, mixed batches with pages and slots
used again, long decoding across many runs of positions, keys made to stand out at the edges of a run, at page
borders and far away, a layer that reads another's rows, each kernel alone, greedy generation through the scheduler,
and the trace replay program as a process."""

from __future__ import annotations

import json

import numpy as np
import pytest
import torch

import nurasun_models as M
import plain_nurasun as P
from helpers import cut, first_bad, random_ids, replay

pytestmark = pytest.mark.gpu

#: bounds on max |difference| / max |logit| of a position, fixed before the first run: float32 against the float64
#: plain run; bfloat16 loosely, because the sharp softmax of these models amplifies the rounding of queries and keys
TOL = {"float32": 2e-5, "bfloat16": 8e-2}
MODELS = {"small": (M.SMALL, 11), "ones": (M.ONES, 12), "wide": (M.WIDE, 13), "odd": (M.ODD, 14)}
DEV = "cuda:0"

_made = {}


def _folder_of(raw, seed, tensors=None):
    """A model folder for ``raw`` (cached by its text); ``tensors(state)`` may change the drawn weights."""
    import tempfile

    from safetensors.torch import save_file

    from pyre_amd.registry import config_from_dict
    from pyre_amd.weights import model_tensor_specs, random_state

    key = (json.dumps(raw, sort_keys=True), seed, tensors)
    if key not in _made:
        d = tempfile.mkdtemp(prefix="nurasun_")
        cfg = config_from_dict(raw)
        cfg.save(d)
        state = random_state(model_tensor_specs(cfg), seed, 0.2, 0.2)
        if tensors is not None:
            tensors(state)
        save_file({k: v.contiguous() for k, v in state.items()}, d + "/model.safetensors")
        _made[key] = (d, *P.read_folder(d))
    return _made[key]


@pytest.fixture(scope="module")
def folders():
    return {name: _folder_of(raw, seed) for name, (raw, seed) in MODELS.items()}


def engine_of(folder, dtype, **kw):
    from pyre_amd.config.engine import EngineConfig
    from pyre_amd.engine.engine import Engine

    args = dict(dtype=dtype, page_size=8, max_cached_tokens=1024, max_num_seqs=4, max_num_batched_tokens=512,
                use_graphs=False)
    args.update(kw)
    return Engine.from_folder(folder, EngineConfig(**args))


def plain_rows(cfg, w, ids):
    return P.forward(w, cfg, ids).float()


def whole(reqs):
    return [([(r, ids, list(range(len(ids))))], [r]) for r, ids in reqs.items()]


def in_portions(reqs, sizes):
    steps = []
    for r, ids in reqs.items():
        pos, parts = 0, cut(len(ids), sizes)
        for k, n in enumerate(parts):
            steps.append(([(r, ids[pos:pos + n], list(range(n)))], [r] if k == len(parts) - 1 else []))
            pos += n
    return steps


def one_by_one(reqs, first):
    steps = []
    for r, ids in reqs.items():
        steps.append(([(r, ids[:first], list(range(first)))], []))
        steps += [([(r, [ids[t]], [0])], [r] if t == len(ids) - 1 else []) for t in range(first, len(ids))]
    return steps


#: a 16-bit run is not compared where the plain router's choice hangs on less than this much of a score
CLOSE_CALL = 0.02


def assert_close(got, want, tol, calls=None):
    """``calls``: request -> :func:`plain_nurasun.closest_call` of its tokens (16-bit runs)."""
    if calls is not None:
        got = {(r, pos): row for (r, pos), row in got.items() if float(calls[r][pos]) >= CLOSE_CALL}
    bad, worst = first_bad(got, want, tol)
    assert bad is None, bad
    return worst


def all_given_back(eng):
    eng.cache.check_invariants()
    return all(g.allocator.num_used == 0 for g in eng.cache.page_groups) and eng.cache.slots.num_used == 0


# ----------------------------------------------------------------------------- whole prompts, layer by layer


@pytest.mark.parametrize("name", list(MODELS))
def test_every_layer_of_a_whole_prompt(name, folders):
    from pyre_amd.engine.batch import Entry

    folder, cfg, w = folders[name]
    ids = random_ids(cfg["vocab"], 75, seed=3)
    want, layers = P.forward(w, cfg, ids, return_hidden=True)
    eng = engine_of(folder, "float32")
    seen = {}
    got = eng.step([Entry("a", ids, list(range(len(ids))))], tap=lambda pos, rows: seen.__setitem__(pos, rows.double().cpu()))
    for pos, ref in enumerate(layers):
        d = float((seen[pos] - ref).abs().max() / ref.abs().max())
        assert d <= TOL["float32"], f"layer {pos}: {d:.2e}"
    d = float((got.double().cpu() - want).abs().max() / want.abs().max())
    assert d <= TOL["float32"], d


# (the model of single heads of one to six elements runs in float32 only: in 16 bits its logits are mostly rounding)
@pytest.mark.parametrize("name,dtype,page", [("small", "float32", 8), ("small", "bfloat16", 16), ("small", "float32", 4),
                                             ("ones", "float32", 4), ("wide", "float32", 16), ("wide", "bfloat16", 8),
                                             ("odd", "float32", 8), ("odd", "bfloat16", 4)])
def test_prefill_decode_and_portions_agree_with_plain(name, dtype, page, folders):
    folder, cfg, w = folders[name]
    reqs = {r: random_ids(cfg["vocab"], n, seed=n) for r, n in (("a", 90), ("b", 1), ("c", 37))}
    want = {r: plain_rows(cfg, w, ids) for r, ids in reqs.items()}
    calls = {r: P.closest_call(w, cfg, ids) for r, ids in reqs.items()} if dtype == "bfloat16" else None
    eng = engine_of(folder, dtype, page_size=page)
    assert_close(replay(eng, whole(reqs)), want, TOL[dtype], calls)
    # most of the prompt, then token by token: the runs of positions end and begin under decoded tokens
    tail = {r: ids for r, ids in reqs.items() if len(ids) > 1}
    assert_close(replay(eng, one_by_one(tail, 6)), want, TOL[dtype], calls)
    # the first tokens of a sequence one by one from the very start
    assert_close(replay(eng, one_by_one({"c": reqs["c"][:12]}, 1)), want, TOL[dtype], calls)
    for sizes in ([2], [3, 2, 17, 2, 31, 5], [64, 2, 9], [7, 1, 1, 24]):
        assert_close(replay(eng, in_portions(tail, sizes)), want, TOL[dtype], calls)
    assert all_given_back(eng)


@pytest.mark.parametrize("name,dtype,poison", [("small", "float32", True), ("wide", "float32", True), ("small", "bfloat16", False),
                                               ("ones", "float32", True)])
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype, poison, folders):
    folder, cfg, w = folders[name]
    reqs = {r: random_ids(cfg["vocab"], n, seed=7 * n) for r, n in (("a", 61), ("b", 9), ("c", 100), ("d", 33), ("e", 2), ("f", 47))}
    want = {r: plain_rows(cfg, w, ids) for r, ids in reqs.items()}
    # three slots, a pool that holds three of the requests at most: everything is used again
    eng = engine_of(folder, dtype, max_num_seqs=3, max_cached_tokens=232, debug_poison=poison)
    fed = {r: 0 for r in reqs}
    live, waiting, steps, k = [], list(reqs), [], 0
    while live or waiting:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in live:
            n = min([5, 1, 13, 2, 1, 40, 1][k % 7], len(reqs[r]) - fed[r])
            k += 1
            entries.append((r, reqs[r][fed[r]:fed[r] + n], list(range(n))))
            fed[r] += n
            if fed[r] == len(reqs[r]):
                end.append(r)
        steps.append((entries, end))
        live = [r for r in live if r not in end]
    got = replay(eng, steps)
    assert_close(got, want, TOL[dtype], {r: P.closest_call(w, cfg, ids) for r, ids in reqs.items()} if dtype == "bfloat16" else None)
    assert all_given_back(eng)
    if dtype == "float32":
        # each request alone gives what it gave among the others
        alone = replay(eng, whole({"c": reqs["c"], "d": reqs["d"]}))
        for key, row in alone.items():
            assert float((row - got[key]).abs().max() / row.abs().max()) <= TOL[dtype]


def test_long_decoding_across_many_runs_of_positions(folders):
    folder, cfg, w = folders["small"]
    ids = random_ids(cfg["vocab"], 260, seed=1)
    want = {"a": plain_rows(cfg, w, ids)}
    eng = engine_of(folder, "float32", page_size=8, max_cached_tokens=272, debug_poison=True)
    assert_close(replay(eng, one_by_one({"a": ids}, 2)), want, TOL["float32"])
    assert all_given_back(eng)


def test_long_decoding_in_a_pool_that_only_ended_runs_make_fit():
    """260 tokens one by one through a model whose layers all see runs of positions: the pages of a run go back when
    the next run begins, so a pool of 64 tokens is enough (freed pages are filled with NaN: a read of one would show)."""
    raw = M.model(113, 40, [M.SMALL["layers"][0], M.SMALL["layers"][3]], eps=1e-5, mult=0.45, softcap=9.0)
    folder, cfg, w = _folder_of(raw, 21)
    ids = random_ids(cfg["vocab"], 260, seed=1)
    want = {"a": plain_rows(cfg, w, ids)}
    eng = engine_of(folder, "float32", page_size=8, max_cached_tokens=64, max_model_len=512, debug_poison=True)
    assert_close(replay(eng, one_by_one({"a": ids}, 2)), want, TOL["float32"])
    assert_close(replay(eng, in_portions({"a": ids}, [5, 2, 19, 1, 7, 30])), want, TOL["float32"])
    assert all_given_back(eng)


# ----------------------------------------------------------------------------- keys made to stand out


EDGE = M.model(53, 32, [M.layer(M.attention(2, 1, 16, 1.5, chunk=12, rot=2, base=1e6), M.dense(24))], mult=0.8, softcap=0.0)


def _keys_like_queries(state):
    # the key head is made by the first head's query matrix and bias: a token's key points where the same token's
    # query points (two of sixteen elements turn with the position), so a query gives nearly all its weight to the
    # earlier copies of its own token that it sees
    state["l0.mix.k"] = state["l0.mix.q"][:16].clone()
    state["l0.mix.k.b"] = state["l0.mix.q.b"][:16].clone()


def test_a_copy_of_the_token_just_inside_and_just_outside_its_run():
    folder, cfg, w = _folder_of(EDGE, 31, _keys_like_queries)
    run, T = 12, 52
    eng = engine_of(folder, "float32", page_size=8)
    base = [1 + (i % 50) for i in range(60)]           # no token twice within 50 positions; T appears nowhere
    # the query at 46 sits in the run 36..47, the one at 48 is the first of its run
    cases = {"inside": (46, 36), "outside": (46, 35), "page_border": (47, 40), "neighbour": (46, 45), "run_start": (48, 47),
             "far_outside": (57, 9)}
    reqs = {}
    for name, (i, j) in cases.items():
        ids = list(base)
        ids[i] = ids[j] = T
        reqs[name] = ids
    want = {r: plain_rows(cfg, w, ids) for r, ids in reqs.items()}
    # the construction works: whether the copy is seen decides the logits at the query
    seen = float((want["inside"][46] - want["outside"][46]).abs().max() / want["inside"][46].abs().max())
    assert seen > 500 * TOL["float32"], seen
    for steps in (whole(reqs), one_by_one(reqs, 30), in_portions(reqs, [35, 2, 9, 2]), in_portions(reqs, [2, 3]),
                  in_portions(reqs, [36, 11, 1, 12])):
        assert_close(replay(eng, steps), want, TOL["float32"])


FAR = M.model(61, 24, [M.layer(M.latent(1, 16, 8, 16, 2.5), M.moe(3, 1, 8, shared=4))], mult=1.0, softcap=20.0)


def _latent_keys_for_the_opposite_token(state):
    # the compressed row is made by minus the query matrix and carried up by the identity, the norm has no shift, and
    # token 59's embedding is minus token 60's: the key of a 59 is the query of a 60 (divided by its root mean
    # square) while a 60's own key points the other way, so a query 60 gives nearly all its weight to the 59s before
    # it, however far back, and their value is not its own
    state["l0.mix.dkv"] = -state["l0.mix.q"]
    state["l0.mix.dkv.norm"] = torch.ones_like(state["l0.mix.dkv.norm"])
    state["l0.mix.uk"] = torch.eye(16).to(state["l0.mix.uk"].dtype)
    state["l0.norm1.b"] = torch.zeros_like(state["l0.norm1.b"])
    state["embed"][59] = -state["embed"][60]


def test_a_far_key_among_hundreds():
    folder, cfg, w = _folder_of(FAR, 33, _latent_keys_for_the_opposite_token)
    base = [1 + (i % 58) for i in range(420)]          # neither 59 nor 60 appears
    with_key, without = list(base), list(base)
    with_key[3], with_key[409] = 59, 60
    without[409] = 60
    other = list(base)
    other[127], other[128], other[409] = 59, 59, 60   # at a page's last and first place
    reqs = {"far": with_key, "none": without, "border": other}
    want = {r: plain_rows(cfg, w, ids) for r, ids in reqs.items()}
    moved = float((want["far"][409] - want["none"][409]).abs().max() / want["far"][409].abs().max())
    assert moved > 500 * TOL["float32"], moved
    eng = engine_of(folder, "float32", page_size=16, max_cached_tokens=1344, max_num_batched_tokens=1024)
    for steps in (whole(reqs), one_by_one(reqs, 400), in_portions(reqs, [250, 2, 129, 37])):
        assert_close(replay(eng, steps), want, TOL["float32"])
    eng16 = engine_of(folder, "bfloat16", page_size=16, max_cached_tokens=1344, max_num_batched_tokens=1024)
    assert_close(replay(eng16, one_by_one(reqs, 405)), want, TOL["bfloat16"], {r: P.closest_call(w, cfg, ids) for r, ids in reqs.items()})


def test_a_layer_that_reads_another_layers_rows():
    """Two layers over the same compressed rows: the second has no rows of its own, and what it reads are the first
    one's, not rows made of its own input."""
    raw = M.model(47, 32, [M.layer(M.latent(2, 8, 12, 24, 1.2), M.dense(16)), M.layer(M.latent(4, 6, 4, 24, 1.6, kv_from=0))],
                  mult=0.7)
    folder, cfg, w = _folder_of(raw, 35)
    ids = random_ids(47, 70, seed=2)
    want = {"a": plain_rows(cfg, w, ids)}
    eng = engine_of(folder, "float32", page_size=4)
    assert [len(c) for c in eng.model.cache_specs()] == [1, 0] and len(eng.cache.page_groups) == 1
    for steps in (whole({"a": ids}), one_by_one({"a": ids}, 50), in_portions({"a": ids}, [9, 2, 30])):
        assert_close(replay(eng, steps), want, TOL["float32"])


@pytest.mark.parametrize("kind", ["attention", "latent", "latent_wide"])
def test_each_mixer_alone(kind):
    mixer = {"attention": M.attention(6, 3, 20, 0.7, chunk=9, rot=12, base=33.0), "latent": M.latent(5, 7, 9, 19, 1.1),
             "latent_wide": M.latent(2, 24, 8, 200, 0.3)}[kind]
    raw = M.model(71, 40, [M.layer(mixer)], mult=1.3, softcap=5.0)
    folder, cfg, w = _folder_of(raw, 41)
    reqs = {r: random_ids(71, n, seed=n) for r, n in (("a", 70), ("b", 19))}
    want = {r: plain_rows(cfg, w, ids) for r, ids in reqs.items()}
    eng = engine_of(folder, "float32")
    for steps in (whole(reqs), in_portions(reqs, [5, 2, 30]), one_by_one(reqs, 4)):
        assert_close(replay(eng, steps), want, TOL["float32"])


# ----------------------------------------------------------------------------- each kernel alone


@pytest.mark.parametrize("hidden,dtype", [(48, torch.float32), (701, torch.float32), (2100, torch.bfloat16)])
def test_tanh_norm_with_two_pending_terms(hidden, dtype):
    from pyre_amd.hip import ops

    g = torch.Generator().manual_seed(hidden)
    n = 9
    resid = torch.randn(n, hidden, generator=g) * 3 + 1.5
    a, b = torch.randn(3, n, hidden, generator=g), torch.randn(1, n, hidden, generator=g)
    bias = torch.randn(hidden, generator=g)
    w = {"n": (1 + 0.3 * torch.randn(hidden, generator=g)).double(), "n.b": torch.randn(hidden, generator=g).double(),
         "n.alpha": torch.tensor(0.37, dtype=P.F)}
    w = {k: v.to(dtype).double() for k, v in w.items()}    # the parameters as the kernel holds them
    want_resid = resid.double() + 0.3 * (a.double().sum(0) + bias.double()) + 0.3 * b.double().sum(0)
    want_out = P.squash_norm(want_resid, w, "n")
    par = [w[k].to(dtype).reshape(-1).to(DEV) for k in ("n.alpha", "n", "n.b")]
    for bias_dev in (bias.to(DEV), None):          # with a pending bias (one element a thread) and without (four)
        if bias_dev is None:
            want_resid = want_resid - 0.3 * bias.double()
            want_out = P.squash_norm(want_resid, w, "n")
        r = resid.to(DEV)
        out = torch.empty(n, hidden, device=DEV, dtype=dtype)
        terms = ops.Partials(a.to(DEV), bias_dev, scale=0.3, more=ops.Partials(b.to(DEV), scale=0.3))
        ops.add_tanhnorm(r, terms, *par, out)
        tol = 1e-5 if dtype == torch.float32 else 1e-2
        assert float((r.cpu().double() - want_resid).abs().max()) < 1e-5 * float(want_resid.abs().max())
        assert float((out.cpu().double() - want_out).abs().max()) < tol * float(want_out.abs().max())
        # some rows only, the stream untouched
        r2 = resid.to(DEV)
        rows = torch.tensor([7, 0, 3], dtype=torch.int32, device=DEV)
        out2 = torch.empty(3, hidden, device=DEV, dtype=dtype)
        ops.add_tanhnorm(r2, terms, *par, out2, rows)
        assert torch.equal(r2.cpu(), resid)
        assert float((out2.cpu().double() - want_out[[7, 0, 3]]).abs().max()) < tol * float(want_out.abs().max())
    # nothing pending: the first layer's norm
    out3 = torch.empty(n, hidden, device=DEV, dtype=dtype)
    ops.add_tanhnorm(resid.to(DEV), None, *par, out3)
    assert float((out3.cpu().double() - P.squash_norm(resid.double(), w, "n")).abs().max()) < tol * float(want_out.abs().max())
    with pytest.raises(Exception):
        ops.add_rmsnorm(r, terms, par[1], 1e-6, out)


def test_gelu_gated_unit_and_softcap():
    from pyre_amd.hip import ops

    g = torch.Generator().manual_seed(5)
    n, inter = 6, 37
    gu = torch.randn(2, n, 2 * inter, generator=g) * 2
    total = gu.double().sum(0)
    want = P.gelu_tanh(total[:, :inter]) * total[:, inter:]
    out = torch.empty(n, inter, device=DEV)
    ops.clipped_glu(ops.Partials(gu.to(DEV)), out, n, 0.0, ops.GELU_TANH_SLOPE, 0.0, ops.GELU_TANH_CUBIC)
    assert float((out.cpu().double() - want).abs().max()) < 1e-5
    x = torch.randn(5, 33, generator=g) * 30
    y = x.to(DEV)
    ops.softcap_(y, 7.5)
    assert float((y.cpu().double() - 7.5 * torch.tanh(x.double() / 7.5)).abs().max()) < 1e-5


@pytest.mark.parametrize("rows", [1, 8, 40, 64, 100, 200])
def test_gelu_gated_unit_in_the_gate_up_products_epilogue(rows):
    from pyre_amd.hip import ops

    g = torch.Generator().manual_seed(rows)
    k, inter = 512, 384
    x = (torch.randn(rows, k, generator=g) * 0.5).bfloat16()
    w = (torch.randn(2 * inter, k, generator=g) * 0.08).bfloat16()
    both = x.double() @ w.double().T
    want = P.gelu_tanh(both[:, :inter]) * both[:, inter:]
    xd, wd = x.to(DEV), w.to(DEV)
    ran = 0
    for name, supports, fn in (("skinny", ops.gemm_skinny_supports, ops.gemm_skinny_silu_bf16),
                               ("mid", ops.gemm_mid_supports, ops.gemm_mid_silu_bf16)):
        if rows > (64 if name == "skinny" else 256) or not supports(rows, 2 * inter, k, xd.stride(0), wd.stride(0)):
            continue
        out = torch.zeros(rows, inter, device=DEV, dtype=torch.bfloat16)
        fn(xd, wd, out, rows, (0.0, ops.GELU_TANH_SLOPE, 0.0, ops.GELU_TANH_CUBIC))
        assert float((out.cpu().double() - want).abs().max()) < 1e-2 * float(want.abs().max()), name
        ran += 1
    assert ran


@pytest.mark.parametrize("experts,top,parts", [(5, 2, 1), (64, 8, 3), (70, 6, 2), (200, 1, 1), (3, 3, 1)])
def test_routing_and_the_experts_activation(experts, top, parts):
    from pyre_amd.hip import ops

    g = torch.Generator().manual_seed(experts)
    n, hidden, ff, shared = 13, 24, 6, 4
    h = torch.randn(n, hidden, generator=g).double()
    w = {"m.router": torch.randn(experts, hidden, generator=g).double() * 0.2}   # scores well inside (0, 1)
    z = (h @ w["m.router"].T).float()
    split = torch.randn(parts, n, experts, generator=g)
    split[0] = z - split[1:].sum(0)
    gates = torch.full((n, experts), 7.0, device=DEV)
    ops.route_topk(ops.Partials(split.contiguous().to(DEV)), gates, n, top)
    want = torch.zeros(n, experts, dtype=P.F)
    for t, chosen in enumerate(P.route(h, w, "m", top)):
        for e, weight in chosen:
            want[t, e] = weight
    assert float((gates.cpu().double() - want).abs().max()) < 1e-5
    assert int((gates != 0).sum()) == n * top
    up = torch.randn(2, n, experts * ff + shared, generator=g)
    act = torch.empty(n, experts * ff + shared, device=DEV)
    ops.expert_act(ops.Partials(up.to(DEV)), gates, act, n, experts, ff, shared)
    total = torch.relu(up.double().sum(0)) ** 2
    total[:, :experts * ff] *= gates.cpu().double().repeat_interleave(ff, dim=1)
    assert float((act.cpu().double() - total).abs().max()) < 1e-5 * float(total.abs().max())


def test_routing_tells_experts_apart_whose_scores_round_to_one():
    """Logits of 15 to 40: their sigmoids are all 1 in float32, the experts are still chosen by the larger logit."""
    from pyre_amd.hip import ops

    g = torch.Generator().manual_seed(3)
    n, experts, top = 9, 12, 3
    z = 15 + 25 * torch.rand(n, experts, generator=g)
    gates = torch.zeros(n, experts, device=DEV)
    ops.route_topk(ops.Partials(z[None].contiguous().to(DEV)), gates, n, top)
    chosen = (gates.cpu() > 0)
    want = torch.zeros(n, experts, dtype=torch.bool)
    want.scatter_(1, z.double().topk(top, dim=1).indices, True)
    assert torch.equal(chosen, want) and float((gates.cpu().sum(1) - 1).abs().max()) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,heads,din,dout", [(1, 3, 7, 19), (37, 5, 40, 24), (70, 2, 136, 300)])
def test_the_product_per_head(dtype, n, heads, din, dout):
    from pyre_amd.hip import ops

    g = torch.Generator().manual_seed(n)
    x = torch.randn(n + 2, heads * din + 3, generator=g).to(dtype)
    w = (torch.randn(heads, din, dout, generator=g) * 0.3).to(dtype)
    out = torch.zeros(n, heads * dout, device=DEV, dtype=dtype)
    ops.head_matmul(x.to(DEV), w.to(DEV), out, n)
    want = torch.einsum("nhi,hio->nho", x[:n, :heads * din].double().view(n, heads, din), w.double()).reshape(n, -1)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert float((out.cpu().double() - want).abs().max()) < tol * float(want.abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_what_stands_between_the_input_product_and_attention(dtype):
    from pyre_amd.hip import ops
    from pyre_amd.parts.rotary import rotary_tables

    g = torch.Generator().manual_seed(9)
    n, nq, nkv, d, rot, page, pages = 11, 4, 2, 10, 6, 4, 8
    width = (nq + nkv) * d
    parts = torch.randn(2, n, width + 5, generator=g)
    bias = torch.randn(width, generator=g)
    positions = torch.tensor([0, 1, 2, 3, 4, 500, 501, 77, 9, 10, 11], dtype=torch.int32)
    slots = torch.tensor([4, 5, 6, 7, 12, 0, 1, -1, 29, 30, 31], dtype=torch.int32)
    cos, sin = rotary_tables(rot, 50.0, 600, exact=True)
    full = (parts.double().sum(0)[:, 2:2 + width] + bias.double()).view(n, nq + nkv, d)
    turned = P.rotate(full, [int(p) for p in positions], rot, 50.0)
    q = torch.zeros(n, nq * d, device=DEV, dtype=dtype)
    kc = torch.zeros(pages, nkv, page, d, device=DEV, dtype=dtype)
    vc = torch.zeros_like(kc)
    ops.rope_tied_write(ops.Partials(parts.to(DEV), bias.to(DEV)), 2, q, kc, vc, cos.to(DEV), sin.to(DEV), rot, positions.to(DEV),
                        slots.to(DEV), n, nq, nkv, d, page)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    scale = float(full.abs().max())
    assert float((q.cpu().double().view(n, nq, d) - turned[:, :nq]).abs().max()) < tol * scale
    for t, slot in enumerate(slots.tolist()):
        if slot < 0:
            continue
        assert float((kc[slot // page, :, slot % page].cpu().double() - turned[t, nq:]).abs().max()) < tol * scale
        assert float((vc[slot // page, :, slot % page].cpu().double() - full[t, nq:]).abs().max()) < tol * scale
    assert int((kc != 0).any(-1).sum()) == 10 * nkv    # the token without a slot is stored nowhere
    # the compressed row
    qw, rank = 14, 9
    gain = (1 + 0.3 * torch.randn(rank, generator=g))
    q2 = torch.zeros(n, qw, device=DEV, dtype=dtype)
    cc = torch.zeros(pages, 1, page, rank, device=DEV, dtype=dtype)
    ops.latent_write(ops.Partials(parts.to(DEV)), 1, q2, cc, gain.to(dtype).to(DEV), 1e-3, slots.to(DEV), n, qw, rank, page)
    total = parts.double().sum(0)[:, 1:]
    assert float((q2.cpu().double() - total[:, :qw]).abs().max()) < tol * scale
    rows = P.unit_rms(total[:, qw:qw + rank], 1e-3) * gain.to(dtype).double()
    for t, slot in enumerate(slots.tolist()):
        if slot >= 0:
            assert float((cc[slot // page, 0, slot % page].cpu().double() - rows[t]).abs().max()) < tol * float(rows.abs().max())


@pytest.mark.parametrize("nq,nkv,dk,dv,chunk", [(4, 2, 64, 64, 0), (6, 1, 128, 128, 0), (3, 3, 24, 40, 37), (5, 1, 136, 136, 0),
                                                 (7, 1, 64, 64, 0), (14, 2, 32, 32, 50), (28, 1, 16, 16, 0)])
def test_attention_over_pages_in_16_bits_is_the_32_bit_one_rounded_once(nq, nkv, dk, dv, chunk):
    """Prompt tiles and single tokens of bfloat16 queries, keys and values against float64 on the same values: the
    16-bit kernels multiply exactly and keep scores and weights in float32, so what is left is the rounding of the
    output (two to the minus eight of a value's size), not that of the weights (which would grow with the scores)."""
    from pyre_amd.hip import ops

    g = torch.Generator().manual_seed(nq * dk)
    page, n = 16, 150
    pages = (n + page - 1) // page
    q = (torch.randn(n, nq * dk, generator=g)).bfloat16()
    k = (torch.randn(n, nkv, dk, generator=g)).bfloat16()
    v = k if dk == dv else (torch.randn(n, nkv, dv, generator=g)).bfloat16()
    order = torch.randperm(pages + 3, generator=g)[:pages].to(torch.int32)      # the request's pages lie anywhere
    kc = torch.zeros(pages + 3, nkv, page, dk, dtype=torch.bfloat16)
    vc = torch.zeros(pages + 3, nkv, page, dv, dtype=torch.bfloat16)
    for t in range(n):
        kc[order[t // page], :, t % page], vc[order[t // page], :, t % page] = k[t], v[t]
    scale = 2.0 / dk ** 0.5
    want = torch.zeros(n, nq, dv, dtype=P.F)
    visible = P.same_chunk(chunk) if chunk else P.causal
    for head in range(nq):
        kv = head // (nq // nkv)
        a = P.softmax_rows((q.double().view(n, nq, dk)[:, head] @ k.double()[:, kv].T) * scale, visible)
        want[:, head] = a @ v.double()[:, kv]
    want = want.reshape(n, -1)
    dev = lambda t: t.to(DEV)  # noqa: E731
    positions, seqs = torch.arange(n, dtype=torch.int32), torch.zeros(n, dtype=torch.int32)
    tiles = torch.tensor([[t0, min(32, n - t0)] for t0 in range(0, n, 32)], dtype=torch.int32)
    shape = (nq, nkv, dk, dv, page, scale, 0.0, None, 0, 0, 0)
    kcd, vcd = dev(kc), dev(vc)
    if dk == dv:
        vcd = kcd                                                                # one tensor as keys and values
    ulp = 2.0 ** -8
    if dk <= ops.ATTN_BIASED_TILE_MAX_KEY_HEAD:
        out = torch.zeros(n, nq * dv, device=DEV, dtype=torch.bfloat16)
        ops.attn_biased_tile(dev(q), out, kcd, vcd, None, 1.0, dev(tiles), len(tiles), dev(positions), dev(seqs),
                             dev(order.view(1, -1)), *shape, chunk=chunk)
        assert bool(((out.cpu().double() - want).abs() <= ulp * want.abs() + 1e-6).all())
    out = torch.zeros(n, nq * dv, device=DEV, dtype=torch.bfloat16)
    spans = ops.attn_biased_spans(pages, page, 0, 0, chunk)
    scratch = torch.empty(n * nq * spans * (dv + 2), device=DEV)
    ops.attn_biased_single(dev(q), out, kcd, vcd, None, 1.0, None, n, dev(positions), dev(seqs), dev(order.view(1, -1)), *shape,
                           scratch=scratch if spans > 1 else None, chunk=chunk)
    assert bool(((out.cpu().double() - want).abs() <= ulp * want.abs() + 1e-6).all())
    # some of the tokens only: other numbers of blocks, so other numbers of heads to a block, and the same rows
    for count in (60, 33, 7):
        some = torch.arange(n - count, n, dtype=torch.int32)
        out2 = torch.zeros(n, nq * dv, device=DEV, dtype=torch.bfloat16)
        ops.attn_biased_single(dev(q), out2, kcd, vcd, None, 1.0, dev(some), count, dev(positions), dev(seqs),
                               dev(order.view(1, -1)), *shape, scratch=scratch if spans > 1 else None, chunk=chunk)
        assert torch.equal(out2[n - count:], out[n - count:]) and not bool(out2[:n - count].any())


# ----------------------------------------------------------------------------- the entry points


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_scheduler(graphs, folders):
    from pyre_amd.api import generate, load_model

    folder, cfg, w = folders["small"]
    prompts = [random_ids(cfg["vocab"], n, seed=n + 1) for n in (1, 9, 40, 23)]
    eng, _ = load_model(str(folder), device=DEV, dtype="float32", page_size=8, max_cached_tokens=1024, max_num_seqs=4,
                        max_num_batched_tokens=64, prefill_chunk=16, use_graphs=graphs)
    got = generate(eng, prompts, max_new_tokens=30)
    for p, g in zip(prompts, got):
        assert len(g) == 30
        ids = list(p)
        for k, tok in enumerate(g):
            row = P.forward(w, cfg, ids)[-1]
            twin = int(row.argmax())
            if twin != tok:
                margin = float((row[twin] - row[tok]) / row.abs().max())
                assert margin < TOL["float32"], f"token {k} is {tok}, plainly {twin} (margin {margin:.2e})"
            ids.append(tok)
    assert all(g.allocator.num_used == 0 for g in eng.cache.page_groups) and eng.cache.slots.num_used == 0
    if graphs:
        assert eng.graph_replays > 0


def test_the_generate_program_as_a_process(folders, tmp_path):
    import subprocess
    import sys
    from pathlib import Path

    folder, cfg, w = folders["wide"]
    root = Path(__file__).resolve().parent.parent
    out = tmp_path / "res.json"
    proc = subprocess.run([sys.executable, str(root / "bin" / "pyre_generate"), "--model", str(folder), "--dtype", "float32",
                           "--prompt-ids", "7,3,3,41,9,60,5", "--prompt-ids", "11", "--tokens", "12", "--num-blocks", "32",
                           "--max-batch", "2", "--out", str(out)], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    res = json.loads(out.read_text())
    assert res["dtype"] == "float32" and [len(g) for g in res["generated"]] == [12, 12]
    for prompt, tokens in zip(res["prompts"], res["generated"]):
        ids = list(prompt)
        for k, tok in enumerate(tokens):
            row = P.forward(w, cfg, ids)[-1]
            twin = int(row.argmax())
            if twin != tok:
                margin = float((row[twin] - row[tok]) / row.abs().max())
                assert margin < TOL["float32"], f"token {k} is {tok}, plainly {twin} (margin {margin:.2e})"
            ids.append(tok)


@pytest.mark.parametrize("dtype,extra", [("float32", ("--page-size", "8", "--poison")), ("bfloat16", ("--graphs",))])
def test_trace_run_as_a_process(dtype, extra, folders, tmp_path):
    from test_trace_run_gpu import run_trace

    folder, cfg, w = folders["small"]
    vocab = cfg["vocab"]
    reqs = {"a": random_ids(vocab, 70, 1), "b": random_ids(vocab, 40, 2), "c": random_ids(vocab, 64, 3), "d": random_ids(vocab, 3, 4),
            "e": random_ids(vocab, 61, 5)}
    fed = {r: 0 for r in reqs}
    sizes = [13, 2, 30, 1, 7, 64, 3]
    live, waiting, steps, k, wanted = [], list(reqs), [], 0, {}
    while live or waiting:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in live:
            n = min(sizes[k % len(sizes)], len(reqs[r]) - fed[r])
            k += 1
            want = [] if k % 5 == 0 else list(range(0, n, 2))
            entries.append({"id": r, "tokens": reqs[r][fed[r]:fed[r] + n], "want": want})
            wanted.setdefault(len(steps), []).extend((r, fed[r] + x) for x in want)
            fed[r] += n
            if fed[r] == len(reqs[r]):
                end.append(r)
        steps.append({"step": len(steps), "entries": entries, "end": end})
        live = [r for r in live if r not in end]
    out = tmp_path / "out"
    run_trace(folder, dtype, out, 4 * 128, steps, extra)
    ref = {r: plain_rows(cfg, w, ids) for r, ids in reqs.items()}
    calls = {r: P.closest_call(w, cfg, ids) for r, ids in reqs.items()}
    checked = 0
    for st, rows in wanted.items():
        if not rows:
            assert not (out / f"{st}.f32").exists()
            continue
        got = torch.from_numpy(np.fromfile(out / f"{st}.f32", dtype="<f4").reshape(len(rows), vocab))
        for i, (r, pos) in enumerate(rows):
            if dtype == "bfloat16" and float(calls[r][pos]) < CLOSE_CALL:
                continue
            d = float((got[i] - ref[r][pos]).abs().max() / ref[r][pos].abs().max())
            assert d <= TOL[dtype], f"step {st} request {r} position {pos}: {d:.3e}"
            checked += 1
    assert checked > 50
