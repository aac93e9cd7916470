"""Tumitar on the GPU against the plain implementation (tests/plain_tumitar.py): every mechanism
alone, whole prompts, token-by-token decoding, portions, mixed batches with pages and state slots
used again, keys and states made to stand out at the places where a cache can lose them, long
decoding, and greedy generation through the entry point."""
import copy
import random

import numpy as np
import pytest
import torch

from tests import plain_tumitar as P
from tests.helpers import steps_portions, steps_prefill_then_decode, steps_whole
from tests.samovik_helpers import LIMIT, rel_error, run_steps
from tests.test_samovik_gpu import mixed_steps
from tests.tumitar_helpers import (CFG_A, CFG_B, CONFIGS, build, one_layer, run_steps_with_routes, typed, _dense, _left, _moe,
                                   _parallel, _right)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]


def tokens_for(cfg, n, seed):
    rng = random.Random(seed)
    return [rng.randrange(cfg["vocab"]) for _ in range(n)]


def run_and_check(model, steps, cfg, w, reqs, dtype, what="", **kw):
    """Run the steps and hold every position against the plain implementation.  In float32 the plain run
    routes by itself.  In bfloat16 a router's close call may fall the other way (the rounding of its input
    is enough) and then changes every later position through the states and caches: there the plain run is
    told which experts the framework chose, and every such choice must be the router's own or so close to
    it that rounding explains it (under a tenth of the root mean square of the token's logits)."""
    if dtype == "float32":
        got, routes = run_steps(model, steps, **kw), {}
    else:
        got, routes = run_steps_with_routes(model, steps, **kw)
    for rid, toks in reqs.items():
        regrets = []
        forced = iter(routes[rid]) if routes.get(rid) else None
        want = P.forward(toks, w, cfg, margins=regrets if forced is not None else None, forced=forced).numpy()
        if forced is not None:
            assert next(forced, None) is None, f"{what}: the framework routed more often than the plain run"
            worst_choice = float(torch.stack(regrets).max())
            assert worst_choice < 0.1, f"{what}: request {rid}: an expert {worst_choice:.2f} (in units of the logits' size) under the router's own was chosen"
        rows = got[rid]
        assert sorted(rows) == list(range(len(toks))), f"{what}: {rid} is missing positions"
        errs = {p: rel_error(rows[p], want[p]) for p in rows}
        first_bad = next((p for p in sorted(rows) if not errs[p] <= LIMIT[dtype]), None)
        assert first_bad is None, (f"{what} {dtype}: request {rid}: first wrong position {first_bad} of {len(toks)}, "
                                   f"worst error {max(errs.values()):.3e}")


def _session(model, page=16, blocks=64, slots=4):
    from tensorline_amd.cache.manager import CacheManager
    from tensorline_amd.engine.runner import ModelRunner
    cache = CacheManager(model.cache_needs(), model.schedule, model.state_needs(), page_size=page, num_blocks=blocks,
                         max_requests=slots, dtype=model.dtype, device=DEV)
    return cache, ModelRunner(model, cache)


def _step_context(cache, runner, portions):
    """``portions``: (request, first position, tokens).  Returns the step's context and cache views."""
    from tensorline_amd.engine.batch import StepEntry
    entries = []
    for rid, lo, n in portions:
        if lo == 0:
            cache.add_request(rid)
        cache.grow(rid, lo + n)
        entries.append(StepEntry(rid, [0] * n, lo, [0]))
    packed = runner.pack(entries)
    return runner.context(packed, runner._upload(packed.data))


def _rms_error(got, want):
    return ((got - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt()).item()


# ---- every mechanism alone -------------------------------------------------------------------------
MIXERS = [
    ("parallel", _parallel(_left(4, 2, 24, 40, every=7), _right(4, 16, 24, 2, conv=4, norm_groups=2))),
    ("parallel", _parallel(_left(1, 1, 10, 7, scale=1.3, every=1), _right(1, 5, 9, 1, conv=1), 1.0, 1.0)),   # all sizes odd, one of each, one tap
    ("parallel", _parallel(_left(6, 1, 64, 64, every=50), _right(6, 64, 128, 3, conv=4, norm_groups=6), 0.5, 0.5)),  # matrix-core attention, state of 128
    ("parallel", _parallel(_left(2, 2, 128, 32, scale=0.02, every=9), _right(2, 20, 200, 2, conv=7), 2.0, 0.1)),     # value size under the key size, state of 200
    ("parallel", _parallel(_left(18, 2, 32, 48, every=1000), _right(4, 8, 16, 4, conv=2, norm_groups=1), 1.0, 0.0)),  # nine query heads a group; values wider than keys
    ("rglru", {"width": 64, "blocks": 4, "conv": 3}),
    ("rglru", {"width": 90, "blocks": 1, "conv": 1}),
    ("rglru", {"width": 35, "blocks": 7, "conv": 6}),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", range(len(MIXERS)))
def test_mixer_alone(case, dtype):
    """Three sequences in one batch, each from its first token, then each continued by a second step of
    other sizes (one token among them): the mixer's outputs against the plain ones of the whole sequences."""
    kind, mixer = MIXERS[case]
    cfg = one_layer(kind, mixer, width=72)
    model, w = build(cfg, dtype, seed=case)
    first, second = [37, 1, 150], [1, 20, 3]
    torch.manual_seed(case)
    hs = [torch.randn(a + b, 72).to(torch.bfloat16).float() for a, b in zip(first, second)]
    fn = (lambda x: P.parallel_mixer(x, w, "l0.mix.", mixer, 1e-6)[0]) if kind == "parallel" else \
         (lambda x: P.rglru_mixer(x, w, "l0.mix.", mixer)[0])
    cache, runner = _session(model)
    mix = model.blocks[0].mixer
    ctx, views = _step_context(cache, runner, [(i, 0, n) for i, n in enumerate(first)])
    got1 = mix.forward(torch.cat([h[:n] for h, n in zip(hs, first)]).to(DEV).to(model.dtype), ctx, views[0]).float().cpu()
    ctx, views = _step_context(cache, runner, [(i, a, b) for i, (a, b) in enumerate(zip(first, second))])
    got2 = mix.forward(torch.cat([h[n:] for h, n in zip(hs, first)]).to(DEV).to(model.dtype), ctx, views[0]).float().cpu()
    at1 = at2 = 0
    for h, a, b in zip(hs, first, second):
        want = fn(h)
        got = torch.cat((got1[at1:at1 + a], got2[at2:at2 + b]))
        err = _rms_error(got, want)
        assert err < (1e-5 if dtype == "float32" else 3e-2), f"{kind} {mixer}: sequence of {a} + {b}: {err:.3e}"
        at1, at2 = at1 + a, at2 + b


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mlp", [_dense(136), _dense(7), _moe(6, 2, 40), _moe(3, 3, 20, scale=0.5), _moe(1, 1, 100, scale=3.0), _moe(40, 5, 16)])
def test_feed_forward_alone(mlp, dtype):
    """Few rows and many (the grouped product's tiles of 16 and of 64 rows)."""
    cfg = one_layer("rglru", {"width": 8, "blocks": 1, "conv": 1}, mlp, width=88)
    model, w = build(cfg, dtype, seed=3)
    ff = model.blocks[0].feed_forward
    for rows in (1, 5, 300):
        torch.manual_seed(rows)
        h = (torch.randn(rows, 88) * 2).to(torch.bfloat16).float()
        got = ff.forward(h.to(DEV).to(model.dtype), None).float().cpu()
        want = P.feed_forward(h, w, "l0.mlp.", mlp)
        err = (got - want).abs().max().item() / want.abs().max().item()
        assert err < (1e-5 if dtype == "float32" else 3e-2), f"{rows} rows: {err:.3e}"


def test_router_weighs_each_choice_by_its_own_score():
    from tensorline_amd.ops import kernels
    z = torch.tensor([[0.5, 3.0, -1.0, 3.0, 2.0], [-4.0, -9.0, -2.0, -3.0, -8.0]], device=DEV)
    ids, wts = kernels.moe_route(z, 3, "sigmoid", 1.5)
    assert ids.tolist() == [[1, 3, 4], [2, 3, 0]]              # equal logits: the lower index first
    for r in range(2):
        assert torch.allclose(wts[r], 1.5 * torch.sigmoid(z[r, ids[r].long()]), atol=1e-6)
    assert float(wts[0].sum()) > 1.5                            # nothing is renormalised


@pytest.mark.parametrize("taps", [1, 2, 4, 5])
def test_convolution_keeps_its_last_inputs_across_steps_of_any_size(taps):
    """Portions shorter than the taps reach back (one and two tokens), portions that start at a sequence's
    first token (zeros before it), two sequences in a step, and a slot that another request used before."""
    from tensorline_amd.ops import kernels
    C = 70
    torch.manual_seed(taps)
    w, b = torch.randn(C, taps), torch.randn(C)
    cfg = one_layer("rglru", {"width": C, "blocks": 1, "conv": taps}, width=32)
    model, _ = build(cfg, "float32", seed=0)
    cache, runner = _session(model, slots=2)
    state = cache.state[0]
    xs = {"a": torch.randn(30, C), "b": torch.randn(12, C)}
    want = {k: P.causal_conv(v, w, b)[0] for k, v in xs.items()}
    ctx, _ = _step_context(cache, runner, [("old", 0, 9)])                    # leaves its inputs in slot 0 ...
    kernels.causal_conv(torch.randn(9, C, device=DEV), w.to(DEV), b.to(DEV), ctx, state, C, act="none")
    cache.release("old")                                                      # ... which "a" gets, zeroed
    at = {"a": 0, "b": 0}
    for step in ([("a", 1), ("b", 5)], [("a", 2)], [("a", 1), ("b", 1)], [("b", 2), ("a", 19)], [("a", 7), ("b", 4)]):
        ctx, _ = _step_context(cache, runner, [(r, at[r], n) for r, n in step])
        x = torch.cat([xs[r][at[r]:at[r] + n] for r, n in step])
        got = kernels.causal_conv(x.to(DEV), w.to(DEV), b.to(DEV), ctx, state, C, act="none").cpu()
        row = 0
        for r, n in step:
            assert torch.allclose(got[row:row + n], want[r][at[r]:at[r] + n], atol=1e-5), f"{r} at {at[r]}, {n} tokens"
            row, at[r] = row + n, at[r] + n
    assert at == {"a": 30, "b": 12}


# ---- whole models in the cuttings ----------------------------------------------------------------------
CUTS = {"whole": steps_whole, "decode": lambda r: steps_prefill_then_decode(r, tail=9), "portions": steps_portions}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cut", list(CUTS))
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_cuttings_against_plain(name, cut, dtype):
    cfg = CONFIGS[name]
    model, w = build(cfg, dtype, seed=11)
    reqs = {"x": tokens_for(cfg, 75, 1), "y": tokens_for(cfg, 1, 2), "z": tokens_for(cfg, 34, 3)}
    run_and_check(model, CUTS[cut](reqs), cfg, w, reqs, dtype, f"{name} {cut}", page_size=16 if name != "B" else 8, max_tokens=128)


@pytest.mark.parametrize("dtype", DTYPES)
def test_portions_down_to_two_tokens_and_one(dtype):
    cfg = CFG_A
    model, w = build(cfg, dtype, seed=4)
    reqs = {"x": tokens_for(cfg, 61, 5)}
    for sizes in ((2,), (1,), (2, 1, 3), (17, 2, 2, 1, 30)):
        run_and_check(model, steps_portions(reqs, sizes=sizes), cfg, w, reqs, dtype, f"portions of {sizes}", max_tokens=128)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype):
    cfg = CONFIGS[name]
    model, w = build(cfg, dtype, seed=12)
    rng = random.Random(5)
    reqs = {f"r{i}": tokens_for(cfg, n, 20 + i) for i, n in enumerate([50, 3, 33, 1, 64, 17, 48, 2, 31])}
    # a pool that holds four live requests and no more: every page and slot is handed out several times
    run_and_check(model, mixed_steps(reqs, rng), cfg, w, reqs, dtype, f"{name} mixed", page_size=16, max_tokens=4 * 64, max_requests=4)


def test_a_request_alone_and_in_a_batch_give_the_same_logits():
    cfg = CFG_A
    model, _ = build(cfg, "float32", seed=2)
    reqs = {"a": tokens_for(cfg, 40, 9), "b": tokens_for(cfg, 23, 8), "c": tokens_for(cfg, 5, 7)}
    alone = {r: run_steps(model, steps_portions({r: t}, sizes=(6, 1, 9)))[r] for r, t in reqs.items()}
    rng = random.Random(1)
    together = run_steps(model, mixed_steps(reqs, rng), max_tokens=192, max_requests=3)
    for r, t in reqs.items():
        for p in range(len(t)):
            assert rel_error(together[r][p], alone[r][p]) < 2e-6, f"{r} at {p}"


def test_float32_bits_do_not_depend_on_the_cutting_in_recurrent_layers():
    """The recurrences and the convolutions walk a sequence token by token whatever the step brings: a
    position's state, and so its 32-bit logits, are the same bits for portions and for one token at a time
    (17 rows or more per step and 16 or fewer take different product kernels, so both runs stay at few rows)."""
    cfg = {"architecture": "Tumitar", "vocab": 64, "width": 48, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0},
           "loop": {"start": 0, "stop": 1, "times": 2},
           "layers": [{"type": "rglru", "mixer": {"width": 40, "blocks": 2, "conv": 4}, "mlp": _dense(24)}]}
    model, _ = build(cfg, "float32", seed=2)
    reqs = {"a": tokens_for(cfg, 40, 9)}
    one = run_steps(model, steps_portions(reqs, sizes=(1,)))
    many = run_steps(model, steps_portions(reqs, sizes=(5, 2, 16, 3, 9)))
    for p in range(40):
        assert np.array_equal(one["a"][p], many["a"][p]), f"position {p}"


# ---- keys and states made to stand out -----------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("place", [0, 1, 15, 16, 17, 255, 256, 300])
def test_a_far_key_that_takes_all_the_weight_is_found(place, dtype):
    """The attention side alone (the other side's scale is 0) over 330 tokens.  The input rows are arranged so
    that the last token's query puts nearly all of its weight on the key at ``place`` (the first tokens, both
    sides of a page's border, hundreds of tokens back): the row whose key scores highest is moved there and
    the query's norm weight is scaled up (the projection itself is normed away).  A cache that loses or
    misplaces that one key gives another output altogether; the sink, which would take the weight of a lost
    key, gives nearly zero.  Checked for the key seen from inside a prompt portion and from a token decoded
    alone."""
    left = _left(2, 1, 16, 24, scale=0.25, coef=0.2, every=50)
    mixer = _parallel(left, _right(1, 8, 8, 1, conv=2), 1.0, 0.0)
    cfg = one_layer("parallel", mixer, width=64)
    _, w = build(cfg, "float32", seed=7, device="cpu")
    T, p = 330, "l0.mix.left."

    def scores(hh, wts):
        q = P.rms_norm(hh[-1:] @ wts[p + "q"].T + wts[p + "q.b"], wts[p + "q.norm"], 1e-6) * P.query_temperature(torch.tensor([T - 1]), 0.2, 50).float()
        k = P.rms_norm(hh @ wts[p + "k"].T + wts[p + "k.b"], wts[p + "k.norm"], 1e-6)
        return (q.view(2, 16) @ k.T) * 0.25                                  # [heads, T]

    for attempt in range(20):                              # until the row moved to ``place`` still wins there
        torch.manual_seed(1000 * attempt + place)
        h = torch.randn(T, 64).to(torch.bfloat16).float()
        best = int(scores(h, w)[0, :-1].argmax())
        h[[best, place]] = h[[place, best]]
        sc = scores(h, w)[0]
        gap = (sc[place] - torch.cat((sc[:place], sc[place + 1:])).max()).item()
        if gap > 0 and sc[place] > 0:
            break
    assert gap > 0 and sc[place] > 0
    sharpen = 2.0 ** np.ceil(np.log2(12.0 / min(gap, sc[place].item())))       # the winner leads every key and the sink by 12 or more

    def edit(wts):
        wts[p + "q.norm"] *= sharpen
    model, w = build(cfg, dtype, seed=7, edit=edit)
    sc = torch.cat((scores(h, w)[0], torch.zeros(1)))
    weight = torch.softmax(sc, -1)[place].item()
    assert weight > 0.9, f"the arrangement failed: the key at {place} has weight {weight:.3f}"
    want = P.parallel_mixer(h, w, "l0.mix.", mixer, 1e-6)[0][-1]
    mix = model.blocks[0].mixer
    hg = h.to(DEV).to(model.dtype)
    for tail in (1, 40):                                  # the query decoded alone; the query inside a portion of 40
        cache, runner = _session(model, blocks=24, slots=2)
        out = None
        for lo, hi in ((0, T - tail), (T - tail, T)):
            ctx, views = _step_context(cache, runner, [("q", lo, hi - lo)])
            out = mix.forward(hg[lo:hi], ctx, views[0]).float().cpu()
        err = (out[-1] - want).abs().max().item() / want.abs().max().item()
        assert err < (1e-4 if dtype == "float32" else 4e-2), f"key at {place}, last {tail} tokens in their own step: {err:.3e}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_sink_takes_the_weight_when_no_key_scores(dtype):
    """Scores far below zero: the sink holds nearly all of the weight and the attention side gives nearly
    nothing, in a prompt and decoded; a softmax without the sink would give an average of the values."""
    left = _left(2, 2, 16, 16, scale=4.0, coef=0.0, every=1)
    mixer = _parallel(left, _right(1, 8, 8, 1, conv=2), 1.0, 0.0)
    cfg = one_layer("parallel", mixer, width=32)

    def edit(wts):                                         # queries and keys of opposite sign: every score is negative
        wts["l0.mix.left.q"].zero_(), wts["l0.mix.left.k"].zero_()
        wts["l0.mix.left.q.b"].fill_(1.0), wts["l0.mix.left.k.b"].fill_(-1.0)
        wts["l0.mix.left.q.norm"].fill_(1.0), wts["l0.mix.left.k.norm"].fill_(1.0)
    model, w = build(cfg, dtype, seed=1, edit=edit)
    h = torch.randn(40, 32).to(torch.bfloat16).float()
    want = P.parallel_mixer(h, w, "l0.mix.", mixer, 1e-6)[0]
    loud = (h @ w["l0.mix.left.v"].T + w["l0.mix.left.v.b"]) @ w["l0.mix.left.o"].T
    assert want.abs().max() < 1e-6 * loud.abs().max()
    cache, runner = _session(model)
    ctx, views = _step_context(cache, runner, [("q", 0, 39)])
    got = model.blocks[0].mixer.forward(h[:39].to(DEV).to(model.dtype), ctx, views[0]).float().cpu()
    ctx, views = _step_context(cache, runner, [("q", 39, 1)])
    got = torch.cat((got, model.blocks[0].mixer.forward(h[39:].to(DEV).to(model.dtype), ctx, views[0]).float().cpu()))
    assert got.abs().max() < 1e-5 * loud.abs().max()


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_state_that_hardly_decays_reaches_back_hundreds_of_tokens(dtype):
    """The state-space side alone (the attention side's scale is 0) with a rate near zero: the state adds up
    all the tokens of a sequence and the first hundreds weigh as much at the end as the last ones, in
    prompts, across step borders and in a slot that was used before."""
    mixer = _parallel(_left(1, 1, 16, 16), _right(2, 12, 16, 1, conv=3, norm_groups=1), 0.0, 6.0)
    cfg = one_layer("parallel", mixer, None, width=48)
    toks = tokens_for(cfg, 400, 3)

    def edit(wts):
        wts["l0.mix.right.A_log"].fill_(-12.0)
    model, w = build(cfg, dtype, seed=9, edit=edit)
    reqs = {"first": tokens_for(cfg, 30, 8), "long": toks}
    steps = steps_whole({"first": reqs["first"]}) + steps_portions({"long": toks}, sizes=(3, 64, 2, 200, 1, 1, 50, 1))
    run_and_check(model, steps, cfg, w, reqs, dtype, "slow decay", max_tokens=512, max_requests=1)   # one slot: "long" inherits it
    assert rel_error(P.forward(toks[300:], w, cfg)[-1].numpy(), P.forward(toks, w, cfg)[-1].numpy()) > 2 * LIMIT[dtype], \
        "the first 300 tokens do not show at the end: the test would not see a lost state"


# ---- long decoding, graphs, the entry point ------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_eager_and_from_graphs(dtype):
    cfg = CFG_A
    model, w = build(cfg, dtype, seed=13)
    reqs = {"a": tokens_for(cfg, 150, 1), "b": tokens_for(cfg, 140, 2)}
    steps = [{"entries": [{"id": r, "tokens": t[:6], "want": list(range(6))} for r, t in reqs.items()], "end": []}]
    for i in range(6, 150):
        entries = [{"id": r, "tokens": [t[i]], "want": [0]} for r, t in reqs.items() if i < len(t)]
        steps.append({"entries": entries, "end": [r for r, t in reqs.items() if i == len(t) - 1]})
    run_and_check(model, copy.deepcopy(steps), cfg, w, reqs, dtype, "long decoding", max_tokens=512)
    # a replayed step computes what its eager twin computes
    eager = run_steps(model, copy.deepcopy(steps), max_tokens=512)
    replayed = run_steps(model, copy.deepcopy(steps), max_tokens=512, graphs=True)
    for rid, toks in reqs.items():
        for p in range(len(toks)):
            assert rel_error(replayed[rid][p], eager[rid][p]) < 1e-6, f"{rid} at {p}: a graph's step differs from the eager one"


def _greedy(cfg, w, prompts, n):
    want = []
    for p in prompts:
        seq = list(p)
        for _ in range(n):
            seq.append(int(P.forward(seq, w, cfg)[-1].argmax()))
        want.append(seq[len(p):])
    return want


def _folder_weights(folder):
    from safetensors import safe_open
    w = {}
    with safe_open(folder + "/model.safetensors", "pt") as f:
        for k in f.keys():
            w[k] = f.get_tensor(k).float()
    return w


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_point(name, tmp_path):
    """``LLM.generate`` with its scheduler, portions under a small token budget, more requests than
    slots at a time, and graphs: in 32-bit the greedy tokens are the plain implementation's."""
    from tensorline_amd import LLM, SamplingParams
    from tensorline_amd.weights.random_init import write_random_model
    cfg = CONFIGS[name]
    folder = write_random_model(typed(cfg), str(tmp_path / "model"), seed=21)
    w = _folder_weights(folder)
    prompts = [tokens_for(cfg, n, 40 + n) for n in (41, 3, 77, 18, 1, 30)]
    want = _greedy(cfg, w, prompts, 12)
    for options in (dict(graphs=False, max_batched_tokens=32, max_num_seqs=3), dict(graphs=True, max_batched_tokens=64, max_num_seqs=4)):
        llm = LLM(folder, dtype="float32", block_size=16 if name == "A" else 8, num_blocks=40 if name == "A" else 80,
                  max_model_len=128, graph_warmup_tokens=0, **options)
        outs = llm.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0))
        assert [o.token_ids for o in outs] == want
        assert llm.cache.all_free()


def test_command_line_random_model_generate_and_trace_program(tmp_path):
    """The programs a user runs: ``tensorline random-model`` from a config.json, ``tensorline generate`` on the
    folder (greedy, and sampled with a seed twice), and ``bin/trace_run`` fed steps on its standard input."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = copy.deepcopy(CFG_B)
    (tmp_path / "cfg.json").write_text(json.dumps(cfg))
    tl = [sys.executable, os.path.join(root, "bin", "tensorline")]
    folder = str(tmp_path / "m")
    proc = subprocess.run(tl + ["random-model", "--config", str(tmp_path / "cfg.json"), "--out", folder, "--seed", "4"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    w = _folder_weights(folder)
    prompts = [tokens_for(cfg, 19, 1), tokens_for(cfg, 4, 2)]
    want = _greedy(cfg, w, prompts, 6)
    base = tl + ["generate", "--model", folder, "--dtype", "float32", "--num-blocks", "32", "--block-size", "8",
                 "--max-tokens", "6", "--stop-token-id", "-1"]
    for p in prompts:
        base += ["--prompt-ids", " ".join(map(str, p))]
    proc = subprocess.run(base, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    recs = [json.loads(l) for l in proc.stdout.splitlines() if l.startswith("{")]
    assert [r["token_ids"] for r in recs] == want
    sampled = []
    for _ in range(2):
        proc = subprocess.run(base + ["--temperature", "0.9", "--top-p", "0.8", "--seed", "7"], capture_output=True, text=True, timeout=300)
        assert proc.returncode == 0, proc.stderr[-2000:]
        sampled.append([json.loads(l)["token_ids"] for l in proc.stdout.splitlines() if l.startswith("{")])
    assert sampled[0] == sampled[1] and all(len(t) == 6 for t in sampled[0])
    # the trace program: a prompt in two portions, then one token; logits at three places
    toks = prompts[0]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:7], "want": [6]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[7:18], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": toks[18:], "want": [0]}], "end": ["a"]}]
    out = tmp_path / "out"
    proc = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(out),
                           "--max-tokens", "64"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    ref = P.forward(toks, w, cfg).numpy()
    assert not (out / "1.f32").exists()
    for step, place in ((0, 6), (2, 18)):
        got = np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(1, -1)
        assert rel_error(got[0], ref[place]) < LIMIT["float32"]


# ---- seeded random configurations ----------------------------------------------------------------------------
@pytest.mark.parametrize("seed", range(14))
def test_random_configurations_in_mixed_batches(seed):
    """Sizes, head groupings, layer orders, loops and constants drawn from the seed, a page size of 8, 16 or 32,
    five requests cut at random over a pool that holds three: float32 for even seeds, bfloat16 for odd ones."""
    from tests.tumitar_helpers import random_config
    rng = random.Random(1000 + seed)
    cfg = random_config(rng)
    dtype = "float32" if seed % 2 == 0 else "bfloat16"
    model, w = build(cfg, dtype, seed=seed)
    reqs = {f"r{i}": tokens_for(cfg, n, 50 + i) for i, n in enumerate([rng.randint(1, 70) for _ in range(5)])}
    page = rng.choice([8, 16, 32])
    run_and_check(model, mixed_steps(reqs, rng, live=3), cfg, w, reqs, dtype, f"seed {seed}: {cfg}", page_size=page,
                  max_tokens=3 * 96, max_requests=3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_long_prompt_in_portions_then_decoded_across_the_key_splits(dtype):
    """2,300 tokens: a portion of 1,500, one of 700 behind it (its work-groups walk their keys as two chains of
    tiles), one of 64, then tokens decoded one by one, whose keys are split into runs that a second kernel merges:
    the sink's term enters once in each of these, and the states carry everything before.  The last position of
    every step is held against the plain implementation."""
    cfg = {"architecture": "Tumitar", "vocab": 150, "width": 64, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0}, "layers": [
        {"type": "parallel", "mixer": _parallel(_left(4, 2, 64, 64, scale=0.125, every=512), _right(2, 16, 16, 1, conv=4), 1.0, 0.5), "mlp": _dense(96)},
        {"type": "rglru", "mixer": {"width": 48, "blocks": 3, "conv": 4}, "mlp": None}]}
    model, w = build(cfg, dtype, seed=31)
    toks = tokens_for(cfg, 2300, 6)
    want = P.forward(toks, w, cfg).numpy()
    steps, at = [], 0
    for n in [1500, 700, 64] + [1] * 36:
        steps.append({"entries": [{"id": "a", "tokens": toks[at:at + n], "want": [n - 1]}], "end": ["a"] if at + n == len(toks) else []})
        at += n
    assert at == len(toks)
    got = run_steps(model, steps, max_tokens=2304)["a"]
    assert len(got) == len(steps)
    for p, row in got.items():
        assert rel_error(row, want[p]) < LIMIT[dtype], f"position {p}: {rel_error(row, want[p]):.3e}"


# ---- the state-space recurrence in chunks against the token-by-token walk -----------------------------------------
@pytest.mark.parametrize("case", [
    # heads, share, N, P, tokens of each sequence, first column of q and k in their matrix
    (4, 2, 32, 48, [150, 1, 64], 0),
    (6, 3, 128, 64, [333, 17], 4),
    (2, 1, 16, 8, [65, 128, 63, 2], 0),
    (3, 3, 64, 100, [200], 3),             # value size no multiple of 16; rows that start at no 16-byte border
    (8, 8, 48, 128, [70, 70], 8),
])
def test_state_space_recurrence_in_chunks_equals_the_walk(case, monkeypatch):
    """Prompt portions compute the state-space form in chunks of 64 tokens on the matrix cores; the walk computes it
    token by token.  Same operands, states that enter non-zero: outputs and the states left behind agree within
    float rounding, for chunks that are full, partial and single, several sequences in a step, and operands that
    are column blocks of wider matrices."""
    from types import SimpleNamespace
    from tensorline_amd.engine.batch import StepFacts
    from tensorline_amd.ops import kernels
    H, share, N, P, lens, col0 = case
    G, T = H // share, sum(lens)
    torch.manual_seed(sum(lens) + N)
    wide = torch.randn(T, col0 + 2 * G * N + 5, device=DEV)
    q, k = wide[:, col0:col0 + G * N], wide[:, col0 + G * N:col0 + 2 * G * N]
    v = torch.randn(T, H * P, device=DEV)
    steps, rate_log = torch.randn(T, H, device=DEV), torch.randn(H, device=DEV) - 1.0
    bias, skip = torch.randn(H, device=DEV), torch.randn(H, device=DEV)
    starts = [0]
    for n in lens:
        starts.append(starts[-1] + n)
    ctx = SimpleNamespace(
        facts=StepFacts(max_context=max(lens), max_query_len=max(lens), decode_only=False, num_seqs=len(lens), q_lens=list(lens),
                        starts=[0] * len(lens)),
        num_seqs=len(lens), state_slots=torch.arange(len(lens), dtype=torch.int32, device=DEV),
        q_start=torch.tensor(starts, dtype=torch.int32, device=DEV))
    state0 = torch.randn(len(lens) + 1, H * N * P + 7, device=DEV)

    def run():
        state = state0.clone()
        out = kernels.linear_recurrence(q, k, v, ctx, state, H, N, P, steps=steps, rate_log=rate_log, step_bias=bias, skip=skip,
                                        share=share)
        return out, state
    called = []
    call = kernels._call
    monkeypatch.setattr(kernels, "_call", lambda name, *a: (called.append(name), call(name, *a))[1])
    chunked, state_c = run()
    monkeypatch.setattr(kernels, "SSD_WALK_MAX_TOKENS", 1 << 30)
    walked, state_w = run()
    assert called == ["tl_ssd_chunked", "tl_linear_recurrence"]
    scale = walked.abs().max().item()
    assert (chunked - walked).abs().max().item() < 2e-5 * scale
    assert (state_c - state_w).abs().max().item() < 2e-5 * state_w.abs().max().item()
    assert torch.equal(state_c[:, H * N * P:], state0[:, H * N * P:])         # what lies behind the state is not touched
