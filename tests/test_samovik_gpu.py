"""Samovik on the GPU against the plain implementation (tests/plain_samovik.py): every mechanism
alone, whole prompts, token-by-token decoding, portions, mixed batches with pages and state slots
used again, keys made to stand out at the places where a cache can lose one, long decoding, and
greedy generation through the entry point."""
import copy
import random

import numpy as np
import pytest
import torch

from tests import plain_samovik as P
from tests.helpers import steps_portions, steps_prefill_then_decode, steps_whole
from tests.samovik_helpers import CFG_A, CFG_B, CFG_C, CONFIGS, LIMIT, build, one_layer, rel_error, run_steps, typed, _latent, _moe

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]


def tokens_for(cfg, n, seed):
    rng = random.Random(seed)
    return [rng.randrange(cfg["vocab"]) for _ in range(n)]


def plain_logits(cfg, w, toks):
    return P.forward(toks, w, cfg).numpy()


def check_against_plain(got, cfg, w, reqs, dtype, what=""):
    """Every position within the limit.  In bfloat16 a router's close call may fall the other way (the
    rounding of its input is enough): positions where the plain router's margin is under 1% are only
    required to be finite, and there may be few of them."""
    for rid, toks in reqs.items():
        margins = []
        want = P.forward(toks, w, cfg, margins=margins).numpy()
        rows = got[rid]
        assert sorted(rows) == list(range(len(toks))), f"{what}: {rid} is missing positions"
        close = set()
        if dtype == "bfloat16" and margins:
            close = set(torch.nonzero(torch.stack(margins).min(0).values < 0.01).flatten().tolist())
            assert len(close) <= max(3, len(toks) // 5), f"{what}: too many close calls for a test: {len(close)} of {len(toks)}"
        assert all(np.isfinite(rows[p]).all() for p in rows)
        worst = max(rel_error(rows[p], want[p]) for p in rows if p not in close)
        first_bad = next((p for p in sorted(rows) if p not in close and rel_error(rows[p], want[p]) > LIMIT[dtype]), None)
        assert first_bad is None, f"{what} {dtype}: request {rid}: first wrong position {first_bad} of {len(toks)}, worst error {worst:.3e}"


# ---- every mechanism alone -------------------------------------------------------------------------
def _context(model, token_lists, page=16):
    from tensorline_amd.cache.manager import CacheManager
    from tensorline_amd.engine.batch import StepEntry
    from tensorline_amd.engine.runner import ModelRunner
    cache = CacheManager(model.cache_needs(), model.schedule, model.state_needs(), page_size=page, num_blocks=64,
                         max_requests=4, dtype=model.dtype, device=DEV)
    entries = []
    for i, toks in enumerate(token_lists):
        cache.add_request(i)
        cache.grow(i, len(toks))
        entries.append(StepEntry(i, toks, 0, [0]))
    r = ModelRunner(model, cache)
    packed = r.pack(entries)
    return r.context(packed, r._upload(packed.data))


MIXERS = [
    ("latent_attention", _latent(3, 24, 8, 40, 48, scaling={"factor": 3.0, "original": 32, "fast": 8.0, "slow": 1.0})),
    ("latent_attention", _latent(1, 10, 6, 7, 20, base=20.0)),
    ("latent_attention", _latent(5, 16, 16, 32, 112, base=1e6, scale=0.3)),        # rows of 128: the bfloat16 matrix-core kernels
    ("latent_attention", _latent(4, 32, 8, 16, 200, base=500.0)),                     # rows of 256
    ("latent_attention", _latent(18, 8, 8, 8, 140)),                                  # rows of 256, more heads than a tile of 16
    ("latent_attention", _latent(3, 16, 12, 20, 300, base=100.0)),                    # wider than 256: the plain wide-row kernel
    ("lightning", {"heads": 2, "dim": 24, "vdim": 48, "decay": [0.9, 0.999]}),
    ("lightning", {"heads": 1, "dim": 130, "vdim": 66, "decay": [1.0]}),
    ("lightning", {"heads": 3, "dim": 7, "vdim": 5, "decay": [0.1, 0.5, 0.7]}),
    ("wkv", {"heads": 3, "dim": 16, "decay_rank": 8}),
    ("wkv", {"heads": 1, "dim": 72, "decay_rank": 3}),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", range(len(MIXERS)))
def test_mixer_alone(case, dtype):
    kind, mixer = MIXERS[case]
    cfg = one_layer(kind, mixer, width=72)
    model, w = build(cfg, dtype, seed=case)
    lens = [37, 1, 150] if kind == "latent_attention" else [37, 1, 18]
    ctx, views = _context(model, [tokens_for(cfg, n, s) for s, n in enumerate(lens)])
    torch.manual_seed(case)
    h = torch.randn(sum(lens), 72).to(torch.bfloat16).float()
    got = model.blocks[0].mixer.forward(h.to(DEV).to(model.dtype), ctx, views[0]).float().cpu()
    fn = {"latent_attention": lambda x: P.latent_attention(x, w, "l0.mix.", mixer, 1e-6),
          "lightning": lambda x: P.lightning(x, w, "l0.mix.", mixer, 1e-6)[0],
          "wkv": lambda x: P.wkv(x, w, "l0.mix.", mixer, 1e-6)[0]}[kind]
    at = 0
    for n in lens:                                   # three sequences in one batch, each from its first token
        want = fn(h[at:at + n])
        # root mean square of the difference over that of the output (a single element of a head with a
        # small root mean square may be off by more in bfloat16 and says little)
        err = ((got[at:at + n] - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt()).item()
        assert err < (1e-5 if dtype == "float32" else 3e-2), f"{kind} {mixer}: sequence of {n}: {err:.3e}"
        at += n


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mlp", [_moe(6, 2, 40, 3.0, {"ff": 56, "limit": 1.5}), _moe(3, 3, 20, 0.5), _moe(7, 1, 36, 9.0, {"ff": 12, "limit": 0.25}),
                                 _moe(1, 1, 100, 2.0), _moe(40, 5, 16, 2.0)])
def test_routed_experts_alone(mlp, dtype):
    """Few rows (tiles of 16 rows) and many (tiles of 64), clamps that bite and clamps that do not."""
    cfg = one_layer("lightning", {"heads": 1, "dim": 8, "vdim": 8, "decay": [0.5]}, mlp, width=88)
    model, w = build(cfg, dtype, seed=3)
    ff = model.blocks[0].feed_forward
    for rows in (1, 5, 300):
        torch.manual_seed(rows)
        h = (torch.randn(rows, 88) * 2).to(torch.bfloat16).float()
        got = ff.forward(h.to(DEV).to(model.dtype), None).float().cpu()
        want = P.routed_experts(h, w, "l0.mlp.", mlp)
        err = (got - want).abs().max().item() / want.abs().max().item()
        assert err < (1e-5 if dtype == "float32" else 3e-2), f"{rows} rows: {err:.3e}"


def test_router_picks_the_largest_and_weighs_only_those():
    from tensorline_amd.ops import kernels
    z = torch.tensor([[0.5, 3.0, -1.0, 3.0, 2.0], [-4.0, -9.0, -2.0, -3.0, -8.0]], device=DEV)
    ids, wts = kernels.moe_route(z, 3)
    assert ids.tolist() == [[1, 3, 4], [2, 3, 0]]              # equal logits: the lower index first
    for r in range(2):
        want = torch.softmax(z[r, ids[r].long()], 0)
        assert torch.allclose(wts[r], want, atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
def test_dynamic_tanh_and_token_input_alone(dtype):
    cfg = one_layer("lightning", {"heads": 1, "dim": 8, "vdim": 8, "decay": [0.5]}, None, width=40, vocab=30, side=6)
    cfg["layers"] = cfg["layers"] * 3                       # three slices of the table
    model, w = build(cfg, dtype, seed=5)
    toks = tokens_for(cfg, 9, 1)
    ctx, _ = _context(model, [toks])
    x = (torch.randn(9, 40) * 3).float()
    res = torch.randn(9, 40).float()
    tol = 1e-5 if dtype == "float32" else 2e-2
    norm = model.blocks[1].mixer_norm
    xg = x.to(DEV)
    got = norm.forward(xg, res.to(DEV)).float().cpu()
    assert torch.allclose(xg.cpu(), x + res)                 # the residual is added in place, in float32
    assert (got - P.dynamic_tanh(x + res, w, "l1.norm1")).abs().max() < tol * 3
    rows = torch.tensor([4, 0, 8], dtype=torch.int32, device=DEV)
    got = model.final_norm.forward(xg, res.to(DEV), rows=rows).float().cpu()
    assert (got - P.dynamic_tanh((x + 2 * res)[[4, 0, 8]], w, "final.norm")).abs().max() < tol * 3
    for layer in (0, 2):
        xs = x.to(DEV).contiguous()
        carry = model.blocks[layer].token_input.forward(xs, res.to(DEV), ctx).cpu()
        want = P.token_side_input(x + res, torch.tensor(toks), w, layer, 6, 1e-6)
        assert ((xs.cpu() + carry) - want).abs().max() < tol * want.abs().max()


# ---- whole models in the four cuttings ---------------------------------------------------------------
CUTS = {"whole": steps_whole, "decode": lambda r: steps_prefill_then_decode(r, tail=9), "portions": steps_portions}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cut", list(CUTS))
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_cuttings_against_plain(name, cut, dtype):
    cfg = CONFIGS[name]
    model, w = build(cfg, dtype, seed=11)
    reqs = {"x": tokens_for(cfg, 75, 1), "y": tokens_for(cfg, 1, 2), "z": tokens_for(cfg, 34, 3)}
    got = run_steps(model, CUTS[cut](reqs), page_size=16 if name != "B" else 8, max_tokens=128)
    check_against_plain(got, cfg, w, reqs, dtype, f"{name} {cut}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_latent_wider_than_the_matrix_core_kernels_take(dtype):
    """kv_rank + rot_dim above 256 is served by the plain wide-row attention: whole, decoded, in portions and mixed."""
    cfg = {"architecture": "Samovik", "vocab": 90, "width": 80, "norm": {"eps": 1e-6}, "layers": [
        {"type": "latent_attention", "mixer": _latent(2, 24, 8, 16, 260, base=1000.0), "mlp": None},
        {"type": "wkv", "mixer": {"heads": 2, "dim": 16, "decay_rank": 4}, "mlp": _moe(4, 2, 24, 2.0)}]}
    model, w = build(cfg, dtype, seed=17)
    assert model.cache_needs()[0].planes[0].shape == (1, 272)
    reqs = {"x": tokens_for(cfg, 70, 1), "y": tokens_for(cfg, 2, 2), "z": tokens_for(cfg, 41, 3)}
    for name, cut in CUTS.items():
        check_against_plain(run_steps(model, cut(reqs), max_tokens=128), cfg, w, reqs, dtype, f"wide latent, {name}")
    got = run_steps(model, mixed_steps(reqs, random.Random(3)), max_tokens=192, max_requests=3)
    check_against_plain(got, cfg, w, reqs, dtype, "wide latent, mixed")


def mixed_steps(reqs, rng, live=4):
    """Up to ``live`` requests at a time; each step gives every live request a portion of a random size
    (two tokens and one among them); a finished request ends and the next one takes its slot and pages."""
    waiting, at, running, steps = list(reqs), {}, [], []
    while waiting or running:
        while waiting and len(running) < live:
            rid = waiting.pop(0)
            running.append(rid)
            at[rid] = 0
        entries, end = [], []
        for rid in list(running):
            if rng.random() < 0.2 and len(running) > 1:
                continue                                   # left out of this step, goes on later
            left = len(reqs[rid]) - at[rid]
            n = min(left, rng.choice([1, 1, 2, 2, 3, 7, 16, 17, 40]))
            entries.append({"id": rid, "tokens": reqs[rid][at[rid]:at[rid] + n], "want": list(range(n))})
            at[rid] += n
            if at[rid] == len(reqs[rid]):
                end.append(rid)
                running.remove(rid)
        if entries:
            steps.append({"entries": entries, "end": end})
    return steps


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype):
    cfg = CONFIGS[name]
    model, w = build(cfg, dtype, seed=12)
    rng = random.Random(5)
    reqs = {f"r{i}": tokens_for(cfg, n, 20 + i) for i, n in enumerate([50, 3, 33, 1, 64, 17, 48, 2, 31])}
    # a pool that holds four live requests and no more: every page and slot is handed out several times
    got = run_steps(model, mixed_steps(reqs, rng), page_size=16, max_tokens=4 * 64, max_requests=4)
    check_against_plain(got, cfg, w, reqs, dtype, f"{name} mixed")


def test_float32_bits_do_not_depend_on_the_cutting_in_recurrent_layers():
    """The recurrences walk a sequence token by token whatever the step brings: a position's state, and
    so its 32-bit logits, are the same bits for portions and for one token at a time (17 rows or more per
    step and 16 or fewer take different product kernels, so both runs stay at few rows)."""
    cfg = CFG_C
    model, _ = build(cfg, "float32", seed=2)
    reqs = {"a": tokens_for(cfg, 40, 9)}
    one = run_steps(model, steps_portions(reqs, sizes=(1,)))
    many = run_steps(model, steps_portions(reqs, sizes=(5, 2, 16, 3, 9)))
    for p in range(40):
        assert np.array_equal(one["a"][p], many["a"][p]), f"position {p}"


# ---- keys made to stand out ------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("place", [0, 1, 15, 16, 17, 255, 256, 300])
def test_a_far_key_that_takes_all_the_weight_is_found(place, dtype):
    """One layer of latent attention over 330 tokens.  The input rows are arranged so that the last
    token's query puts nearly all of its weight on the key at ``place`` (the first tokens, both sides of
    a page's border, hundreds of tokens back): the row whose key scores highest is moved there and the
    query is scaled up.  A cache that loses or misplaces that one key gives another output altogether.
    Checked for the key seen from inside a prompt portion and from a token decoded alone."""
    mixer = _latent(2, 16, 8, 24, 40, base=10000.0, scaling={"factor": 2.0, "original": 128, "fast": 16.0, "slow": 2.0})
    cfg = one_layer("latent_attention", mixer, width=64)
    _, w = build(cfg, "float32", seed=7, device="cpu")
    T = 330
    H, d, r, rank = 2, 16, 8, 40

    def scores(hh, wq):
        pos = torch.arange(T)
        q = (hh[-1:] @ wq.T).view(1, H, d + r)
        dkv = hh @ w["l0.mix.dkv"].T
        c = P.rms_divide(dkv[:, :rank], 1e-6) * w["l0.mix.dkv.norm"]
        kp = (c @ w["l0.mix.uk"].T).view(T, H, d)
        kr = P.rotate(dkv[:, None, rank:], pos, mixer["rot"])[:, 0]
        qr = P.rotate(q[..., d:], pos[-1:], mixer["rot"])
        return (torch.einsum("ihd,jhd->hj", q[..., :d], kp) + torch.einsum("ihd,jd->hj", qr, kr)) * mixer["scale"]

    for attempt in range(20):                              # until the row moved to ``place`` still wins there
        torch.manual_seed(1000 * attempt + place)
        h = torch.randn(T, 64).to(torch.bfloat16).float()
        best = int(scores(h, w["l0.mix.q"])[0, :-1].argmax())
        h[[best, place]] = h[[place, best]]
        sc = scores(h, w["l0.mix.q"])[0]
        gap = (sc[place] - torch.cat((sc[:place], sc[place + 1:])).max()).item()
        if gap > 0:
            break
    assert gap > 0
    sharpen = 2.0 ** np.ceil(np.log2(12.0 / gap))          # queries scaled so that the winner leads by 12 or more

    def edit(wts):
        wts["l0.mix.q"] *= sharpen
    model, w = build(cfg, dtype, seed=7, edit=edit)
    weight = torch.softmax(scores(h, w["l0.mix.q"]), -1)[0, place].item()
    assert weight > 0.9, f"the arrangement failed: the key at {place} has weight {weight:.3f}"
    want = P.latent_attention(h, w, "l0.mix.", mixer, 1e-6)[-1]
    mix = model.blocks[0].mixer
    hg = h.to(DEV).to(model.dtype)
    for tail in (1, 40):                                  # the query decoded alone; the query inside a portion of 40
        from tensorline_amd.cache.manager import CacheManager
        from tensorline_amd.engine.batch import StepEntry
        from tensorline_amd.engine.runner import ModelRunner
        cache = CacheManager(model.cache_needs(), model.schedule, model.state_needs(), page_size=16, num_blocks=24,
                             max_requests=2, dtype=model.dtype, device=DEV)
        cache.add_request("q")
        runner = ModelRunner(model, cache)
        out = None
        for lo, hi in ((0, T - tail), (T - tail, T)):
            cache.grow("q", hi)
            packed = runner.pack([StepEntry("q", [0] * (hi - lo), lo, [0])])
            ctx, views = runner.context(packed, runner._upload(packed.data))
            out = mix.forward(hg[lo:hi], ctx, views[0]).float().cpu()
        err = (out[-1] - want).abs().max().item() / want.abs().max().item()
        assert err < (1e-4 if dtype == "float32" else 4e-2), f"key at {place}, last {tail} tokens in their own step: {err:.3e}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_state_of_a_slow_decay_reaches_back_hundreds_of_tokens(dtype):
    """Linear attention with a decay of 1 and one token, far back, whose key and value are large: every
    later output is dominated by it, in prompts, across step borders and in a slot that was used before."""
    mixer = {"heads": 2, "dim": 16, "vdim": 24, "decay": [1.0, 0.999]}
    cfg = one_layer("lightning", mixer, None, width=48)
    model, w = build(cfg, dtype, seed=9)
    toks = tokens_for(cfg, 400, 3)

    def edit(wts):
        wts["embed"][toks[5]] *= 6.0
    toks = [t if (t != toks[5] or i == 5) else (t + 1) % cfg["vocab"] for i, t in enumerate(toks)]
    model, w = build(cfg, dtype, seed=9, edit=edit)
    reqs = {"first": tokens_for(cfg, 30, 8), "long": toks}
    steps = steps_whole({"first": reqs["first"]}) + steps_portions({"long": toks}, sizes=(3, 64, 2, 200, 1, 1, 50, 1))
    got = run_steps(model, steps, max_tokens=512, max_requests=1)          # one slot: "long" inherits it
    check_against_plain(got, cfg, w, reqs, dtype, "slow decay")


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
    for graphs in (False, True):
        got = run_steps(model, copy.deepcopy(steps), max_tokens=512, graphs=graphs)
        check_against_plain(got, cfg, w, reqs, dtype, f"long decoding, graphs={graphs}")


@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_entry_point(name, tmp_path):
    """``LLM.generate`` with its scheduler, portions under a small token budget, more requests than
    slots at a time, and graphs: in 32-bit the greedy tokens are the plain implementation's."""
    from tensorline_amd import LLM, SamplingParams
    from tensorline_amd.weights.random_init import write_random_model
    cfg = CONFIGS[name]
    folder = write_random_model(typed(cfg), str(tmp_path / "model"), seed=21)
    from safetensors import safe_open
    w = {}
    with safe_open(folder + "/model.safetensors", "pt") as f:
        for k in f.keys():
            w[k] = f.get_tensor(k).float()
    prompts = [tokens_for(cfg, n, 40 + n) for n in (41, 3, 77, 18, 1, 30)]
    want = []
    for p in prompts:
        seq = list(p)
        for _ in range(12):
            seq.append(int(P.forward(seq, w, cfg)[-1].argmax()))
        want.append(seq[len(p):])
    for options in (dict(graphs=False, max_batched_tokens=32, max_num_seqs=3), dict(graphs=True, max_batched_tokens=64, max_num_seqs=4)):
        llm = LLM(folder, dtype="float32", block_size=16, num_blocks=40, max_model_len=128, graph_warmup_tokens=0, **options)
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
    # the folder's config.json may leave the decay's bottleneck width to the tensor's shape
    raw = json.load(open(folder + "/config.json"))
    del raw["layers"][1]["mixer"]["decay_rank"]
    json.dump(raw, open(folder + "/config.json", "w"))
    from safetensors import safe_open
    w = {}
    with safe_open(folder + "/model.safetensors", "pt") as f:
        for k in f.keys():
            w[k] = f.get_tensor(k).float()
    prompts = [tokens_for(cfg, 19, 1), tokens_for(cfg, 4, 2)]
    want = []
    for p in prompts:
        seq = list(p)
        for _ in range(6):
            seq.append(int(P.forward(seq, w, cfg)[-1].argmax()))
        want.append(seq[len(p):])
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
