"""Bikovik on the GPU against the plain implementation (tests/plain/bikovik_plain.py): the kernels
of each mechanism alone, one-layer models of each mixer, whole prompts against token-by-token
decoding and portions down to two tokens, mixed batches against each request alone with pages
and state slots that are freed and used again, the edges of the window and of the kept first
tokens in prompts and in decoding (with weights on which a window one key off shows, and a
control that it does), long decoding through replayed graphs, and generation through the
scheduler.  The 32-bit path is compared to a bound a little above its rounding, the bfloat16 path
to a bound some three times what it measures on these weights."""

from __future__ import annotations

import copy
import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from bikovik_cases import CASES, SINGLE, make_tensors, write_model
from helpers import feed, make_mixed_trace, max_live_tokens, random_tokens, rel_err, replay_in_process
from plain import bikovik_plain as plain

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
F64 = torch.float64

# Bounds on max |engine - plain| / max |plain logit| over a request, some three times the largest error
# measured on the MI355X on these weights: float32 3.9e-6 (case B; the others below 1.1e-6); bfloat16 7.5e-3
# (A), 2.0e-3 (C, one-layer attention), 1.1e-2 (one-layer HGRN2), 2.2e-3 (one-layer retention) and 3.3e-2 for
# case B, whose soft cap of 8 makes the largest logit small and whose gated unit clamps at 0.7, where a
# rounded bfloat16 input lands on the other side of the bound.  The cuttings of a request agree with each
# other to all printed digits in both precisions.
TOL = {"float32": 1.5e-5, "bfloat16": 3.5e-2}
TOL_CASE = {("B", "bfloat16"): 1e-1}


def tol(dtype, name=None):
    return TOL_CASE.get((name, dtype), TOL[dtype])


def K():
    from lockstep_amd.ops import kernels
    return kernels()


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """(case, dtype, sharpen) -> (loaded model, plain model, raw config, page size), made once."""
    made = {}

    def get(name, dtype="float32", sharpen=1.0, table=CASES, seed=11):
        from lockstep_amd import load_model

        key = (name, dtype, sharpen, seed)
        if key not in made:
            case = table[name]
            tensors = make_tensors(case["raw"], seed=seed, sharpen=sharpen)
            folder = write_model(tmp_path_factory.mktemp(f"bikovik{name}"), case["raw"], tensors)
            made[key] = (load_model(folder, dtype=dtype), plain.PlainBikovik(case["raw"], tensors), case["raw"],
                         case["page_size"], folder)
        return made[key]

    return get


def new_cache(model, page_size, tokens=512, requests=4, poison=True):
    return model.make_cache(num_pages=-(-tokens // page_size), page_size=page_size, max_requests=requests,
                            max_tokens_per_request=tokens, poison_on_free=poison)


# ---------------------------------------------------------------------------
# the kernels of each mechanism alone
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dynamic_tanh_with_row_list_and_with_a_pending_addition(dtype):
    g = torch.Generator().manual_seed(0)
    h = torch.randn(7, 70, generator=g) * 3
    w, b, alpha = torch.randn(70, generator=g), torch.randn(70, generator=g), torch.tensor([0.37])
    parts = torch.randn(3, 7, 70, generator=g)
    want = plain.dynamic_tanh(h.double(), w.double(), b.double(), alpha.double())
    out = torch.empty(7, 70, dtype=dtype, device="cuda")
    K().dyt(h.cuda(), w.cuda(), b.cuda(), alpha.cuda(), out)
    tol = 1e-6 if dtype is torch.float32 else 1e-2
    assert rel_err(out.float().cpu(), want) < tol
    rows = torch.tensor([5, 0, 3], dtype=torch.int32)
    picked = torch.empty(3, 70, dtype=dtype, device="cuda")
    K().dyt(h.cuda(), w.cuda(), b.cuda(), alpha.cuda(), picked, rows.cuda())
    assert torch.equal(picked, out[rows.long().cuda()])
    stream = h.cuda()
    K().dyt(stream, w.cuda(), b.cuda(), alpha.cuda(), out, partials=parts.cuda())
    summed = h.double() + parts.double().sum(0)
    assert rel_err(stream.cpu(), summed) < 1e-6
    assert rel_err(out.float().cpu(), plain.dynamic_tanh(summed, w.double(), b.double(), alpha.double())) < tol
    only = h.cuda()
    K().dyt(only, None, None, None, None, partials=parts.cuda())
    assert torch.equal(only, stream)


def test_clamped_gated_unit_and_soft_cap_kernels():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(9, 2 * 50, generator=g) * 3
    out = torch.empty(9, 50, device="cuda")
    K().glu_clamped(x.cuda(), out, 1.5, 1.702)
    assert rel_err(out.cpu(), plain.clamped_gated_unit(x[:, :50].double(), x[:, 50:].double(), 1.5)) < 1e-6
    logits = (torch.randn(4, 300, generator=g) * 40)
    dev = logits.cuda()
    K().softcap(dev, 25.0)
    assert rel_err(dev.cpu(), plain.soft_cap(logits.double(), 25.0)) < 1e-6
    assert float(dev.abs().max()) <= 25.0


@pytest.mark.parametrize("heads, vdim", [(2, 40), (3, 64), (1, 200)])
def test_per_head_norm_with_and_without_weight_and_gate(heads, vdim):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(6, heads * vdim, generator=g) * 5
    w, gate = torch.randn(vdim, generator=g), torch.randn(6, heads * vdim, generator=g)
    normed = plain.root_mean_square_norm(x.double().view(6, heads, vdim), 1e-3)
    out = torch.empty(6, heads * vdim, device="cuda")
    K().head_norm_gate(x.cuda(), heads, vdim, w.cuda(), None, 1e-3, out)
    assert rel_err(out.cpu(), (normed * w.double()).reshape(6, -1)) < 1e-6
    K().head_norm_gate(x.cuda(), heads, vdim, None, gate.cuda(), 1e-3, out)
    assert rel_err(out.cpu(), normed.reshape(6, -1) * torch.nn.functional.silu(gate.double())) < 1e-6


class _Seqs:
    """The step's per-request rows as the kernels read them, for launches outside a model."""

    def __init__(self, lengths, starts, slots):
        rows, at = [], 0
        for n, s, slot in zip(lengths, starts, slots):
            rows.append([at, n, s, s + n, slot, 0, 0, 0])
            at += n
        self.dev = torch.tensor(rows, dtype=torch.int32).reshape(-1).cuda()
        self.positions = torch.tensor([s + i for n, s in zip(lengths, starts) for i in range(n)], dtype=torch.int32).cuda()
        self.n = len(lengths)


@pytest.mark.parametrize("heads, dim, vdim", [(2, 16, 32), (1, 40, 24), (3, 24, 100), (2, 128, 64)])
def test_recurrence_kernel_both_modes_over_unequal_requests_in_two_steps(heads, dim, vdim):
    """Three requests with their own state slots, fed in two steps of unequal portions (one request
    starts in the second step only): the state carries over, o_t equals the plain recurrence."""
    g = torch.Generator().manual_seed(3)
    total = [23, 5, 40]
    cut = [17, 0, 1]
    width = 2 * heads * dim + heads * vdim
    raws = [torch.randn(n, width, generator=g) for n in total]
    lower, f_bias = torch.rand(heads * dim, generator=g), torch.randn(heads * dim, generator=g)
    decay = torch.tensor([0.9, 0.99, 0.5][:heads])
    rot, base = (dim // 2) // 2 * 2, 100.0
    half = rot // 2
    positions = torch.arange(64)
    freq = torch.tensor([base ** (-2.0 * i / rot) for i in range(half)], dtype=F64)
    cos, sin = (positions.double()[:, None] * freq).cos().float().cuda(), (positions.double()[:, None] * freq).sin().float().cuda()
    for mode in (K().LINREC_HGRN2, K().LINREC_RETENTION):
        state = torch.full((4, heads, dim, vdim), float("nan"), device="cuda")
        state[[0, 2, 3]] = 0.0
        got = [[] for _ in total]
        for step in range(2):
            lengths = [c if step == 0 else n - c for n, c in zip(total, cut)]
            starts = [0 if step == 0 else c for c in cut]
            live = [i for i, n in enumerate(lengths) if n]
            seqs = _Seqs([lengths[i] for i in live], [starts[i] for i in live], [[0, 2, 3][i] for i in live])
            raw = torch.cat([raws[i][starts[i]:starts[i] + lengths[i]] for i in live]).cuda()
            out = torch.empty(raw.shape[0], heads * vdim, device="cuda")
            p0, p1 = (lower.cuda(), f_bias.cuda()) if mode == K().LINREC_HGRN2 else (decay.cuda(), None)
            gates = torch.empty(K().linrec_gate_floats(raw.shape[0], heads, dim), device="cuda")
            K().linrec(mode, raw, 0, heads * dim, 2 * heads * dim, heads, dim, vdim, p0, p1, cos, sin, rot, 63,
                       seqs.positions, seqs.dev, seqs.n, state, gates, out)
            at = 0
            for i in live:
                got[i].append(out[at:at + lengths[i]].cpu())
                at += lengths[i]
        assert bool(state[1].isnan().all())                 # a slot of no request is not touched
        for i, n in enumerate(total):
            r = raws[i].double()
            q = r[:, :heads * dim].view(n, heads, dim)
            ab = r[:, heads * dim:2 * heads * dim].view(n, heads, dim)
            v = r[:, 2 * heads * dim:].view(n, heads, vdim)
            for h in range(heads):
                if mode == K().LINREC_HGRN2:
                    lo = lower.double().view(heads, dim)[h]
                    f = lo + (1 - lo) * torch.sigmoid(ab[:, h] + f_bias.double().view(heads, dim)[h])
                    want, last = plain.gated_outer_product_recurrence(torch.nn.functional.silu(q[:, h]), f, 1 - f, v[:, h])
                else:
                    qr = plain.rotate_pairs(q[:, h:h + 1], torch.arange(n), rot, base)[:, 0]
                    kr = plain.rotate_pairs(ab[:, h:h + 1], torch.arange(n), rot, base)[:, 0] * dim ** -0.5
                    want, last = plain.gated_outer_product_recurrence(qr, decay.double()[h].expand(n, dim), kr, v[:, h])
                assert rel_err(torch.cat(got[i])[:, h * vdim:(h + 1) * vdim], want) < 2e-5, (mode, i, h)
                assert rel_err(state[[0, 2, 3][i], h].cpu(), last) < 2e-5


# ---------------------------------------------------------------------------
# one-layer models: each mixer alone, whole and cut
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("kind", ["attention", "hgrn2", "retention"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_each_mixer_alone_whole_and_in_portions(models, kind, dtype):
    model, oracle, raw, page, _ = models(kind, dtype, table=SINGLE)
    tokens = random_tokens(75, raw["vocab"], seed=4)
    want = oracle.forward(tokens)
    for cuts in ([], [2, 31, 2, 17, 1, 1, 1], [1] * 75):
        cache = new_cache(model, page)
        got = feed(model, cache, "r", tokens, cuts)
        assert rel_err(got, want) < TOL[dtype], (kind, cuts[:3])
        cache.close("r")
        cache.audit()


# ---------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_portions_and_token_by_token_agree_with_the_plain_model(models, name, dtype):
    model, oracle, raw, page, _ = models(name, dtype)
    tokens = random_tokens(150, raw["vocab"], seed=5)
    want = oracle.forward(tokens)
    runs = {}
    for label, cuts in (("whole", []), ("portions", [2, 47, 3, 16, 2, 33, 5, 1, 1, 2]), ("tail", [110] + [1] * 40),
                        ("single", [1] * 150)):
        cache = new_cache(model, page)
        runs[label] = feed(model, cache, "r", tokens, cuts)
        assert rel_err(runs[label], want) < tol(dtype, name), (name, label)
        cache.close("r")
        cache.audit()
    if dtype == "float32":              # the cuttings agree with each other far below the bound against the plain model
        for label in ("portions", "tail", "single"):
            assert rel_err(runs[label], runs["whole"]) < 1e-5, label


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_whose_late_row_blocks_are_cut_into_runs(models, dtype):
    """A window of a thousand keys and a prompt of 700 tokens: the late row blocks of the prompt see
    enough key tiles for the attention to deal them to several work items and fold the results (the
    buffer of partial results exists afterwards); decoding goes on from there."""
    model, oracle, raw, page, _ = models("B", dtype)
    tokens = random_tokens(720, raw["vocab"], seed=13)
    want = oracle.forward(tokens)
    for cuts in ([700] + [1] * 20, [333, 2, 365] + [1] * 20):
        cache = new_cache(model, page, tokens=1024)
        got = feed(model, cache, "r", tokens, cuts)
        assert rel_err(got, want) < tol(dtype, "B"), cuts[:3]
        cache.close("r")
    assert any(name == "talking.part" for name, _, _ in model.workspace._buffers)


@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens_and_prompts_of_one_and_two_tokens(models, name):
    model, oracle, raw, page, _ = models(name)
    for n in (1, 2, 3, page, page + 1):
        tokens = random_tokens(n, raw["vocab"], seed=20 + n)
        cache = new_cache(model, page)
        assert rel_err(feed(model, cache, "r", tokens, []), oracle.forward(tokens)) < TOL["float32"], n


@pytest.mark.parametrize("name, dtype", [("A", "float32"), ("B", "float32"), ("C", "float32"), ("A", "bfloat16")])
def test_mixed_batches_of_unequal_requests_with_pages_and_slots_used_again(models, name, dtype):
    """Seven requests of unequal lengths through four slots and a pool that holds the live ones only:
    portions beside single tokens, requests that sit steps out, finished requests whose (poisoned)
    pages and state slots the next ones take.  Each request's logits equal those of the request alone."""
    model, oracle, raw, page, _ = models(name, dtype)
    lengths = [1, 23, 97, 150, 61, 2, 130]
    requests = {f"r{i}": random_tokens(n, raw["vocab"], seed=40 + i) for i, n in enumerate(lengths)}
    steps = make_mixed_trace(requests, seed=3, max_live=4, decode_tail=12, max_portion=29)
    assert any(len(s["entries"]) > 1 and {len(e["tokens"]) for e in s["entries"]} != {1} for s in steps)
    tokens = max_live_tokens(steps, round_to=page)
    cache = model.make_cache(num_pages=-(-tokens // page), page_size=page, max_requests=4,
                             max_tokens_per_request=max(lengths) + page, poison_on_free=True)
    got = replay_in_process(model, cache, steps)
    assert cache.free_slots == 4 and all(g.pool.taken_total > g.pool.num_pages for g in cache.groups)
    for rid, toks in requests.items():
        assert rel_err(got[rid], oracle.forward(toks)) < tol(dtype, name), rid


# ---------------------------------------------------------------------------
# the window's edge and the kept first tokens, on weights that show them
# ---------------------------------------------------------------------------

PLANTED = 7          # the token id whose key every query answers


def _edge_case():
    """One attention layer and weights on which one key decides: the planted token's key gets a strong
    component along a direction (an unrotated dimension of every head) that the bias of every query
    points along, and its value a strong component of its own.  Wherever the planted token is visible
    its score stands out by e^40 among hundreds and the output is its value; where it is hidden the
    output is something else entirely.  A window or a number of kept tokens that is one off moves the
    logits at the edge by a large part of their size, in either precision."""
    raw = copy.deepcopy(SINGLE["attention"]["raw"])
    mixer = raw["layers"][0]["mixer"]
    mixer["mask"], mixer["rot"] = {"size": 37, "keep_first": 5}, {"dims": 16, "base": 10000.0}
    tensors = make_tensors(raw, seed=21)
    heads, groups, dim, vdim, at = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"], 20
    embedded = tensors["embed"][PLANTED].double() * raw["embedding"]["scale"]
    seen = plain.dynamic_tanh(embedded, tensors["l0.norm1"].double(), tensors["l0.norm1.b"].double(),
                              tensors["l0.norm1.alpha"].double())
    along = seen / seen.norm()
    k, v, qb = tensors["l0.mix.k"].float(), tensors["l0.mix.v"].float(), tensors["l0.mix.q.b"].float()
    g = torch.Generator().manual_seed(5)
    for group in range(groups):
        k[group * dim + at] += 8.0 * along.float()
        v[group * vdim:(group + 1) * vdim] += 3.0 * torch.randn(vdim, 1, generator=g) * along.float()[None, :]
    for head in range(heads):
        qb[head * dim + at] = 8.0
    tensors["l0.mix.k"], tensors["l0.mix.v"], tensors["l0.mix.q.b"] = k.bfloat16(), v.bfloat16(), qb.bfloat16()
    return raw, tensors


def _with_mask(raw, size, keep_first):
    other = copy.deepcopy(raw)
    other["layers"][0]["mixer"]["mask"] = {"size": size, "keep_first": keep_first}
    return other


def _sequence_with_planted(vocab, n, places, seed):
    tokens = [t if t != PLANTED else PLANTED + 1 for t in random_tokens(n, vocab, seed)]
    for p in places:
        tokens[p] = PLANTED
    return tokens


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_keys_just_inside_and_just_outside_the_window_and_the_kept_tokens(tmp_path, dtype):
    """Window 37, five kept tokens.  Three sequences: the planted token at 50 and 95 (queries 86 and
    131 are the last to see it, 87 and 132 the first not to), at 4 (the last kept place: seen for
    ever) and at 5 (the first place that is not kept: gone from query 42 on).  Controls: the plain
    model with the window or the kept tokens one off differs at those places by many times the
    bound.  The engine follows the plain model with the edges inside a prompt, inside portions cut
    at and around the edges, and in tokens decoded one by one, on pages of 8 and of 16."""
    from lockstep_amd import load_model

    raw, tensors = _edge_case()
    model = load_model(write_model(tmp_path / "edge", raw, tensors), dtype=dtype)
    oracle = plain.PlainBikovik(raw, tensors)
    bound = TOL[dtype]
    cases = [([50, 95], [(38, 5, 87), (36, 5, 86), (38, 5, 132), (36, 5, 131)]),
             ([4], [(37, 4, 41), (37, 4, 139)]),
             ([5], [(37, 6, 42), (37, 6, 139)])]
    for places, controls in cases:
        tokens = _sequence_with_planted(raw["vocab"], 140, places, seed=6 + places[0])
        want = oracle.forward(tokens)
        for size, keep, where in controls:
            moved = plain.PlainBikovik(_with_mask(raw, size, keep), tensors).forward(tokens)
            assert rel_err(moved[where], want[where]) > 3 * bound, (places, size, keep, where)
        for page in (8, 16):
            for cuts in ([], [80] + [1] * 60, [30] + [1] * 110, [37, 2, 36, 5, 2, 11, 2, 38]):
                cache = new_cache(model, page)
                got = feed(model, cache, "r", tokens, cuts)
                worst = (got.double() - want).abs().max(dim=1)[0] / want.abs().max()
                assert float(worst.max()) < bound, (places, page, cuts[:2], int(worst.argmax()))
                cache.close("r")
                cache.audit()


def test_a_far_key_that_a_recurrent_layer_must_still_hold(models):
    """A long request through the recurrent layers: the same prompt with one early token replaced
    moves the last logits (the state remembers it), and the engine follows the plain model in both."""
    model, oracle, raw, page, _ = models("B")
    tokens = random_tokens(260, raw["vocab"], seed=7)
    other = list(tokens)
    other[3] = (other[3] + 17) % raw["vocab"]
    want, want_other = oracle.forward(tokens), oracle.forward(other)
    assert rel_err(want_other[-20:], want[-20:]) > 20 * TOL["float32"]
    for toks, expected in ((tokens, want), (other, want_other)):
        cache = new_cache(model, page)
        got = feed(model, cache, "r", toks, [200] + [1] * 60)
        assert rel_err(got[-20:], expected[-20:]) < TOL["float32"]


# ---------------------------------------------------------------------------
# long decoding (replayed graphs), the device-side loop, generation through the scheduler
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("name", ["A", "C"])
def test_long_decoding_of_two_requests_through_replayed_graphs(models, name):
    from lockstep_amd.engine.batch import StepEntry

    model, oracle, raw, page, _ = models(name)
    a, b = random_tokens(230, raw["vocab"], seed=8), random_tokens(215, raw["vocab"], seed=9)
    cache = new_cache(model, page, tokens=512)
    cache.open("a"), cache.open("b")
    model.step(cache, [StepEntry("a", a[:30], []), StepEntry("b", b[:15], [])])
    replays = model.graph_replays
    rows = {"a": [], "b": []}
    for t in range(200):
        logits = model.step(cache, [StepEntry("a", [a[30 + t]], [0]), StepEntry("b", [b[15 + t]], [0])])
        rows["a"].append(logits[0].cpu()), rows["b"].append(logits[1].cpu())
    assert model.graph_replays - replays >= 150
    assert rel_err(torch.stack(rows["a"]), oracle.forward(a)[30:]) < TOL["float32"]
    assert rel_err(torch.stack(rows["b"]), oracle.forward(b)[15:]) < TOL["float32"]


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_scheduler_and_the_single_prompt_entry_point(models, name):
    from lockstep_amd import LLM, Request

    _, oracle, raw, page, folder = models(name, seed=12)
    prompts = [random_tokens(n, raw["vocab"], seed=60 + n) for n in (5, 41, 18)]
    want = [oracle.generate_greedy(p, 24) for p in prompts]
    llm = LLM(folder, dtype="float32", num_pages=64, page_size=page)
    got = llm.generate([Request(uid=f"r{i}", prompt=p, max_new_tokens=24) for i, p in enumerate(prompts)])
    assert [got[f"r{i}"] for i in range(3)] == want
    alone, _ = llm.generate_greedy(prompts[1], 24)
    assert alone == want[1]
    # the bfloat16 path generates too (its tokens may part from the exact ones after a near tie)
    half = LLM(folder, dtype="bfloat16", num_pages=64, page_size=page)
    tokens = half.generate([Request(uid="x", prompt=prompts[0], max_new_tokens=8)])["x"]
    assert len(tokens) == 8 and tokens[:2] == want[0][:2]


def test_trace_replay_program_on_a_model_folder(models, tmp_path):
    """bin/trace_run as a subprocess on a Bikovik folder: a mixed schedule through four slots."""
    _, oracle, raw, page, folder = models("A")
    requests = {f"q{i}": random_tokens(n, raw["vocab"], seed=80 + i) for i, n in enumerate([40, 3, 77, 52, 19])}
    steps = make_mixed_trace(requests, seed=5, max_live=4, decode_tail=6, max_portion=19)
    out = tmp_path / "out"
    proc = subprocess.Popen([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32",
                             "--out", str(out), "--max-tokens", str(max_live_tokens(steps)), "--page-size", str(page)],
                            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for step in steps:
            proc.stdin.write(json.dumps(step) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {step['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    rows: dict = {}
    for step in steps:
        data = np.fromfile(out / f"{step['step']}.f32", dtype="<f4").reshape(-1, raw["vocab"])
        at = 0
        for e in step["entries"]:
            rows.setdefault(e["id"], []).append(data[at:at + len(e["want"])])
            at += len(e["want"])
    for rid, toks in requests.items():
        assert rel_err(np.concatenate(rows[rid]), oracle.forward(toks)) < TOL["float32"], rid


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_preempted_requests_recompute_state_and_pages_to_the_same_tokens(models, dtype):
    """The scheduler preempts one request twice while two others run beside it (one of them draws
    its tokens): its pages and its state slot are given back, its context runs again in portions
    from an empty state, and every request's tokens and logits are those of the request alone."""
    from lockstep_amd import Request, Scheduler
    from lockstep_amd.engine.policy import PreemptAtStepsPolicy

    model, oracle, raw, page, _ = models("A", dtype, seed=12)
    vocab = raw["vocab"]
    wave = [Request(uid="p0", prompt=random_tokens(2 * page + 3, vocab, seed=41), max_new_tokens=14),
            Request(uid="p1", prompt=random_tokens(37, vocab, seed=42), max_new_tokens=9),
            Request(uid="p2", prompt=random_tokens(5, vocab, seed=43), max_new_tokens=12, temperature=0.9, seed=7)]

    def alone(request):
        s = Scheduler(model, num_blocks=16, block_size=page, keep_logits=True, audit=False)
        s.submit(Request(**vars(request)))
        return s.run()[request.uid], torch.stack(s.emitted_logits[request.uid])

    policy = PreemptAtStepsPolicy("p0", (5, 9), chunk=page + 3)
    cache = model.make_cache(num_pages=40, page_size=page, max_requests=4, poison_on_free=True)
    s = Scheduler(model, num_blocks=40, block_size=page, cache=cache, keep_logits=True, audit=True, policy=policy,
                  max_batched_tokens=40)
    for r in wave:
        s.submit(Request(**vars(r)))
    out = s.run()
    s.counters.require_fired("preempt_fired", "resume", "prefill_chunk", "decode_step")
    assert {q.uid: q.preemptions for q in s.done}["p0"] == 2
    for r in wave:
        tokens, rows = alone(r)
        assert out[r.uid] == tokens, r.uid
        assert rel_err(torch.stack(s.emitted_logits[r.uid]).cpu(), rows.cpu()) < 1e-5 if dtype == "float32" else True
    if dtype == "float32":
        assert out["p0"] == oracle.generate_greedy(wave[0].prompt, 14)
    cache.audit()
    assert cache.free_slots == 4
