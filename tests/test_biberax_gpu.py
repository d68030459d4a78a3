"""Biberax on the GPU against the plain implementation (tests/plain/biberax_plain.py): the kernels of
each mechanism alone (the pass before the attention, the attention with every mask, sink, bias and
gate and every shape of work, the routing and the experts' products), one-layer models of each
mixer and feed-forward, whole prompts against token-by-token decoding and portions down to two
tokens, mixed batches against each request alone with pages and slots that are freed and used
again, keys at the edges of chunks and far away among hundreds (on weights where one key decides,
with controls that a chunk one off, a lost sink or a lost bias shows), long decoding through
replayed graphs, and generation through the scheduler.  The 32-bit path is compared to a bound a
little above its rounding, the bfloat16 path to a bound some three times what it measures."""

from __future__ import annotations

import copy
import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from biberax_cases import CASES, SINGLE, make_tensors, write_model
from helpers import feed, make_mixed_trace, max_live_tokens, random_tokens, rel_err, replay_in_process
from plain import biberax_plain as plain

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
F64 = torch.float64

# Bounds on max |engine - plain| / max |plain logit| over a request, some three times the largest error
# measured on the MI355X on these weights.
TOL = {"float32": 1.5e-5, "bfloat16": 4e-2}


def K():
    from lockstep_amd.ops import kernels
    return kernels()


def assert_follows(got, want, dtype, what):
    """Every position within the bound in float32.  In bfloat16 a router's near tie may fall the other way for
    a token now and then (its input is rounded), and that token's logits then belong to another expert: almost
    all positions within the bound, and the typical position far inside it."""
    rows = (torch.as_tensor(np.asarray(got)).double() - want).abs().max(dim=1)[0] / want.abs().max()
    if dtype == "float32":
        assert float(rows.max()) < TOL[dtype], (what, int(rows.argmax()), float(rows.max()))
        return
    beyond = int((rows >= TOL[dtype]).sum())
    assert beyond <= max(1, 0.04 * len(rows)) and float(rows.median()) < TOL[dtype] / 4, \
        (what, beyond, len(rows), float(rows.median()), float(rows.max()))


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """(case, dtype, sharpen) -> (loaded model, plain model, raw config, page size, folder), made once."""
    made = {}

    def get(name, dtype="float32", sharpen=1.0, table=CASES, seed=11):
        from lockstep_amd import load_model

        key = (name, dtype, sharpen, seed)
        if key not in made:
            case = table[name]
            tensors = make_tensors(case["raw"], seed=seed, sharpen=sharpen)
            folder = write_model(tmp_path_factory.mktemp(f"biberax{name}"), case["raw"], tensors)
            made[key] = (load_model(folder, dtype=dtype), plain.PlainBiberax(case["raw"], tensors), case["raw"],
                         case["page_size"], folder)
        return made[key]

    return get


def new_cache(model, page_size, tokens=512, requests=4, poison=True):
    return model.make_cache(num_pages=-(-tokens // page_size), page_size=page_size, max_requests=requests,
                            max_tokens_per_request=tokens, poison_on_free=poison)


# ---------------------------------------------------------------------------
# the kernels of each mechanism alone
# ---------------------------------------------------------------------------

def paged(n_pages, groups, page, d, dv, dtype):
    keys = torch.full((n_pages, groups, page, d), float("nan"), dtype=dtype, device="cuda")
    values = torch.full((n_pages, groups, dv, page), float("nan"), dtype=dtype, device="cuda")
    return keys, values


def step_meta(lengths, starts, slots):
    """tok_seq, tok_pos, seqs [n, 8] as the engine's upload lays them out."""
    seqs, tok_seq, tok_pos, off = [], [], [], 0
    for i, (n, s, slot) in enumerate(zip(lengths, starts, slots)):
        seqs.append([off, n, s, s + n, slot, 0, 0, 0])
        tok_seq += [i] * n
        tok_pos += list(range(s, s + n))
        off += n
    as_dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    return as_dev(tok_seq), as_dev(tok_pos), as_dev(seqs).reshape(-1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("norm, rot, neighbours, shared", [(True, 0, False, True), (False, 12, True, False),
                                                          (False, 16, False, False), (True, 8, True, False)])
def test_the_pass_before_the_attention(dtype, norm, rot, neighbours, shared):
    """Biases, the norm over the whole of q and of k, rotation of neighbouring pairs or of halves, keys as
    values: two requests in one step on scattered pages, compared element by element."""
    g = torch.Generator().manual_seed(3)
    heads, groups, d, page = 3, 1, 16, 8
    dv = d if shared else 12
    lengths, starts, slots = [5, 9], [11, 0], [1, 0]
    t = sum(lengths)
    width = heads * d + groups * d + (0 if shared else groups * dv)
    raw = torch.randn(t, width + 7, generator=g) * 2          # (columns beyond the projections are left alone)
    bias = torch.randn(width, generator=g)
    qw, kw = torch.rand(heads * d, generator=g) + 0.5, torch.rand(groups * d, generator=g) + 0.5
    table = torch.tensor([[3, 0, 5, -1], [4, 1, 2, -1]], dtype=torch.int32, device="cuda")
    keys, values = paged(6, groups, page, d, dv, dtype)
    tok_seq, tok_pos, seqs = step_meta(lengths, starts, slots)
    freq = plain.scaled_frequencies(rot, 50.0) if rot else None
    cos = sin = None
    if rot:
        angles = torch.arange(32, dtype=F64)[:, None] * freq[None, :]
        cos, sin = angles.cos().float().cuda(), angles.sin().float().cuda()
    q_out = torch.empty(t, heads * d, dtype=dtype, device="cuda")
    K().qkv_post(raw.cuda(), t, heads, groups, d, dv, bias.cuda(), qw.cuda() if norm else None, kw.cuda() if norm else None,
                 1e-5, cos, sin, rot, neighbours, max(s + n for s, n in zip(starts, lengths)) - 1, tok_seq, tok_pos, seqs,
                 table, q_out, keys, values, page, keys_are_values=shared)
    x = raw.double()[:, :width] + bias.double()
    q, k = x[:, :heads * d], x[:, heads * d:heads * d + groups * d]
    v = k if shared else x[:, heads * d + groups * d:]
    if norm:
        q, k = plain.root_mean_square_norm(q, 1e-5, qw.double()), plain.root_mean_square_norm(k, 1e-5, kw.double())
    q, k = q.reshape(t, heads, d), k.reshape(t, groups, d)
    if rot:
        pos = tok_pos.cpu()
        if neighbours:
            q, k = plain.rotate_neighbours(q, pos, freq), plain.rotate_neighbours(k, pos, freq)
        else:
            def halves(y):
                order = list(range(0, rot, 2)) + list(range(1, rot, 2)) + list(range(rot, d))   # pairs (i, i + rot/2) as neighbours
                back = torch.argsort(torch.tensor(order))
                return plain.rotate_neighbours(y[..., back], pos, freq)[..., order]
            q, k = halves(q), halves(k)
    bound = 1e-6 if dtype is torch.float32 else 1e-2
    assert rel_err(q_out.float().cpu(), q.reshape(t, -1)) < bound
    for row in range(t):
        slot, position = slots[int(tok_seq[row])], int(tok_pos[row])
        pg = int(table[slot, position // page])
        assert rel_err(keys[pg, :, position % page].float().cpu(), k[row]) < bound
        assert rel_err(values[pg, :, :, position % page].float().cpu(), v[row].reshape(groups, dv)) < bound


def run_attention_kernel(dtype, heads, groups, d, dv, lengths, starts, page, row_tiles, runs, scale, window, chunk, sink,
                         bias, gate, seed):
    """Keys, values and queries for requests that hold ``starts[i] + lengths[i]`` tokens and bring the last
    ``lengths[i]`` as queries; pages dealt in a scattered order.  Returns (kernel output, plain output)."""
    g = torch.Generator().manual_seed(seed)
    totals = [s + n for s, n in zip(starts, lengths)]
    t = sum(lengths)
    per = [-(-n // page) for n in totals]
    order = torch.randperm(sum(per) + 3, generator=g).tolist()
    table = torch.full((len(lengths), max(per) + 1), -1, dtype=torch.int32)
    keys, values = paged(sum(per) + 3, groups, page, d, dv, dtype)
    ks, vs, qs = [], [], []
    for i, total in enumerate(totals):
        k = (torch.randn(total, groups, d, generator=g) * 1.5).to(dtype)
        v = torch.randn(total, groups, dv, generator=g).to(dtype)
        q = (torch.randn(lengths[i], heads, d, generator=g) * 1.5).to(dtype)
        for logical in range(per[i]):
            pg = order.pop()
            table[i, logical] = pg
            n = min(page, total - logical * page)
            keys[pg, :, :n] = k[logical * page:logical * page + n].transpose(0, 1).cuda()
            values[pg, :, :, :n] = v[logical * page:logical * page + n].permute(1, 2, 0).cuda()
        ks.append(k), vs.append(v), qs.append(q)
    _, _, seqs = step_meta(lengths, starts, list(range(len(lengths))))
    items, folds = [], []
    block_rows = K().sink_staged_rows(heads, groups) if row_tiles == 8 else 16 * row_tiles if row_tiles else 1
    off = 0
    for i, n in enumerate(lengths):
        for b in range(-(-n // block_rows) if row_tiles else 1):
            if runs > 1:
                folds.append([len(items), runs, off + b * block_rows, min(block_rows, n - b * block_rows)])
            items += [[i, b, r, runs] for r in range(runs)]
        off += n
    as_dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda").reshape(-1)
    gate_rows = torch.randn(t, heads * dv, generator=g) * 2 if gate else None
    out = torch.empty(t, heads * dv, dtype=dtype, device="cuda")
    part = torch.full((len(items) * block_rows * heads * (dv + 2),), float("nan"), device="cuda") if folds else None
    q_all = torch.cat(qs).reshape(t, heads * d).cuda()
    K().sink_attention(q_all, heads, groups, d, dv, keys, values, page, table.cuda(), seqs, as_dev(items), len(items),
                       row_tiles, scale, window, chunk, None if sink is None else sink.cuda(),
                       None if bias is None else bias.cuda(), None if gate_rows is None else gate_rows.cuda(), out,
                       as_dev(folds) if folds else None, len(folds), part)
    want = []
    for i, total in enumerate(totals):
        i_pos, j_pos = torch.arange(starts[i], total)[:, None], torch.arange(total)[None, :]
        visible = j_pos <= i_pos
        if window:
            visible &= i_pos - j_pos < window
        if chunk:
            visible &= i_pos // chunk == j_pos // chunk
        full_bias = None
        if bias is not None:
            dist = (i_pos - j_pos).clamp(0, bias.shape[1] - 1)
            full_bias = bias.double()[:, dist]
        q_full = torch.zeros(total, heads, d, dtype=F64)
        q_full[starts[i]:] = qs[i].double()
        # (the plain function takes square score matrices: pad the queries and keep the rows that exist)
        pad_visible = torch.zeros(total, total, dtype=torch.bool)
        pad_visible[starts[i]:] = visible
        pad_visible[:starts[i]] = torch.eye(total, dtype=torch.bool)[:starts[i]]
        pad_bias = None
        if full_bias is not None:
            pad_bias = torch.zeros(heads, total, total, dtype=F64)
            pad_bias[:, starts[i]:] = full_bias
        o = plain.attention_with_sink(q_full, ks[i].double(), vs[i].double(), scale, pad_visible,
                                      None if sink is None else sink.double(), pad_bias)[starts[i]:]
        want.append(o.reshape(lengths[i], heads * dv))
    want = torch.cat(want)
    if gate_rows is not None:
        want = want * torch.sigmoid(gate_rows.double())
    return out.float().cpu(), want


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, groups, d, dv, page", [(4, 2, 32, 16, 8), (6, 1, 40, 40, 16), (2, 2, 16, 16, 4),
                                                        (20, 1, 24, 24, 8), (3, 3, 128, 128, 16)])
def test_attention_kernel_with_every_mask_sink_bias_and_gate(dtype, heads, groups, d, dv, page):
    g = torch.Generator().manual_seed(7)
    bound = 6e-6 if dtype is torch.float32 else 2e-2      # (measured: up to 2.5e-6 at keys of 128 elements, whose scores are widest)
    sink = torch.randn(heads, generator=g) * 2
    bias = torch.randn(heads, 23, generator=g)
    for label, kwargs in (
            ("plain causal, no sink", dict(window=0, chunk=0, sink=None, bias=None, gate=False)),
            ("chunks", dict(window=0, chunk=37, sink=torch.zeros(heads), bias=None, gate=True)),
            ("window", dict(window=29, chunk=0, sink=sink, bias=None, gate=False)),
            ("bias, sink and gate", dict(window=0, chunk=0, sink=sink, bias=bias, gate=True))):
        for row_tiles, runs, lengths, starts in ((1, 1, [40, 3, 17], [0, 100, 31]), (2, 3, [70, 33], [5, 130]),
                                                 (4, 2, [150], [61]), (0, 1, [1, 1, 1], [0, 77, 160]),
                                                 (0, 4, [1, 1], [250, 36]), (8, 1, [40, 3, 170], [0, 100, 31]),
                                                 (8, 3, [70, 133], [5, 130])):
            if row_tiles == 8 and not (K().sink_staged_keys(d, dv, dtype) and page % (8 if dtype is torch.bfloat16 else 4) == 0):
                continue        # (the kernel with tiles staged in LDS takes pages of at least 16 bytes of keys)
            got, want = run_attention_kernel(dtype, heads, groups, d, dv, lengths, starts, page, row_tiles, runs, 0.2,
                                             seed=row_tiles + runs, **kwargs)
            assert rel_err(got, want) < bound, (label, row_tiles, runs)


def test_a_sink_left_out_or_a_chunk_one_off_shows_in_the_kernel_test():
    """Controls of the test above: the same inputs against a plain result without the sink, or with the
    chunk one larger, differ by many times the bound."""
    heads = 4
    sink = torch.full((heads,), 1.0)
    got, want = run_attention_kernel(torch.float32, heads, 2, 32, 16, [40], [20], 8, 1, 1, 0.2, 0, 0, sink, None, False, 1)
    _, no_sink = run_attention_kernel(torch.float32, heads, 2, 32, 16, [40], [20], 8, 1, 1, 0.2, 0, 0, None, None, False, 1)
    assert rel_err(got, want) < 2e-6 and rel_err(got, no_sink) > 1e-2
    got, want = run_attention_kernel(torch.float32, heads, 2, 32, 16, [40], [20], 8, 1, 1, 0.2, 0, 15, None, None, False, 1)
    _, off = run_attention_kernel(torch.float32, heads, 2, 32, 16, [40], [20], 8, 1, 1, 0.2, 0, 16, None, None, False, 1)
    assert rel_err(got, want) < 2e-6 and rel_err(got, off) > 1e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("tokens, experts, top, width, ff", [(1, 4, 2, 32, 24), (37, 7, 3, 64, 40), (300, 5, 1, 48, 16),
                                                            (260, 3, 3, 40, 72), (9, 40, 16, 32, 8)])
def test_routing_and_the_experts_products(dtype, tokens, experts, top, width, ff):
    g = torch.Generator().manual_seed(tokens + experts)
    k = K()
    x = torch.randn(tokens, width, generator=g).to(dtype)
    logits = torch.randn(tokens, experts, generator=g) * 2
    logits[0, :2] = 0.75                                        # a tie: the lower index wins
    rb = torch.randn(experts, generator=g)
    rb[:2] = 0.0
    w = {f"m.e{e}.{n}": (torch.randn(*shape, generator=g) * 0.3).to(dtype) for e in range(experts)
         for n, shape in (("gate", (ff, width)), ("up", (ff, width)), ("down", (width, ff)))}
    stack = lambda n: torch.stack([w[f"m.e{e}.{n}"] for e in range(experts)]).cuda()
    for rows in (16, 32, 64):
        cap = k.experts_tile_capacity(tokens, experts, top, rows)
        i32 = lambda n: torch.full((n,), -7, dtype=torch.int32, device="cuda")
        chosen, order, tiles, counts = i32(tokens * top), i32(tokens * top), i32(4 * cap), i32(experts)
        share = torch.empty(tokens * top, device="cuda")
        k.experts_route(logits.cuda(), rb.cuda(), top, rows, chosen, share, order, tiles, counts)
        z = logits.double() + rb.double()
        for t in range(tokens):
            want = sorted(range(experts), key=lambda e: (-float(z[t, e]), e))[:top]
            assert chosen[t * top:(t + 1) * top].tolist() == want, (t, rows)
            assert rel_err(share[t * top:(t + 1) * top].cpu(), torch.softmax(z[t, want], dim=0)) < 1e-6
        sorted_pairs = order.tolist()
        assert sorted(sorted_pairs) == list(range(tokens * top))
        by_expert = [chosen[p].item() for p in sorted_pairs]
        assert by_expert == sorted(by_expert)
        used = [tl for tl in tiles.reshape(-1, 4).tolist() if tl[0] >= 0]
        assert sum(tl[2] for tl in used) == tokens * top and all(0 < tl[2] <= rows for tl in used)
        act = torch.empty(tokens * top, ff, dtype=dtype, device="cuda")
        partials = torch.full((top, tokens, width), float("nan"), device="cuda")
        k.experts_apply(x.cuda(), stack("gate"), stack("up"), stack("down"), top, rows, order, tiles, share, 1.3, 1.702,
                        act, partials)
        mlp = {"router": {"experts": experts, "top": top}, "expert": {"limit": 1.3}}
        full = dict(w, **{"m.router": torch.zeros(experts, width), "m.router.b": z[0] * 0})
        want = torch.zeros(tokens, width, dtype=F64)
        for t in range(tokens):          # the plain feed-forward with the router's logits given
            picks = chosen[t * top:(t + 1) * top].tolist()
            sh = torch.softmax(z[t, picks], dim=0)
            for s, e in zip(sh, picks):
                want[t] += s * plain.bounded_gated_unit(x[t:t + 1].double(), full, f"m.e{e}", 1.3)[0]
        assert rel_err(partials.sum(0).cpu(), want) < (2e-6 if dtype is torch.float32 else 2e-2), rows


# ---------------------------------------------------------------------------
# one-layer models of each mechanism, then whole models
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("kind", ["rotary", "biased", "dense", "routed"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_each_mechanism_alone_whole_and_in_portions(models, kind, dtype):
    model, oracle, raw, page, _ = models(kind, dtype, table=SINGLE)
    tokens = random_tokens(75, raw["vocab"], seed=4)
    want = oracle.forward(tokens)
    for cuts in ([], [2, 31, 2, 17, 1, 1, 1], [1] * 75):
        cache = new_cache(model, page)
        got = feed(model, cache, "r", tokens, cuts)
        assert rel_err(got, want) < TOL[dtype], (kind, cuts[:3])
        cache.close("r")
        cache.audit()


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_portions_and_token_by_token_agree_with_the_plain_model(models, name, dtype):
    model, oracle, raw, page, _ = models(name, dtype)
    tokens = random_tokens(150, raw["vocab"], seed=5)
    want = oracle.forward(tokens, round_router_input=torch.bfloat16 if dtype == "bfloat16" else None)
    runs = {}
    for label, cuts in (("whole", []), ("portions", [2, 47, 3, 16, 2, 33, 5, 1, 1, 2]), ("tail", [110] + [1] * 40),
                        ("single", [1] * 150)):
        cache = new_cache(model, page)
        runs[label] = feed(model, cache, "r", tokens, cuts)
        assert_follows(runs[label], want, dtype, (name, label))
        cache.close("r")
        cache.audit()
    if dtype == "float32":              # the cuttings agree with each other far below the bound against the plain model
        for label in ("portions", "tail", "single"):
            assert rel_err(runs[label], runs["whole"]) < 1e-5, label


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_whose_keys_are_dealt_to_runs(models, dtype):
    """A prompt of 1,100 tokens: the late row blocks of the layers that see all keys are dealt to several
    work items and folded (the buffer of partial results exists afterwards); decoding goes on from
    there, also cut into runs."""
    model, oracle, raw, page, _ = models("B", dtype)
    tokens = random_tokens(1120, raw["vocab"], seed=13)
    want = oracle.forward(tokens, round_router_input=torch.bfloat16 if dtype == "bfloat16" else None)
    for cuts in ([1100] + [1] * 20, [433, 2, 665] + [1] * 20):
        cache = new_cache(model, page, tokens=1536)
        got = feed(model, cache, "r", tokens, cuts)
        assert_follows(got, want, dtype, cuts[:3])
        cache.close("r")
    assert any(name == "sink.part" for name, _, _ in model.workspace._buffers)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_first_tokens_and_prompts_of_one_and_two_tokens(models, name):
    model, oracle, raw, page, _ = models(name)
    for n in (1, 2, 3, page, page + 1):
        tokens = random_tokens(n, raw["vocab"], seed=20 + n)
        cache = new_cache(model, page)
        assert rel_err(feed(model, cache, "r", tokens, []), oracle.forward(tokens)) < TOL["float32"], n


@pytest.mark.parametrize("name, dtype", [("A", "float32"), ("B", "float32"), ("C", "float32"), ("D", "float32"), ("A", "bfloat16")])
def test_mixed_batches_of_unequal_requests_with_pages_and_slots_used_again(models, name, dtype):
    """Seven requests of unequal lengths through four slots and a pool that holds the live ones only:
    portions beside single tokens, requests that sit steps out, finished requests whose (poisoned)
    pages the next ones take.  Each request's logits equal those of the request alone."""
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
    rounded = torch.bfloat16 if dtype == "bfloat16" else None
    for rid, toks in requests.items():
        assert_follows(got[rid], oracle.forward(toks, round_router_input=rounded), dtype, rid)


# ---------------------------------------------------------------------------
# one key that decides: the edges of chunks, a far key among hundreds, the sink, the bias
# ---------------------------------------------------------------------------

PLANTED = 7                       # the token id whose key every query answers
SECOND = 6                        # another one, with the same score and another value
OTHERS = list(range(8, 28))       # the ids all other tokens of these tests' sequences are drawn from


def _planted_case(kind):
    """One mixer layer and weights on which one key decides.  Every embedding gets a common component that the
    queries of all heads read into one dimension of the head (beyond the rotated ones); the planted token's key
    gets a large entry in that dimension through a direction of its normalised embedding that is orthogonal
    to the embeddings of the other tokens in use, whose keys are therefore small there; and (where the layer
    has a value projection) its value gets a strong component of its own.  Wherever the planted token is
    visible its score stands out among hundreds and the output is mostly its value."""
    raw = copy.deepcopy(SINGLE[kind]["raw"])
    mixer = raw["layers"][0]["mixer"]
    if kind == "biased":
        mixer["scale"] = 1.0          # (the norm over the whole projection bounds a query's and a key's entries)
    tensors = make_tensors(raw, seed=21)
    heads, groups, dim, vdim, at = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"], 20
    g = torch.Generator().manual_seed(5)
    embed = tensors["embed"].float()
    embed[:, 0] += 6.0                                # every token carries this component: the queries read it
    tensors["embed"] = embed.bfloat16()
    seen = plain.root_mean_square_norm(tensors["embed"].double(), raw["norm"]["eps"], tensors["l0.norm1"].double())

    def own_direction(token, other):
        basis = torch.linalg.qr(torch.cat([seen[OTHERS + [other]], torch.eye(raw["width"], dtype=F64)[:1]]).T).Q
        rest = seen[token] - basis @ (basis.T @ seen[token])
        return (rest / rest.norm()).float()

    along, along_second = own_direction(PLANTED, SECOND), own_direction(SECOND, PLANTED)
    k, q = tensors["l0.mix.k"].float(), tensors["l0.mix.q"].float()
    for group in range(groups):
        k[group * dim + at] = 10.0 * (along + along_second)
        k[group * dim + at + 1] = 10.0 * (along - along_second)      # (no query reads it: where the values are the keys, it tells the two apart)
    for head in range(heads):
        q[head * dim + at] = q[head * dim + at + 1] = 0.0
        q[head * dim + at, 0] = (30.0 if kind == "biased" else 3.0) / float(seen[:, 0].mean())
    tensors["l0.mix.k"], tensors["l0.mix.q"] = k.bfloat16(), q.bfloat16()
    if kind == "rotary":
        v = tensors["l0.mix.v"].float()
        for group in range(groups):
            v[group * vdim:(group + 1) * vdim] += 3.0 * torch.randn(vdim, 1, generator=g) * along[None, :]
        tensors["l0.mix.v"] = v.bfloat16()
    else:      # the values are the keys: the planted key's large entry is its value too
        for name in ("l0.mix.q.norm", "l0.mix.k.norm"):
            tensors[name] = torch.ones_like(tensors[name])
        for name in ("l0.mix.q.b", "l0.mix.k.b"):
            tensors[name] = torch.zeros_like(tensors[name])
        tensors["l0.mix.sink"] = torch.full_like(tensors["l0.mix.sink"], 2.0)
    return raw, tensors


def _sequence_with_planted(n, places, seed):
    g = torch.Generator().manual_seed(seed)
    tokens = [OTHERS[i] for i in torch.randint(0, len(OTHERS), (n,), generator=g).tolist()]
    for p in places:
        tokens[p] = PLANTED
    return tokens


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_keys_just_inside_and_just_outside_a_chunk(tmp_path, dtype):
    """Chunks of 20.  The planted token at 43 (seen by 43..59, gone at 60), at 59 (the last place of its
    chunk: seen by its own query alone) and at 60 (the first of the next).  Controls: the plain model
    with chunks of 19 or 21 differs at those places by many times the bound.  The engine follows the
    plain model with the edges inside a prompt, inside portions cut at and around the edges, and in
    tokens decoded one by one, on pages of 8 and of 16."""
    from lockstep_amd import load_model

    raw, tensors = _planted_case("rotary")
    model = load_model(write_model(tmp_path / "edge", raw, tensors), dtype=dtype)
    oracle = plain.PlainBiberax(raw, tensors)
    bound = TOL[dtype]
    for places, wheres in (([43], [59, 60]), ([59], [59, 60]), ([60, 100], [79, 80, 119, 120])):
        tokens = _sequence_with_planted(140, places, seed=6 + places[0])
        want = oracle.forward(tokens)
        for size in (19, 21):
            other = copy.deepcopy(raw)
            other["layers"][0]["mixer"]["mask"]["size"] = size
            moved = plain.PlainBiberax(other, tensors).forward(tokens)
            assert max(rel_err(moved[w], want[w]) for w in wheres) > 3 * bound, (places, size)
        for page in (8, 16):
            for cuts in ([], [80] + [1] * 60, [30] + [1] * 110, [20, 2, 37, 1, 2, 18, 2, 38]):
                cache = new_cache(model, page)
                got = feed(model, cache, "r", tokens, cuts)
                worst = (got.double() - want).abs().max(dim=1)[0] / want.abs().max()
                assert float(worst.max()) < bound, (places, page, cuts[:2], int(worst.argmax()))
                cache.close("r")
                cache.audit()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds_the_sink_and_the_bias_by_distance(tmp_path, dtype):
    """The mixer that sees every earlier key.  The planted token at place 3 of 600 decides the output of the
    queries up to 559 (a key far away, across many pages and runs); from 560 on a second planted token (the same score, another value) shares
    the weight with it according to the bias by distance (the far one in the table's last row, the near one
    moving through the rows before it); the first queries see few keys and so mostly the sink.  Controls on
    the plain side: without the early token, with the sink left out, or with a bias table whose last rows
    are swapped, the logits at those places move by many times the bound.  The engine follows the plain
    model in a prompt, in portions and decoded one by one, on pages of 8 and of 16."""
    from lockstep_amd import load_model

    raw, tensors = _planted_case("biased")
    model = load_model(write_model(tmp_path / "far", raw, tensors), dtype=dtype)
    oracle = plain.PlainBiberax(raw, tensors)
    bound = TOL[dtype]
    tokens = _sequence_with_planted(600, [3, 560], seed=9)
    tokens[560] = SECOND
    want = oracle.forward(tokens)
    without = list(tokens)
    without[3] = OTHERS[0]
    assert rel_err(oracle.forward(without)[500:560], want[500:560]) > 3 * bound
    no_sink = dict(tensors, **{"l0.mix.sink": torch.full_like(tensors["l0.mix.sink"], -100.0)})
    assert rel_err(plain.PlainBiberax(raw, no_sink).forward(tokens)[:3], want[:3]) > 3 * bound
    swapped = tensors["l0.mix.rel"].clone()
    swapped[[-1, -2]] = swapped[[-2, -1]]
    assert rel_err(plain.PlainBiberax(raw, dict(tensors, **{"l0.mix.rel": swapped})).forward(tokens)[560:], want[560:]) > 3 * bound
    for page in (8, 16):
        for cuts in ([], [550] + [1] * 50, [255, 2, 300, 13] + [1] * 30):
            cache = new_cache(model, page, tokens=640)
            got = feed(model, cache, "r", tokens, cuts)
            worst = (got.double() - want).abs().max(dim=1)[0] / want.abs().max()
            assert float(worst.max()) < bound, (page, cuts[:2], int(worst.argmax()))
            cache.close("r")


# ---------------------------------------------------------------------------
# long decoding (replayed graphs), generation through the scheduler, the programs
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
    half = LLM(folder, dtype="bfloat16", num_pages=64, page_size=page)
    tokens = half.generate([Request(uid="x", prompt=prompts[0], max_new_tokens=8)])["x"]
    assert len(tokens) == 8 and tokens[:2] == want[0][:2]


def test_trace_replay_program_on_a_model_folder(models, tmp_path):
    """bin/trace_run as a subprocess on a Biberax folder: a mixed schedule through four slots."""
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
