"""Ziferax in the framework against the plain implementation (``plain_ziferax``, 64-bit): each mechanism's kernels
alone; whole prompts; a prompt and then token by token, also from the very first token; portions down to two
tokens; unequal requests in one batch against each alone, in a pool and slots that are used again; windows that
pass over pages, tiles and portions with scores scaled so that single keys decide a row; sinks that outweigh the
keys; routers whose identity experts, correction and top count take every special value; long decoding through
captured steps; sizes that differ wherever they can; greedy generation through the entry point.  In 32-bit against
the plain implementation to rounding; in bfloat16, where a rounded router input may choose another expert at a
close call, most rows to rounding and every row within a bound that a lost key or a stale slot exceeds."""
import json
import math
import os

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

import plain_ziferax as plain
from gpu_util import DEV

pytestmark = pytest.mark.gpu

REL = {"float32": 2e-5, "bfloat16": 3e-2}


def att(heads, kv, dim, window, rot, scale, base=10000.0):
    return dict(heads=heads, kv_heads=kv, dim=dim, vdim=dim, mask=dict(size=window), rot=dict(base=base, dims=rot), scale=scale)


def moe(experts, identity, top, ff, limit, shared=None):
    out = dict(kind="moe", router=dict(experts=experts, identity=identity, top=top), expert=dict(ff=ff, limit=limit))
    if shared:
        out["shared"] = dict(ff=shared[0], limit=shared[1])
    return out


def layer(mixer, mlp=None, weights_of=None):
    out = dict(type="attention", mixer=mixer, mlp=mlp)
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def config(width, vocab, layers, mult=0.3, eps=1e-5):
    return dict(architecture="Ziferax", vocab=vocab, width=width, layers=layers, norm=dict(eps=eps), residual_mult=mult)


_A0, _A1 = layer(att(4, 2, 32, 24, 8, 0.2), moe(6, 2, 2, 24, 1.5, (40, 2.0))), layer(att(2, 1, 64, 40, 64, 0.15, 500.0), moe(4, 0, 1, 32, 1.0))
# A: the usual shape: two layers with tensors and two that use them again with caches of their own; a window that is
# no multiple of a page; rotation of a part of the head in one layer and of the whole head in the other
CFG_A = config(64, 97, [_A0, _A1, dict(_A0, weights_of=0), dict(_A1, weights_of=1)])
# B: sizes that differ wherever they can: heads stored padded (24 as 32), as many key heads as query heads, a window
# shorter than a page, an expert size that no 16-byte access fits, every router output chosen (top = all), a layer
# without a feed-forward, one whose experts are all identity but one, no multiplier
CFG_B = config(40, 131, [layer(att(3, 3, 24, 7, 6, 0.3), moe(3, 1, 4, 12, 0.7)), layer(att(1, 1, 16, 19, 2, 0.25)),
                         layer(att(5, 1, 8, 33, 8, 0.4), moe(1, 3, 2, 20, 5.0, (8, 0.5)))], mult=1.0, eps=1e-3)
# C: head sizes the matrix-core kernels take (128, 64, 96 and 256), windows beside tile and page borders and one
# longer than any test sequence, expert sizes the matrix-core products take, many experts
CFG_C = config(128, 113, [layer(att(4, 1, 128, 100, 32, 0.09), moe(8, 0, 2, 64, 1.5, (64, 2.0))),
                          layer(att(8, 2, 64, 32, 16, 0.12), moe(24, 8, 4, 32, 2.5)),
                          layer(att(2, 2, 96, 1000, 96, 0.1), moe(5, 1, 3, 72, 1.5, (136, 1.0))),
                          layer(att(1, 1, 256, 65, 2, 0.06))], mult=0.5)
# S: scores scaled so that a softmax row is nearly one key of the window, windows that cross page and tile borders
_S0 = layer(att(2, 1, 16, 33, 4, 5.0), moe(2, 1, 1, 16, 1.5))
CFG_S = config(32, 50, [_S0, layer(att(2, 2, 32, 47, 32, 4.0)), dict(_S0, weights_of=0)])
# K: sinks that outweigh the keys in some heads and vanish in others
CFG_K = config(32, 50, [layer(att(4, 2, 16, 21, 8, 0.3), moe(3, 0, 2, 8, 1.5))])
MODELS = {"A": (CFG_A, 1, {}), "B": (CFG_B, 2, {}), "C": (CFG_C, 3, {}), "S": (CFG_S, 4, {}),
          "K": (CFG_K, 5, dict(sink_std=6.0))}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """{name: (folder, config, 64-bit weights)}; the folders hold bfloat16 tensors under the design's names."""
    out = {}
    for name, (cfg, seed, kw) in MODELS.items():
        d = tmp_path_factory.mktemp(f"ziferax{name}")
        w = plain.random_weights(cfg, seed, **kw)
        with open(os.path.join(d, "config.json"), "w") as f:
            json.dump(cfg, f)
        save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(d, "model.safetensors"))
        out[name] = (str(d), cfg, {k: v.double() for k, v in w.items()})
    return out


_oracle_cache = {}


def oracle(models, name, toks):
    key = (name, tuple(toks))
    if key not in _oracle_cache:
        _, cfg, w = models[name]
        _oracle_cache[key] = plain.forward(w, cfg, list(toks)).float().numpy()
    return _oracle_cache[key]


# bfloat16 bounds (median, 85th of 100 rows, largest row).  A rounded router input may pick another expert where two
# choice scores nearly tie (a few rows in a hundred, and the rows that attend to them a little), so most rows are
# held to rounding and every row to a bound that a lost key, a window off by one or a stale slot exceeds on peaked
# rows.  Model C (four layers, 32 router outputs of which four are chosen) moves that far by rounding alone: its
# 64-bit implementation with nothing but the normed layer inputs rounded to bfloat16 differs from itself by 1.1e-2
# (median), 2.5e-2 (85th) and 8.5e-2 (largest) of the largest logit over the same prompts.
BF16_BOUNDS = {"C": (3e-2, 6e-2, 0.3)}


def close(got, want, dtype, name=""):
    err = np.abs(got - want).max(-1) / float(np.abs(want).max())
    if dtype == "float32":
        assert err.max() <= REL[dtype], f"max {err.max():.3e} at row {int(err.argmax())}"
        return
    mid, most, top = BF16_BOUNDS.get(name, (2e-2, REL[dtype], 0.3))
    assert np.median(err) <= mid and (len(err) < 8 or np.quantile(err, 0.85) <= most) and err.max() <= top, \
        f"median {np.median(err):.3e}, 85th {np.quantile(err, 0.85):.3e}, max {err.max():.3e} at row {int(err.argmax())}"


def tokens(vocab, n, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


@pytest.fixture(scope="module")
def replayers(models):
    from ullm_amd.replay import Replayer
    made = {}

    def get(name, dtype, max_tokens=512, max_requests=4, use_graphs=True):
        key = (name, dtype, max_tokens, max_requests, use_graphs)
        if key not in made:
            made[key] = Replayer(models[name][0], dtype, max_tokens, 16, DEV, max_requests=max_requests, use_graphs=use_graphs)
        rep = made[key]
        assert not rep.live and rep.runner.cache.num_free_pages() == rep.max_tokens // 16
        return rep
    return get


def run(rep, rid, toks, cuts, end=True):
    """Feed ``toks`` in portions of the sizes ``cuts`` (the rest one by one); logits of every position."""
    got, at, step = [], 0, 0
    sizes = list(cuts) + [1] * len(toks)
    while at < len(toks):
        n = min(sizes[step], len(toks) - at)
        got.append(rep.step({"step": step, "entries": [{"id": rid, "tokens": toks[at:at + n], "want": list(range(n))}],
                             "end": [rid] if end and at + n == len(toks) else []}))
        at, step = at + n, step + 1
    return np.concatenate(got)


CASES = [(n, d) for n in ("A", "B", "C") for d in ("float32", "bfloat16")]


@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompts(replayers, models, name, dtype):
    rep = replayers(name, dtype)
    for i, n in enumerate((1, 2, 15, 16, 17, 75)):
        toks = tokens(models[name][1]["vocab"], n, 10 + i)
        close(run(rep, "r", toks, [n]), oracle(models, name, toks), dtype, name)


def test_the_stream_after_every_layer(models):
    """Layer by layer in 32-bit: the stream after a layer is the stream before it plus the multiplier times the
    branch that the layer leaves pending."""
    from ullm_amd.engine.loading import load_model
    from ullm_amd.engine.runner import ModelRunner, StepEntry
    from ullm_amd.kernels import ops
    d, cfg, w = models["A"]
    toks = tokens(cfg["vocab"], 50, 3)
    want = []
    plain.forward(w, cfg, toks, want)
    _, model, env = load_model(d, "float32", DEV, context_len=64)
    runner = ModelRunner(model, env, page_size=16, num_pages=4, max_requests=1, use_graphs=False)
    rc = runner.cache.admit("r")
    assert runner.cache.reserve(rc, len(toks))
    ctx, _ = runner.build_context([StepEntry(rc, toks, [])])
    stream, pending = ops.embedding(ctx.token_ids, model.embedding), None
    for idx, (block, cache_id) in enumerate(model.run_order):
        stream, pending = model.blocks[block].forward(stream, pending, ctx, runner.caches[cache_id])
        after = (stream + pending.mult * pending.branch).double().cpu()
        assert (after - want[idx]).abs().max() <= 2e-5 * want[idx].abs().max(), idx


@pytest.mark.parametrize("name,dtype", CASES)
def test_a_prompt_and_then_token_by_token(replayers, models, name, dtype):
    toks = tokens(models[name][1]["vocab"], 75, 15)
    for graphs in (True, False):
        close(run(replayers(name, dtype, use_graphs=graphs), "r", toks, [40]), oracle(models, name, toks), dtype, name)


@pytest.mark.parametrize("name,dtype", CASES)
def test_token_by_token_from_the_first_token(replayers, models, name, dtype):
    toks = tokens(models[name][1]["vocab"], 45, 16)
    close(run(replayers(name, dtype), "r", toks, []), oracle(models, name, toks), dtype, name)


@pytest.mark.parametrize("name,dtype", CASES)
@pytest.mark.parametrize("cuts", [(2, 2, 3, 2, 14, 2, 17, 31, 2), (1, 1, 2, 30, 3, 3, 33), (16, 16, 16, 2, 25)])
def test_portions_of_changing_size(replayers, models, name, dtype, cuts):
    toks = tokens(models[name][1]["vocab"], 75, 15)
    close(run(replayers(name, dtype), "r", toks, cuts), oracle(models, name, toks), dtype, name)


@pytest.mark.parametrize("name,dtype", CASES)
def test_unequal_requests_together_in_pages_and_slots_used_again(replayers, models, name, dtype):
    """Six requests through two slots and a pool of 128 tokens: portions beside single tokens, a request left out
    of a step, a request that starts in the slot and pages another has just given back."""
    rep = replayers(name, dtype, max_tokens=128, max_requests=2)
    vocab = models[name][1]["vocab"]
    reqs = {f"q{i}": tokens(vocab, n, 30 + i) for i, n in enumerate((50, 33, 1, 64, 20, 47))}
    plan = [[("q0", 20), ("q1", 2)], [("q0", 1), ("q1", 31)], [("q0", 29)],          # q1 ends; q0 goes on alone
            [("q2", 1)], [("q3", 17)], [("q3", 1)], [("q3", 2)], [("q3", 44)],        # q2 and q3 use q1's and q0's slots again
            [("q4", 3), ("q5", 30)], [("q5", 1)], [("q4", 16), ("q5", 1)], [("q4", 1), ("q5", 15)]]
    at = {r: 0 for r in reqs}
    got = {r: [] for r in reqs}
    for s, entries in enumerate(plan):
        msg = {"step": s, "entries": [], "end": []}
        for r, n in entries:
            msg["entries"].append({"id": r, "tokens": reqs[r][at[r]:at[r] + n], "want": list(range(n))})
            at[r] += n
            if at[r] == len(reqs[r]):
                msg["end"].append(r)
        out, row = rep.step(msg), 0
        for r, n in entries:
            got[r].append(out[row:row + n])
            row += n
    assert at == {r: len(t) for r, t in reqs.items()}
    for r, toks in reqs.items():
        close(np.concatenate(got[r]), oracle(models, name, toks), dtype, name)
    rep.runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_while_windows_pass_and_pages_return(replayers, models, dtype):
    """190 tokens one by one: the windows (24 and 40 keys) pass over many pages, which go back to the pool while the
    request lives; a second request then takes them."""
    rep = replayers("A", dtype, max_tokens=192)
    toks = tokens(models["A"][1]["vocab"], 190, 40)
    got = run(rep, "r", toks, [3], end=False)
    assert rep.runner.cache.num_free_pages() >= 12 - 4          # of 12 pages the request still holds 40 keys' worth
    other = tokens(models["A"][1]["vocab"], 100, 41)
    close(run(rep, "s", other, [60]), oracle(models, "A", other), dtype, "A")
    rep.step({"step": 999, "entries": [], "end": ["r"]})
    close(got, oracle(models, "A", toks), dtype, "A")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cuts", [(260,), (200,), (17, 64, 2, 130, 2, 30), (33, 33, 1, 1, 47, 47, 2, 16)])
def test_scores_scaled_so_that_single_keys_of_the_window_decide(replayers, models, dtype, cuts):
    """With scores of many units a softmax row is close to one key among the window's 33 or 47 (for one query in
    thirty the key at the window's far edge, and as often the key just outside would win if it were seen): a key
    lost or doubled at a page's or a tile's border, a window off by one in a prompt portion or for a single token,
    takes a whole value out of the sum."""
    toks = tokens(models["S"][1]["vocab"], 260, 42)
    want = oracle(models, "S", toks)
    got = run(replayers("S", dtype), "r", toks, cuts)
    if dtype == "float32":
        close(got, want, dtype)
    else:
        # one key's weight moves by percents under bfloat16 rounding of peaked scores
        err = np.abs(got - want).max(-1) / np.abs(want).max()
        assert np.median(err) < 3e-2 and err.max() < 0.3, (np.median(err), err.max())


def test_the_window_edge_moves_the_oracle():
    """The plain implementation itself: a window one key longer or shorter changes the peaked model's logits by
    far more than the bounds above, so those bounds do test the edge."""
    cfg, seed, kw = MODELS["S"]
    w = {k: v.double() for k, v in plain.random_weights(cfg, seed, **kw).items()}
    toks = tokens(cfg["vocab"], 120, 42)
    base = plain.forward(w, cfg, toks)
    for delta in (-1, 1):
        other = json.loads(json.dumps(cfg))
        for L in other["layers"]:
            L["mixer"]["mask"]["size"] += delta
        moved = (plain.forward(w, other, toks) - base).abs().max(-1).values / base.abs().max()
        assert float(moved[50:].max()) > 0.05 and float((moved[50:] > 1e-3).float().mean()) > 0.1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cuts", [(70,), (30,), (2, 2, 21, 21, 2)])
def test_sinks_that_outweigh_the_keys(replayers, models, dtype, cuts):
    toks = tokens(models["K"][1]["vocab"], 70, 43)
    close(run(replayers("K", dtype), "r", toks, cuts), oracle(models, "K", toks), dtype)
    # and the sinks matter: without them the oracle's logits move by percents
    _, cfg, w = models["K"]
    none = dict(w)
    none["l0.mix.sink"] = torch.full_like(w["l0.mix.sink"], -1e4)
    moved = (plain.forward(none, cfg, toks) - plain.forward(w, cfg, toks)).abs().max() / plain.forward(w, cfg, toks).abs().max()
    assert float(moved) > 0.05


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_greedy_generation_through_the_entry_point(models, name):
    from ullm_amd import LLM, EngineConfig, SamplingParams
    d, cfg, w = models[name]
    g = torch.Generator().manual_seed(50)
    prompts = [torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for n in (5, 19, 1, 33)]
    for kw in (dict(), dict(max_num_batched_tokens=12, max_prefill_chunk=5, max_bs=3), dict(enforce_eager=True, disable_async_scheduling=True)):
        args = dict(model=d, dtype="float32", max_bs=8, context_len=128, page_size=16, num_pages=24, device=DEV)
        args.update(kw)
        llm = LLM(EngineConfig(**args))
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_new_tokens=10, ignore_eos=True))
        for p, o in zip(prompts, outs):
            assert o.token_ids == plain.greedy_generate(w, cfg, p, 10)
        llm.engine.runner.cache.check()
        assert llm.engine.runner.cache.num_free_pages() == 24
        llm.shutdown()


def test_the_trace_program_runs_the_design(models, trace_run):
    d, cfg, _ = models["A"]
    toks = tokens(cfg["vocab"], 40, 60)
    want = oracle(models, "A", toks)
    tr = trace_run(d, "float32", 128)
    a = tr.step([("a", toks[:21], [0, 20])])
    b = tr.step([("a", toks[21:], [18])], end=["a"])
    tr.close()
    close(np.concatenate((a, b)), want[[0, 20, 39]], "float32")


# ------------------------------------------------------------------------------------------- kernels alone

@pytest.mark.parametrize("window", [0, 40, 33])
@pytest.mark.parametrize("hd,nq,nkv", [(64, 10, 2), (128, 6, 2), (32, 20, 1), (96, 4, 4), (256, 2, 1)])
def test_matrix_core_attention_with_sinks_and_a_window(hd, nq, nkv, window):
    """The bfloat16 kernels (single tokens cut over splits and their reduce; prompt tiles) against 64-bit softmax
    attention with one more term exp(sink) in the denominator, on the same rounded operands: sinks from far below
    the scores to far above them; contexts that end at and beside tile and page borders, one past 1 100 keys; a
    prompt portion that starts in the middle of a page beside single tokens; the same in the general kernel."""
    from types import SimpleNamespace
    from gpu_util import paged_cache, table_tensor
    from ullm_amd.kernels import ops
    from ullm_amd.parts import GroupView, StepShape
    from ullm_amd.parts.attention import plan_attention_step
    g = torch.Generator().manual_seed(hd + nq)
    starts, lens = [1130, 31, 64, 200, 0], [1, 1, 1, 45, 33]            # tokens before the step, new tokens
    sink = torch.linspace(-8.0, 6.0, nq)[torch.randperm(nq, generator=g)].float()
    seqs_k = [torch.randn(s + n, nkv, hd, generator=g).bfloat16().float() for s, n in zip(starts, lens)]
    seqs_v = [torch.randn(s + n, nkv, hd, generator=g).bfloat16().float() for s, n in zip(starts, lens)]
    k_pool, v_pool, tables = paged_cache(seqs_k, seqs_v, 16, torch.bfloat16, DEV, fill=0.0)
    T = sum(lens)
    q = torch.randn(T, nq, hd, generator=g).bfloat16()
    positions = torch.tensor([s + i for s, n in zip(starts, lens) for i in range(n)], dtype=torch.int32, device=DEV)
    entry = torch.tensor([b for b, n in enumerate(lens) for _ in range(n)], dtype=torch.int32, device=DEV)
    plan = plan_attention_step(StepShape(tuple(lens), tuple(starts)))
    plan.arrays = {k: torch.tensor(v, dtype=torch.int32, device=DEV) for k, v in plan.arrays.items()}
    group = GroupView(table_tensor(tables, DEV), 0, 16, window)
    ctx = SimpleNamespace(positions=positions, token_entry=entry)
    scale = 1.5 / math.sqrt(hd)
    out = ops.paged_attention(q.view(T, nq * hd).to(DEV), k_pool, v_pool, ctx, group, nq, nkv, hd, scale, window, plan,
                              sink=sink.to(DEV), sink_log2=(sink * math.log2(math.e)).to(DEV))
    general = ops.paged_attention_generic(q.view(T, nq * hd).to(DEV), k_pool, v_pool, positions, entry, group.block_table,
                                          16, nq, nkv, hd, scale, window, sink=sink.to(DEV))
    out, general = out.float().cpu().view(T, nq, hd), general.float().cpu().view(T, nq, hd)
    t = 0
    for b, (s, n) in enumerate(zip(starts, lens)):
        for i in range(n):
            pos = s + i
            lo = max(0, pos - window + 1) if window else 0
            for h in range(nq):
                kv = h // (nq // nkv)
                sc = (seqs_k[b][lo:pos + 1, kv].double() @ q[t, h].double()) * scale
                top = max(float(sc.max()), float(sink[h]))
                e = torch.exp(sc - top)
                want = (e / (e.sum() + math.exp(float(sink[h]) - top))) @ seqs_v[b][lo:pos + 1, kv].double()
                for res in (out, general):
                    err = (res[t, h].double() - want).abs().max()
                    assert err <= 2e-2 * max(1.0, float(want.abs().max())), (b, i, h, float(err))
            t += 1


@pytest.mark.parametrize("hd,nq,nkv,rot,T", [(24, 3, 3, 6, 5), (96, 4, 2, 24, 9), (64, 8, 2, 16, 150), (128, 2, 1, 128, 1100)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotation_and_cache_write_with_the_values_taken_from_the_keys(hd, nq, nkv, rot, T, dtype):
    """q rotated to its buffer, k rotated into the key pool, and the same k as projected, not rotated, into the value
    pool (no value columns in the row): the one-head-a-wave kernel and the 16-byte kernel with its runs of eight."""
    from ullm_amd.kernels import ops
    from ullm_amd.parts.position import Rotary
    g = torch.Generator().manual_seed(hd)
    P, start = 16, 5
    row = (torch.randn(T, (nq + nkv) * hd, generator=g)).to(dtype)
    pages = -(-(start + T) // P)
    order = torch.randperm(pages + 2, generator=g)[:pages]
    table = order.to(torch.int32).view(1, pages).to(DEV)
    k_pool = torch.zeros(pages + 2, nkv, P, hd, dtype=dtype, device=DEV)
    v_pool = torch.zeros(pages + 2, nkv, hd, P, dtype=dtype, device=DEV)
    q_out = torch.empty(T, nq * hd, dtype=dtype, device=DEV)
    positions = torch.arange(start, start + T, dtype=torch.int32, device=DEV)
    cos_sin = Rotary.make_table(rot, 500.0, start + T).to(DEV)
    ops.qk_norm_rope_write(row.to(DEV), q_out, None, None, 0.0, cos_sin, rot, 2, positions, torch.zeros(T, dtype=torch.int32, device=DEV),
                           table, k_pool, v_pool, P, nq, nkv, hd, write_kv=True, values_from_keys=True)
    x = row.double()
    pos = torch.arange(start, start + T)
    want_q = plain.rotate_adjacent_pairs(x[:, :nq * hd].reshape(T, nq, hd), pos, rot, 500.0)
    k = x[:, nq * hd:].reshape(T, nkv, hd)
    want_k = plain.rotate_adjacent_pairs(k, pos, rot, 500.0)
    # the angles are 32-bit products of position and frequency: their rounding grows with the position
    tol = 1e-5 + 2e-7 * (start + T) if dtype == torch.float32 else 1.6e-2
    assert (q_out.double().cpu().view(T, nq, hd) - want_q).abs().max() <= tol * want_q.abs().max()
    for t in range(T):
        page, off = int(order[(start + t) // P]), (start + t) % P
        assert (k_pool[page, :, off].double().cpu() - want_k[t]).abs().max() <= tol * want_k.abs().max()
        assert torch.equal(v_pool[page, :, :, off].cpu(), row[t, nq * hd:].view(nkv, hd))


@pytest.mark.parametrize("R,top,correction", [(20, 3, True), (5, 5, True), (64, 1, False), (200, 8, True), (2, 1, True)])
def test_router_scores_choice_and_weights(R, top, correction):
    from ullm_amd.kernels import ops
    g = torch.Generator().manual_seed(R)
    T = 37
    z = torch.randn(T, R, generator=g) * 3
    z[3] = 0.0                                                   # every score equal: the lowest indices win
    z[4, :] = -1e4
    z[4, R - 1] = 50.0                                           # one output has all the weight
    c = torch.randn(R, generator=g) * 0.3 if correction else None
    ids, wts = ops.moe_route(z.to(DEV), c.to(DEV) if correction else None, top)
    s = torch.softmax(z.float(), -1).double()
    choice = s + (c.double() if correction else 0)
    for t in range(T):
        # the largest choice scores, equal ones by rising index
        want = sorted(range(R), key=lambda e: (-float(choice[t, e]), e))[:top]
        assert ids[t].tolist() == want, t
        picked = s[t, want]
        assert (wts[t].double().cpu() - picked / (picked.sum() + 1e-20)).abs().max() < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,R,top", [(40, 4, 4), (256, 20, 3), (2048, 36, 4), (100, 130, 8)])
def test_router_product_and_routing_in_one_kernel(dtype, H, R, top):
    """The fused kernel against the 64-bit product of the same (rounded) rows and the plain routing; a token's
    choice and weights are the same bits whatever else is in the batch."""
    from ullm_amd.kernels import ops
    g = torch.Generator().manual_seed(H + R)
    x = torch.randn(50, H, generator=g).to(dtype)
    w = (torch.randn(R, H, generator=g) * 0.3).float()
    c = (torch.randn(R, generator=g) * 0.1).float()
    ids, wts = ops.moe_router(x.to(DEV), w.to(DEV), c.to(DEV), top)
    one_ids, one_wts = ops.moe_router(x[17:18].to(DEV), w.to(DEV), c.to(DEV), top)
    assert torch.equal(one_ids[0], ids[17]) and torch.equal(one_wts[0], wts[17])
    # many tokens take the variant with four tokens a block: the same bits again
    many = torch.cat([x] * 13)[:-3]
    many_ids, many_wts = ops.moe_router(many.to(DEV), w.to(DEV), c.to(DEV), top)
    assert torch.equal(many_ids[:50], ids) and torch.equal(many_wts[600:], wts[:47]) and torch.equal(many_wts[:50], wts)
    s = torch.softmax(x.double() @ w.double().T, -1)
    choice = s + c.double()
    for t in range(50):
        order = sorted(range(R), key=lambda e: (-float(choice[t, e]), e))
        if top < R and float(choice[t, order[top - 1]] - choice[t, order[top]]) < 1e-5:
            continue                                              # a close call: either choice is right
        if min(float(choice[t, order[i]] - choice[t, order[i + 1]]) for i in range(top - 1)) < 1e-5 if top > 1 else False:
            assert sorted(ids[t].tolist()) == sorted(order[:top])
            continue
        assert ids[t].tolist() == order[:top], t
        picked = s[t, order[:top]]
        assert (wts[t].double().cpu() - picked / (picked.sum() + 1e-20)).abs().max() < 1e-5


@pytest.mark.parametrize("T,top,E,extra,rows", [(1, 3, 16, 4, 16), (7, 2, 3, 1, 16), (300, 4, 8, 0, 64), (129, 1, 40, 8, 32), (33, 8, 9, 3, 16),
                                                (700, 3, 5, 1, 128)])
def test_grouping_pairs_by_expert(T, top, E, extra, rows):
    from ullm_amd.kernels import ops
    g = torch.Generator().manual_seed(T + E)
    ids = torch.stack([torch.randperm(E + extra, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    if T > 5:
        ids[:, 0] = 1 if E > 1 else 0                            # one expert takes a row of every token
    slot, token, tiles, offsets = (x.cpu() for x in ops.moe_sort(ids.to(DEV), E, rows))
    flat = ids.view(-1)
    counts = torch.bincount(flat[flat < E], minlength=E)
    assert offsets.tolist() == [0] + torch.cumsum(counts, 0).tolist()
    real = flat < E
    assert (slot[~real] == -1).all()
    assert sorted(slot[real].tolist()) == list(range(int(counts.sum())))         # every slot taken once
    for p in torch.nonzero(real).view(-1).tolist():
        e, s = int(flat[p]), int(slot[p])
        assert offsets[e] <= s < offsets[e + 1] and int(token[s]) == p // top
    assert tiles[-1].tolist() == [int((tiles[:-1, 2] > 0).sum()), 0, 0]          # behind the list: the tiles in use
    covered = []
    for e, first, n in tiles[:-1].tolist():
        assert 0 <= n <= rows
        if n:
            assert offsets[e] <= first and first + n <= offsets[e + 1]
            covered += list(range(first, first + n))
    assert sorted(covered) == list(range(int(counts.sum())))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,top,E,H,ff,rows", [(5, 2, 4, 64, 32, 16), (70, 3, 5, 136, 72, 16), (200, 2, 3, 128, 64, 64),
                                               (90, 4, 6, 96, 40, 32), (9, 2, 3, 40, 12, 16), (3, 1, 2, 72, 8, 16),
                                               (300, 3, 4, 200, 136, 64), (130, 2, 2, 72, 200, 64), (500, 3, 4, 264, 72, 128),
                                               (600, 2, 3, 136, 200, 128), (400, 2, 2, 512, 256, 128)])
def test_expert_products_over_grouped_rows_and_their_weighted_sum(dtype, T, top, E, H, ff, rows):
    """gate | up with the clamped unit, down, and the sum with identity experts, a shared branch, another branch and a
    bias, against 64-bit products of the same operands; sizes the matrix-core tiles take and sizes they do not (an
    inner size that is no multiple of 8, outputs that do not fill a tile, an inner size that ends inside a step)."""
    from ullm_amd.kernels import ops
    g = torch.Generator().manual_seed(T * E + ff)
    limit, alpha = 1.2, 1.702
    x = torch.randn(T, H, generator=g).to(dtype)
    wgu = (torch.randn(E, 2 * ff, H, generator=g) * 0.2).to(dtype)
    wd = (torch.randn(E, H, ff, generator=g) * 0.2).to(dtype)
    ids = torch.stack([torch.randperm(E + 2, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    wts = torch.rand(T, top, generator=g).float()
    base, shared = torch.randn(T, H, generator=g).float(), torch.randn(T, H, generator=g).to(dtype)
    bias = torch.randn(H, generator=g).float()
    slot, token, tiles, _ = ops.moe_sort(ids.to(DEV), E, rows)
    act = ops.moe_rows(x.to(DEV), token, wgu.to(DEV), tiles, rows, T * top, gated=True, limit=limit, alpha=alpha)
    y = ops.moe_rows(act, None, wd.to(DEV), tiles, rows, T * top, gated=False)
    out = ops.moe_combine(y, x.to(DEV), ids.to(DEV), wts.to(DEV), slot, E, base=base.to(DEV), bias=bias.to(DEV),
                          shared=shared.to(DEV)).double().cpu()
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    slot = slot.cpu()
    xd = x.double()
    want = base.double() + bias.double() + shared.double()
    for t in range(T):
        for k in range(top):
            e = int(ids[t, k])
            if e >= E:
                want[t] += float(wts[t, k]) * xd[t]
                continue
            gu = wgu[e].double() @ xd[t]
            a = plain.clamped_unit(gu[:ff], gu[ff:], limit)
            got_a = act[int(slot[t * top + k])].double().cpu()
            assert (got_a - a).abs().max() <= tol * max(1.0, float(a.abs().max())), (t, k)
            want[t] += float(wts[t, k]) * (wd[e].double() @ got_a)      # the second product of the first's rounded result
    assert (out - want).abs().max() <= tol * want.abs().max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_clamped_gated_unit(dtype):
    from ullm_amd.kernels import ops
    g = torch.Generator().manual_seed(1)
    for I in (7, 64):
        gu = (torch.randn(13, 2 * I, generator=g) * 3).to(dtype)
        got = ops.glu_clamped(gu.to(DEV), 1.5, 1.702).double().cpu()
        want = plain.clamped_unit(gu[:, :I].double(), gu[:, I:].double(), 1.5)
        assert (got - want).abs().max() <= (1e-6 if dtype == torch.float32 else 1e-2) * want.abs().max()


@pytest.mark.parametrize("M", [1, 9, 40, 64])
def test_clamped_gated_unit_on_store_of_the_few_rows_products(M):
    """gate | up with the clamped unit applied to the 32-bit sums inside the product kernels (the weight-streaming
    kernel up to 64 rows, the rows kernel up to 128) against 64-bit products of the same operands; with no limit the
    same kernels still give silu(gate) * up."""
    from ullm_amd.kernels import ops
    g = torch.Generator().manual_seed(M)
    K, I, limit = 256, 192, 1.3
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(2 * I, K, generator=g) * 0.15).bfloat16()
    gu = x.double() @ w.double().T
    want = plain.clamped_unit(gu[:, :I], gu[:, I:], limit)
    silu = gu[:, :I] * torch.sigmoid(gu[:, :I]) * gu[:, I:]
    got = []
    if M <= 64:
        got.append((ops.gemm_skinny_silu(x.to(DEV), w.to(DEV), limit=limit, alpha=1.702), want))
        got.append((ops.gemm_skinny_silu(x.to(DEV), w.to(DEV)), silu))
    if ops.gemm_rows_supports(x.to(DEV), w.to(DEV), silu=True):
        got.append((ops.gemm_rows(x.to(DEV), w.to(DEV), silu=True, limit=limit, alpha=1.702), want))
        got.append((ops.gemm_rows(x.to(DEV), w.to(DEV), silu=True), silu))
    assert got
    for out, ref in got:
        assert (out.double().cpu() - ref).abs().max() <= 1e-2 * ref.abs().max()
