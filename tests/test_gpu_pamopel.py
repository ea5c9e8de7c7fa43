"""Pamopel in the framework against the plain implementation (``plain_pamopel``, 64-bit): each mechanism's kernels
alone; whole prompts; a prompt and then token by token, also from the very first token; portions down to two
tokens; unequal requests in one batch against each alone, in a pool and slots that are used again; a distance bias
that decides every weight (every bucket's edge, in prompts and in decoding); scores scaled so that single far keys
stand out; long decoding through captured steps; sizes that differ wherever they can; greedy generation through the
entry point.  In 32-bit and in bfloat16."""
import json
import os

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

import plain_pamopel as plain
from gpu_util import DEV

pytestmark = pytest.mark.gpu

REL = {"float32": 2e-5, "bfloat16": 3e-2}


def attn(heads, kv, dim, vdim, far, scale, ff=None, kv_from=None):
    m = dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, bias_max=far, scale=scale)
    if kv_from is not None:
        m["kv_from"] = kv_from
    return dict(type="attention", mixer=m, mlp=dict(kind="dense", ff=ff) if ff else None)


def mamba(heads, vdim, state, groups, conv, norm_groups, ff=None):
    return dict(type="mamba2", mixer=dict(heads=heads, vdim=vdim, state=state, groups=groups, conv=conv,
                                          norm_groups=norm_groups), mlp=dict(kind="dense", ff=ff) if ff else None)


def config(width, vocab, layers, bigram=(61, 7, 3), scale=3.0, mult=0.5, logit_scale=1.5, eps=1e-5):
    emb = dict(scale=scale)
    if bigram:
        emb["bigram"] = dict(buckets=bigram[0], mul_prev=bigram[1], mul_cur=bigram[2])
    return dict(architecture="Pamopel", vocab=vocab, width=width, layers=layers, embedding=emb, norm=dict(eps=eps),
                residual_mult=mult, logit_scale=logit_scale)


# P: the usual shape: a layer on another's keys and values, a state-space layer without a feed-forward
CFG_P = config(48, 97, [attn(4, 2, 16, 16, 40, 0.3, ff=80), attn(4, 2, 16, 16, 40, 0.3, ff=64, kv_from=0),
                        mamba(3, 16, 8, 1, 4, 3), attn(2, 1, 32, 32, 24, 0.2, ff=56)])
# Q: sizes that differ wherever they can: key size != value size (both padded in the cache), as many key heads as
# query heads, a group per state-space head, one norm part, two taps, a feed-forward behind the state-space layer and
# none behind attention, no multiplier, few table rows
CFG_Q = config(40, 131, [mamba(4, 12, 20, 4, 2, 1, ff=72), attn(3, 3, 24, 40, 50, 0.25), attn(3, 3, 24, 40, 9, 0.25, kv_from=1),
                         mamba(2, 24, 6, 2, 3, 2)], bigram=(17, 1000003, 999983), scale=1.0, mult=1.0, logit_scale=1.0, eps=1e-3)
# R: no bigram table, a convolution of one tap (nothing carried), a state larger than the head
CFG_R = config(32, 64, [mamba(2, 8, 24, 1, 1, 2), attn(2, 2, 8, 16, 30, 0.5, ff=48)], bigram=None, mult=0.25)
# S: attention alone with scores scaled so that a softmax row is nearly one key, and a flat distance table
CFG_S = config(32, 50, [attn(2, 1, 16, 16, 100, 6.0, ff=40), attn(2, 1, 16, 16, 100, 6.0, kv_from=0)])
# B: a distance table that decides every weight (queries scaled away)
CFG_B = config(32, 50, [attn(3, 1, 16, 16, 37, 0.01)])
# T: head sizes the matrix-core kernels take, keys and values of different size (32 | 64 and 64 | 32), a state-space
# layer first and last with sizes that cut into 16-byte pieces (the vector convolution, the register scan), a
# feed-forward behind one of them, three query heads a key head
CFG_T = config(64, 113, [mamba(4, 16, 16, 2, 4, 2, ff=96), attn(6, 2, 32, 64, 64, 0.2, ff=96),
                         attn(6, 2, 32, 64, 64, 0.2, kv_from=1), attn(4, 4, 64, 32, 20, 0.15), mamba(4, 16, 64, 1, 3, 1)],
               bigram=(251, 5, 11), mult=0.7)
MODELS = {"P": (CFG_P, 1, 32, 1.0), "Q": (CFG_Q, 2, 6, 1.0), "R": (CFG_R, 3, 32, 1.0), "S": (CFG_S, 4, 32, 0.1),
          "B": (CFG_B, 5, 13, 4.0), "T": (CFG_T, 6, 24, 1.0)}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """{name: (folder, config, 64-bit weights)}; the folders hold bfloat16 tensors under the design's names."""
    out = {}
    for name, (cfg, seed, rel_rows, rel_std) in MODELS.items():
        d = tmp_path_factory.mktemp(f"pamopel{name}")
        w = plain.random_weights(cfg, seed, rel_rows, rel_std)
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


def close(got, want, dtype, name=""):
    if dtype == "bfloat16" and name in ("P", "Q", "R", "T"):
        # A state-space layer norms its gated output in parts, and the block norms the branch again: at a token where
        # a part happens to be ten times smaller than usual, the rounding of the layer's input comes out ten times
        # larger (seen: one row of 75 at 6e-2 of the largest logit where the 64-bit implementation with weights
        # perturbed by 2^-9 moves by 1e-2 to 2e-2).  So in bfloat16 these models are held to the usual bound on 95 of
        # 100 rows and to a bound that a lost key, a wrong state or a stale slot exceeds on every row.
        err = np.abs(got - want).max(-1) / float(np.abs(want).max())
        assert np.median(err) <= 1.5e-2 and np.quantile(err, 0.95) <= REL[dtype] and err.max() <= 0.2, \
            f"median {np.median(err):.3e}, 95th {np.quantile(err, 0.95):.3e}, max {err.max():.3e} at row {int(err.argmax())}"
        return
    bound = REL[dtype] * float(np.abs(want).max()) + 1e-6
    err = float(np.abs(got - want).max())
    assert err <= bound, f"max |diff| {err:.3e} > {bound:.3e} (first bad row {int(np.argmax(np.abs(got - want).max(-1) > bound))})"


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


CASES = [(n, d) for n in ("P", "Q", "R", "T") for d in ("float32", "bfloat16")]


@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompts(replayers, models, name, dtype):
    rep = replayers(name, dtype)
    for i, n in enumerate((1, 2, 15, 16, 17, 75)):
        toks = tokens(models[name][1]["vocab"], n, 10 + i)
        close(run(rep, "r", toks, [n]), oracle(models, name, toks), dtype, name)


@pytest.mark.parametrize("name,dtype", CASES)
def test_a_prompt_and_then_token_by_token(replayers, models, name, dtype):
    toks = tokens(models[name][1]["vocab"], 75, 15)
    for graphs in (True, False):
        close(run(replayers(name, dtype, use_graphs=graphs), "r", toks, [40]), oracle(models, name, toks), dtype, name)


@pytest.mark.parametrize("name,dtype", CASES)
def test_token_by_token_from_the_first_token(replayers, models, name, dtype):
    toks = tokens(models[name][1]["vocab"], 40, 16)
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
def test_long_decoding_over_many_pages(replayers, models, dtype):
    toks = tokens(models["P"][1]["vocab"], 150, 40)
    close(run(replayers("P", dtype), "r", toks, [3]), oracle(models, "P", toks), dtype, "P")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cuts", [(90,), (5,), (31, 2, 2, 29, 2, 2)])
def test_a_distance_table_that_decides_every_weight(replayers, models, dtype, cuts):
    """The queries are scaled away and the table's entries are several units apart: a key counted into the wrong
    row, or the rows beyond the table's reach, change the logits by far more than rounding.  Prompts and single
    tokens both pass every edge of the 13 rows (reach 37) and go on beyond it."""
    toks = tokens(models["B"][1]["vocab"], 90, 41)
    close(run(replayers("B", dtype), "r", toks, cuts), oracle(models, "B", toks), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cuts", [(260,), (200,), (17, 64, 2, 130, 2, 30)])
def test_scores_scaled_so_that_single_far_keys_stand_out(replayers, models, dtype, cuts):
    """With the scores multiplied by six a softmax row is close to one key, somewhere among up to 260: a key lost
    or doubled at a page's border, or one that a portion or a single token does not reach, takes a whole value
    out of the sum."""
    toks = tokens(models["S"][1]["vocab"], 260, 42)
    want = oracle(models, "S", toks)
    _, cfg, w = models["S"]
    got = run(replayers("S", dtype), "r", toks, cuts)
    if dtype == "float32":
        close(got, want, dtype)
    else:
        # one key's weight moves by percents under bfloat16 rounding of peaked scores: the rows must agree where
        # the 32-bit engine agrees, within a bound a lost key would exceed many times
        err = np.abs(got - want).max(-1) / np.abs(want).max()
        assert np.median(err) < 3e-2 and err.max() < 0.25, (np.median(err), err.max())


# (heads, head size, state, groups, taps, norm parts, tokens of the first step, of the second): sizes that no 16-byte
# access fits; one row of state a thread; a head that does not cut into whole slices and a state below the rows a
# block covers, over several staged chunks; the usual sizes; whole heads a block (many heads), with a state that
# fills the rows and one that does not; a state of many rows a thread
SSM_SHAPES = [(4, 12, 10, 2, 3, 2, (5, 1, 2), (1, 4, 1)),
              (4, 16, 8, 2, 4, 2, (5, 1, 2), (1, 4, 1)),
              (6, 40, 44, 3, 4, 2, (37, 1, 20), (1, 40, 3)),
              (8, 64, 128, 2, 4, 4, (33, 2, 16), (17, 1, 32)),
              (344, 64, 24, 8, 2, 8, (18, 1, 2), (1, 21, 1)),
              (342, 64, 72, 2, 3, 2, (3, 17, 1), (16, 2, 1)),
              (2, 16, 200, 1, 2, 1, (19, 1, 2), (1, 4, 30))]


@pytest.mark.parametrize("heads,P,N,groups,taps,parts,lens1,lens2", SSM_SHAPES)
def test_kernels_of_the_state_space_mixer_alone(heads, P, N, groups, taps, parts, lens1, lens2):
    """Convolution with carried inputs, the recurrence with carried state, gate and grouped norm: two steps of a
    batch of three entries against the plain functions run over each entry's whole sequence.  (In the first shape
    entry 1 brings fewer tokens than taps-1 and then more.)"""
    from ullm_amd.kernels import ops
    g = torch.Generator().manual_seed(7)
    inner, ch = heads * P, heads * P + 2 * groups * N
    cols = inner + ch + heads
    conv_w, conv_b = torch.randn(ch, taps, generator=g) * 0.5, torch.randn(ch, generator=g) * 0.2
    dt_bias, a_log, d_skip = (torch.randn(heads, generator=g) * 0.5 for _ in range(3))
    gain = 1 + 0.2 * torch.randn(inner, generator=g)
    seqs = [torch.randn(a + b, cols, generator=g) for a, b in zip(lens1, lens2)]
    state = torch.zeros(4, (taps - 1) * ch + heads * N * P, device=DEV)
    slots = torch.tensor([2, 0, 3], dtype=torch.int32, device=DEV)
    dev = lambda t: t.to(DEV).contiguous()                                      # noqa: E731
    outs = [[], [], []]
    for lens, first in ((lens1, [0, 0, 0]), (lens2, list(lens1))):
        proj = torch.cat([s[f:f + n] for s, f, n in zip(seqs, first, lens)])
        q_start = torch.tensor(np.concatenate(([0], np.cumsum(lens))), dtype=torch.int32, device=DEV)
        entry = torch.repeat_interleave(torch.arange(3), torch.tensor(lens)).to(torch.int32).to(DEV)
        pj = dev(proj)
        xbc = ops.conv_silu(pj, inner, ch, dev(conv_w), dev(conv_b), state, entry, q_start, slots, 3)
        y = ops.ssm_scan(xbc, pj, inner + ch, dev(dt_bias), dev(a_log), dev(d_skip), state, (taps - 1) * ch, q_start, slots, 3,
                         heads, groups, N, P)
        out = ops.gated_group_norm(y, pj, 0, dev(gain), 1e-5, parts, torch.float32).cpu()
        t = 0
        for b, n in enumerate(lens):
            outs[b].append(out[t:t + n])
            t += n
    for b, s in enumerate(seqs):
        s = s.double()
        T = s.shape[0]
        xbc = plain.causal_conv_silu(s[:, inner:inner + ch], conv_w.double(), conv_b.double())
        y, S = plain.ssm_recurrence(xbc[:, :inner].reshape(T, heads, P), xbc[:, inner:inner + groups * N].reshape(T, groups, N),
                                    xbc[:, inner + groups * N:].reshape(T, groups, N),
                                    plain.softplus(s[:, inner + ch:] + dt_bias.double()), a_log.double(), d_skip.double())
        want = plain.gated_group_rms(y.reshape(T, inner), s[:, :inner], gain.double(), parts, 1e-5)
        got = torch.cat(outs[b]).double()
        assert (got - want).abs().max() <= 2e-5 * want.abs().max()
        kept = state[int(slots[b]), (taps - 1) * ch:].cpu().double().view(heads, N, P)
        assert (kept - S).abs().max() <= 2e-5 * S.abs().max()
        carried = state[int(slots[b]), :(taps - 1) * ch].cpu().double().view(taps - 1, ch)
        assert torch.equal(carried.float(), s[T - (taps - 1):, inner:inner + ch].float())


def test_embedding_sum_with_the_id_before_a_portion_carried():
    from ullm_amd.kernels import ops
    from ullm_amd.parts.embedding import sinusoid_table
    g = torch.Generator().manual_seed(8)
    V, H, buckets = 30, 20, 11
    cfg = dict(width=H, embedding=dict(scale=2.5, bigram=dict(buckets=buckets, mul_prev=2000003, mul_cur=5)))
    w = dict(embed=torch.randn(V, H, generator=g), bigram=torch.randn(buckets + 1, H, generator=g))
    seqs = [tokens(V, 7, 1), tokens(V, 3, 2)]
    last = torch.full((3, 1), 77, dtype=torch.int32, device=DEV)            # stale ids of earlier requests
    table = sinusoid_table(16, H).to(DEV)
    got = [[], []]
    for (a0, a1), (b0, b1) in (((0, 4), (0, 1)), ((4, 5), (1, 3)), ((5, 7), (3, 3))):
        parts = [(0, seqs[0][a0:a1], a0), (1, seqs[1][b0:b1], b0)]
        parts = [p for p in parts if p[1]]
        ids = torch.tensor([t for _, ts, _ in parts for t in ts], dtype=torch.int32, device=DEV)
        pos = torch.tensor([s + i for _, ts, s in parts for i in range(len(ts))], dtype=torch.int32, device=DEV)
        ent = torch.tensor([e for e, (_, ts, _) in enumerate(parts) for _ in ts], dtype=torch.int32, device=DEV)
        q_start = torch.tensor(np.concatenate(([0], np.cumsum([len(ts) for _, ts, _ in parts]))), dtype=torch.int32, device=DEV)
        slot = torch.tensor([2 if r == 0 else 0 for r, _, _ in parts], dtype=torch.int32, device=DEV)
        out = ops.embedding_sum(ids, w["embed"].to(DEV), 2.5, w["bigram"].to(DEV), 2000003, 5, table, pos, ent, q_start, slot, last).cpu()
        t = 0
        for r, ts, _ in parts:
            got[r].append(out[t:t + len(ts)])
            t += len(ts)
    for r in range(2):
        want = plain.embed({k: v.double() for k, v in w.items()}, cfg, seqs[r])
        assert (torch.cat(got[r]).double() - want).abs().max() < 1e-5


@pytest.mark.parametrize("kind,post_kind", [(1, 1), (0, 1), (1, 0), (1, None)])
def test_norm_behind_a_branch_the_add_and_the_next_norm_in_one_pass(kind, post_kind):
    from ullm_amd.kernels import ops
    g = torch.Generator().manual_seed(9)
    T, H, eps = 5, 70, 1e-3
    branch, res = torch.randn(T, H, generator=g) * 3 + 1, torch.randn(T, H, generator=g)
    gain, post_gain = 1 + 0.3 * torch.randn(H, generator=g), 1 + 0.3 * torch.randn(H, generator=g)
    norm = {0: lambda x, w: plain.rms(x, eps) * w, 1: lambda x, w: plain.layer_norm(x, w, eps)}
    b = branch.double() if post_kind is None else norm[post_kind](branch.double(), post_gain.double())
    stream = res.double() + 0.3 * b
    want = norm[kind](stream, gain.double())
    for dt, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        r = res.to(DEV).clone()
        bb = branch.to(DEV, dt)
        if dt == torch.bfloat16:
            b = bb.double().cpu() if post_kind is None else norm[post_kind](bb.double().cpu(), post_gain.double())
            stream, want = res.double() + 0.3 * b, norm[kind](res.double() + 0.3 * b, gain.double())
        got = ops.add_norm_general(bb, r, gain.to(DEV), eps, kind, dt, post_gain=None if post_kind is None else post_gain.to(DEV),
                                   post_eps=eps, post_kind=post_kind or 0, mult=0.3)
        assert (got.double().cpu() - want).abs().max() <= tol * want.abs().max()
        assert (r.double().cpu() - stream).abs().max() <= 1e-5 * stream.abs().max()
        rows = torch.tensor([3, 0], dtype=torch.int32, device=DEV)
        r2 = res.to(DEV).clone()
        some = ops.add_norm_general(bb, r2, gain.to(DEV), eps, kind, dt, rows=rows, post_gain=None if post_kind is None else post_gain.to(DEV),
                                    post_eps=eps, post_kind=post_kind or 0, mult=0.3)
        assert torch.equal(some, got[[3, 0]]) and torch.equal(r2.cpu(), res)


@pytest.mark.parametrize("name", ["P", "Q", "T"])
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
    d, cfg, _ = models["P"]
    toks = tokens(cfg["vocab"], 40, 60)
    want = oracle(models, "P", toks)
    tr = trace_run(d, "float32", 128)
    a = tr.step([("a", toks[:21], [0, 20])])
    b = tr.step([("a", toks[21:], [18])], end=["a"])
    tr.close()
    close(np.concatenate((a, b)), want[[0, 20, 39]], "float32")


@pytest.mark.parametrize("rows", [70, 2100])        # 2100: more distances than the prompt kernel keeps in shared memory
@pytest.mark.parametrize("hd,nq,nkv", [(64, 10, 2), (128, 6, 2), (32, 20, 1), (96, 4, 4), (256, 2, 1)])
def test_matrix_core_attention_with_distance_bias_and_head_gates(hd, nq, nkv, rows):
    """The bfloat16 kernels (single tokens cut over splits and their reduce; prompt tiles) against 64-bit softmax
    attention on the same rounded operands: a bias by distance whose entries are units apart, clamped at the
    table's last entry, and a gate per head; contexts that end at and beside tile and page borders, one past 1 100
    keys; a prompt portion that starts in the middle of a page beside single tokens."""
    import math
    from types import SimpleNamespace
    from gpu_util import paged_cache, table_tensor
    from ullm_amd.kernels import ops
    from ullm_amd.parts import GroupView, StepShape
    from ullm_amd.parts.attention import plan_attention_step
    g = torch.Generator().manual_seed(hd + nq)
    starts, lens = [1130, 31, 64, 200, 0], [1, 1, 1, 45, 33]            # tokens before the step, new tokens
    bias = (torch.randn(nq, rows, generator=g) * 2).float()
    seqs_k = [torch.randn(s + n, nkv, hd, generator=g).bfloat16().float() for s, n in zip(starts, lens)]
    seqs_v = [torch.randn(s + n, nkv, hd, generator=g).bfloat16().float() for s, n in zip(starts, lens)]
    k_pool, v_pool, tables = paged_cache(seqs_k, seqs_v, 16, torch.bfloat16, DEV, fill=0.0)
    T = sum(lens)
    q = torch.randn(T, nq, hd, generator=g).bfloat16()
    gate = torch.randn(T, nq + 3, generator=g).bfloat16()
    positions = torch.tensor([s + i for s, n in zip(starts, lens) for i in range(n)], dtype=torch.int32, device=DEV)
    entry = torch.tensor([b for b, n in enumerate(lens) for _ in range(n)], dtype=torch.int32, device=DEV)
    plan = plan_attention_step(StepShape(tuple(lens), tuple(starts)))
    plan.arrays = {k: torch.tensor(v, dtype=torch.int32, device=DEV) for k, v in plan.arrays.items()}
    group = GroupView(table_tensor(tables, DEV), 0, 16, 0)
    ctx = SimpleNamespace(positions=positions, token_entry=entry)
    scale = 0.7 / math.sqrt(hd)
    out = ops.paged_attention(q.view(T, nq * hd).to(DEV), k_pool, v_pool, ctx, group, nq, nkv, hd, scale, 0, plan,
                              bias=bias.to(DEV), bias_log2=(bias * math.log2(math.e)).to(DEV), gate=gate.to(DEV))
    out = out.float().cpu().view(T, nq, hd)
    t = 0
    for b, (s, n) in enumerate(zip(starts, lens)):
        for i in range(n):
            pos = s + i
            dist = (pos - torch.arange(pos + 1)).clamp(max=rows - 1)
            for h in range(nq):
                kv = h // (nq // nkv)
                sc = (seqs_k[b][:pos + 1, kv].double() @ q[t, h].double()) * scale + bias[h][dist].double()
                want = (torch.softmax(sc, 0) @ seqs_v[b][:pos + 1, kv].double()) * torch.sigmoid(gate[t, h].double())
                err = (out[t, h].double() - want).abs().max()
                assert err <= 2e-2 * max(1.0, float(want.abs().max())), (b, i, h, float(err))
            t += 1
