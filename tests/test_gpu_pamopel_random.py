"""Pamopel configurations drawn at random (sizes, layer order, which layers read another's keys, taps, groups, table
rows) through the replayer in 32-bit against the plain 64-bit implementation: whole prompts, portions of drawn sizes
followed by single tokens, and a schedule of up to four live requests in a pool and slots that are used again."""
import json
import os
import random

import numpy as np
import pytest
from safetensors.torch import save_file

import plain_pamopel as plain
from gpu_util import DEV

pytestmark = pytest.mark.gpu


def drawn_config(rng):
    width = rng.choice([24, 32, 40, 48, 64, 72, 96, 128, 160, 256])
    layers, own = [], []
    for i in range(rng.randint(2, 6)):
        mlp = dict(kind="dense", ff=rng.choice([16, 24, 40, 64, 100, 128, 200])) if rng.random() < 0.7 else None
        if rng.random() < 0.6:
            if own and rng.random() < 0.35:
                src = rng.choice(own)
                m = dict(layers[src]["mixer"], kv_from=src, scale=rng.choice([0.1, 0.2, 0.5]), bias_max=rng.randint(40, 400))
            else:
                kv = rng.choice([1, 1, 2, 3, 4])
                m = dict(heads=kv * rng.choice([1, 2, 3, 4, 8]), kv_heads=kv, dim=rng.choice([8, 16, 24, 32, 48, 64, 80, 96, 128]),
                         vdim=rng.choice([8, 16, 24, 32, 48, 64, 96, 128]), scale=rng.choice([0.05, 0.125, 0.3]),
                         bias_max=rng.randint(40, 400))
                own.append(i)
            layers.append(dict(type="attention", mixer=m, mlp=mlp))
        else:
            groups = rng.choice([1, 1, 2, 3, 4])
            heads, P = groups * rng.choice([1, 2, 3, 4]), rng.choice([4, 8, 12, 16, 24, 32, 40, 64])
            # parts of at least eight values: the root mean square of two or three values is now and then tiny, and
            # such a token multiplies every rounding before it by hundreds
            parts = rng.choice([d for d in (1, 2, 3, 4, 6, 8) if (heads * P) % d == 0 and heads * P // d >= 8])
            m = dict(heads=heads, vdim=P, state=rng.choice([4, 8, 10, 16, 24, 32, 64, 100, 128]), groups=groups,
                     conv=rng.randint(1, 6), norm_groups=parts)
            layers.append(dict(type="mamba2", mixer=m, mlp=mlp))
    emb = dict(scale=rng.choice([1.0, 3.0, width ** 0.5]))
    if rng.random() < 0.8:
        emb["bigram"] = dict(buckets=rng.choice([7, 61, 251, 4093]), mul_prev=rng.randint(1, 100000), mul_cur=rng.randint(1, 100000))
    return dict(architecture="Pamopel", vocab=rng.randint(40, 700), width=width, layers=layers, embedding=emb,
                norm=dict(eps=rng.choice([1e-5, 1e-6, 1e-3])), residual_mult=rng.choice([0.3, 0.5, 1.0, 0.7]),
                logit_scale=rng.choice([1.0, 2.0, 0.5]))


def worst_error(got, want):
    return float(np.abs(got - want).max() / np.abs(want).max())


@pytest.mark.parametrize("seed", range(8))
def test_drawn_configurations_in_32_bit(seed, tmp_path):
    from ullm_amd.replay import Replayer
    rng = random.Random(4000 + seed)
    cfg = drawn_config(rng)
    rows = rng.choice([4, 6, 13, 16, 24, 64])
    for L in cfg["layers"]:
        if L["type"] == "attention":
            L["mixer"]["bias_max"] = max(L["mixer"]["bias_max"], rows // 2 + 2)
    w = plain.random_weights(cfg, seed, rows, 1.0)
    with open(os.path.join(tmp_path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(tmp_path, "model.safetensors"))
    wide = {k: v.double() for k, v in w.items()}
    reqs = {f"r{i}": [rng.randrange(cfg["vocab"]) for _ in range(rng.randint(20, 110))] for i in range(6)}
    want = {k: plain.forward(wide, cfg, t).float().numpy() for k, t in reqs.items()}
    narrow = {k: v.float() for k, v in w.items()}
    bound = {k: max(3e-5, 4 * worst_error(plain.forward(narrow, cfg, t).numpy(), want[k])) for k, t in reqs.items()}
    rep = Replayer(str(tmp_path), "float32", 512, 16, DEV, max_requests=4)

    # one request alone: whole, then in portions of drawn sizes and token by token
    toks = reqs["r0"]
    got = rep.step({"step": 0, "entries": [{"id": "w", "tokens": toks, "want": list(range(len(toks)))}], "end": ["w"]})
    assert worst_error(got, want["r0"]) <= bound["r0"]
    at, step, parts = 0, 0, []
    sizes = [rng.choice([2, 3, 5, 16, 17, 31]) for _ in range(4)] + [1] * len(toks)
    while at < len(toks):
        n = min(sizes[step], len(toks) - at)
        parts.append(rep.step({"step": step, "entries": [{"id": "c", "tokens": toks[at:at + n], "want": list(range(n))}],
                               "end": ["c"] if at + n == len(toks) else []}))
        at, step = at + n, step + 1
    assert worst_error(np.concatenate(parts), want["r0"]) <= bound["r0"]

    # all of them, at most four alive, some left out of a step; ended requests give their slots and pages back
    waiting, live, at, got = list(reqs), [], {}, {k: [] for k in reqs}
    step = 0
    while waiting or live:
        while waiting and len(live) < 4 and rng.random() < 0.7:
            k = waiting.pop(0)
            live.append(k)
            at[k] = 0
        entries, end = [], []
        for k in list(live):
            if rng.random() < 0.25 and len(live) > 1:
                continue
            n = min(len(reqs[k]) - at[k], rng.choice([1, 1, 1, 2, 3, 7, 16, 17, 40]))
            entries.append({"id": k, "tokens": reqs[k][at[k]:at[k] + n], "want": list(range(n))})
            at[k] += n
            if at[k] == len(reqs[k]):
                end.append(k)
                live.remove(k)
        if not entries:
            continue
        out, o = rep.step({"step": step, "entries": entries, "end": end}), 0
        for e in entries:
            got[e["id"]].append(out[o:o + len(e["tokens"])])
            o += len(e["tokens"])
        step += 1
    for k in reqs:
        assert worst_error(np.concatenate(got[k]), want[k]) <= bound[k], (k, bound[k])
