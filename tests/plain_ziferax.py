"""Plain, slow Ziferax: whole sequences, no cache, one function per mechanism, written from the design's
equations.  It shares no code with ``ullm_amd``; the framework is tested against it.

A model is a dict ``cfg`` (the config.json keys) and a dict ``w`` of tensors by checkpoint name.  Everything is
computed in the dtype of ``w`` (the tests widen to float64 for a sharp oracle).

The design: x_0 = embed[token]; every layer is  x <- x + m * (attention(h) + experts(h)),  h = rms(x) * gain,
with one norm for both sublayers; logits = embed @ (rms(x_L) * final gain).  A layer with ``weights_of: j`` uses
layer j's tensors.
"""
import math
from typing import Dict, List, Optional

import torch

SWISH_SLOPE = 1.702


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rotate_adjacent_pairs(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, d]: for i < dims/2 the pair (x[2i], x[2i+1]) is turned by the angle p * base^(-2i/dims);
    dims from ``dims`` on pass unchanged."""
    if dims == 0:
        return x
    i = torch.arange(dims // 2, dtype=torch.float64)
    angle = positions.to(torch.float64)[:, None] * torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims)
    cos, sin = angle.cos().to(x.dtype)[:, None, :], angle.sin().to(x.dtype)[:, None, :]
    even, odd = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = even * cos - odd * sin
    out[..., 1:dims:2] = odd * cos + even * sin
    return out


def window_mask(T: int, size: int) -> torch.Tensor:
    """[T, T] bool: query i sees key j iff 0 <= i - j < size (size 0: every j <= i)."""
    d = torch.arange(T)[:, None] - torch.arange(T)[None, :]
    return (d >= 0) & ((d < size) if size else torch.ones_like(d, dtype=torch.bool))


def softmax_with_sink(scores: torch.Tensor, sink: torch.Tensor) -> torch.Tensor:
    """Rows of ``scores`` [T, S] (-inf where masked) to weights whose denominator also holds exp(sink)."""
    top = torch.maximum(scores.max(-1).values, sink)
    e = torch.exp(scores - top[:, None])
    return e / (e.sum(-1) + torch.exp(sink - top))[:, None]


def attention(w, prefix: str, m: dict, h: torch.Tensor) -> torch.Tensor:
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w[f"{prefix}.q"].T + w[f"{prefix}.q.b"]).view(T, H, d)
    k = (h @ w[f"{prefix}.k"].T + w[f"{prefix}.k.b"]).view(T, G, d)
    v = k                                                     # the values are the keys as projected
    rot = m.get("rot") or {}
    pos = torch.arange(T)
    qr = rotate_adjacent_pairs(q, pos, rot.get("dims", 0), rot.get("base", 10000.0))
    kr = rotate_adjacent_pairs(k, pos, rot.get("dims", 0), rot.get("base", 10000.0))
    seen = window_mask(T, (m.get("mask") or {}).get("size", 0))
    heads = []
    for a in range(H):
        g = a // (H // G)
        s = (qr[:, a] @ kr[:, g].T) * m["scale"]
        s = s.masked_fill(~seen, -math.inf)
        heads.append(softmax_with_sink(s, w[f"{prefix}.sink"][a]) @ v[:, g])
    return torch.cat(heads, -1) @ w[f"{prefix}.o"].T + w[f"{prefix}.o.b"]


def clamped_unit(gate: torch.Tensor, up: torch.Tensor, limit: float) -> torch.Tensor:
    g = torch.clamp(gate, max=limit)
    u = torch.clamp(up, -limit, limit)
    return g * torch.sigmoid(SWISH_SLOPE * g) * (u + 1)


def expert(w, prefix: str, limit: float, h: torch.Tensor) -> torch.Tensor:
    return clamped_unit(h @ w[f"{prefix}.gate"].T, h @ w[f"{prefix}.up"].T, limit) @ w[f"{prefix}.down"].T


MARGINS = None      # a list: route() then appends, per call, every token's gap between the last choice score taken and the first left


def route(w, prefix: str, r: dict, h: torch.Tensor):
    """(indices [T, top], weights [T, top]): softmax over all router outputs, the choice by score + correction,
    the weights by the chosen scores over their sum."""
    s = torch.softmax(h @ w[f"{prefix}.router"].T, -1)
    if MARGINS is not None:
        ranked = torch.sort(s + w[f"{prefix}.correction"], dim=-1, descending=True).values
        MARGINS.append(ranked[:, r["top"] - 1] - ranked[:, r["top"]] if r["top"] < ranked.shape[1]
                       else torch.full((h.shape[0],), math.inf, dtype=h.dtype))
    chosen = torch.topk(s + w[f"{prefix}.correction"], r["top"], dim=-1).indices
    picked = torch.gather(s, 1, chosen)
    return chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20)


def experts(w, prefix: str, mlp: dict, h: torch.Tensor) -> torch.Tensor:
    r = mlp["router"]
    chosen, weight = route(w, prefix, r, h)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t].tolist(), weight[t]):
            if e >= r["experts"]:                              # an identity expert: its output is its input
                out[t] += a * h[t]
            else:
                out[t] += a * expert(w, f"{prefix}.e{e}", mlp["expert"]["limit"], h[t:t + 1])[0]
    if mlp.get("shared"):
        out = out + expert(w, f"{prefix}.shared", mlp["shared"]["limit"], h)
    return out


def forward(w, cfg: dict, tokens: List[int], streams: Optional[list] = None, round_to=None) -> torch.Tensor:
    """Logits [len(tokens), vocab]; with ``streams`` the residual stream after every layer is appended to it.
    With ``round_to`` (a dtype) every normed layer input and the head's input is rounded to it and widened again:
    what rounding of the sublayers' inputs alone does to the logits, a floor for any engine that computes in it."""
    def rounded(h):
        return h if round_to is None else h.to(round_to).to(h.dtype)

    x = w["embed"][torch.tensor(tokens)]
    eps, mult = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    for i, L in enumerate(cfg["layers"]):
        p = f"l{L['weights_of'] if L.get('weights_of') is not None else i}"
        h = rounded(rms(x, eps) * w[f"{p}.norm1"])
        y = attention(w, f"{p}.mix", L["mixer"], h)
        if L.get("mlp") is not None:
            y = y + experts(w, f"{p}.mlp", L["mlp"], h)
        x = x + mult * y
        if streams is not None:
            streams.append(x.clone())
    return rounded(rms(x, eps) * w["final.norm"]) @ w["embed"].T


def greedy_generate(w, cfg, prompt: List[int], n: int) -> List[int]:
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(forward(w, cfg, toks)[-1].argmax())
        toks.append(nxt)
        out.append(nxt)
    return out


def random_weights(cfg: dict, seed: int, std: float = 0.08, sink_std: float = 1.0, correction_std: float = 0.05,
                   router_std: Optional[float] = None) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors under the design's names.  Sinks of about one unit and a router whose scores differ: a sink
    left out, or a correction that leaks into the weights, then moves the logits far beyond rounding.  The router's
    logits are about a unit and a half wide whatever the width (a saturated softmax leaves the choice among the
    others to the corrections, whose bfloat16 values tie)."""
    g = torch.Generator().manual_seed(seed)
    H = cfg["width"]
    if router_std is None:
        router_std = 1.5 / math.sqrt(H)

    def mat(*shape, s=std):
        return (torch.randn(*shape, generator=g) * s).bfloat16()

    w = {"embed": mat(cfg["vocab"], H, s=0.5), "final.norm": (1 + 0.2 * torch.randn(H, generator=g)).bfloat16()}
    for i, L in enumerate(cfg["layers"]):
        if L.get("weights_of") is not None:
            continue
        p, m = f"l{i}", L["mixer"]
        w[f"{p}.norm1"] = (1 + 0.2 * torch.randn(H, generator=g)).bfloat16()
        w[f"{p}.mix.q"], w[f"{p}.mix.q.b"] = mat(m["heads"] * m["dim"], H, s=0.25), mat(m["heads"] * m["dim"], s=0.3)
        w[f"{p}.mix.k"], w[f"{p}.mix.k.b"] = mat(m["kv_heads"] * m["dim"], H, s=0.25), mat(m["kv_heads"] * m["dim"], s=0.3)
        w[f"{p}.mix.o"], w[f"{p}.mix.o.b"] = mat(H, m["heads"] * m["dim"]), mat(H, s=0.3)
        w[f"{p}.mix.sink"] = mat(m["heads"], s=sink_std)
        mlp = L.get("mlp")
        if mlp is None:
            continue
        r = mlp["router"]
        n_out = r["experts"] + r.get("identity", 0)
        w[f"{p}.mlp.router"], w[f"{p}.mlp.correction"] = mat(n_out, H, s=router_std), mat(n_out, s=correction_std)
        names = [f"e{e}" for e in range(r["experts"])]
        sizes = [mlp["expert"]["ff"]] * r["experts"]
        if mlp.get("shared"):
            names.append("shared")
            sizes.append(mlp["shared"]["ff"])
        for name, ff in zip(names, sizes):
            w[f"{p}.mlp.{name}.gate"], w[f"{p}.mlp.{name}.up"] = mat(ff, H, s=0.3), mat(ff, H, s=0.3)
            w[f"{p}.mlp.{name}.down"] = mat(H, ff)
    return w
