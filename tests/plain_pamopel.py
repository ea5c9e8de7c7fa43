"""Plain, slow Pamopel: whole sequences, no cache, one function per mechanism, written from the
design's equations.  It shares no code with ``ullm_amd``; the framework is tested against it.

A model is a dict ``cfg`` (the config.json keys) and a dict ``w`` of tensors by checkpoint name.
Everything is computed in the dtype of ``w`` (the tests widen to float64 for a sharp oracle).
"""
import math
from typing import Dict, List

import torch


def layer_norm(x, gain, eps):
    mean = x.mean(-1, keepdim=True)
    dev = x - mean
    return dev / torch.sqrt((dev * dev).mean(-1, keepdim=True) + eps) * gain


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def sinusoid(positions: torch.Tensor, width: int, dtype) -> torch.Tensor:
    """[len, width]: entry 2i = sin(p * 10000^(-2i/width)), entry 2i+1 = cos of the same angle."""
    i = torch.arange((width + 1) // 2, dtype=torch.float64)
    freq = torch.pow(torch.tensor(10000.0, dtype=torch.float64), -2.0 * i / width)
    angle = positions.to(torch.float64)[:, None] * freq[None, :]
    out = torch.zeros(len(positions), 2 * len(i), dtype=torch.float64)
    out[:, 0::2] = angle.sin()
    out[:, 1::2] = angle.cos()
    return out[:, :width].to(dtype)


def embed(w, cfg, tokens: List[int]) -> torch.Tensor:
    e = cfg["embedding"]
    ids = torch.tensor(tokens)
    x = w["embed"][ids] * e["scale"]
    big = e.get("bigram")
    if big:
        rows = [big["buckets"]] + [(tokens[t - 1] * big["mul_prev"] + tokens[t] * big["mul_cur"]) % big["buckets"]
                                   for t in range(1, len(tokens))]
        x = x + w["bigram"][torch.tensor(rows)]
    return x + sinusoid(torch.arange(len(tokens)), cfg["width"], x.dtype)


def distance_bucket(n: int, rows: int, far: int) -> int:
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def attention(w, p: str, m: dict, h: torch.Tensor, eps: float, shared_kv: dict, layer: int):
    """One attention mixer on the normed input h [T, width]; ``shared_kv`` maps a layer to its (k, v)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ w[f"{p}.q"].T
    q = rms(q, eps) * w[f"{p}.q.norm"]
    if "kv_from" in m and m["kv_from"] is not None:
        k, v = shared_kv[m["kv_from"]]
    else:
        k = rms(h @ w[f"{p}.k"].T, eps) * w[f"{p}.k.norm"]
        v = h @ w[f"{p}.v"].T
        shared_kv[layer] = (k, v)
    q, k, v = q.view(T, H, d), k.view(T, G, d), v.view(T, G, dv)
    rel = w[f"{p}.rel"]
    rows = rel.shape[0]
    gate = torch.sigmoid(h @ w[f"{p}.g"].T)                      # [T, H]
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        kv = head // (H // G)
        for i in range(T):
            s = (k[: i + 1, kv] @ q[i, head]) * m["scale"]
            s = s + torch.stack([rel[distance_bucket(i - j, rows, m["bias_max"]), head] for j in range(i + 1)])
            out[i, head] = torch.softmax(s, 0) @ v[: i + 1, kv]
    out = out * gate[:, :, None]
    return out.reshape(T, H * dv) @ w[f"{p}.o"].T


def mamba2(w, p: str, m: dict, h: torch.Tensor, eps: float):
    T = h.shape[0]
    nh, P, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = nh * P
    proj = h @ w[f"{p}.in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    padded = torch.cat((torch.zeros(taps - 1, xbc.shape[1], dtype=h.dtype), xbc), 0)
    conv = w[f"{p}.conv.b"].clone()[None, :].repeat(T, 1)
    for j in range(taps):                                        # the last column is the current token's
        conv = conv + padded[j:j + T] * w[f"{p}.conv"][:, j]
    xbc = silu(conv)
    x = xbc[:, :inner].view(T, nh, P)
    Bm = xbc[:, inner:inner + G * N].view(T, G, N)
    Cm = xbc[:, inner + G * N:].view(T, G, N)
    dt = torch.nn.functional.softplus(dt + w[f"{p}.dt_bias"], threshold=1e9)
    decay = torch.exp(-torch.exp(w[f"{p}.A_log"]) * dt)          # [T, nh]
    y = torch.zeros(T, nh, P, dtype=h.dtype)
    for head in range(nh):
        g = head // (nh // G)
        S = torch.zeros(N, P, dtype=h.dtype)
        for t in range(T):
            S = decay[t, head] * S + dt[t, head] * torch.outer(Bm[t, g], x[t, head])
            y[t, head] = S.T @ Cm[t, g] + w[f"{p}.D"][head] * x[t, head]
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * w[f"{p}.norm"]
    return y @ w[f"{p}.o"].T


def dense_ff(w, p: str, h: torch.Tensor):
    return (silu(h @ w[f"{p}.gate"].T) * (h @ w[f"{p}.up"].T)) @ w[f"{p}.down"].T


def forward(w: Dict[str, torch.Tensor], cfg: dict, tokens: List[int], streams: list = None) -> torch.Tensor:
    """Logits [T, vocab] of a whole sequence; ``streams`` (a list) receives the stream after every layer."""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = embed(w, cfg, tokens)
    shared_kv = {}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}"
        h = layer_norm(x, w[f"{p}.norm1"], eps)
        if L["type"] == "attention":
            y = attention(w, f"{p}.mix", L["mixer"], h, eps, shared_kv, i)
        elif L["type"] == "mamba2":
            y = mamba2(w, f"{p}.mix", L["mixer"], h, eps)
        else:
            raise ValueError(L["type"])
        x = x + mult * layer_norm(y, w[f"{p}.norm1b"], eps)
        if L.get("mlp"):
            y = dense_ff(w, f"{p}.mlp", layer_norm(x, w[f"{p}.norm2"], eps))
            x = x + mult * layer_norm(y, w[f"{p}.norm2b"], eps)
        if streams is not None:
            streams.append(x.clone())
    return (layer_norm(x, w["final.norm"], eps) @ w["head"].T) * cfg["logit_scale"]
