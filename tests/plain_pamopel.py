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


def distance_bias(rel: torch.Tensor, T: int, far: int) -> torch.Tensor:
    """[heads, T, T]: entry [h, i, j] = rel[bucket(i - j), h] for j <= i, -inf above the diagonal."""
    rows = rel.shape[0]
    by_distance = rel[torch.tensor([distance_bucket(n, rows, far) for n in range(T)])]       # [T, heads]
    i = torch.arange(T)
    dist = i[:, None] - i[None, :]
    bias = by_distance[dist.clamp(min=0)].permute(2, 0, 1).clone()
    bias[:, dist < 0] = float("-inf")
    return bias


def attention(w, p: str, m: dict, h: torch.Tensor, eps: float, shared_kv: dict, layer: int):
    """One attention mixer on the normed input h [T, width]; ``shared_kv`` maps a layer to its (k, v)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms(h @ w[f"{p}.q"].T, eps) * w[f"{p}.q.norm"]           # over the whole projection, then split
    if m.get("kv_from") is not None:
        k, v = shared_kv[m["kv_from"]]
    else:
        k = rms(h @ w[f"{p}.k"].T, eps) * w[f"{p}.k.norm"]
        v = h @ w[f"{p}.v"].T
        shared_kv[layer] = (k, v)
    q, k, v = q.view(T, H, d), k.view(T, G, d), v.view(T, G, dv)
    bias = distance_bias(w[f"{p}.rel"], T, m["bias_max"])
    gate = torch.sigmoid(h @ w[f"{p}.g"].T)                      # [T, H]
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        kv = head // (H // G)
        scores = (q[:, head] @ k[:, kv].T) * m["scale"] + bias[head]
        out[:, head] = torch.softmax(scores, dim=-1) @ v[:, kv]
    out = out * gate[:, :, None]
    return out.reshape(T, H * dv) @ w[f"{p}.o"].T


def causal_conv_silu(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, before: torch.Tensor = None):
    """x [T, channels]; weight [channels, taps], last column for the current token; ``before``: the taps-1 inputs
    ahead of x (zeros at a sequence's start)."""
    T, taps = x.shape[0], weight.shape[1]
    if before is None:
        before = torch.zeros(taps - 1, x.shape[1], dtype=x.dtype)
    padded = torch.cat((before, x), 0)
    out = bias[None, :].repeat(T, 1)
    for j in range(taps):
        out = out + padded[j:j + T] * weight[:, j]
    return silu(out)


def ssm_recurrence(x, Bm, Cm, dt, a_log, d_skip, S0=None):
    """x [T, heads, P], Bm/Cm [T, groups, N], dt [T, heads] (after softplus); returns (y [T, heads, P], S [heads, N, P])."""
    T, nh, P = x.shape
    G, N = Bm.shape[1:]
    S = torch.zeros(nh, N, P, dtype=x.dtype) if S0 is None else S0.clone()
    y = torch.zeros(T, nh, P, dtype=x.dtype)
    for t in range(T):
        for head in range(nh):
            g = head // (nh // G)
            decay = torch.exp(-torch.exp(a_log[head]) * dt[t, head])
            S[head] = decay * S[head] + dt[t, head] * torch.outer(Bm[t, g], x[t, head])
            y[t, head] = S[head].T @ Cm[t, g] + d_skip[head] * x[t, head]
    return y, S


def gated_group_rms(y, z, gain, parts: int, eps: float):
    T, inner = y.shape
    v = y * silu(z)
    return rms(v.view(T, parts, inner // parts), eps).reshape(T, inner) * gain


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + z.clamp(min=0)


def mamba2(w, p: str, m: dict, h: torch.Tensor, eps: float):
    T = h.shape[0]
    nh, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = nh * P
    proj = h @ w[f"{p}.in"].T                                    # z | x | B | C | dt
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = causal_conv_silu(xbc, w[f"{p}.conv"], w[f"{p}.conv.b"])
    x = xbc[:, :inner].reshape(T, nh, P)
    Bm = xbc[:, inner:inner + G * N].reshape(T, G, N)
    Cm = xbc[:, inner + G * N:].reshape(T, G, N)
    y, _ = ssm_recurrence(x, Bm, Cm, softplus(dt + w[f"{p}.dt_bias"]), w[f"{p}.A_log"], w[f"{p}.D"])
    y = gated_group_rms(y.reshape(T, inner), z, w[f"{p}.norm"], m["norm_groups"], eps)
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


def greedy_generate(w, cfg, prompt: List[int], n_new: int) -> List[int]:
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(forward(w, cfg, toks)[-1].argmax()))
    return toks[len(prompt):]


def tensor_shapes(cfg: dict, rel_rows: int = 32) -> Dict[str, tuple]:
    """Every tensor name of a configuration with its shape, as a checkpoint of the design holds them."""
    W, out = cfg["width"], {}
    out["embed"] = (cfg["vocab"], W)
    if cfg["embedding"].get("bigram"):
        out["bigram"] = (cfg["embedding"]["bigram"]["buckets"] + 1, W)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}", L["mixer"]
        out[f"{p}.norm1"] = out[f"{p}.norm1b"] = (W,)
        if L["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out[f"{p}.mix.q"], out[f"{p}.mix.q.norm"] = (H * d, W), (H * d,)
            if m.get("kv_from") is None:
                out[f"{p}.mix.k"], out[f"{p}.mix.v"], out[f"{p}.mix.k.norm"] = (G * d, W), (G * dv, W), (G * d,)
            out[f"{p}.mix.rel"], out[f"{p}.mix.g"], out[f"{p}.mix.o"] = (rel_rows, H), (H, W), (W, H * dv)
        else:
            nh, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            ch = nh * P + 2 * G * N
            out[f"{p}.mix.in"] = (nh * P + ch + nh, W)
            out[f"{p}.mix.conv"], out[f"{p}.mix.conv.b"] = (ch, m["conv"]), (ch,)
            out[f"{p}.mix.dt_bias"] = out[f"{p}.mix.A_log"] = out[f"{p}.mix.D"] = (nh,)
            out[f"{p}.mix.norm"], out[f"{p}.mix.o"] = (nh * P,), (W, nh * P)
        if L.get("mlp"):
            ff = L["mlp"]["ff"]
            out[f"{p}.norm2"] = out[f"{p}.norm2b"] = (W,)
            out[f"{p}.mlp.gate"] = out[f"{p}.mlp.up"] = (ff, W)
            out[f"{p}.mlp.down"] = (W, ff)
    out["final.norm"], out["head"] = (W,), (cfg["vocab"], W)
    return out


def random_weights(cfg: dict, seed: int, rel_rows: int = 32, rel_std: float = 1.0) -> Dict[str, torch.Tensor]:
    """Random bfloat16 tensors sized so that activations stay of order one."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg, rel_rows).items():
        leaf = name.split(".")[-1]
        if name.endswith(("norm1", "norm1b", "norm2", "norm2b", "final.norm", "q.norm", "k.norm", "mix.norm")):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf == "rel":
            t = rel_std * torch.randn(shape, generator=g)
        elif leaf in ("dt_bias", "A_log"):
            t = 0.5 * torch.randn(shape, generator=g)
        elif leaf == "D":
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif leaf == "b":
            t = 0.2 * torch.randn(shape, generator=g)
        elif leaf == "conv":
            t = 0.5 * torch.randn(shape, generator=g)
        elif name in ("embed", "bigram"):
            t = 0.1 * torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / shape[-1] ** 0.5
        w[name] = t.to(torch.bfloat16)
    return w
