"""Ziferax as a plan.  Every layer is a parallel block: one RMS norm whose output both the attention mixer and
the routed feed-forward read, and a multiplier on their sum.  Attention has biases on q, k and the output, no
value projection (the values are the keys before rotation), rotation of adjacent pairs over the first dims of
each head, a sliding window and a sink per head; the feed-forward routes each token to a few of many small
clamped gated units (some of them identity experts without tensors) and adds a shared one.  A layer may use
another layer's tensors with a cache of its own: it runs that layer's parts under its own cache id.  The head is
the embedding table.  Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.mix.q / q.b / k / k.b / o / o.b / sink``,
``l<i>.mlp.router / correction / e<j>.gate|up|down / shared.gate|up|down``, ``final.norm``.
"""
from __future__ import annotations

from ..config.model_config import ZiferaxConfig
from .model import Choice, ModelPlan
from .registry import register_architecture

ATTENTION_NAMES = {"q": "q", "k": "k", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "o_bias": "o.b", "sink": "sink"}
SWISH_SLOPE = 1.702          # the gated unit's sigmoid takes this times the gate


def ziferax_plan(cfg: ZiferaxConfig) -> ModelPlan:
    H, eps = cfg.hidden_size, cfg.norm_eps
    layers, index_of, order = [], {}, []
    for i, L in enumerate(cfg.layers):
        if L.weights_of is not None:
            continue
        p, m = f"l{i}", L.mixer
        position = None
        if m.rot_dims:
            position = Choice("position", "rotary", dict(head_dim=m.dim, theta=m.rot_base, rotary_dim=m.rot_dims,
                                                         pairing="adjacent", max_positions=None))
        mixer = Choice("mixer", "gqa_attention", dict(
            hidden_size=H, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, prefix=f"{p}.mix",
            position=position, bias=True, out_bias=True, window=m.window, scale=m.scale, values="keys", sink=True,
            names=ATTENTION_NAMES))
        params = dict(norm=Choice("norm", "rmsnorm", dict(size=H, eps=eps, weight_name=f"{p}.norm1")), mixer=mixer,
                      mult=cfg.residual_mult)
        if L.mlp is not None:
            f = L.mlp
            params["ffn"] = Choice("ffn", "routed_experts", dict(
                hidden_size=H, experts=f.experts, intermediate_size=f.ff, top=f.top, limit=f.limit, identity=f.identity,
                alpha=SWISH_SLOPE, shared_size=f.shared_ff, shared_limit=f.shared_limit, prefix=f"{p}.mlp"))
        index_of[i] = len(layers)
        layers.append(Choice("block", "parallel", params))
    for i, L in enumerate(cfg.layers):
        # a layer that uses another's tensors runs that layer's parts on a cache of its own
        order.append((index_of[i if L.weights_of is None else L.weights_of], i))
    return ModelPlan(
        vocab_size=cfg.vocab_size, hidden_size=H, embedding_weight="embed", layers=layers,
        final_norm=Choice("norm", "rmsnorm", dict(size=H, eps=eps, weight_name="final.norm")),
        head_weight="head", tie_head_to_embedding=True, run_order=order, init_std=0.05)


register_architecture("Ziferax", ZiferaxConfig.from_dict, ziferax_plan)
