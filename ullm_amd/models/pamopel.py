"""Pamopel as a plan.  The stream starts as the token's row (scaled) plus a hashed-bigram row plus a sinusoidal
position row; every layer norms on both sides of each sublayer (layer norms without bias) and scales what
joins the stream; a layer's mixer is attention (q/k norm over the whole projection, no rotation, a learned
bias by distance on the scores, a sigmoid gate per head, possibly on another layer's keys and values) or a
Mamba-2 state-space mixer; its feed-forward, where it has one, is the dense gated one.  Tensor names:
``l<i>.norm1 / norm1b / norm2 / norm2b``, ``l<i>.mix.*``, ``l<i>.mlp.gate / up / down``, ``embed``, ``bigram``,
``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.model_config import PamopelConfig
from .model import Choice, ModelPlan
from .registry import register_architecture

ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "gate": "g"}
MAMBA_NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "a_log": "A_log", "d": "D",
               "norm": "norm", "out": "o"}
SWIGLU_NAMES = {"gate": "gate", "up": "up", "down": "down"}
SINUSOID_BASE = 10000.0


def pamopel_plan(cfg: PamopelConfig) -> ModelPlan:
    H, eps = cfg.hidden_size, cfg.norm_eps
    layers, order = [], []
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}", L.mixer_dict()
        norm = lambda name: Choice("norm", "layernorm", dict(size=H, eps=eps, weight_name=f"{p}.{name}"))  # noqa: E731
        if L.type == "attention":
            # the table has as many rows as the checkpoint gives it; its shape is read when the weights are bound
            bias = Choice("position", "log_distance_bias", dict(heads=m["heads"], far=m["bias_max"],
                                                                weight_name=f"{p}.mix.rel"))
            mixer = Choice("mixer", "gqa_attention", dict(
                hidden_size=H, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"], value_dim=m["vdim"],
                prefix=f"{p}.mix", position=bias, qk_norm_eps=eps, qk_norm="whole", scale=m["scale"], head_gate=True,
                own_kv="kv_from" not in m, names=ATTENTION_NAMES))
            order.append((i, m.get("kv_from", i)))
        else:
            mixer = Choice("mixer", "mamba2", dict(
                hidden_size=H, heads=m["heads"], head_dim=m["vdim"], state=m["state"], groups=m["groups"],
                conv=m["conv"], norm_groups=m["norm_groups"], norm_eps=eps, prefix=f"{p}.mix", names=MAMBA_NAMES))
            order.append((i, i))
        params = dict(mixer_norm=norm("norm1"), mixer=mixer, mixer_post=norm("norm1b"), mult=cfg.residual_mult)
        mlp = L.mlp_dict()
        if mlp is not None:
            params.update(ffn_norm=norm("norm2"), ffn_post=norm("norm2b"),
                          ffn=Choice("ffn", "swiglu", dict(hidden_size=H, intermediate_size=mlp["ff"], prefix=f"{p}.mlp",
                                                           names=SWIGLU_NAMES)))
        layers.append(Choice("block", "sandwich", params))
    embedder = Choice("embedding", "table_sum", dict(
        vocab_size=cfg.vocab_size, hidden_size=H, weight_name="embed", scale=cfg.embedding_scale,
        pair_weight_name="bigram" if cfg.bigram_buckets else None, pair_buckets=cfg.bigram_buckets,
        pair_mul_prev=cfg.bigram_mul_prev, pair_mul_cur=cfg.bigram_mul_cur, sinusoid_base=SINUSOID_BASE))
    return ModelPlan(
        vocab_size=cfg.vocab_size, hidden_size=H, embedding_weight="embed", layers=layers,
        final_norm=Choice("norm", "layernorm", dict(size=H, eps=eps, weight_name="final.norm")),
        head_weight="head", run_order=order, embedder=embedder, logit_scale=cfg.logit_scale, init_std=0.05)


register_architecture("Pamopel", PamopelConfig.from_dict, pamopel_plan)
