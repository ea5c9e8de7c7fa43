"""The Ziferax configuration reader and plan, without a GPU."""
import copy

import pytest

from ullm_amd.config import ConfigError, ZiferaxConfig
from ullm_amd.models import build_model


def base():
    mixer = dict(heads=4, kv_heads=2, dim=32, vdim=32, mask=dict(size=24), rot=dict(base=10000.0, dims=8), scale=0.2)
    mlp = dict(kind="moe", router=dict(experts=6, identity=2, top=2), expert=dict(ff=24, limit=1.5), shared=dict(ff=40, limit=2.0))
    first = dict(type="attention", mixer=mixer, mlp=mlp)
    second = dict(type="attention", mixer=dict(mixer, heads=2, kv_heads=1, dim=64, vdim=64), mlp=None)
    return dict(architecture="Ziferax", vocab=97, width=64, norm=dict(eps=1e-5), residual_mult=0.3,
                layers=[first, second, dict(copy.deepcopy(first), weights_of=0)])


def test_every_size_and_constant_is_read():
    cfg = ZiferaxConfig.from_dict(base())
    assert (cfg.vocab_size, cfg.hidden_size, cfg.norm_eps, cfg.residual_mult, cfg.num_hidden_layers) == (97, 64, 1e-5, 0.3, 3)
    m, f = cfg.layers[0].mixer, cfg.layers[0].mlp
    assert (m.heads, m.kv_heads, m.dim, m.scale, m.window, m.rot_dims, m.rot_base) == (4, 2, 32, 0.2, 24, 8, 10000.0)
    assert (f.experts, f.identity, f.top, f.ff, f.limit, f.shared_ff, f.shared_limit) == (6, 2, 2, 24, 1.5, 40, 2.0)
    assert cfg.layers[1].mlp is None and cfg.layers[2].weights_of == 0 and cfg.layers[0].weights_of is None


def test_a_layer_that_uses_another_layers_tensors_declares_none_and_keeps_a_cache_of_its_own():
    _, model = build_model(base())
    assert model.run_order == [(0, 0), (1, 1), (0, 2)]
    names = [d.name for d in model.weight_decls()]
    assert not any(n.startswith("l2.") for n in names)
    assert {"embed", "l0.norm1", "l0.mix.q", "l0.mix.q.b", "l0.mix.k", "l0.mix.k.b", "l0.mix.o", "l0.mix.o.b", "l0.mix.sink",
            "l0.mlp.router", "l0.mlp.correction", "l0.mlp.e5.down", "l0.mlp.shared.up", "l1.mix.sink", "final.norm"} <= set(names)
    assert not any(n.endswith(".v") or ".mlp.e6." in n or n.startswith("l1.mlp") for n in names)
    router = next(d for d in model.weight_decls() if d.name == "l0.mlp.router")
    assert router.shape == (8, 64) and router.keep_fp32              # experts + identity outputs, held in 32-bit
    head = next(d for d in model.weight_decls() if d.name == "head")
    assert head.alias_of == "embed"                                   # the head is the embedding table
    groups, _, states = model.cache_layout()
    assert not states and sorted(len(g.layers) for g in groups) == [1, 2]
    assert {g.window for g in groups} == {24}


@pytest.mark.parametrize("change,what", [
    (lambda c: c["layers"][0]["mixer"].update(vdim=16), "vdim"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "heads"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "top"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "kind"),
    (lambda c: c["layers"][2].update(weights_of=2), "weights_of"),
    (lambda c: c["layers"][2].update(weights_of=7), "weights_of"),
    (lambda c: c["layers"][2].update(weights_of=1), "differ"),
    (lambda c: c["layers"][1].update(type="mamba2"), "type"),
    (lambda c: c.pop("width"), "width"),
])
def test_configurations_that_cannot_be_served_are_refused(change, what):
    c = base()
    change(c)
    with pytest.raises(ConfigError, match=what):
        ZiferaxConfig.from_dict(c)


def test_keys_a_model_may_leave_out():
    c = base()
    del c["layers"][0]["mlp"]["shared"], c["layers"][2]["mlp"]["shared"]
    c["layers"][0]["mlp"]["router"].pop("identity")
    c["layers"][2]["mlp"]["router"].pop("identity")
    c.pop("residual_mult")
    cfg = ZiferaxConfig.from_dict(c)
    assert cfg.layers[0].mlp.shared_ff == 0 and cfg.layers[0].mlp.identity == 0 and cfg.residual_mult == 1.0


def test_a_chain_of_layers_that_use_anothers_tensors_is_followed():
    c = base()
    c["layers"].append(dict(copy.deepcopy(c["layers"][0]), weights_of=2))
    cfg = ZiferaxConfig.from_dict(c)
    assert cfg.layers[3].weights_of == 0
    assert build_model(c)[1].run_order == [(0, 0), (1, 1), (0, 2), (0, 3)]
