"""Pamopel without a GPU: the configuration reader, the plan it becomes (run order, tensor names and shapes),
the distance table's rows, and a checkpoint's own row count for that table."""
import copy

import pytest
import torch

import plain_pamopel as plain
from ullm_amd.config import ConfigError, PamopelConfig
from ullm_amd.models import build_model
from ullm_amd.parts.position import LogDistanceBias, log_distance_bucket
from ullm_amd.weights.loader import WeightError, check_against

CFG = dict(architecture="Pamopel", vocab=70, width=24, residual_mult=0.4, logit_scale=1.25, norm=dict(eps=1e-4),
           embedding=dict(scale=2.0, bigram=dict(buckets=13, mul_prev=5, mul_cur=9)),
           layers=[dict(type="mamba2", mixer=dict(heads=2, vdim=6, state=10, groups=1, conv=3, norm_groups=2), mlp=None),
                   dict(type="attention", mixer=dict(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.3, bias_max=20),
                        mlp=dict(kind="dense", ff=36)),
                   dict(type="attention", mixer=dict(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.3, bias_max=20, kv_from=1),
                        mlp=None)])


def test_the_plan_names_every_tensor_of_the_design_with_its_shape():
    cfg, model = build_model(CFG)
    assert isinstance(cfg, PamopelConfig) and cfg.num_hidden_layers == 3
    declared = {d.name: tuple(d.shape) for d in model.weight_decls()}
    assert declared == plain.tensor_shapes(CFG, rel_rows=LogDistanceBias.DEFAULT_ROWS)
    assert model.run_order == [(0, 0), (1, 1), (2, 1)]
    groups, cache_group, states = model.cache_layout()
    assert len(groups) == 1 and groups[0].num_kv_heads == 2 and groups[0].head_dim == 32 and groups[0].layers == ((1, 0),)
    assert sorted(states) == [(-1, 0), (0, 0)]
    assert states[(0, 0)].shape == ((3 - 1) * (12 + 20) + 2 * 10 * 6,) and states[(-1, 0)].dtype == torch.int32


def test_a_checkpoint_decides_the_rows_of_its_distance_table():
    _, model = build_model(CFG)
    index = {n: ("f", s, "BF16") for n, s in plain.tensor_shapes(CFG, rel_rows=7).items()}
    check_against(model.weight_decls(), index)
    index["l1.mix.rel"] = ("f", (7, 5), "BF16")
    with pytest.raises(WeightError, match="l1.mix.rel"):
        check_against(model.weight_decls(), index)


@pytest.mark.parametrize("rows,far", [(32, 240), (8, 16), (13, 37), (6, 50), (32, 256), (9, 1000), (2, 5)])
def test_rows_of_the_distance_table(rows, far):
    part = LogDistanceBias(heads=1, far=far, weight_name="t", rows=rows)
    by_distance = part.buckets()
    assert by_distance == [plain.distance_bucket(n, rows, far) for n in range(len(by_distance))]
    assert by_distance[-1] == rows - 1 and rows - 1 not in by_distance[:-1]
    assert all(plain.distance_bucket(n, rows, far) == rows - 1 for n in (len(by_distance), far, 3 * far, 10 ** 6))
    assert all(b - a in (0, 1) or a < rows // 2 for a, b in zip(by_distance, by_distance[1:])) or rows - rows // 2 > 1
    assert [log_distance_bucket(n, rows, far) for n in range(rows // 2)] == list(range(rows // 2))


def test_configurations_that_are_refused():
    for change, text in ((lambda c: c["layers"][2]["mixer"].update(kv_from=0), "kv_from"),
                         (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "kv_from"),
                         (lambda c: c["layers"][1].update(type="conv"), "type"),
                         (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
                         (lambda c: c["layers"][1]["mlp"].update(kind="experts"), "mlp"),
                         (lambda c: c.pop("width"), "width"), (lambda c: c["norm"].pop("eps"), "eps")):
        bad = copy.deepcopy(CFG)
        change(bad)
        with pytest.raises(ConfigError, match=text):
            PamopelConfig.from_dict(bad)
