"""Felavik without a GPU: the reader of config.json, tensor names, the schedule from weights_of, cache groups, the
distance buckets, and the plain implementation's own mechanisms against each other."""

import copy
import math

import pytest
import torch

import plain_felavik as pf
from felavik_configs import SMALL, SMALL_B, SMALL_C, config_of, lightning, moe, parallel

from llmserve.cache.manager import CacheManager, group_layers
from llmserve.config.model_config import ConfigError
from llmserve.config.registry import architecture_of, preset
from llmserve.parts.attention_composed import bias_by_distance, distance_bucket
from llmserve.parts.model import Model
from llmserve.parts.registry import BuildContext
from llmserve.parts.spec import PagedCacheSpec, StateCacheSpec


def build(config):
    arch = architecture_of(config)
    assert arch.name == "Felavik"
    cfg = arch.config_class.from_dict(config)
    return cfg, Model(arch.build_spec(cfg), BuildContext(torch.float32, torch.device("cpu")))


def test_tensor_names_and_shapes_follow_the_configuration():
    _cfg, model = build(SMALL)
    infos = model.param_infos()
    assert infos["embed"].shape == (151, 72) and infos["head"].shape == (151, 72) and infos["final.norm"].shape == (72,)
    assert infos["l0.mix.q"].shape == (3 * 12, 72) and infos["l0.mix.v"].shape == (3 * 20, 72)
    assert infos["l0.mix.g"].shape == (60, 72) and infos["l0.mix.o"].shape == (72, 60) and infos["l0.mix.norm"].shape == (60,)
    assert infos["l1.mix.left.q"].shape == (4 * 16, 72) and infos["l1.mix.left.q.b"].shape == (64,)
    assert infos["l1.mix.left.k"].shape == (2 * 16, 72) and infos["l1.mix.left.v.b"].shape == (2 * 24,)
    assert infos["l1.mix.left.q.norm"].shape == (16,) and infos["l1.mix.left.k.norm"].shape == (16,)
    assert infos["l1.mix.left.rel"].shape == (10, 4)
    assert infos["l1.mix.left.g"].shape == (4 * 24, 72) and infos["l1.mix.left.o"].shape == (72, 96)
    assert infos["l1.mix.right.k"].shape == (2 * 16, 72) and infos["l1.mix.right.v"].shape == (2 * 8, 72)
    assert infos["l1.mix.right.g"].shape == (16, 72) and "l1.mix.right.norm" not in infos and "l1.mix.right.q.b" not in infos
    assert infos["l1.mlp.router"].shape == (6, 72) and infos["l1.mlp.e5.down"].shape == (72, 24) and "l1.mlp.e6.up" not in infos
    assert infos["l2.mlp.router"].shape == (5, 72)
    # a layer on another's tensors has none of its own; a layer without feed-forward has no second norm
    assert not [n for n in infos if n.startswith("l3.")]
    assert "l4.norm1" in infos and "l4.norm2" not in infos and "l4.norm2" in model.spec.unused_tensors


def test_a_layer_on_anothers_tensors_is_a_second_run_with_a_cache_of_its_own():
    cfg, model = build(SMALL)
    assert model.spec.schedule == (0, 1, 2, 1, 3)
    specs = model.cache_specs()
    assert specs[0] == StateCacheSpec((3, 12, 20), "float32")
    for run in (1, 3):
        pages, state = specs[run]
        assert isinstance(pages, PagedCacheSpec) and (pages.num_kv_heads, pages.head_dim, pages.v_dim) == (2, 16, 24)
        assert pages.window is None and not pages.bounded
        assert state == StateCacheSpec((2, 16, 8), "float32")
    groups = group_layers(specs)
    by_layers = {g.layers: g.spec for g in groups}
    assert (1, 3) in by_layers and isinstance(by_layers[(1, 3)], (PagedCacheSpec, StateCacheSpec))
    assert sum(1 for g in groups if g.layers == (1, 3)) == 2  # the pages and the state of the two runs
    cfg_b, model_b = build(SMALL_B)  # a chain: layer 3 names layer 2, which names layer 1
    assert cfg_b.owner(3) == 1 and model_b.spec.schedule == (0, 1, 1, 1)


def test_pages_and_slots_of_both_kinds_are_handed_out_and_come_back():
    _cfg, model = build(SMALL)
    groups = group_layers(model.cache_specs())
    manager = CacheManager(groups, 6, 4, max_seqs=2)
    manager.add_sequence("a")
    manager.add_sequence("b")
    layout = manager.append(["a", "b"], [9, 3])
    assert sorted(layout.fresh_slots) == [0, 1]
    paged = [g.group_id for g in groups if g.paged]
    assert len(paged) == 1 and manager.free_pages()[paged[0]] == 6 - 3 - 1
    manager.free_sequence("a")
    manager.add_sequence("c")
    assert manager.append(["c"], [1]).fresh_slots == [0]  # the slot that came back is cleared before it is used again
    manager.check_invariants()


def test_what_the_reader_refuses():
    def broken(change):
        c = copy.deepcopy(SMALL)
        change(c)
        with pytest.raises(ConfigError):
            architecture_of(c).config_class.from_dict(c)

    broken(lambda c: c["layers"][0].update(type="attention"))
    broken(lambda c: c["layers"][0]["mixer"].update(decay=[0.5]))
    broken(lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=3))
    broken(lambda c: c["layers"][1]["mixer"]["right"]["rot"].update(dims=7))
    broken(lambda c: c["layers"][1]["mlp"]["router"].update(top=7))
    broken(lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=4))
    broken(lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(keep=1, count=6))  # one expert kept, two chosen
    broken(lambda c: c["layers"][3].update(weights_of=9))
    broken(lambda c: (c["layers"][1].update(weights_of=3)))  # a circle
    broken(lambda c: c.update(logit_softcap=0.0))


def test_the_rows_of_a_distance_table_come_from_the_tensors_shape():
    cfg, _model = build(SMALL)
    bare = copy.deepcopy(SMALL)
    for entry in bare["layers"]:
        if entry["type"] == "parallel":
            del entry["mixer"]["left"]["bias_rows"]
    cfg = architecture_of(bare).config_class.from_dict(bare).with_tensor_shapes({"l1.mix.left.rel": (22, 4)})
    model = Model(architecture_of(bare).build_spec(cfg), BuildContext(torch.float32, torch.device("cpu")))
    assert model.param_infos()["l1.mix.left.rel"].shape == (22, 4)
    assert cfg.layers[3]["mixer"]["left"]["bias_rows"] == 22  # the run on layer 1's tensors follows


def test_named_sizes():
    for name in ("felavik-tiny", "felavik-1b"):
        _cfg, model = build(preset(name))
        assert model.graph_safe()
        assert len(model.spec.schedule) > len(model.spec.layers)  # a layer runs twice


@pytest.mark.parametrize("rows,farthest", [(10, 40), (4, 17), (32, 200), (16, 1000), (2, 5)])
def test_distance_buckets(rows, farthest):
    half = rows // 2
    seen = [distance_bucket(n, rows, farthest) for n in range(farthest + 50)]
    assert seen[:half] == list(range(half))  # a row per short distance
    assert seen == sorted(seen) and seen[-1] == rows - 1 and all(b == rows - 1 for b in seen[farthest:])
    assert seen == [pf.distance_bucket(n, rows, farthest) for n in range(farthest + 50)]
    # past the rows of single distances a row's span grows by the same factor from row to row
    for n in range(half, farthest):
        exact = half + math.log(n / half) / math.log(farthest / half) * (rows - half)
        assert seen[n] == min(rows - 1, math.floor(exact))
    table = torch.randn(rows, 3, generator=torch.Generator().manual_seed(rows))
    flat = bias_by_distance(table, farthest)
    reach = flat.shape[1] - 1
    assert reach <= farthest and seen[reach] == rows - 1 and (reach == 0 or seen[reach - 1] < rows - 1 or reach == half)
    for n in range(farthest + 50):
        assert torch.equal(flat[:, min(n, reach)], table[seen[n]].float())


# ------------------------------------------------------------------------------ the plain implementation by itself
def test_the_recurrence_is_the_decayed_sum_over_earlier_keys():
    g = torch.Generator().manual_seed(3)
    t, heads, dk, dv = 9, 2, 5, 4
    q, k, v = (torch.randn(t, heads, d, generator=g, dtype=torch.float64) for d in (dk, dk, dv))
    decay = [0.8, 1.0]
    got = pf.decayed_sums(q, k, v, decay)
    for a in range(heads):
        for i in range(t):
            want = sum(decay[a] ** (i - j) * float(q[i, a] @ k[j, a]) * v[j, a] for j in range(i + 1))
            assert torch.allclose(got[i, a], want, atol=1e-12)


def test_the_rotation_turns_pairs_half_a_rotated_part_apart():
    x = torch.zeros(3, 1, 6, dtype=torch.float64)
    x[:, 0, 0] = 1.0  # partner of dimension 0 is dimension 2 when 4 dimensions turn
    x[:, 0, 5] = 7.0
    y = pf.rotate_half(x, base=10.0, dims=4)
    for p in range(3):
        assert math.isclose(float(y[p, 0, 0]), math.cos(p)) and math.isclose(float(y[p, 0, 2]), math.sin(p), abs_tol=1e-15)
        assert float(y[p, 0, 1]) == 0.0 and float(y[p, 0, 3]) == 0.0 and float(y[p, 0, 5]) == 7.0
    # a score of rotated q and k depends on the distance alone
    g = torch.Generator().manual_seed(5)
    q, k = torch.randn(1, 1, 8, generator=g, dtype=torch.float64), torch.randn(1, 1, 8, generator=g, dtype=torch.float64)
    qs, ks = pf.rotate_half(q.expand(20, 1, 8), 100.0, 6), pf.rotate_half(k.expand(20, 1, 8), 100.0, 6)
    assert math.isclose(float(qs[7, 0] @ ks[3, 0]), float(qs[19, 0] @ ks[15, 0]), rel_tol=1e-9)


def test_only_experts_of_the_best_groups_are_chosen():
    h = torch.eye(8, dtype=torch.float64)[:1]  # logits are the router's first column
    logits = torch.tensor([5.0, 0.0, 4.9, 4.8, 0.1, 0.2, 4.7, 0.3], dtype=torch.float64)
    router = logits[:, None] * torch.eye(1, 8, dtype=torch.float64)  # [experts, hidden]: the first column holds the logits
    chosen, weights = pf.route(h, router, top=2, groups=4, keep=1)
    assert chosen.tolist() == [[0, 1]]  # group 0 holds the best expert; its second is chosen before better ones elsewhere
    chosen, weights = pf.route(h, router, top=3, groups=4, keep=2)
    assert chosen.tolist() == [[0, 2, 3]] and math.isclose(float(weights.sum()), 1.0)
    s = torch.softmax(logits, 0)
    assert torch.allclose(weights[0], s[[0, 2, 3]] / s[[0, 2, 3]].sum())


def test_the_query_factor_steps_up_every_so_many_positions():
    f = pf.query_temperature(30, 0.5, 8, torch.float64)
    assert float(f[0]) == 1.0 and float(f[6]) == 1.0 and math.isclose(float(f[7]), 1 + 0.5 * math.log(2))
    assert math.isclose(float(f[22]), 1 + 0.5 * math.log(3)) and math.isclose(float(f[23]), 1 + 0.5 * math.log(4))
