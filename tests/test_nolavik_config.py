"""Nolavik without a GPU: the configuration reader and what it refuses, the order of layer runs and the shifts of a loop,
tensor names and shapes, what each run keeps between steps, and the frequencies of a stretched rotation."""

import math

import pytest
import torch

import plain_nolavik as pn
from nolavik_configs import SMALL, SMALL_B, SMALL_C, SMALL_D, config_of, delta, latent, moe, parallel


def spec_of(config):
    from llmserve.models.nolavik import NolavikConfig, nolavik_spec

    return nolavik_spec(NolavikConfig.from_dict(config))


def model_of(config):
    from llmserve.parts.model import Model
    from llmserve.parts.registry import BuildContext

    return Model(spec_of(config), BuildContext(torch.float32, torch.device("cpu")))


def test_the_registry_finds_the_design_by_its_name():
    from llmserve.config.registry import architecture_of, preset

    assert architecture_of(SMALL).name == "Nolavik"
    assert architecture_of(preset("nolavik-tiny")).name == "Nolavik"


@pytest.mark.parametrize("config", [SMALL, SMALL_B, SMALL_C, SMALL_D])
def test_layer_runs_and_shifts_follow_the_loop(config):
    spec = spec_of(config)
    runs = pn.layer_runs(config)
    assert list(spec.schedule) == [i for i, _ in runs]
    assert list(spec.shifts) == [(pos, k) for pos, (_, k) in enumerate(runs) if k is not None]
    loop = config.get("loop")
    if loop:
        assert len(spec.shifts) == loop["times"]
        assert len(spec.schedule) == len(config["layers"]) + (loop["times"] - 1) * (loop["stop"] - loop["start"])
    else:
        assert not spec.shifts and "shifts" not in spec.weights


def test_tensor_names_and_shapes():
    infos = model_of(SMALL).param_infos()
    shape = {k: tuple(v.shape) for k, v in infos.items()}
    w = SMALL["width"]
    assert shape["embed"] == (151, w) and shape["head"] == (151, w) and shape["final.norm"] == (w,)
    assert shape["loop.step"] == (3, w)
    for i in range(4):
        for name in ("norm1", "norm1b", "norm2", "norm2b"):
            assert shape[f"l{i}.{name}"] == (w,)
    assert shape["l0.mix.dq"] == (24, w) and shape["l0.mix.dq.norm"] == (24,) and shape["l0.mix.uq"] == (3 * 20, 24)
    assert shape["l0.mix.dkv"] == (48, w) and shape["l0.mix.dkv.norm"] == (40,)
    assert shape["l0.mix.uk"] == (36, 40) and shape["l0.mix.uv"] == (60, 40) and shape["l0.mix.o"] == (w, 60)
    assert shape["l1.mix.q"] == (24, w) and shape["l1.mix.k"] == (24, w) and shape["l1.mix.v"] == (80, w)
    assert shape["l1.mix.q.conv"] == (24, 3) and shape["l1.mix.v.conv"] == (80, 3)
    assert shape["l1.mix.b"] == (4, w) and shape["l1.mix.a"] == (4, w) and shape["l1.mix.A_log"] == (4,)
    assert shape["l1.mix.dt_bias"] == (4,) and shape["l1.mix.norm"] == (20,) and shape["l1.mix.g"] == (80, w)
    assert shape["l1.mix.o"] == (w, 80)
    assert shape["l2.mix.left.q"] == (96, w) and shape["l2.mix.left.k"] == (48, w) and shape["l2.mix.left.v"] == (24, w)
    assert shape["l2.mix.left.o"] == (w, 48)
    assert shape["l2.mix.right.in"] == (112, w) and shape["l2.mix.right.conv"] == (56, 4) and shape["l2.mix.right.conv.b"] == (56,)
    assert shape["l2.mix.right.x"] == (6 + 10, 56) and shape["l2.mix.right.dt"] == (56, 6) and shape["l2.mix.right.dt.b"] == (56,)
    assert shape["l2.mix.right.A_log"] == (56, 5) and shape["l2.mix.right.D"] == (56,) and shape["l2.mix.right.o"] == (w, 56)
    assert shape["l0.mlp.router"] == (6, w) and shape["l0.mlp.router.b"] == (6,)
    assert shape["l0.mlp.e5.gate"] == (24, w) and shape["l0.mlp.e5.down"] == (w, 24)
    assert shape["l0.mlp.shared.gate"] == (40, w) and shape["l0.mlp.shared.down"] == (w, 40) and shape["l0.mlp.shared.sg"] == (1, w)
    assert "l3.mlp.shared.gate" not in shape and "l3.mlp.e4.up" in shape and "l3.mlp.e5.up" not in shape
    # a layer without a feed-forward has no second pair of norms of its own, and a checkpoint may still hold them
    infos_b = model_of(SMALL_B).param_infos()
    assert "l1.norm2" not in infos_b and "l1.norm2b" not in infos_b and "l1.mlp.router" not in infos_b
    assert {"l1.norm2", "l1.norm2b"} <= set(spec_of(SMALL_B).unused_tensors)
    assert "loop.step" not in infos_b


def test_every_run_keeps_a_cache_of_its_own():
    from llmserve.parts.spec import PagedCacheSpec, StateCacheSpec

    specs = model_of(SMALL).cache_specs()
    assert len(specs) == 8  # 0, (1, 2) x 3, 3
    assert isinstance(specs[0], PagedCacheSpec) and specs[0].head_dim == 48 and specs[0].v_heads == 0
    for pos in (1, 3, 5):
        assert specs[pos] == StateCacheSpec((4 * 12 * 20 + 2 * (24 + 24 + 80),), "float32")
    for pos in (2, 4, 6):
        pages, state = specs[pos]
        assert (pages.num_kv_heads, pages.head_dim, pages.v_dim, pages.window) == (2, 24, 12, None)
        assert state == StateCacheSpec((56 * 5 + 3 * 56,), "float32")
    assert specs[7] == StateCacheSpec((2 * 40 * 8 + 1 * (80 + 80 + 16),), "float32")
    # one tap: no ring
    assert model_of(SMALL_B).cache_specs()[0][1] == StateCacheSpec((9 * 24,), "float32")


def test_the_manager_gives_pages_and_a_slot_and_takes_them_back():
    from llmserve.cache.manager import CacheManager  # noqa: F401  (the manager is exercised through the runner on the GPU)

    model = model_of(SMALL_C)
    assert len(model.cache_specs()) == 6 and model.cache_sources() == [None] * 6


@pytest.mark.parametrize("bad", [
    lambda c: c["layers"][0].update(type="attention"),
    lambda c: c.update(loop={"start": 2, "stop": 9, "times": 2}),
    lambda c: c.update(loop={"start": 1, "stop": 3, "times": 0}),
    lambda c: c["layers"][2]["mixer"]["left"].update(heads=3),
    lambda c: c["layers"][2]["mixer"]["left"]["rot"].update(dims=26),
    lambda c: c["layers"][2]["mixer"]["left"]["rot"].update(dims=7),
    lambda c: c["layers"][2]["mixer"]["left"]["rot"]["scaling"].pop("original"),
    lambda c: c["layers"][2]["mixer"]["right"].update(state=0),
    lambda c: c["layers"][1]["mixer"].update(kv_heads=3),
    lambda c: c["layers"][0]["mixer"].pop("scale"),
    lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10),
    lambda c: c["layers"][0]["mlp"]["router"].update(top=7),
    lambda c: c["layers"][0]["mlp"].update(kind="dense"),
    lambda c: c["layers"][0]["mlp"]["shared"].update(ff=0),
    lambda c: c.pop("vocab"),
])
def test_what_the_reader_refuses(bad):
    import copy

    from llmserve.config.model_config import ConfigError
    from llmserve.models.nolavik import NolavikConfig

    config = copy.deepcopy(SMALL)
    bad(config)
    with pytest.raises(ConfigError):
        NolavikConfig.from_dict(config)


def test_the_configuration_goes_to_json_and_back():
    from llmserve.models.nolavik import NolavikConfig

    for config in (SMALL, SMALL_B):
        cfg = NolavikConfig.from_dict(config)
        assert NolavikConfig.from_dict(cfg.to_dict()) == cfg


def test_stretched_frequencies():
    """All three regimes: short wavelengths stay, long ones are divided by the factor, those between are blended."""
    from llmserve.parts.attention_composed import scaled_frequencies

    scaling = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
    got = scaled_frequencies(100.0, 16, scaling)
    want = pn.frequencies(100.0, 16, scaling)
    assert got == pytest.approx(want.tolist(), rel=1e-15)
    plain = [100.0 ** (-2.0 * i / 16) for i in range(8)]
    kinds = set()
    for f, g in zip(plain, got):
        wave = 2 * math.pi / f
        if wave < 16:
            assert g == f
            kinds.add("kept")
        elif wave > 64:
            assert g == pytest.approx(f / 8)
            kinds.add("divided")
        else:
            assert f / 8 < g < f
            kinds.add("blended")
    assert kinds == {"kept", "divided", "blended"}
    assert scaled_frequencies(100.0, 16, None) == plain and scaled_frequencies(10.0, 0, scaling) == []


def test_the_plain_router_takes_the_softmax_over_the_chosen_logits_alone():
    t = {"router": torch.tensor([[1.0], [3.0], [2.0], [-1.0]], dtype=torch.float64), "router.b": torch.tensor([0.0, 0.0, 2.0, 0.0], dtype=torch.float64)}
    idx, w = pn.route(torch.ones(1, 1, dtype=torch.float64), t, "", 2)
    assert idx.tolist() == [[2, 1]]  # the bias lifts expert 2 over expert 1
    assert w[0].tolist() == pytest.approx([math.e / (1 + math.e), 1 / (1 + math.e)])
